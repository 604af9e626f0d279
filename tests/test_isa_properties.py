"""Properties of the compiled device code that neither the oracle nor the emulation can see, read from the compiler's
assembly output for gfx950 (hipcc -S of this repository's own sources, with the Makefile's flags): the hardware rule
around the global->LDS loads' M0 operand, the absence of scratch (spill) accesses in the kernels whose speed rests on
it, and the shape of the hand-ordered K loop of the four-wave kernel. A change that makes the register allocator
spill inside a K loop, or lets the compiler regroup the loop's loads, fails here instead of showing up as a slower
benchmark."""
import collections
import os
import re
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "applied-ai_amd", "csrc")
HIPCC = "/opt/rocm/bin/hipcc"
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-S", "--cuda-device-only"]
FILES = sorted(f for f in os.listdir(CSRC) if f.endswith(".hip") and f != "api.hip")   # every kernel file, compiled once

if not os.path.exists(HIPCC):
    pytest.skip("hipcc not found", allow_module_level=True)


def _compile(name, out_dir):
    out = os.path.join(out_dir, name.replace(".hip", ".s"))
    subprocess.run([HIPCC] + FLAGS + [os.path.join(CSRC, name), "-o", out], check=True, stdout=subprocess.DEVNULL,
                   stderr=subprocess.DEVNULL)
    return open(out).read()


@pytest.fixture(scope="module")
def asm(tmp_path_factory):
    d = str(tmp_path_factory.mktemp("isa"))
    with ThreadPoolExecutor(8) as ex:
        texts = list(ex.map(lambda f: _compile(f, d), FILES))
    shutil.rmtree(d, ignore_errors=True)
    return dict(zip(FILES, texts))


def kernels(text):
    """name -> (instruction lines, metadata text) of every kernel of an assembly file."""
    out = {}
    for m in re.finditer(r"^(_Z[^\n:]+):\s*; @\S+\n(.*?)\n\.Lfunc_end", text, re.S | re.M):
        lines = [re.sub(r"\s*;.*", "", l).strip() for l in m.group(2).splitlines()]
        meta = re.search(r"\.amdhsa_kernel " + re.escape(m.group(1)) + r"\n(.*?)\.end_amdhsa_kernel", text, re.S)
        out[m.group(1)] = ([l for l in lines if l], meta.group(1) if meta else "")
    return out


def scratch_bytes(meta):
    return int(re.search(r"\.amdhsa_private_segment_fixed_size (\d+)", meta).group(1))


def loops(lines):
    """Instruction lists of the backward-branch loops of a kernel."""
    idx = {l[:-1]: i for i, l in enumerate(lines) if l.endswith(":")}
    for i, l in enumerate(lines):
        m = re.match(r"s_c?branch\w*\s+(\.LBB\S+)", l)
        if m and m.group(1) in idx and idx[m.group(1)] < i:
            yield lines[idx[m.group(1)]:i + 1]


def count(seg, prefix):
    return sum(1 for l in seg if l.startswith(prefix))


def test_m0_is_written_one_wait_state_before_every_lds_dma(asm):
    """global_load_lds_* takes its LDS address from M0; the hardware needs one wait state between the scalar write of
    M0 and the load. Every such load in the compiled code must come from the tree's dma helpers (s_mov_b32 m0; s_nop 0;
    load), and no global load with a register destination may come from inline assembly (the emulated build rejects
    unknown asm templates; this checks the compiled result)."""
    seen = 0
    for name, text in asm.items():
        for kname, (lines, _) in kernels(text).items():
            ins = [l for l in lines if not l.endswith(":")]
            for i, l in enumerate(ins):
                if l.startswith("global_load_lds_dword"):
                    seen += 1
                    assert ins[i - 1] == "s_nop 0" and ins[i - 2].startswith("s_mov_b32 m0,"), (name, kname, ins[i - 2:i + 1])
    assert seen > 100


def test_hot_kernels_do_not_touch_scratch(asm):
    k = kernels(asm["gg_pingpong.hip"])
    for want in ("gg_bf16_pingpongE", "gg_f16_pingpongE", "gg_bf16_pingpong_swigluE", "gg_bf16_pingpong_ntE",
                 "gg_bf16_pingpong_wgrad_directE", "gg_bf16_pingpong_wgradE", "gg_fp8_pingpong_rowwiseE"):
        (name, (lines, meta)), = [(n, v) for n, v in k.items() if want in n]
        assert scratch_bytes(meta) == 0, name
    (name, (lines, meta)), = [(n, v) for n, v in k.items() if "gg_fp8_pingpong_blockE" in n]
    assert scratch_bytes(meta) <= 32, name          # a handful of spills outside the K loop
    for seg in loops(lines):
        if count(seg, "v_mfma") >= 32 and len(seg) < 1500:   # the K loops (the tile loop around them is longer)
            assert count(seg, "scratch_") == 0, name
    for name, (lines, meta) in kernels(asm["w4a16.hip"]).items():
        if "w4a16_splitk_g128" in name:
            assert scratch_bytes(meta) == 0, name
            vgpr = int(re.search(r"\.amdhsa_next_free_vgpr (\d+)", meta).group(1))
            four_waves = "ELi4ELi1ELi4E" in name        # <FP16, MF = 4, GA = 1, NWAVES = 4, ...>: one wave per SIMD
            warm = re.search(r"ELi2ELb[01]EEEv8W4Params$", name) is not None   # ten waves: three on some SIMDs
            assert vgpr <= (512 if four_waves else 168 if warm else 256), (name, vgpr)
            lds = int(re.search(r"\.amdhsa_group_segment_fixed_size (\d+)", meta).group(1))
            assert lds <= 160 << 10, (name, lds)        # the staged forms add 4 KB of LDS per wave and fragment


def test_tall_tile_k_loop(asm):
    """The four-wave kernels with tiles of up to 288 rows: the K-step loop has the 128 MFMAs of the plain form plus the
    16 hand-written ones of the ninth activation fragment (VGPR accumulators), 34 fragment reads, 17 slab loads, and
    still no accumulator moves and no scratch access; the hand-written MFMAs keep their accumulators in the same
    registers in both half steps."""
    for want in ("gg_bf16_fourwave_tallE", "gg_f16_fourwave_tallE", "gg_bf16_fourwave_tall_swigluE", "gg_f16_fourwave_tall_swigluE"):
        (name, (lines, meta)), = [(n, v) for n, v in kernels(asm["gg_pingpong.hip"]).items() if want in n]
        main = [seg for seg in loops(lines) if count(seg, "v_mfma") == 144 and count(seg, "global_load_lds_dwordx4") == 17]
        assert main, name
        seg = min(main, key=len)
        assert count(seg, "ds_read_b128") == 34 and count(seg, "s_barrier") == 1
        assert count(seg, "v_accvgpr") == 0 and count(seg, "scratch_") == 0
        assert len(seg) <= 345, len(seg)
        hand = [l for l in seg if re.match(r"v_mfma_f32_16x16x32_\w+ v\[", l)]       # VGPR destination: the hand-written ones
        assert len(hand) == 16
        dst = [re.match(r"v_mfma\S+ (v\[\d+:\d+\]), \S+ \S+ (v\[\d+:\d+\])", l).groups() for l in hand]
        assert all(d == c for d, c in dst) and sorted(d for d, _ in dst[:8]) == sorted(d for d, _ in dst[8:])
        lds = int(re.search(r"\.amdhsa_group_segment_fixed_size (\d+)", meta).group(1))
        assert lds <= 160 << 10, lds


def test_four_wave_k_loop_is_what_the_source_spells_out(asm):
    """gg_bf16_fourwave / gg_f16_fourwave and their SiLU-and-mul forms: one K-step loop of 128 MFMAs with 32 fragment reads and 16 slab loads
    between them, no accumulator moves, no scratch access, no branch but the back edge (and the one around the load
    cursor's tile change), and never more than five other instructions between two MFMAs of a half step."""
    for want in ("gg_bf16_fourwaveE", "gg_f16_fourwaveE", "gg_bf16_fourwave_swigluE", "gg_f16_fourwave_swigluE"):
        (name, (lines, meta)), = [(n, v) for n, v in kernels(asm["gg_pingpong.hip"]).items() if want in n]
        main = [seg for seg in loops(lines) if count(seg, "v_mfma") == 128 and count(seg, "global_load_lds_dwordx4") == 16]
        assert main, name
        seg = min(main, key=len)
        assert count(seg, "ds_read_b128") == 32
        assert count(seg, "v_accvgpr") == 0 and count(seg, "scratch_") == 0
        assert count(seg, "s_barrier") == 1
        assert len(seg) <= 300, len(seg)
        ins = [l for l in seg if not l.endswith(":")]
        gaps, run = [], 0
        for l in ins:
            if l.startswith("v_mfma"):
                gaps.append(run)
                run = 0
            else:
                run += 1
        gaps = sorted(gaps[1:])
        # two long gaps (loop entry / the waits and the barrier between the halves), everything else short
        assert gaps[-3] <= 6, gaps[-8:]
    # the same for the lock-step tiled kernel on four waves
    (name, (lines, meta)), = [(n, v) for n, v in kernels(asm["gg_bf16_prefill.hip"]).items() if "Li256ELi256ELi2ELi2EEELb0ELb0E" in n]
    main = [seg for seg in loops(lines) if count(seg, "v_mfma") == 128 and count(seg, "global_load_lds_dwordx4") == 16]
    assert main and count(min(main, key=len), "v_accvgpr") == 0 and count(min(main, key=len), "scratch_") == 0


def test_pingpong_k_loops_keep_their_instruction_mix(asm):
    """The eight-wave ping-pong kernels: no scratch and no accumulator moves in any loop that holds MFMAs."""
    for name, (lines, meta) in kernels(asm["gg_pingpong.hip"]).items():
        if "fourwave" in name:
            continue
        for seg in loops(lines):
            if count(seg, "v_mfma") >= 32 and len(seg) < 1500:
                assert count(seg, "scratch_") == 0 and count(seg, "v_accvgpr") == 0, (name, len(seg))


def test_default_kernels_are_the_gpu_tested_code(asm):
    """Every kernel of the last commit whose tree passed the GPU suite on an MI355X (tests/golden/isa_fingerprints.json,
    made by tests/golden/make_isa_fingerprints.py) compiles from the working tree to the same instruction stream: the
    kernels that run by default are that code, and what was written since lives in kernels of its own (selectable
    variants). The normalisation is the generator's: labels, the offset of the first hidden kernel argument, the order
    inside runs of scalar register copies."""
    import importlib.util
    import json

    spec = importlib.util.spec_from_file_location("make_isa_fingerprints", os.path.join(ROOT, "tests", "golden", "make_isa_fingerprints.py"))
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    golden = json.load(open(os.path.join(ROOT, "tests", "golden", "isa_fingerprints.json")))
    assert gen.FLAGS == FLAGS
    now = {f: {k: gen.fingerprint(v) for k, v in gen.kernels(asm[f]).items()} for f in FILES}
    checked = 0
    for f, ks in golden["kernels"].items():
        for name, fp in ks.items():
            # the group-size-128 W4A16 kernel has two more template arguments now: <..., WARM = 0, STAGE = false>
            new = name.replace("EEEv8W4Params", "ELi0ELb0EEEv8W4Params") if "w4a16_splitk_g128" in name else name
            assert new in now[f], (f, name)
            assert now[f][new] == fp, (f, name)
            checked += 1
    assert checked >= 80

