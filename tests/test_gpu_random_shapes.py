"""Random shapes and expert-size distributions. The forward product of the generic HIP kernel (one thread per output
element, fp32 accumulation in k order) is checked against the oracle's per-expert fp32 matmul loop on the CPU
(dev/triton_groupGEMM/testing/unit_tests.py:49-55) for every case, and every fast kernel against the generic one; the
fused SiLU-and-mul GEMM and the backward pass are compared with the generic kernel's path only (their oracle tests are
tests/test_gpu_moe_layer.py and tests/test_gpu_backward.py). Covers what the fixed oracle cases miss:
tile tables with many experts, empty experts, sizes around the tile edges, N and K that are not multiples of the
tiles. Bar: the grouped-GEMM bar of the parity tests, 1e-2 + 1e-2 |ref| on bf16 results (the two sides round the
same fp32 sums, accumulated in different orders)."""
import random

import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu

GENERIC, PINGPONG, AUTO = 4, 0, -1


def sizes_for(rng, G, M):
    kind = rng.choice(["even", "rand", "zipf", "sparse"])
    if kind == "even":
        ms = [M // G] * G
    elif kind == "rand":
        cuts = sorted(rng.randint(0, M) for _ in range(G - 1))
        ms = [b - a for a, b in zip([0] + cuts, cuts + [M])]
    elif kind == "zipf":
        w = [1.0 / (i + 1) ** 1.2 for i in range(G)]
        ms = [int(M * v / sum(w)) for v in w]
    else:
        ms = [0] * G
        for _ in range(max(1, G // 4)):
            ms[rng.randrange(G)] += M // max(1, G // 4)
    rng.shuffle(ms)
    return ms


def close(a, b, tol=1e-2):
    d = (a.float() - b.float()).abs()
    return bool((d <= tol + tol * b.float().abs()).all()), float(d.max()) if d.numel() else 0.0


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_fast_paths_against_the_generic_kernel(seed):
    import applied_ai_amd as A
    from applied_ai_amd import _lib

    L = _lib.lib()
    rng = random.Random(seed)
    gen = torch.Generator(device="cuda").manual_seed(seed)
    try:
        for it in range(12):
            G = rng.choice([1, 2, 3, 8, 17, 64, 200])
            M = rng.choice([1, 77, 256, 300, 1000, 2049, 5000])
            N = rng.choice([8, 64, 72, 256, 264, 520, 1024, 1536])
            K = rng.choice([64, 128, 192, 448, 1024])
            ms = sizes_for(rng, G, M)
            R, pad = sum(ms), rng.choice([0, 0, 5])
            print(f"seed {seed} case {it}: G={G} rows={R}+{pad} N={N} K={K}", flush=True)
            x = (torch.randn(R + pad, K, device="cuda", generator=gen) / 4).bfloat16()
            w = (torch.randn(G * N, K, device="cuda", generator=gen) / 4).bfloat16()
            m = torch.tensor(ms, dtype=torch.int32, device="cuda")
            L.moe_gg_set_variant(0, GENERIC)
            ref = A.grouped_gemm(x, w, m)[:R]
            if R > 0:
                cpu = O.grouped_gemm_torch_loop(x[:R].float().cpu(), w.float().cpu(), ms)
                ok, worst = close(ref.cpu(), cpu)
                assert ok, ("generic kernel against the oracle", G, R, N, K, worst)
            for variant in (PINGPONG, AUTO):
                L.moe_gg_set_variant(0, variant)
                ok, worst = close(A.grouped_gemm(x, w, m)[:R], ref)
                assert ok, (variant, G, R, N, K, worst)
            if N % 16 == 0 and R > 0:
                L.moe_gg_set_variant(0, GENERIC)
                two = A.silu_and_mul(A.grouped_gemm(x, w, m))[:R]
                L.moe_gg_set_variant(0, AUTO)
                ok, worst = close(A.grouped_gemm_swiglu(x, w, m)[:R], two, 2e-2)
                assert ok, ("swiglu", G, R, N, K, worst)
            if N % 4 == 0 and K % 4 == 0 and R > 0:
                go = (torch.randn(R + pad, N, device="cuda", generator=gen) / 4).bfloat16()
                L.moe_gg_set_variant(0, GENERIC)
                gx0, gw0 = A.grouped_gemm_backward(go, x, w, m)
                for variant in (AUTO, PINGPONG):
                    L.moe_gg_set_variant(0, variant)
                    gx, gw = A.grouped_gemm_backward(go, x, w, m)
                    ok, worst = close(gx, gx0, 2e-2)
                    assert ok, ("grad_x", variant, G, R, N, K, worst)
                    ok, worst = close(gw, gw0, 2e-2)
                    assert ok, ("grad_w", variant, G, R, N, K, worst)
    finally:
        L.moe_gg_set_variant(0, AUTO)


@pytest.mark.parametrize("seed", [21, 22])
def test_long_reductions_with_few_low_tiles(seed):
    """K >= 8192 and at most 32 experts: the automatic choice may leave the low tiles (an expert's few rows beyond
    its last full 256-row tile) to the small-M kernel, a decision both kernels take on the device. Random expert
    sizes around whole rounds of tiles, where that decision flips; reference = the ping-pong kernel alone."""
    import ctypes

    import applied_ai_amd as A
    from applied_ai_amd import _lib

    L = _lib.lib()
    rng = random.Random(seed)
    gen = torch.Generator(device="cuda").manual_seed(seed)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    nwg = cus - cus % 8
    apart = 0
    try:
        for it in range(8):
            N = rng.choice([256, 512, 1024, 2048])
            K = rng.choice([8192, 8320])
            G = rng.choice([2, 5, 8, 16, 32])
            ntn = N // 256
            # row tiles: about one round of long tiles, dealt to the experts; then tails
            tiles = [0] * G
            for _ in range(nwg // ntn + rng.choice([0, 0, 0, -3, 2])):
                tiles[rng.randrange(G)] += 1
            ms = []
            for t in tiles:
                kind = rng.choice(["full", "low", "low", "long"])
                if kind == "low":
                    ms.append(t * 256 + rng.choice([1, 7, 16, 31, 32, 33, 64, 100, 127]))
                elif kind == "long" and t > 0:
                    ms.append(t * 256 - rng.randint(1, 127))
                else:
                    ms.append(t * 256)
            R = sum(ms)
            arr = (ctypes.c_int32 * G)(*ms)
            hit = L.moe_gg_host_tails_apart(arr, G, R, N, K, nwg)
            apart += hit
            print(f"seed {seed} case {it}: G={G} rows={R} N={N} K={K} apart={hit} m_sizes={ms}", flush=True)
            x = (torch.randn(R, K, device="cuda", generator=gen) / 8).bfloat16()
            w = (torch.randn(G * N, K, device="cuda", generator=gen) / 8).bfloat16()
            m = torch.tensor(ms, dtype=torch.int32, device="cuda")
            L.moe_gg_set_variant(0, PINGPONG)
            ref = A.grouped_gemm(x, w, m)
            L.moe_gg_set_variant(0, AUTO)
            got = A.grouped_gemm(x, w, m)
            ok, worst = close(got, ref)
            assert ok, (G, R, N, K, ms, worst)
            del x, w, ref, got
        assert apart >= 2 or cus != 256, "the cases no longer reach the two-kernel path"
    finally:
        L.moe_gg_set_variant(0, AUTO)


@pytest.mark.parametrize("seed", [31, 32])
def test_fp8_and_w4a16_random_shapes_against_the_oracle(seed):
    """Random expert sizes and shapes for the fp8 grouped GEMM (both scale modes, every kernel variant the automatic
    choice can take) and the grouped W4A16 GEMM, against the CPU oracle; relative Frobenius error <= 2e-2."""
    import numpy as np

    import applied_ai_amd as A
    from oracle import oracle as O
    from tests.gpu_util import rel_fro, to_np

    rng = random.Random(seed)
    nrng = np.random.default_rng(seed)
    F8 = torch.float8_e4m3fn
    for it in range(6):
        G = rng.choice([1, 3, 8, 24])
        M = rng.choice([5, 64, 300, 1100])
        N = rng.choice([128, 256, 384])
        K = rng.choice([128, 256, 1024])
        ms = sizes_for(rng, G, M)
        R = sum(ms)
        print(f"seed {seed} case {it}: G={G} rows={R} N={N} K={K} m_sizes={ms}", flush=True)
        m = torch.tensor(ms, dtype=torch.int32, device="cuda")
        x = nrng.standard_normal((R, K)).astype(np.float32)
        w = (nrng.standard_normal((G * N, K)) * 0.05).astype(np.float32)
        for mode in (0, 1):
            if mode == 1:
                xq, xs = O.fp8_groupwise_quant(x) if R else (np.zeros((0, K), np.uint8), np.zeros((0, K // 128), np.float32))
                wq, ws = O.fp8_block_quant_weight(w)
                fn = A.grouped_gemm_fp8_blockwise
            else:
                xs = np.maximum(np.abs(x).max(axis=1, initial=0.0), 1e-12) / 448.0
                ws = np.abs(w).max(axis=1) / 448.0
                xq = torch.from_numpy(np.clip(x / xs[:, None], -448, 448)).to(F8).view(torch.uint8).numpy()
                wq = torch.from_numpy(np.clip(w / ws[:, None], -448, 448)).to(F8).view(torch.uint8).numpy()
                fn = A.grouped_gemm_fp8_rowwise
            y = fn(torch.from_numpy(np.ascontiguousarray(xq)).view(F8).cuda(), torch.from_numpy(np.ascontiguousarray(wq)).view(F8).cuda(), m,
                   torch.from_numpy(np.ascontiguousarray(xs, dtype=np.float32)).cuda(),
                   torch.from_numpy(np.ascontiguousarray(ws, dtype=np.float32)).cuda())
            if R:
                ref = O.grouped_gemm_fp8(xq, wq, xs, ws, ms, mode)
                assert rel_fro(to_np(y)[:R], ref[:R]) <= 2e-2, (mode, G, R, N, K)
        # grouped W4A16 on the same expert sizes (N % 64 == 0, group 128)
        Nq = 128
        q = nrng.integers(0, 16, size=(G, K, Nq)); zz = nrng.integers(0, 16, size=(G, K // 128, Nq))
        scales = torch.from_numpy(nrng.uniform(0.005, 0.02, size=(G, K // 128, Nq)).astype(np.float32)).bfloat16()
        a = torch.from_numpy(x).bfloat16()
        qw = np.stack([O.pack_int4_along_k(q[g]) for g in range(G)]); qz = np.stack([O.pack_int4_along_n(zz[g]) for g in range(G)])
        c = A.matmul_split_k_grouped(a.cuda(), torch.from_numpy(qw).cuda(), scales.cuda(), torch.from_numpy(qz).cuda(), m)
        row = 0
        for g, mg in enumerate(ms):
            if mg:
                ref = O.w4a16_gemm(to_np(a[row:row + mg]), qw[g], to_np(scales[g]), qz[g], 128, 1)
                assert rel_fro(to_np(c[row:row + mg]), ref) <= 2e-2, ("w4a16", g, mg, K)
            row += mg
