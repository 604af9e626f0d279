"""Builds tests/emu/_build/libmoe_gg_emu.so: the library's .hip sources compiled as host C++ against the stand-in
HIP header of this folder, so that the C ABI of include/moe_gg.h runs on the CPU under the wave emulation of
emu_core.cpp (tests only; the product never loads it).

The sources are used as they are except for two constructs that have no host form, rewritten on the way in:
  * inline assembly: each statement is recognised by its instruction and replaced by the call that models it
    (global->LDS loads, counter waits, the 24-bit multiply-add); an instruction without a rule stops the build;
  * `extern __shared__ T name[];` becomes a pointer into the emulated dynamic LDS range.
"""
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
# EMU_CSRC / EMU_OUT: build another copy of the sources (a kernel under development) into another folder.
CSRC = os.environ.get("EMU_CSRC") or os.path.join(ROOT, "applied-ai_amd", "csrc")
OUT = os.environ.get("EMU_OUT") or os.path.join(HERE, "_build")
CXX = "/opt/rocm/llvm/bin/clang++"
FLAGS = ["-x", "c++", "-std=c++17", "-O1", "-g", "-fPIC", "-fno-strict-aliasing", "-Wno-unknown-attributes", "-Wno-unused-value",
         "-Wno-ignored-attributes", "-I", os.path.join(HERE, "include"), "-I", CSRC]
# EMU_UBSAN (with an EMU_OUT of its own): the kernels trap on misaligned vector accesses, out-of-range shifts, signed
# overflow and indices beyond a fixed-size array (no sanitizer runtime needed: the checks end in a trap instruction).
if os.environ.get("EMU_UBSAN"):
    FLAGS += ["-fsanitize=alignment,shift,signed-integer-overflow,bounds,null", "-fsanitize-trap=all"]


def _split_top(s, sep):
    parts, depth, cur, i, in_str = [], 0, [], 0, False
    while i < len(s):
        c = s[i]
        if in_str:
            cur.append(c)
            if c == "\\":
                cur.append(s[i + 1]); i += 1
            elif c == '"':
                in_str = False
        elif c == '"':
            in_str = True; cur.append(c)
        elif c in "([{":
            depth += 1; cur.append(c)
        elif c in ")]}":
            depth -= 1; cur.append(c)
        elif c == sep and depth == 0:
            parts.append("".join(cur)); cur = []
        else:
            cur.append(c)
        i += 1
    parts.append("".join(cur))
    return parts


def _operands(section):
    """'"s"(a), "v"(b + 1)' -> ['a', 'b + 1']"""
    out = []
    for item in _split_top(section, ","):
        item = item.strip()
        if not item:
            continue
        m = re.match(r'"[^"]*"\s*\((.*)\)\s*$', item, re.S)
        assert m, "operand not understood: " + item
        out.append(m.group(1).strip())
    return out


def _asm_rule(template, outs, ins, where):
    t = template
    if "global_load_lds_dwordx4" in t or "global_load_lds_dword " in t:
        assert "s_mov_b32 m0, %0" in t and len(ins) == 3 and not outs, where
        lds, voff, sbase = ins
        # (the base may be a pointer with a device address space)
        return "emu::dma(%d, (const void*)(uintptr_t)(%s), %s, %s)" % (16 if "dwordx4" in t else 4, sbase, voff, lds)
    m = re.fullmatch(r"\s*s_waitcnt vmcnt\((%0|\d+)\)\s*", t)
    if m:
        return "emu::wait_vm(%s)" % (ins[0] if m.group(1) == "%0" else m.group(1))
    if re.fullmatch(r"\s*s_waitcnt lgkmcnt\(0\)\s*", t):
        return "emu::wait_lds()"
    if re.fullmatch(r"\s*v_mad_u32_u24 %0, %1, %2, %3\s*", t):
        assert len(outs) == 1 and len(ins) == 3, where
        return "%s = ((%s) & 0xFFFFFFu) * ((%s) & 0xFFFFFFu) + (%s)" % (outs[0], ins[0], ins[1], ins[2])
    m = re.fullmatch(r"\s*v_mfma_f32_16x16x32_(bf16|f16) %0, %1, %2, %0\s*", t)
    if m:  # an MFMA with VGPR accumulators, written out: "+v"(c) : "v"(a), "v"(b)
        assert len(outs) == 1 and len(ins) == 2, where
        return "%s = mfma_16x16x32<%s>(__builtin_bit_cast(u32x4_t, %s), __builtin_bit_cast(u32x4_t, %s), %s)" % (
            outs[0], "true" if m.group(1) == "f16" else "false", ins[0], ins[1], outs[0])
    if re.fullmatch(r"\s*s_nop \d+(\s*s_nop \d+)*\s*", t):
        return "((void)0)"  # wait states
    if t.strip() == "":
        return "((void)0)"  # an optimisation barrier on registers
    raise SystemExit("build_emu: no rule for the inline assembly at %s: %r" % (where, template))


def translate(text, name):
    out, pos = [], 0
    for m in re.finditer(r"\basm\s*(?:volatile\s*)?\(", text):
        if m.start() < pos:
            continue
        line_start = text.rfind("\n", 0, m.start()) + 1
        if "//" in text[line_start:m.start()]:
            continue
        i, depth, in_str = m.end(), 1, False
        while depth:
            c = text[i]
            if in_str:
                if c == "\\":
                    i += 1
                elif c == '"':
                    in_str = False
            elif c == '"':
                in_str = True
            elif c == "(":
                depth += 1
            elif c == ")":
                depth -= 1
            i += 1
        body = text[m.end():i - 1]
        sections = _split_top(body, ":")
        template = "".join(bytes(s, "utf-8").decode("unicode_escape") for s in re.findall(r'"((?:[^"\\]|\\.)*)"', sections[0]))
        outs = _operands(sections[1]) if len(sections) > 1 else []
        ins = _operands(sections[2]) if len(sections) > 2 else []
        where = "%s:%d" % (name, text.count("\n", 0, m.start()) + 1)
        out.append(text[pos:m.start()])
        out.append(_asm_rule(re.sub(r"\s+", " ", template).strip(), outs, ins, where))
        pos = i
    out.append(text[pos:])
    text = "".join(out)
    text = re.sub(r"extern\s+__shared__\s+([\w:]+)\s+(\w+)\s*\[\s*\]\s*;", r"\1* \2 = (\1*)emu::dyn_lds();", text)
    assert "asm" not in re.sub(r"//[^\n]*", "", text).replace("emu::", ""), "untranslated asm in " + name
    return text


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def stale(lib):
    if not os.path.exists(lib):
        return True
    t = os.path.getmtime(lib)
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".h"))]
    deps += [os.path.join(HERE, "emu_core.cpp"), os.path.join(HERE, "include", "hip", "hip_runtime.h"), os.path.abspath(__file__),
             os.path.join(ROOT, "include", "moe_gg.h")]
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=False, jobs=8):
    lib = os.path.join(OUT, "libmoe_gg_emu.so")
    if not force and not stale(lib):
        return lib
    os.makedirs(OUT, exist_ok=True)
    procs, objs = [], []
    units = []
    for f in sources():
        cpp = os.path.join(OUT, f.replace(".hip", ".emu.cpp"))
        with open(os.path.join(CSRC, f)) as fh:
            text = translate(fh.read(), f)
        # api.hip includes the public header by a relative path: keep it valid from the build folder
        text = text.replace('#include "../../include/moe_gg.h"', '#include "%s"' % os.path.join(ROOT, "include", "moe_gg.h"))
        with open(cpp, "w") as fh:
            fh.write('#line 1 "%s"\n' % os.path.join(CSRC, f) + text)
        units.append(cpp)
    units.append(os.path.join(HERE, "emu_core.cpp"))
    pending = list(units)
    running = []
    while pending or running:
        while pending and len(running) < jobs:
            src = pending.pop(0)
            obj = os.path.join(OUT, os.path.basename(src).rsplit(".", 1)[0] + ".o")
            objs.append(obj)
            running.append((src, subprocess.Popen([CXX] + FLAGS + ["-c", src, "-o", obj], stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        src, p = running.pop(0)
        log = p.communicate()[0].decode()
        if p.returncode:
            for _, q in running:
                q.kill()
            raise SystemExit("build_emu: %s failed:\n%s" % (src, log[-6000:]))
    subprocess.run([CXX, "-shared", "-o", lib] + objs + ["-lpthread"], check=True)
    return lib


def build_race_check(force=False, jobs=8):
    """tests/emu/_build/tsan/race_check: race_check.cpp + the kernels under ThreadSanitizer + emu_core.cpp with EMU_TSAN
    (itself not instrumented: its tables are shared by all fibers on purpose)."""
    out = os.path.join(OUT, "tsan")
    exe = os.path.join(out, "race_check")
    if not force and not stale(exe) and all(os.path.getmtime(exe) > os.path.getmtime(os.path.join(HERE, f))
                                            for f in ("race_check.cpp", "race_selftest.cpp")):
        return exe
    build(force=False, jobs=jobs)   # leaves the translated sources in OUT
    os.makedirs(out, exist_ok=True)
    tsan = ["-fsanitize=thread", "-mllvm", "-tsan-instrument-func-entry-exit=0"]
    units = [(os.path.join(OUT, f.replace(".hip", ".emu.cpp")), tsan) for f in sources()]
    units.append((os.path.join(HERE, "race_selftest.cpp"), tsan))
    units.append((os.path.join(HERE, "emu_core.cpp"), ["-DEMU_TSAN"]))
    units.append((os.path.join(HERE, "race_check.cpp"), []))
    objs, running, pending = [], [], list(units)
    while pending or running:
        while pending and len(running) < jobs:
            src, extra = pending.pop(0)
            obj = os.path.join(out, os.path.basename(src).rsplit(".", 1)[0] + ".o")
            objs.append(obj)
            running.append((src, subprocess.Popen([CXX] + FLAGS + extra + ["-c", src, "-o", obj], stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        src, p = running.pop(0)
        log = p.communicate()[0].decode()
        if p.returncode:
            for _, q in running:
                q.kill()
            raise SystemExit("build_emu: %s failed:\n%s" % (src, log[-6000:]))
    subprocess.run([CXX, "-fsanitize=thread", "-o", exe] + objs + ["-ldl", "-lpthread"], check=True)
    return exe


if __name__ == "__main__":
    if "--race-check" in sys.argv:
        print(build_race_check(force="--force" in sys.argv))
    else:
        print(build(force="--force" in sys.argv))
