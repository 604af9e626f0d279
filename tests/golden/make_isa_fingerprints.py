"""Fingerprints of the compiled gfx950 code of the kernels, for tests/test_isa_properties.py::test_default_kernels_are_the_gpu_tested_code.

    python tests/golden/make_isa_fingerprints.py <git commit> > tests/golden/isa_fingerprints.json

compiles applied-ai_amd/csrc/*.hip as they are at <commit> (hipcc -S for gfx950, the flags of the Makefile) and writes, per
kernel, the SHA-256 of its instruction stream. The committed file was made from the last commit whose tree passed the
whole GPU suite on an MI355X; the test compiles the working tree the same way and compares the kernels that run by
default. Normalisation (fingerprint() below, shared with the test): comments and directives dropped, local labels
renumbered in order of appearance, the offset of the first hidden kernel argument (it follows the explicit ones, whose
struct has grown by fields only newer kernels read) and runs of adjacent scalar register copies taken as a set.
"""
import hashlib
import json
import os
import re
import subprocess
import sys
import tempfile

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
HIPCC = "/opt/rocm/bin/hipcc"
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-S", "--cuda-device-only"]


def kernels(asm_text):
    """{mangled kernel name: [instruction lines]} of one -S output."""
    out = {}
    for m in re.finditer(r"^(_Z[^\n:]+):\s*; @\S+\n(.*?)\n\.Lfunc_end", asm_text, re.S | re.M):
        lines = [re.sub(r"\s*;.*", "", ln).strip() for ln in m.group(2).splitlines()]
        out[m.group(1)] = [ln for ln in lines if ln and not ln.startswith((".p2align", ".amdhsa", ".section", ".end_amdhsa"))]
    return out


def fingerprint(lines):
    labels = {}

    def label(m):
        return labels.setdefault(m.group(0), "L%d" % len(labels))

    norm, run = [], []
    for ln in lines:
        ln = re.sub(r"\.?LBB\d+_\d+", label, ln)
        ln = re.sub(r"^(s_load_dword\w* \S+ s\[0:1\]), 0x[0-9a-f]+$", lambda m: m.group(1) + ", <arg>", ln) if re.search(r"s\[0:1\], 0x(68|80)$", ln) else ln
        if re.match(r"s_mov_b(32|64) s", ln):
            run.append(ln)
            continue
        norm += sorted(run) + [ln]
        run = []
    norm += sorted(run)
    return hashlib.sha256("\n".join(norm).encode()).hexdigest()


def compile_tree(csrc_dir):
    """{file: {kernel: fingerprint}} of every .hip file of a csrc directory."""
    res = {}
    with tempfile.TemporaryDirectory() as tmp:
        procs = []
        for f in sorted(os.listdir(csrc_dir)):
            if f.endswith(".hip") and f != "api.hip":
                out = os.path.join(tmp, f[:-4] + ".s")
                procs.append((f, out, subprocess.Popen([HIPCC] + FLAGS + [os.path.join(csrc_dir, f), "-o", out],
                                                       stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)))
        for f, out, p in procs:
            if p.wait() != 0:
                raise SystemExit("hipcc failed on " + f)
            res[f] = {k: fingerprint(v) for k, v in kernels(open(out).read()).items()}
    return res


def main(commit):
    with tempfile.TemporaryDirectory() as tmp:
        subprocess.run("git -C %s archive %s applied-ai_amd/csrc include | tar -x -C %s" % (ROOT, commit, tmp), shell=True, check=True)
        res = compile_tree(os.path.join(tmp, "applied-ai_amd", "csrc"))
    full = subprocess.run(["git", "-C", ROOT, "rev-parse", commit], stdout=subprocess.PIPE, check=True).stdout.decode().strip()
    json.dump({"commit": full, "what": "SHA-256 of the normalised instruction stream of every kernel at that commit (make_isa_fingerprints.py)",
               "kernels": res}, sys.stdout, indent=1, sort_keys=True)


if __name__ == "__main__":
    main(sys.argv[1])
