"""ctypes binding of libmoe_gg.so (the C ABI declared in include/moe_gg.h).

The library is built in-tree by ``build_library()`` (hipcc, gfx950). Loading fails loudly when it
has not been built: there is no CPU or eager fallback behind these entry points.
"""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmoe_gg.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

_c_void_p = ctypes.c_void_p
_c_int = ctypes.c_int
_c_i64 = ctypes.c_int64
_i32_p = ctypes.POINTER(ctypes.c_int32)

# name -> (restype, argtypes); must list every symbol include/moe_gg.h declares.
SIGNATURES = {
    "moe_gg_abi_version": (_c_int, []),
    "moe_gg_strerror": (ctypes.c_char_p, [_c_int]),
    "moe_gg_set_variant": (_c_int, [_c_int, _c_int]),
    "moe_gg_grouped_gemm_bf16": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_i64, _c_int, _c_int, _c_i64, _c_int,
         _c_void_p],
    ),
    "moe_gg_grouped_gemm_f16": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_i64, _c_int, _c_int, _c_i64, _c_int,
         _c_void_p],
    ),
    "moe_gg_grouped_gemm_fp8": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_i64, _c_int, _c_int,
         _c_i64, _c_int, _c_void_p],
    ),
    "moe_gg_w4a16_splitk": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
         _c_void_p],
    ),
    "moe_gg_w4a16_grouped": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int,
         _c_int, _c_void_p],
    ),
    "moe_gg_w4a16_grouped_fp8out": (
        _c_int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_i64, _c_int, _c_int,
         _c_int, _c_int, _c_int, _c_void_p],
    ),
    "moe_gg_route_topk": (_c_int, [_c_void_p, _c_i64, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "moe_gg_route_group": (_c_int, [_c_void_p, _c_i64, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "moe_gg_gather_rows": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_void_p, _c_i64, _c_i64, _c_i64, _c_void_p, _c_void_p]),
    "moe_gg_grouped_gemm_backward_workspace": (ctypes.c_size_t, [_c_int, _c_i64, _c_int, _c_int, _c_int]),
    "moe_gg_grouped_gemm_backward_bf16": (
        _c_int,
        [_c_void_p, _c_i64, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_i64, _c_int, _c_int, _c_void_p, _c_void_p,
         _c_void_p, ctypes.c_size_t, _c_void_p],
    ),
    "moe_gg_grouped_gemm_backward_bf16_static": (
        _c_int,
        [_c_void_p, _c_i64, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_i64, _c_int, _c_int, _c_void_p, _c_void_p,
         _c_void_p],
    ),
    "moe_gg_grouped_gemm_swiglu_bf16": (
        _c_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_i64, _c_int, _c_int, _c_i64, _c_void_p]),
    "moe_gg_grouped_gemm_swiglu_f16": (
        _c_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_i64, _c_int, _c_int, _c_i64, _c_void_p]),
    "moe_gg_grouped_gemm_swiglu_gather": (
        _c_int, [_c_void_p, _c_i64, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_i64, _c_int, _c_int, _c_i64,
                 _c_int, _c_void_p]),
    "moe_gg_silu_and_mul": (_c_int, [_c_void_p, _c_void_p, _c_i64, _c_int, _c_void_p]),
    "moe_gg_silu_and_mul_f16": (_c_int, [_c_void_p, _c_void_p, _c_i64, _c_int, _c_void_p]),
    "moe_gg_invert_perm": (_c_int, [_c_void_p, _c_void_p, _c_i64, _c_void_p, _c_void_p]),
    "moe_gg_combine_topk": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_i64, _c_int, _c_int, _c_i64, _c_void_p]),
    "moe_gg_combine_topk_f16": (_c_int, [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_i64, _c_int, _c_int, _c_i64, _c_void_p]),
    "moe_gg_fp8_groupwise_quant": (_c_int, [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_i64, _c_void_p]),
    "moe_gg_fp8_block128_quant": (_c_int, [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_i64, _c_int, _c_void_p]),
    "moe_gg_align_block_size": (_c_int, [_c_void_p, _c_void_p, _c_int, _c_i64, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "moe_gg_host_enumerate_tiles": (
        _c_int,
        [_i32_p, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int, _i32_p, _c_int],
    ),
    "moe_gg_host_enumerate_tiles_two_lists": (
        _c_int,
        [_i32_p, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int, _i32_p, _c_int],
    ),
    "moe_gg_host_tails_apart": (_c_int, [_i32_p, _c_int, _c_i64, _c_int, _c_int, _c_int]),
    "moe_gg_host_tail_pieces": (_c_int, [_c_int, _c_int, _c_int]),
}

_lib = None


def build_library(jobs: int = 8, verbose: bool = False) -> str:
    """Compile every HIP source under csrc/ for gfx950 into lib/libmoe_gg.so (always recompiles)."""
    os.makedirs(os.path.join(_HERE, "lib"), exist_ok=True)
    subprocess.run(["make", "-C", CSRC_DIR, "clean"], check=True, capture_output=not verbose)
    proc = subprocess.run(["make", "-C", CSRC_DIR, f"-j{jobs}"], capture_output=True, text=True)
    if proc.returncode != 0 or not os.path.exists(LIB_PATH):
        raise RuntimeError("building libmoe_gg.so failed:\n" + proc.stdout[-4000:] + proc.stderr[-4000:])
    if verbose:
        print(proc.stdout)
    return LIB_PATH


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it first (python -c 'import __graft_entry__ as g; g.build()'). "
                "There is no fallback implementation."
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        if handle.moe_gg_abi_version() != 1:
            raise RuntimeError("libmoe_gg.so ABI version mismatch; rebuild it")
        _lib = handle
    return _lib


def strerror(code: int) -> str:
    return lib().moe_gg_strerror(code).decode()


def check(code: int, what: str) -> None:
    """Map a C-ABI return code to the exceptions the reference's callers expect: ValueError for
    host-checkable argument errors, RuntimeError for everything else
    (dev/triton_groupGEMM/testing/unit_tests.py:180-212)."""
    if code == 0:
        return
    msg = f"{what}: {strerror(code)} (code {code})"
    if code in (-1, -2, -3):
        raise ValueError(msg)
    raise RuntimeError(msg)
