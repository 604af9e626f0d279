"""numpy front end of the emulated library (tests/emu/_build/libmoe_gg_emu.so): the C ABI of include/moe_gg.h with
host arrays in the place of device pointers. Test infrastructure only."""
import ctypes
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, HERE):
    if p not in sys.path:
        sys.path.insert(0, p)

import build_emu  # noqa: E402
from applied_ai_amd import _lib  # noqa: E402

_L = None
# GUARD = "end" / "start": every array handed to the library is copied into memory that ends (begins) at an
# inaccessible page, so that a kernel reading or writing past the end (before the start) of a tensor faults at once
# instead of touching a neighbour. None: plain numpy arrays.
GUARD = os.environ.get("EMU_GUARD") or None
_keep = []
_libc = ctypes.CDLL(None, use_errno=True)
_libc.mprotect.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
BF16, FP16, FP32 = 0, 1, 2
OP_BF16, OP_FP8, OP_TILE_ORDER, OP_W4A16 = 0, 1, 2, 3


def lib():
    global _L
    if _L is None:
        _L = ctypes.CDLL(build_emu.build())
        for name, (res, args) in _lib.SIGNATURES.items():
            f = getattr(_L, name)
            f.restype, f.argtypes = res, args
        for name in ("emu_nonuniform_readfirstlane", "emu_divergent_exchanges"):
            getattr(_L, name).restype = ctypes.c_ulonglong
        # EMU_TILE_ORDER = 0 / 1: the ping-pong kernels' tile order for this process (MOE_GG_OP_TILE_ORDER)
        if os.environ.get("EMU_TILE_ORDER"):
            assert _L.moe_gg_set_variant(OP_TILE_ORDER, int(os.environ["EMU_TILE_ORDER"])) == 0
    return _L


def guarded(a):
    """A copy of `a` whose last (first) byte, up to 16-byte alignment, is followed (preceded) by a page without access."""
    import mmap

    a = np.ascontiguousarray(a)
    n = (a.nbytes + 15) // 16 * 16
    pages = (n + 4095) // 4096 + 2
    m = mmap.mmap(-1, pages * 4096)
    base = ctypes.addressof(ctypes.c_char.from_buffer(m))
    for page in (0, pages - 1):
        if _libc.mprotect(base + page * 4096, 4096, 0) != 0:
            raise OSError(ctypes.get_errno(), "mprotect")
    off = 4096 if GUARD == "start" else (pages - 1) * 4096 - n
    out = np.frombuffer(m, dtype=a.dtype, count=a.size, offset=off).reshape(a.shape)
    out[...] = a
    _keep.append(m)
    return out


_guarded_ptrs = set()


def G(a):
    """Input or output array as the library sees it (guarded when GUARD is set)."""
    if a is None or GUARD is None or a.size == 0 or a.ctypes.data in _guarded_ptrs:
        return a
    g = guarded(a)
    _guarded_ptrs.add(g.ctypes.data)
    return g


def _full(shape, fill, dtype):
    return G(np.full(shape, fill, dtype=dtype))


def release():
    """Drops the guarded mappings made so far (their arrays must not be used afterwards)."""
    del _keep[:]
    _guarded_ptrs.clear()


def P(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return G(a).ctypes.data   # inputs get their guarded copy here; outputs were made by _full


def ok(rc):
    if rc != 0:
        raise RuntimeError("rc %d: %s" % (rc, lib().moe_gg_strerror(rc).decode()))


def to_bf16(x):
    """fp32 -> bf16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = ((u >> 16) & 1) + 0x7FFF
    return ((u + r) >> 16).astype(np.uint16)


def from_bf16(b):
    return (b.astype(np.uint32) << 16).view(np.float32)


def to16(x, fp16):
    return np.ascontiguousarray(x, dtype=np.float16).view(np.uint16) if fp16 else to_bf16(x)


def from16(b, fp16):
    return b.view(np.float16).astype(np.float32) if fp16 else from_bf16(b)


def i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


NAN16 = 0x7FC0  # a NaN in both 16-bit formats: rows a kernel must not leave unwritten


def grouped_gemm(x16, w16, m_sizes, N, fp16=False, block_layout=False, variant=-1):
    L = lib()
    ms = i32(m_sizes)
    G, (M, K) = len(ms), x16.shape
    ld = N * G if block_layout else N
    y = _full((M, ld), NAN16, dtype=np.uint16)
    L.moe_gg_set_variant(OP_BF16, variant)
    try:
        fn = L.moe_gg_grouped_gemm_f16 if fp16 else L.moe_gg_grouped_gemm_bf16
        ok(fn(P(x16), P(w16), P(y), P(ms), G, M, N, K, ld, 1 if block_layout else 0, None))
    finally:
        L.moe_gg_set_variant(OP_BF16, -1)
    return y


def grouped_gemm_fp8(xq, wq, x_scale, w_scale, mode, m_sizes, N, variant=-1):
    L = lib()
    ms = i32(m_sizes)
    G, (M, K) = len(ms), xq.shape
    y = _full((M, N), NAN16, dtype=np.uint16)
    L.moe_gg_set_variant(OP_FP8, variant)
    try:
        ok(L.moe_gg_grouped_gemm_fp8(P(xq), P(wq), P(y), P(x_scale), P(w_scale), mode, P(ms), G, M, N, K, N, 0, None))
    finally:
        L.moe_gg_set_variant(OP_FP8, -1)
    return y


def grouped_gemm_swiglu(x16, w16, m_sizes, n, fp16=False, variant=-1):
    """variant 7 or 8 (MOE_GG_GG_FOURWAVE_256 / _TALL pinned for the grouped GEMM) selects a four-wave form of the fused kernel."""
    L = lib()
    ms = i32(m_sizes)
    G, (M, K) = len(ms), x16.shape
    y = _full((M, n), NAN16, dtype=np.uint16)
    fn = L.moe_gg_grouped_gemm_swiglu_f16 if fp16 else L.moe_gg_grouped_gemm_swiglu_bf16
    L.moe_gg_set_variant(OP_BF16, variant)
    try:
        ok(fn(P(x16), P(w16), P(y), P(ms), G, M, n, K, n, None))
    finally:
        L.moe_gg_set_variant(OP_BF16, -1)
    return y


def grouped_gemm_swiglu_gather(tokens16, perm, k, w16, m_sizes, n, fp16=False):
    L = lib()
    ms, pm = i32(m_sizes), i32(perm)
    G, (T, K), M = len(ms), tokens16.shape, len(pm)
    y = _full((M, n), NAN16, dtype=np.uint16)
    ok(L.moe_gg_grouped_gemm_swiglu_gather(P(tokens16), T, P(pm), k, P(w16), P(y), P(ms), G, M, n, K, n, FP16 if fp16 else BF16, None))
    return y


def backward(go16, x16, w16, m_sizes, N, block_layout=False, static=False):
    L = lib()
    ms = i32(m_sizes)
    G, (M, K) = len(ms), x16.shape
    gx = _full((M, K), NAN16, dtype=np.uint16)
    gw = _full((G * N, K), NAN16, dtype=np.uint16)
    layout = 1 if block_layout else 0
    if static:
        ok(L.moe_gg_grouped_gemm_backward_bf16_static(P(go16), go16.shape[1], layout, P(x16), P(w16), P(ms), G, M, N, K, P(gx), P(gw), None))
    else:
        nbytes = L.moe_gg_grouped_gemm_backward_workspace(G, M, N, K, layout)
        raw = _full(nbytes // 256 * 256 + 512, 0, np.uint8)   # ends at the guard page when guarded
        off = (-raw.ctypes.data) % 256
        ws = raw[off:off + nbytes]
        ok(L.moe_gg_grouped_gemm_backward_bf16(P(go16), go16.shape[1], layout, P(x16), P(w16), P(ms), G, M, N, K, P(gx), P(gw),
                                               ws.ctypes.data, nbytes, None))
    return gx, gw


def w4a16(a16, qweight, scales16, qzeros, group_size=128, zero_offset=1, fp16=False, m_sizes=None, fp8out=False, variant=-1):
    L = lib()
    L.moe_gg_set_variant(OP_W4A16, variant)
    try:
        return _w4a16(L, a16, qweight, scales16, qzeros, group_size, zero_offset, fp16, m_sizes, fp8out)
    finally:
        L.moe_gg_set_variant(OP_W4A16, -1)


def _w4a16(L, a16, qweight, scales16, qzeros, group_size, zero_offset, fp16, m_sizes, fp8out):
    M, K = a16.shape
    dt = FP16 if fp16 else BF16
    if m_sizes is None:
        N = qweight.shape[1]
        c = _full((M, N), NAN16, dtype=np.uint16)
        ok(L.moe_gg_w4a16_splitk(P(a16), P(qweight), P(scales16), P(qzeros), P(c), M, N, K, group_size, zero_offset, dt, None))
        return c
    ms = i32(m_sizes)
    G, N = len(ms), qweight.shape[2]
    if fp8out:
        cq = _full((M, N), 0x7F, dtype=np.uint8)
        cs = _full((M, N // 128), np.nan, dtype=np.float32)
        ok(L.moe_gg_w4a16_grouped_fp8out(P(a16), P(qweight), P(scales16), P(qzeros), P(cq), P(cs), P(ms), G, M, N, K, group_size,
                                         zero_offset, dt, None))
        return cq, cs
    c = _full((M, N), NAN16, dtype=np.uint16)
    ok(L.moe_gg_w4a16_grouped(P(a16), P(qweight), P(scales16), P(qzeros), P(c), P(ms), G, M, N, K, group_size, zero_offset, dt, None))
    return c


def route_topk(logits, k):
    L = lib()
    T, E = logits.shape
    ids = _full((T, k), -7, dtype=np.int32)
    perm = _full(T * k, -7, dtype=np.int32)
    ms = _full(E, -7, dtype=np.int32)
    off = _full(E + 1, -7, dtype=np.int32)
    ok(L.moe_gg_route_topk(P(np.ascontiguousarray(logits, dtype=np.float32)), T, E, k, P(ids), P(perm), P(ms), P(off), None))
    return ids, perm, ms, off


def route_group(flat_ids, E):
    L = lib()
    flat = i32(flat_ids).ravel()
    n = flat.size
    perm = _full(n, -7, dtype=np.int32)
    ms = _full(E, -7, dtype=np.int32)
    off = _full(E + 1, -7, dtype=np.int32)
    ok(L.moe_gg_route_group(P(flat), n, E, P(perm), P(ms), P(off), None))
    return perm, ms, off


def align_block_size(perm, m_sizes, block_size):
    L = lib()
    E, n = len(m_sizes), len(perm)
    sorted_ids = _full(n + E * (block_size - 1), -7, dtype=np.int32)
    expert_ids = _full(n + E, -7, dtype=np.int32)
    post = _full(1, -7, dtype=np.int32)
    ok(L.moe_gg_align_block_size(P(i32(perm)), P(i32(m_sizes)), E, n, block_size, P(sorted_ids), P(expert_ids), P(post), None))
    return sorted_ids, expert_ids, int(post[0])


def gather_rows(x, perm, k, n_valid=None):
    L = lib()
    x = np.ascontiguousarray(x)
    n = len(perm)
    out = _full((n,) + x.shape[1:], 0xAB, dtype=x.dtype) if x.dtype.kind in "ui" else _full((n,) + x.shape[1:], np.nan, dtype=x.dtype)
    nv = None if n_valid is None else np.array([n_valid], dtype=np.int32)
    ok(L.moe_gg_gather_rows(P(x), P(i32(perm)), k, P(out), n, x[0].nbytes, x.shape[0], P(nv), None))
    return out


def fp8_groupwise_quant(x, bf16_in=False):
    L = lib()
    src = to_bf16(x) if bf16_in else np.ascontiguousarray(x, dtype=np.float32)
    q = _full(x.shape, 0x7F, dtype=np.uint8)
    s = _full(x.size // 128, np.nan, dtype=np.float32)
    ok(L.moe_gg_fp8_groupwise_quant(P(src), BF16 if bf16_in else FP32, P(q), P(s), x.size, None))
    return q, s.reshape(x.shape[:-1] + (x.shape[-1] // 128,))


def fp8_block128_quant(w, bf16_in=False):
    L = lib()
    rows, K = w.shape
    src = to_bf16(w) if bf16_in else np.ascontiguousarray(w, dtype=np.float32)
    q = _full(w.shape, 0x7F, dtype=np.uint8)
    s = _full((rows // 128, K // 128), np.nan, dtype=np.float32)
    ok(L.moe_gg_fp8_block128_quant(P(src), BF16 if bf16_in else FP32, P(q), P(s), rows, K, None))
    return q, s


def silu_and_mul(x16, fp16=False):
    L = lib()
    rows, n2 = x16.shape
    out = _full((rows, n2 // 2), NAN16, dtype=np.uint16)
    ok((L.moe_gg_silu_and_mul_f16 if fp16 else L.moe_gg_silu_and_mul)(P(x16), P(out), rows, n2 // 2, None))
    return out


def invert_perm(perm, n_valid=None):
    L = lib()
    n = len(perm)
    inv = _full(n, -7, dtype=np.int32)
    nv = None if n_valid is None else np.array([n_valid], dtype=np.int32)
    ok(L.moe_gg_invert_perm(P(i32(perm)), P(inv), n, P(nv), None))
    return inv


def combine_topk(y16, inv, weights, T, k, fp16=False, weights_16bit=False):
    L = lib()
    d = y16.shape[1]
    out = _full((T, d), NAN16, dtype=np.uint16)
    wt = to16(weights, fp16) if weights_16bit else np.ascontiguousarray(weights, dtype=np.float32)
    wd = (FP16 if fp16 else BF16) if weights_16bit else FP32
    fn = L.moe_gg_combine_topk_f16 if fp16 else L.moe_gg_combine_topk
    ok(fn(P(y16), P(i32(inv)), P(wt), wd, P(out), T, k, d, y16.shape[0], None))
    return out


def counters():
    L = lib()
    return int(L.emu_nonuniform_readfirstlane()), int(L.emu_divergent_exchanges())
