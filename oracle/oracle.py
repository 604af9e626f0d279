"""numpy front end of the C oracle (moe_oracle.c) plus the torch per-expert loop used as CPU baseline.

TEST INFRASTRUCTURE ONLY - see the header of moe_oracle.c. All functions take and return numpy arrays
(bf16 / fp8 data is passed as float32 values or uint8 codes); nothing here touches a GPU.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmoe_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _SO


def _l():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.orc_e4m3_to_f32.restype = ctypes.c_float
        _lib.orc_e4m3_to_f32.argtypes = [ctypes.c_uint8]
        _lib.orc_f32_to_e4m3.restype = ctypes.c_uint8
        _lib.orc_f32_to_e4m3.argtypes = [ctypes.c_float]
        _lib.orc_round_bf16.restype = ctypes.c_float
        _lib.orc_round_bf16.argtypes = [ctypes.c_float]
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def offsets(m_sizes):
    """Exclusive prefix sum [G+1] of m_sizes (groupgemm.py:159-165)."""
    m = _i32(m_sizes)
    out = np.empty(m.shape[0] + 1, dtype=np.int32)
    _l().orc_offsets(_p(m), ctypes.c_int(m.shape[0]), _p(out))
    return out


def grouped_gemm(x, w, m_sizes, block_layout=False, fill=np.nan):
    """fp32 per-expert x_g @ w_g^T (unit_tests.py:49-55). Unwritten entries hold `fill`."""
    x, w, m = _f32(x), _f32(w), _i32(m_sizes)
    G = m.shape[0]
    M, K = x.shape
    N = w.shape[0] // G
    cols = N * G if block_layout else N
    y = np.full((M, cols), fill, dtype=np.float32)
    _l().orc_grouped_gemm(_p(x), _p(w), _p(m), ctypes.c_int(G), ctypes.c_int64(M), ctypes.c_int(N),
                          ctypes.c_int(K), _p(y), ctypes.c_int64(cols), ctypes.c_int(N if block_layout else 0))
    return y


def grouped_gemm_backward(grad_output, x, w, m_sizes):
    """fp32 (grad_x [M, K], grad_w [G*N, K]) of the grouped GEMM (pytorch_reference_backwards.py:165-197).
    grad_output is [M, N*G] (each expert reads its own column block) or [M, N]."""
    go, x, w, m = _f32(grad_output), _f32(x), _f32(w), _i32(m_sizes)
    G = m.shape[0]
    M, K = x.shape
    N = w.shape[0] // G
    block = go.shape[1] == N * G and G > 1
    gx = np.empty((M, K), dtype=np.float32)
    gw = np.empty((G * N, K), dtype=np.float32)
    _l().orc_grouped_gemm_backward(_p(go), ctypes.c_int64(go.shape[1]), ctypes.c_int(N if block else 0), _p(x), _p(w),
                                   _p(m), ctypes.c_int(G), ctypes.c_int64(M), ctypes.c_int(N), ctypes.c_int(K),
                                   _p(gx), _p(gw))
    return gx, gw


def topk(logits, k):
    """Top-k expert ids per token, descending score, ties to the lower index (test_moe_gemm.py:54-57)."""
    lg = _f32(logits)
    T, E = lg.shape
    ids = np.empty((T, k), dtype=np.int32)
    _l().orc_topk(_p(lg), ctypes.c_int64(T), ctypes.c_int(E), ctypes.c_int(k), _p(ids))
    return ids


def route(topk_ids, num_experts):
    """(perm, m_sizes): flat indices grouped by ascending expert, stable (v0_moe_fused.py:141-166)."""
    flat = _i32(np.asarray(topk_ids).reshape(-1))
    perm = np.empty(flat.shape[0], dtype=np.int32)
    m = np.empty(num_experts, dtype=np.int32)
    _l().orc_route(_p(flat), ctypes.c_int64(flat.shape[0]), ctypes.c_int(num_experts), _p(perm), _p(m))
    return perm, m


def moe_align_block_size(topk_ids, block_size, num_experts):
    flat = _i32(np.asarray(topk_ids).reshape(-1))
    n = flat.shape[0]
    sorted_ids = np.full(n + num_experts * (block_size - 1), n, dtype=np.int32)
    expert_ids = np.full(n + num_experts, -1, dtype=np.int32)
    post = np.zeros(1, dtype=np.int32)
    _l().orc_moe_align_block_size(_p(flat), ctypes.c_int64(n), ctypes.c_int(num_experts),
                                  ctypes.c_int(block_size), _p(sorted_ids), _p(expert_ids), _p(post))
    return sorted_ids, expert_ids, int(post[0])


def w4_dequant(qweight, scales, qzeros, group_size=128, zero_offset=1):
    """[K, N] fp32 weights from GPTQ-packed int4 (splitk_dequant_gemm.py:56-77)."""
    qw, s, qz = _i32(qweight), _f32(scales), _i32(qzeros)
    K, N = qw.shape[0] * 8, qw.shape[1]
    out = np.empty((K, N), dtype=np.float32)
    _l().orc_w4_dequant(_p(qw), _p(s), _p(qz), ctypes.c_int(K), ctypes.c_int(N), ctypes.c_int(group_size),
                        ctypes.c_int(zero_offset), _p(out))
    return out


def w4a16_gemm(a, qweight, scales, qzeros, group_size=128, zero_offset=1):
    a, qw, s, qz = _f32(a), _i32(qweight), _f32(scales), _i32(qzeros)
    M, K = a.shape
    N = qw.shape[1]
    c = np.empty((M, N), dtype=np.float32)
    _l().orc_w4a16_gemm(_p(a), _p(qw), _p(s), _p(qz), ctypes.c_int(M), ctypes.c_int(N), ctypes.c_int(K),
                        ctypes.c_int(group_size), ctypes.c_int(zero_offset), _p(c))
    return c


def e4m3_to_f32(codes):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    lut = np.array([_l().orc_e4m3_to_f32(i) for i in range(256)], dtype=np.float32)
    return lut[codes]


def f32_to_e4m3(x):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.uint8)
    flat_in, flat_out = x.reshape(-1), out.reshape(-1)
    f = _l().orc_f32_to_e4m3
    for i in range(flat_in.shape[0]):
        flat_out[i] = f(float(flat_in[i]))
    return out


def fp8_groupwise_quant(x, block=128):
    """(codes uint8 like x, scales [..., K/block] fp32) - float8_groupwise_quant.py:36-50."""
    x = _f32(x)
    q = np.empty(x.shape, dtype=np.uint8)
    scales = np.empty(x.shape[:-1] + (x.shape[-1] // block,), dtype=np.float32)
    _l().orc_fp8_groupwise_quant(_p(x), ctypes.c_int64(x.size), ctypes.c_int(block), _p(q), _p(scales))
    return q, scales


def fp8_block_quant_weight(w, block=128):
    """128x128 block quantiser for [rows, K] weights (rule of float8_groupwise_quant.py:36-50 per block)."""
    w = _f32(w)
    rows, K = w.shape
    q = np.empty(w.shape, dtype=np.uint8)
    scales = np.empty((rows // block, K // block), dtype=np.float32)
    _l().orc_fp8_block_quant_weight(_p(w), ctypes.c_int64(rows), ctypes.c_int(K), ctypes.c_int(block), _p(q), _p(scales))
    return q, scales


def grouped_gemm_fp8(xq, wq, x_scale, w_scale, m_sizes, scale_mode, block_layout=False, fill=np.nan):
    """fp8 grouped GEMM oracle; scale_mode 0 = row-wise (base_testing.py:83-88), 1 = 1x128 / 128x128 blocks."""
    xq = np.ascontiguousarray(xq, dtype=np.uint8)
    wq = np.ascontiguousarray(wq, dtype=np.uint8)
    xs, ws, m = _f32(x_scale), _f32(w_scale), _i32(m_sizes)
    G = m.shape[0]
    M, K = xq.shape
    N = wq.shape[0] // G
    cols = N * G if block_layout else N
    y = np.full((M, cols), fill, dtype=np.float32)
    _l().orc_grouped_gemm_fp8(_p(xq), _p(wq), _p(xs), _p(ws), ctypes.c_int(scale_mode), _p(m), ctypes.c_int(G),
                              ctypes.c_int64(M), ctypes.c_int(N), ctypes.c_int(K), _p(y), ctypes.c_int64(cols),
                              ctypes.c_int(N if block_layout else 0))
    return y


def round_bf16(x):
    """fp32 -> bf16 -> fp32, round-to-nearest-even (vectorised restatement of orc_round_bf16)."""
    u = _f32(x).view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) & 0xFFFF0000).astype(np.uint32)
    return r.view(np.float32).reshape(np.shape(x))


def pack_int4_along_k(q):
    """[K, N] values 0..15 -> int32 [K/8, N], nibble j of a word = row 8*i + j (splitk_dequant_gemm.py:56,76)."""
    q = np.asarray(q, dtype=np.uint32)
    K, N = q.shape
    out = np.zeros((K // 8, N), dtype=np.uint32)
    for j in range(8):
        out |= q[j::8, :] << np.uint32(4 * j)
    return out.view(np.int32)


def pack_int4_along_n(z):
    """[G, N] values 0..15 -> int32 [G, N/8], nibble j of a word = column 8*i + j (splitk_dequant_gemm.py:57,70)."""
    z = np.asarray(z, dtype=np.uint32)
    G, N = z.shape
    out = np.zeros((G, N // 8), dtype=np.uint32)
    for j in range(8):
        out |= z[:, j::8] << np.uint32(4 * j)
    return out.view(np.int32)


def grouped_gemm_torch_loop(x, w, m_sizes):
    """The reference's CPU-expressible path: a per-expert torch.matmul loop over the expert-sorted rows
    (dev/triton_groupGEMM/testing/unit_tests.py:49-55), fp32 on the host cores. Used by tests as a second
    opinion on the C oracle and by bench.py as the timed CPU baseline."""
    import torch

    G = len(m_sizes)
    N = w.shape[0] // G
    y = torch.zeros((x.shape[0], N), dtype=torch.float32)
    start = 0
    for g in range(G):
        m = int(m_sizes[g])
        if m > 0:
            y[start:start + m] = x[start:start + m] @ w[g * N:(g + 1) * N].T
        start += m
    return y


def grouped_gemm_backward_torch_loop(grad_output, x, w, m_sizes):
    """Both gradients of the grouped GEMM as a per-expert loop of fp32 torch matmuls on the host cores
    (grad_x_g = dY_g @ w_g, grad_w_g = dY_g^T @ x_g; kernels/MoE/group_GEMM/triton/testing/
    pytorch_reference_backwards.py:165-197). grad_output [M, N], x [M, K], w [G*N, K] float tensors; only the experts
    listed in m_sizes are computed (a prefix of all experts is allowed). bench.py times it as the CPU baseline of the
    backward workload; tests check it against the scalar C form."""
    import torch

    G = len(m_sizes)
    N = grad_output.shape[1]
    K = x.shape[1]
    rows = int(sum(int(m) for m in m_sizes))
    gx = torch.zeros((rows, K), dtype=torch.float32)
    gw = torch.zeros((G * N, K), dtype=torch.float32)
    start = 0
    for g in range(G):
        m = int(m_sizes[g])
        if m > 0:
            dy = grad_output[start:start + m]
            gx[start:start + m] = dy @ w[g * N:(g + 1) * N]
            gw[g * N:(g + 1) * N] = dy.T @ x[start:start + m]
        start += m
    return gx, gw


def w4a16_grouped_torch_loop(a, qweight, scales, qzeros, m_sizes, group_size=128, zero_offset=1):
    """Per-expert W4A16 product over expert-sorted rows on the host cores: w4a16_torch (dequantisation included) for
    every expert of m_sizes that has rows (the GEMM of gptq/mixtral/w4a16_fused_dequant_gemm.py:49-149). qweight
    [E', K/8, N], scales [E', K/g, N], qzeros [E', K/g, N/8] with E' >= len(m_sizes). fp32 tensor out [sum m, N]."""
    import torch

    rows = int(sum(int(m) for m in m_sizes))
    out = torch.zeros((rows, qweight.shape[2]), dtype=torch.float32)
    start = 0
    for e, m in enumerate(m_sizes):
        m = int(m)
        if m > 0:
            out[start:start + m] = w4a16_torch(a[start:start + m], qweight[e], scales[e], qzeros[e], group_size, zero_offset)
        start += m
    return out


def w4a16_torch(a, qweight, scales, qzeros, group_size=128, zero_offset=1):
    """W4A16 on the host cores the way the reference's path states it: dequantise the GPTQ-packed weights with the
    closed form of kernels/triton/inference/gptq/splitk_dequant_gemm.py:56-77 (vectorised torch ops, fp32), then
    torch.matmul. Tensors in (a [M, K] float, qweight [K/8, N] int32, scales [K/g, N] float, qzeros [K/g, N/8] int32),
    fp32 tensor out. bench.py times it (dequantisation included) as the CPU baseline of the W4A16 workloads; tests
    check it against the scalar C form."""
    import torch

    K8, N = qweight.shape
    shifts = torch.arange(8, dtype=torch.int32) * 4
    q = ((qweight[:, None, :] >> shifts[None, :, None]) & 15).reshape(K8 * 8, N)
    z = ((qzeros[:, :, None] >> shifts[None, None, :]) & 15).reshape(qzeros.shape[0], N) + zero_offset
    w = (q - z.repeat_interleave(group_size, dim=0)).float() * scales.float().repeat_interleave(group_size, dim=0)
    return a.float() @ w


def grouped_gemm_fp8_block_torch_loop(xq, wq, x_scale, w_scale, m_sizes, N, block=128):
    """Block-scaled fp8 grouped GEMM on the host cores: per expert, dequantise codes with their 1 x 128 / 128 x 128
    scales (torch's e4m3fn cast and broadcasting) and torch.matmul, streamed one expert at a time (the per-expert
    loop of dev/triton_groupGEMM/testing/unit_tests.py:49-55 with the dequantisation of base_testing.py:83-88 inside
    it). xq [R, K] / wq [G*N, K] torch.float8_e4m3fn (or uint8 codes), x_scale [R, K/128], w_scale [G*N/128, K/128];
    only the experts listed in m_sizes are computed (len(m_sizes) may be a prefix of all experts). fp32 out [R', N]."""
    import torch

    f8 = torch.float8_e4m3fn
    if xq.dtype == torch.uint8:
        xq = xq.view(f8)
    if wq.dtype == torch.uint8:
        wq = wq.view(f8)
    K = xq.shape[1]
    rows = int(sum(int(m) for m in m_sizes))
    y = torch.zeros((rows, N), dtype=torch.float32)
    start = 0
    for g, m in enumerate(m_sizes):
        m = int(m)
        if m > 0:
            xd = xq[start:start + m].float() * x_scale[start:start + m].repeat_interleave(block, dim=1)
            sw = w_scale[g * N // block:(g + 1) * N // block]
            wd = (wq[g * N:(g + 1) * N].float().view(N // block, block, K // block, block) * sw[:, None, :, None]).view(N, K)
            y[start:start + m] = xd @ wd.T
        start += m
    return y


def silu_and_mul(x):
    """out = silu(x[:, :n]) * x[:, n:] (ops.silu_and_mul, v0_moe_fused.py:284)."""
    x = _f32(x)
    rows, n = x.shape[0], x.shape[1] // 2
    out = np.empty((rows, n), dtype=np.float32)
    _l().orc_silu_and_mul(_p(x), ctypes.c_int64(rows), ctypes.c_int(n), _p(out))
    return out


def fused_moe(a, w1, w2, topk_weight, topk_ids, round_intermediate=True):
    """torch_moe of test_moe_gemm.py:16-30 in double precision: a [T, K], w1 [E, 2n, K], w2 [E, d, n],
    topk_weight / topk_ids [T, k] -> out [T, d]. round_intermediate rounds the stored intermediates to bf16."""
    a, w1, w2, tw, ids = _f32(a), _f32(w1), _f32(w2), _f32(topk_weight), _i32(topk_ids)
    T, K = a.shape
    E, two_n, _ = w1.shape
    d = w2.shape[1]
    k = ids.shape[1]
    out = np.empty((T, d), dtype=np.float32)
    _l().orc_fused_moe(_p(a), _p(w1), _p(w2), _p(tw), _p(ids), ctypes.c_int64(T), ctypes.c_int(K), ctypes.c_int(E),
                       ctypes.c_int(two_n // 2), ctypes.c_int(d), ctypes.c_int(k), ctypes.c_int(1 if round_intermediate else 0),
                       _p(out))
    return out


def fused_moe_torch(a, w1, w2, topk_weight, topk_ids):
    """The same layer as a per-expert loop of fp32 torch matmuls on the CPU (the shape of the reference's
    torch_moe, test_moe_gemm.py:16-30), for sizes the scalar C loop would take minutes on. Tensors in, tensor out."""
    import torch

    a, w1, w2 = a.float(), w1.float(), w2.float()
    T, k = topk_ids.shape
    n = w1.shape[1] // 2
    rep = a.repeat_interleave(k, dim=0)
    out = torch.zeros(T * k, w2.shape[1])
    flat = topk_ids.reshape(-1)
    for e in range(w1.shape[0]):
        mask = flat == e
        if mask.any():
            h = rep[mask] @ w1[e].t()
            h = torch.nn.functional.silu(h[:, :n]) * h[:, n:]
            out[mask] = h @ w2[e].t()
    return (out.view(T, k, -1) * topk_weight.float().view(T, k, 1)).sum(dim=1)


def w4a16_grouped(a, qweight, scales, qzeros, m_sizes, group_size=128, zero_offset=1, fill=np.nan):
    """Per-expert W4A16 product over expert-sorted rows (the GEMM of w4a16_fused_moe_kernel,
    gptq/mixtral/w4a16_fused_dequant_gemm.py:49-149): qweight [E, K/8, N], scales [E, K/g, N], qzeros [E, K/g, N/8].
    Composition of w4a16_gemm (pinned on its own) over the offsets of m_sizes; unwritten rows hold `fill`."""
    a = _f32(a)
    E = len(m_sizes)
    N = qweight.shape[2]
    out = np.full((a.shape[0], N), fill, dtype=np.float32)
    start = 0
    for e in range(E):
        m = int(m_sizes[e])
        if m:
            out[start:start + m] = w4a16_gemm(a[start:start + m], qweight[e], scales[e], qzeros[e], group_size, zero_offset)
        start += m
    return out


def dequant_gemm_moe(a, qw1, qw2, s1, s2, z1, z2, topk_ids, topk_weight=None, group_size=128, zero_offset=1,
                     round_intermediate=True):
    """The W4A16 MoE layer (dequant_gemm_moe, gptq/mixtral/w4a16_fused_dequant_gemm.py:255-318): both expert weight
    sets dequantised with w4_dequant, then fused_moe. The reference sums the top-k rows without routed weights
    (:316-317), which is topk_weight = None here."""
    E = qw1.shape[0]
    w1 = np.stack([w4_dequant(qw1[e], s1[e], z1[e], group_size, zero_offset).T for e in range(E)])   # [E, 2n, K]
    w2 = np.stack([w4_dequant(qw2[e], s2[e], z2[e], group_size, zero_offset).T for e in range(E)])   # [E, d, n]
    ids = _i32(topk_ids)
    tw = np.ones(ids.shape, dtype=np.float32) if topk_weight is None else _f32(topk_weight)
    return fused_moe(a, w1, w2, tw, ids, round_intermediate)
