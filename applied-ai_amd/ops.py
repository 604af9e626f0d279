"""Host-side mirror of the reference's Python entry functions for the MoE grouped-GEMM path.

Same names, argument meaning and return values as the reference launchers; the work is done by
hand-written gfx950 kernels behind the C ABI in include/moe_gg.h. torch is used for device
memory and the current stream only.
"""
from typing import Optional

import torch

from . import _lib

OUT_MN = 0
OUT_BLOCK = 1


def _stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _require_cuda(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    for t in tensors:
        if t.device.type != "cuda":
            raise RuntimeError(
                "applied_ai_amd ops run on a HIP device only (got a %s tensor); there is no CPU path"
                % t.device.type
            )
        if t.device != dev:
            raise RuntimeError("all tensors must be on the same device")
    return dev


def check_m_sizes(m_sizes: torch.Tensor, M: int) -> None:
    """The opt-in host check behind validate=True: one copy of m_sizes to the host, ValueError for a negative entry
    or a sum beyond the M rows of x - the two cases the reference's tests expect an exception for
    (dev/triton_groupGEMM/testing/unit_tests.py:191-212). Without it the kernels clamp such sizes on the device
    (negative -> 0, running sum capped at M), so nothing out of bounds is ever touched; the check costs a device
    synchronisation, which is why it is off by default."""
    sizes = m_sizes.detach().to("cpu", torch.int64)
    if sizes.numel() and int(sizes.min()) < 0:
        raise ValueError(f"m_sizes has a negative entry: {sizes.tolist()}")
    total = int(sizes.sum())
    if total > M:
        raise ValueError(f"sum(m_sizes) = {total} exceeds the {M} rows of x")


def _grouped_gemm_bf16(x: torch.Tensor, w: torch.Tensor, m_sizes: torch.Tensor, out_layout: int,
                       validate: bool = False) -> torch.Tensor:
    # Mirrors _grouped_gemm (dev/triton_groupGEMM/groupgemm.py:407-427): contiguity asserts,
    # G from m_sizes, N = w.shape[0] // G, K check, torch.empty output.
    assert x.is_contiguous()
    assert w.is_contiguous()
    assert m_sizes.is_contiguous()
    if x.dim() != 2 or w.dim() != 2 or m_sizes.dim() != 1:
        raise ValueError("x must be [M, K], w must be [G*N, K], m_sizes must be [G]")
    G = m_sizes.shape[0]
    M, K = x.shape
    if G == 0 or w.shape[0] % G != 0:
        raise ValueError(f"w.shape[0]={w.shape[0]} is not a multiple of G={G}")
    N = w.shape[0] // G
    assert K == w.shape[1], f"K mismatch: x has {K}, w has {w.shape[1]}"
    if x.dtype not in (torch.bfloat16, torch.float16) or w.dtype != x.dtype:
        raise ValueError("grouped_gemm takes bf16 (or fp16) x and w of the same dtype")
    if m_sizes.dtype != torch.int32:
        raise ValueError("m_sizes must be int32")
    if validate:
        check_m_sizes(m_sizes, M)
    dev = _require_cuda(x, w, m_sizes)
    cols = N * G if out_layout == OUT_BLOCK else N
    y = torch.empty((M, cols), device=dev, dtype=x.dtype)
    with torch.cuda.device(dev):
        L = _lib.lib()
        fn = L.moe_gg_grouped_gemm_f16 if x.dtype == torch.float16 else L.moe_gg_grouped_gemm_bf16
        rc = fn(
            x.data_ptr(), w.data_ptr(), y.data_ptr(), m_sizes.data_ptr(), G, M, N, K, cols, out_layout,
            _stream_ptr(dev),
        )
    _lib.check(rc, "moe_gg_grouped_gemm_bf16")
    return y


def grouped_gemm(x: torch.Tensor, w: torch.Tensor, m_sizes: torch.Tensor, validate: bool = False) -> torch.Tensor:
    """y[off_g:off_g+m_g] = x[off_g:off_g+m_g] @ w[g*N:(g+1)*N].T for every expert g; y is [M, N] in the dtype of
    x and w (bf16 as in the reference, or fp16).

    Drop-in for grouped_gemm (dev/triton_groupGEMM/groupgemm.py:518-521). Rows at or beyond
    sum(m_sizes) are left uninitialised, as in the reference (torch.empty, groupgemm.py:427).
    validate=True adds the host check of check_m_sizes (ValueError for negative sizes or sum(m_sizes) > M).
    """
    return _grouped_gemm_bf16(x, w, m_sizes, OUT_MN, validate)


def grouped_gemm_forward(x: torch.Tensor, w: torch.Tensor, m_sizes: torch.Tensor, validate: bool = False) -> torch.Tensor:
    """Same product with the [M, N*G] output of the MoE-training copy: expert g writes columns
    [g*N, (g+1)*N) of its own rows (kernels/MoE/group_GEMM/triton/tgroup_gemm_forward.py:626-629,
    280-289); everything else is left uninitialised."""
    return _grouped_gemm_bf16(x, w, m_sizes, OUT_BLOCK, validate)


def grouped_gemm_swiglu(x: torch.Tensor, w: torch.Tensor, m_sizes: torch.Tensor) -> torch.Tensor:
    """silu(x @ w_gate.T) * (x @ w_up.T) per expert in one kernel: x [M, K] expert-sorted, w [G*2n, K] with the
    reference's w1 layout (per expert n gate rows, then n up rows), result [M, n] bf16.

    The first GEMM of fused_moe with ops.silu_and_mul folded into its epilogue
    (kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:271-284); bit-identical to
    silu_and_mul(grouped_gemm(x, w, m_sizes))."""
    assert x.is_contiguous()
    assert w.is_contiguous()
    assert m_sizes.is_contiguous()
    if x.dim() != 2 or w.dim() != 2 or m_sizes.dim() != 1:
        raise ValueError("x must be [M, K], w must be [G*2n, K], m_sizes must be [G]")
    G = m_sizes.shape[0]
    M, K = x.shape
    if G == 0 or w.shape[0] % (2 * G) != 0:
        raise ValueError(f"w.shape[0]={w.shape[0]} is not a multiple of 2*G={2 * G}")
    n = w.shape[0] // (2 * G)
    assert K == w.shape[1], f"K mismatch: x has {K}, w has {w.shape[1]}"
    if x.dtype not in (torch.bfloat16, torch.float16) or w.dtype != x.dtype:
        raise ValueError("grouped_gemm_swiglu takes bf16 (or fp16) x and w of the same dtype")
    if m_sizes.dtype != torch.int32:
        raise ValueError("m_sizes must be int32")
    dev = _require_cuda(x, w, m_sizes)
    y = torch.empty((M, n), device=dev, dtype=x.dtype)
    with torch.cuda.device(dev):
        L = _lib.lib()
        fn = L.moe_gg_grouped_gemm_swiglu_f16 if x.dtype == torch.float16 else L.moe_gg_grouped_gemm_swiglu_bf16
        rc = fn(x.data_ptr(), w.data_ptr(), y.data_ptr(), m_sizes.data_ptr(), G, M, n, K, n, _stream_ptr(dev))
    _lib.check(rc, "moe_gg_grouped_gemm_swiglu_bf16")
    return y


def grouped_gemm_swiglu_gathered(tokens: torch.Tensor, perm: torch.Tensor, k: int, w: torch.Tensor,
                                 m_sizes: torch.Tensor) -> torch.Tensor:
    """grouped_gemm_swiglu(tokens[perm // k], w, m_sizes) without the gathered copy: the kernel reads row perm[i] // k
    of tokens [T, K] where the plain form reads sorted row i, as the reference's kernel reads A through
    sorted_token_ids (kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:75-80). perm [M] int32 and m_sizes
    as route_group returns them; rows at or beyond sum(m_sizes) are left unwritten. Same bits as the two-step form.
    Needs T * K * 2 < 2**31 bytes of tokens (ValueError beyond: gather first)."""
    assert tokens.is_contiguous()
    assert w.is_contiguous()
    assert m_sizes.is_contiguous() and perm.is_contiguous()
    if tokens.dim() != 2 or w.dim() != 2 or m_sizes.dim() != 1 or perm.dim() != 1:
        raise ValueError("tokens must be [T, K], perm [M], w [G*2n, K], m_sizes [G]")
    G = m_sizes.shape[0]
    T, K = tokens.shape
    M = perm.shape[0]
    if G == 0 or w.shape[0] % (2 * G) != 0:
        raise ValueError(f"w.shape[0]={w.shape[0]} is not a multiple of 2*G={2 * G}")
    n = w.shape[0] // (2 * G)
    assert K == w.shape[1], f"K mismatch: tokens have {K}, w has {w.shape[1]}"
    if tokens.dtype not in (torch.bfloat16, torch.float16) or w.dtype != tokens.dtype:
        raise ValueError("grouped_gemm_swiglu_gathered takes bf16 (or fp16) tokens and w of the same dtype")
    if m_sizes.dtype != torch.int32 or perm.dtype != torch.int32:
        raise ValueError("m_sizes and perm must be int32")
    if k < 1:
        raise ValueError("k must be at least 1")
    dev = _require_cuda(tokens, w, m_sizes, perm)
    y = torch.empty((M, n), device=dev, dtype=tokens.dtype)
    with torch.cuda.device(dev):
        rc = _lib.lib().moe_gg_grouped_gemm_swiglu_gather(tokens.data_ptr(), T, perm.data_ptr(), k, w.data_ptr(), y.data_ptr(),
                                                          m_sizes.data_ptr(), G, M, n, K, n, 1 if tokens.dtype == torch.float16 else 0,
                                                          _stream_ptr(dev))
    _lib.check(rc, "moe_gg_grouped_gemm_swiglu_gather")
    return y


def grouped_gemm_backward(grad_output: torch.Tensor, x: torch.Tensor, w: torch.Tensor, m_sizes: torch.Tensor):
    """Backward pass of the bf16 grouped GEMM: returns (grad_x [M, K], grad_w [G*N, K]).

    Drop-in for grouped_gemm_backward (kernels/MoE/group_GEMM/triton/tgroup_gemm_backwards.py:382-590):
    grad_output is the gradient of grouped_gemm_forward's [M, N*G] output, of which only the expert's own column
    block of each row is read; the [M, N] gradient of grouped_gemm is accepted as well. As in the reference, a K
    mismatch raises ValueError, inputs are made contiguous, grad_x rows at or beyond sum(m_sizes) are zero
    (torch.zeros_like, :442-443) and an expert without rows gets a zero grad_w block."""
    if grad_output.dim() != 2 or x.dim() != 2 or w.dim() != 2 or m_sizes.dim() != 1:
        raise ValueError("grad_output must be [M, N*G] or [M, N], x [M, K], w [G*N, K], m_sizes [G]")
    G = m_sizes.shape[0]
    M, K = x.shape
    if K != w.shape[1]:
        raise ValueError("K dimensions must match for grouped GEMM backward")
    if G == 0 or w.shape[0] % G != 0:
        raise ValueError(f"w.shape[0]={w.shape[0]} is not a multiple of G={G}")
    N = w.shape[0] // G
    if grad_output.shape == (M, N * G) and G > 1:
        layout = OUT_BLOCK
    elif grad_output.shape == (M, N):
        layout = OUT_MN
    else:
        raise ValueError(f"grad_output is {tuple(grad_output.shape)}, expected [{M}, {N * G}] or [{M}, {N}]")
    if grad_output.dtype != torch.bfloat16 or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise ValueError("grouped_gemm_backward takes bf16 grad_output, x and w")
    if m_sizes.dtype != torch.int32:
        raise ValueError("m_sizes must be int32")
    dev = _require_cuda(grad_output, x, w, m_sizes)
    grad_output, x, w, m_sizes = grad_output.contiguous(), x.contiguous(), w.contiguous(), m_sizes.contiguous()
    grad_x = torch.zeros_like(x)
    grad_w = torch.empty_like(w)
    with torch.cuda.device(dev):
        L = _lib.lib()
        nbytes = L.moe_gg_grouped_gemm_backward_workspace(G, max(M, 1), N, K, layout)
        workspace = torch.empty(max(nbytes, 256), device=dev, dtype=torch.uint8)
        rc = L.moe_gg_grouped_gemm_backward_bf16(
            grad_output.data_ptr(), grad_output.shape[1], layout, x.data_ptr(), w.data_ptr(), m_sizes.data_ptr(),
            G, M, N, K, grad_x.data_ptr(), grad_w.data_ptr(), workspace.data_ptr(), workspace.numel(), _stream_ptr(dev),
        )
    _lib.check(rc, "moe_gg_grouped_gemm_backward_bf16")
    return grad_x, grad_w


def matmul_split_k(a: torch.Tensor, b: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor,
                   zero_offset: int = 1, groupsize: Optional[int] = None) -> torch.Tensor:
    """W4A16 split-K dequant GEMM: c = a @ dequant(b, scales, zeros).

    Drop-in for matmul_split_k (kernels/triton/inference/gptq/splitk_dequant_gemm.py:91-141):
    a [M, K] fp16 or bf16; b [K/8, N] int32 (8 nibbles along K, LSB = lowest k); scales [K/g, N] in a's
    dtype; zeros [K/g, N/8] int32 (8 nibbles along N); returns c [M, N] in a's dtype.
    w = (q - (z + zero_offset)) * s with zero_offset = 1 as in the reference (:73-74); zero_offset = 0 gives
    (q - z) * s. The group size defaults to K // scales.shape[0] (128 in the reference, :94).
    Unlike the reference there is no atomic accumulation: the result is deterministic and c needs no
    zero-initialisation."""
    if a.dim() != 2 or b.dim() != 2 or scales.dim() != 2 or zeros.dim() != 2:
        raise ValueError("a, b, scales and zeros must be 2-D")
    m, k = a.shape
    kw, n = b.shape
    if kw * 8 != k:
        raise ValueError(f"b has {kw} packed rows, expected K/8 = {k // 8}")
    if b.dtype != torch.int32 or zeros.dtype != torch.int32:
        raise ValueError("b and zeros must be int32")
    if a.dtype not in (torch.bfloat16, torch.float16) or scales.dtype != a.dtype:
        raise ValueError("a and scales must both be bf16 or both fp16")
    g = groupsize if groupsize is not None else k // scales.shape[0]
    if scales.shape != (k // g, n) or zeros.shape != (k // g, n // 8):
        raise ValueError("scales must be [K/g, N] and zeros [K/g, N/8]")
    dev = _require_cuda(a, b, scales, zeros)
    a, b, scales, zeros = a.contiguous(), b.contiguous(), scales.contiguous(), zeros.contiguous()
    c = torch.empty((m, n), device=dev, dtype=a.dtype)
    with torch.cuda.device(dev):
        rc = _lib.lib().moe_gg_w4a16_splitk(
            a.data_ptr(), b.data_ptr(), scales.data_ptr(), zeros.data_ptr(), c.data_ptr(), m, n, k, g,
            zero_offset, 1 if a.dtype == torch.float16 else 0, _stream_ptr(dev),
        )
    _lib.check(rc, "moe_gg_w4a16_splitk")
    return c


def a100_qlinear(a: torch.Tensor, b: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor) -> torch.Tensor:
    """Drop-in for the reference's data-parallel (not split-K) W4A16 linear layers a100_qlinear / h100_qlinear /
    small_qlinear (kernels/triton/inference/gptq/a100_qlinear.py:76-121, h100_qlinear.py:87-121,
    small_benchmark_cuda_graphs.py:109-150): the same packing, group size 128 and (q - (z + 1)) * s as
    matmul_split_k (a100_qlinear.py:44-65), so one kernel serves all of them; the result has a's dtype."""
    return matmul_split_k(a, b, scales, zeros, zero_offset=1, groupsize=128)


h100_qlinear = a100_qlinear
small_qlinear = a100_qlinear


def matmul_split_k_grouped(a: torch.Tensor, b: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor,
                           m_sizes: torch.Tensor, zero_offset: int = 1, groupsize: Optional[int] = None,
                           quantize_output: bool = False):
    """W4A16 grouped GEMM over expert-sorted rows: c[rows of expert g] = a[rows of g] @ dequant(b[g], scales[g], zeros[g]).

    quantize_output=True returns float8_groupwise_quantize(c)
    (kernels/triton/inference/fp8/float8_groupwise_quant.py:53-91) instead of c - (q [M, N] float8_e4m3fn, scales
    [M, N/128] fp32), computed in the GEMM's epilogue; needs N % 128 == 0. Rows beyond sum(m_sizes) are zero then.

    The GEMM of the reference's W4A16 fused MoE kernel
    (kernels/triton/inference/gptq/mixtral/w4a16_fused_dequant_gemm.py:49-149) without its padded token lists:
    a [M, K] fp16 or bf16, rows sorted by expert; b [E, K/8, N] int32; scales [E, K/g, N]; zeros [E, K/g, N/8] int32;
    m_sizes [E] int32 on the device. Packing and zero_offset as in matmul_split_k."""
    if a.dim() != 2 or b.dim() != 3 or scales.dim() != 3 or zeros.dim() != 3 or m_sizes.dim() != 1:
        raise ValueError("a must be 2-D, b / scales / zeros 3-D, m_sizes 1-D")
    m, k = a.shape
    e, kw, n = b.shape
    if kw * 8 != k:
        raise ValueError(f"b has {kw} packed rows per expert, expected K/8 = {k // 8}")
    if b.dtype != torch.int32 or zeros.dtype != torch.int32 or m_sizes.dtype != torch.int32:
        raise ValueError("b, zeros and m_sizes must be int32")
    if a.dtype not in (torch.bfloat16, torch.float16) or scales.dtype != a.dtype:
        raise ValueError("a and scales must both be bf16 or both fp16")
    g = groupsize if groupsize is not None else k // scales.shape[1]
    if scales.shape != (e, k // g, n) or zeros.shape != (e, k // g, n // 8) or m_sizes.shape[0] != e:
        raise ValueError("scales must be [E, K/g, N], zeros [E, K/g, N/8], m_sizes [E]")
    dev = _require_cuda(a, b, scales, zeros, m_sizes)
    a, b, scales, zeros, m_sizes = a.contiguous(), b.contiguous(), scales.contiguous(), zeros.contiguous(), m_sizes.contiguous()
    if quantize_output:
        if n % 128 != 0:
            raise ValueError(f"quantize_output needs N % 128 == 0, got N = {n}")
        q = torch.zeros((m, n), device=dev, dtype=torch.float8_e4m3fn)
        qs = torch.zeros((m, n // 128), device=dev, dtype=torch.float32)
        with torch.cuda.device(dev):
            rc = _lib.lib().moe_gg_w4a16_grouped_fp8out(
                a.data_ptr(), b.data_ptr(), scales.data_ptr(), zeros.data_ptr(), q.data_ptr(), qs.data_ptr(),
                m_sizes.data_ptr(), e, m, n, k, g, zero_offset, 1 if a.dtype == torch.float16 else 0, _stream_ptr(dev),
            )
        _lib.check(rc, "moe_gg_w4a16_grouped_fp8out")
        return q, qs
    c = torch.empty((m, n), device=dev, dtype=a.dtype)
    with torch.cuda.device(dev):
        rc = _lib.lib().moe_gg_w4a16_grouped(
            a.data_ptr(), b.data_ptr(), scales.data_ptr(), zeros.data_ptr(), c.data_ptr(), m_sizes.data_ptr(), e, m, n,
            k, g, zero_offset, 1 if a.dtype == torch.float16 else 0, _stream_ptr(dev),
        )
    _lib.check(rc, "moe_gg_w4a16_grouped")
    return c


SCALE_ROWWISE = 0
SCALE_BLOCK128 = 1


def _grouped_gemm_fp8(x, w, m_sizes, x_scale, w_scale, scale_mode: int, out_layout: int = OUT_MN,
                      validate: bool = False) -> torch.Tensor:
    # Mirrors _grouped_gemm with scales (dev/triton_groupGEMM/groupgemm.py:407-427, 478-494).
    assert x.is_contiguous()
    assert w.is_contiguous()
    assert m_sizes.is_contiguous()
    assert x_scale.is_contiguous()
    assert w_scale.is_contiguous()
    if x.dim() != 2 or w.dim() != 2 or m_sizes.dim() != 1:
        raise ValueError("x must be [M, K], w must be [G*N, K], m_sizes must be [G]")
    G = m_sizes.shape[0]
    M, K = x.shape
    if G == 0 or w.shape[0] % G != 0:
        raise ValueError(f"w.shape[0]={w.shape[0]} is not a multiple of G={G}")
    N = w.shape[0] // G
    assert K == w.shape[1], f"K mismatch: x has {K}, w has {w.shape[1]}"
    if x.dtype != torch.float8_e4m3fn or w.dtype != torch.float8_e4m3fn:
        raise ValueError("x and w must be torch.float8_e4m3fn (gfx950 computes in OCP e4m3)")
    if x_scale.dtype != torch.float32 or w_scale.dtype != torch.float32 or m_sizes.dtype != torch.int32:
        raise ValueError("scales must be float32 and m_sizes int32")
    if scale_mode == SCALE_ROWWISE:
        want_x, want_w = (M,), (G * N,)
    else:
        if K % 128 or (G * N) % 128:
            raise ValueError("block scales need K and G*N to be multiples of 128")
        want_x, want_w = (M, K // 128), (G * N // 128, K // 128)
    if tuple(x_scale.shape) != want_x or tuple(w_scale.shape) != want_w:
        raise ValueError(f"scale shapes must be {want_x} and {want_w}")
    if validate:
        check_m_sizes(m_sizes, M)
    dev = _require_cuda(x, w, m_sizes, x_scale, w_scale)
    cols = N * G if out_layout == OUT_BLOCK else N
    y = torch.empty((M, cols), device=dev, dtype=torch.bfloat16)
    with torch.cuda.device(dev):
        rc = _lib.lib().moe_gg_grouped_gemm_fp8(
            x.data_ptr(), w.data_ptr(), y.data_ptr(), x_scale.data_ptr(), w_scale.data_ptr(), scale_mode,
            m_sizes.data_ptr(), G, M, N, K, cols, out_layout, _stream_ptr(dev),
        )
    _lib.check(rc, "moe_gg_grouped_gemm_fp8")
    return y


def grouped_gemm_fp8_rowwise(x: torch.Tensor, w: torch.Tensor, m_sizes: torch.Tensor, x_scale: torch.Tensor,
                             w_scale: torch.Tensor, validate: bool = False) -> torch.Tensor:
    """fp8 grouped GEMM with one scale per activation row and per weight row:
    y = (x @ w_g.T) * x_scale[:, None] * w_scale[g*N:(g+1)*N][None, :], bf16 out.
    Drop-in for grouped_gemm_fp8_rowwise (dev/triton_groupGEMM/groupgemm.py:524-531)."""
    return _grouped_gemm_fp8(x, w, m_sizes, x_scale, w_scale, SCALE_ROWWISE, validate=validate)


def grouped_gemm_fp8_rowwise_forward(x: torch.Tensor, w: torch.Tensor, m_sizes: torch.Tensor, x_scale: torch.Tensor,
                                     w_scale: torch.Tensor, validate: bool = False) -> torch.Tensor:
    """The same with the [M, N*G] output of the MoE-training copy: expert g writes columns [g*N, (g+1)*N) of its
    own rows, the rest stays uninitialised. Drop-in for that copy's grouped_gemm_fp8_rowwise
    (kernels/MoE/group_GEMM/triton/tgroup_gemm_forward.py:632-639, store at :468-480)."""
    return _grouped_gemm_fp8(x, w, m_sizes, x_scale, w_scale, SCALE_ROWWISE, OUT_BLOCK, validate)


def grouped_gemm_fp8_blockwise(x: torch.Tensor, w: torch.Tensor, m_sizes: torch.Tensor, x_scale: torch.Tensor,
                               w_scale: torch.Tensor, validate: bool = False) -> torch.Tensor:
    """fp8 grouped GEMM with 1x128 activation scales x_scale[M, K/128] (the output layout of
    float8_groupwise_quantize, kernels/triton/inference/fp8/float8_groupwise_quant.py:53-91) and 128x128
    weight scales w_scale[G*N/128, K/128]; bf16 out. No counterpart in the reference (its fp8 grouped GEMM is
    row-wise only); it is the block-scaled extension of that entry point."""
    return _grouped_gemm_fp8(x, w, m_sizes, x_scale, w_scale, SCALE_BLOCK128, validate=validate)
