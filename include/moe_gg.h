/*
 * moe_gg.h - C ABI of libmoe_gg.so: MI355X (gfx950) MoE grouped-GEMM inference path.
 *
 * Plain pointers and sizes only; no torch types. Every pointer marked "device" must be HIP device
 * memory on the current device. All entry points are asynchronous: they enqueue kernels on `stream`
 * (a hipStream_t passed as void*; NULL = the default stream) and return without synchronising.
 * The library keeps no per-call state, never allocates device memory and never synchronises. Its only mutable
 * state is process-wide and set explicitly: the kernel-variant pins of moe_gg_set_variant (a test / tuning hook,
 * see there) and the per-device address of the static scratch array of moe_gg_grouped_gemm_backward_bf16_static.
 *
 * Return value: 0 on success, a negative MOE_GG_E* code for a rejected argument (nothing was
 * launched), or a positive hipError_t from the HIP runtime.
 *
 * The boundary follows the reference's own native pattern: an extern "C" launcher taking raw
 * pointers + dims + stream and returning an error code
 * (kernels/blackwell/cute_gemm_01/sm100_gemm.h:33-35), wrapped by host code that checks
 * device / dtype / contiguity / shape (kernels/blackwell/cute_gemm_01/sm100_gemm_pytorch.cpp:49-100).
 */
#ifndef MOE_GG_H
#define MOE_GG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOE_GG_ABI_VERSION 1

#define MOE_GG_OK 0
#define MOE_GG_EINVAL (-1)       /* null pointer, negative size, bad enum value */
#define MOE_GG_ESHAPE (-2)       /* dimensions inconsistent with each other */
#define MOE_GG_EALIGN (-3)       /* pointer or leading dimension not aligned as required */
#define MOE_GG_EUNSUPPORTED (-4) /* valid request outside what the kernels cover (e.g. G > 1024) */
#define MOE_GG_EDEVICE (-5)      /* no usable gfx950 device */

#define MOE_GG_MAX_GROUPS_ABI 1024 /* largest G the grouped kernels accept */

/* Output layouts of the grouped GEMM. */
#define MOE_GG_OUT_MN 0     /* y is [M, N]: dev/triton_groupGEMM/groupgemm.py:427 */
#define MOE_GG_OUT_BLOCK 1  /* y is [M, N*G], expert g writes columns [g*N, (g+1)*N):
                               kernels/MoE/group_GEMM/triton/tgroup_gemm_forward.py:280-289 */

int moe_gg_abi_version(void);
const char* moe_gg_strerror(int code);

/*
 * bf16 grouped GEMM forward. Replaces grouped_gemm -> _grouped_gemm -> _kernel_grouped_gemm
 * (dev/triton_groupGEMM/groupgemm.py:518-521, 407-515, 130-254) and, with
 * out_layout = MOE_GG_OUT_BLOCK, grouped_gemm_forward
 * (kernels/MoE/group_GEMM/triton/tgroup_gemm_forward.py:626-629).
 *
 *   x        device, bf16 [M, K] row-major, rows sorted by expert
 *   w        device, bf16 [G*N, K] row-major (stacked expert weights)
 *   y        device, bf16, leading dimension ldy elements; rows >= sum(m_sizes) are not written
 *   m_sizes  device, int32 [G]; rows per expert. Consumed on the device (no host copy, no sync).
 *            Negative entries count as 0 and the running sum is clamped at M.
 * fp32 accumulation, round-to-nearest-even bf16 output.
 */
int moe_gg_grouped_gemm_bf16(const void* x, const void* w, void* y, const int32_t* m_sizes, int G,
                             int64_t M, int N, int K, int64_t ldy, int out_layout, void* stream);
/* The same on IEEE half x, w and y (the reference's MoE layer and its test run in fp16 as well:
 * kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:216, test_moe_gemm.py:33-60). Same kernels with the f16
 * MFMA. */
int moe_gg_grouped_gemm_f16(const void* x, const void* w, void* y, const int32_t* m_sizes, int G,
                            int64_t M, int N, int K, int64_t ldy, int out_layout, void* stream);

#define MOE_GG_SCALE_ROWWISE 0  /* x_scale [M], w_scale [G*N] */
#define MOE_GG_SCALE_BLOCK128 1 /* x_scale [M, K/128], w_scale [G*N/128, K/128] */

/*
 * fp8 (OCP e4m3fn) grouped GEMM forward, bf16 output, fp32 accumulation and scales.
 * scale_mode = MOE_GG_SCALE_ROWWISE replaces grouped_gemm_fp8_rowwise -> _kernel_grouped_gemm_fp8_rowwise
 * (dev/triton_groupGEMM/groupgemm.py:524-531, 269-404): y = (x @ w_g^T) * x_scale[m] * w_scale[g*N + n].
 * scale_mode = MOE_GG_SCALE_BLOCK128 is the block-scaled extension used by the DeepSeek-V3-style
 * configuration: per-1x128 activation scales as produced by float8_groupwise_quantize
 * (kernels/triton/inference/fp8/float8_groupwise_quant.py:53-91) and per-128x128 weight scales; each
 * 128-wide K block is scaled by x_scale[m, kb] * w_scale[(g*N + n) / 128, kb] before it is summed.
 * x, w: device fp8 [M, K] / [G*N, K]; other arguments as for moe_gg_grouped_gemm_bf16.
 * Requires K % 128 == 0 (and N % 128 == 0 for block scales).
 */
int moe_gg_grouped_gemm_fp8(const void* x, const void* w, void* y, const float* x_scale, const float* w_scale,
                            int scale_mode, const int32_t* m_sizes, int G, int64_t M, int N, int K,
                            int64_t ldy, int out_layout, void* stream);

#define MOE_GG_DTYPE_BF16 0
#define MOE_GG_DTYPE_FP16 1
#define MOE_GG_DTYPE_FP32 2

/*
 * W4A16 split-K dequant GEMM. Replaces matmul_split_k -> matmul_split_k_kernel
 * (kernels/triton/inference/gptq/splitk_dequant_gemm.py:91-141, 23-89).
 *
 *   a        device, [M, K] row-major, bf16 or fp16 (dtype)
 *   qweight  device, int32 [K/8, N]; nibble j of a word is row 8*i + j (LSB = lowest k)
 *   scales   device, [K/group_size, N], same 16-bit type as a
 *   qzeros   device, int32 [K/group_size, N/8]; nibble j of a word is column 8*i + j
 *   c        device, [M, N], same type as a; fully overwritten (no zero-initialisation needed)
 *   w(k, n) = (q(k, n) - (z(k/group_size, n) + zero_offset)) * s(k/group_size, n);
 *   zero_offset = 1 is the reference's convention (splitk_dequant_gemm.py:73-74), 0 gives (q - z) * s.
 * K is split over the eight waves of a workgroup and reduced in a fixed order (deterministic, no
 * atomics). Requires N % 64 == 0 and group_size % 32 == 0.
 */
int moe_gg_w4a16_splitk(const void* a, const int32_t* qweight, const void* scales, const int32_t* qzeros,
                        void* c, int M, int N, int K, int group_size, int zero_offset, int dtype,
                        void* stream);

/*
 * W4A16 grouped (MoE) GEMM: every expert has its own int4 weights; rows of a and c are sorted by expert.
 * Replaces the GEMM of the reference's W4A16 fused MoE kernel (w4a16_fused_moe_kernel / invoke_dequant_gemm_moe,
 * kernels/triton/inference/gptq/mixtral/w4a16_fused_dequant_gemm.py:49-149, 153-208) on expert-sorted rows instead
 * of its padded token lists:  c[off_g + i, :] = a[off_g + i, :] @ dequant(qweight[g], scales[g], qzeros[g]).
 *   a device [M, K], c device [M, N] (bf16 or fp16, dtype); m_sizes device int32 [G] (consumed on the device);
 *   qweight device int32 [G, K/8, N]; scales device [G, K/group_size, N]; qzeros device int32 [G, K/group_size, N/8];
 *   nibble order, dequantisation formula, zero_offset and requirements as for moe_gg_w4a16_splitk
 *   (the reference kernel uses zero_offset = 1: w4a16_fused_dequant_gemm.py:133-137).
 * Rows >= sum(m_sizes) of c are not written. Built for a few rows per expert (decode): an expert with more
 * than 64 rows is computed in several passes over its weights.
 */
int moe_gg_w4a16_grouped(const void* a, const int32_t* qweight, const void* scales, const int32_t* qzeros, void* c,
                         const int32_t* m_sizes, int G, int64_t M, int N, int K, int group_size, int zero_offset,
                         int dtype, void* stream);

/*
 * The same grouped W4A16 GEMM with the 1 x 128 fp8 activation quantiser as its epilogue: instead of the 16-bit
 * result c it stores float8_groupwise_quantize(c) (kernels/triton/inference/fp8/float8_groupwise_quant.py:20-50,
 * 53-91), ready to be the x / x_scale of moe_gg_grouped_gemm_fp8 with MOE_GG_SCALE_BLOCK128. The reference runs
 * the quantiser as a kernel of its own on a result read back from memory (float8_groupwise_quant.py:53-91); here
 * the 16-bit result never leaves the chip. Bit-identical to moe_gg_w4a16_grouped followed by
 * moe_gg_fp8_groupwise_quant.
 *   c_q device [M, N] e4m3fn; c_scale device fp32 [M, N/128]; everything else as for moe_gg_w4a16_grouped,
 *   and N % 128 == 0. Rows >= sum(m_sizes) of c_q and c_scale are not written.
 */
int moe_gg_w4a16_grouped_fp8out(const void* a, const int32_t* qweight, const void* scales, const int32_t* qzeros,
                                void* c_q, float* c_scale, const int32_t* m_sizes, int G, int64_t M, int N, int K,
                                int group_size, int zero_offset, int dtype, void* stream);

#define MOE_GG_MAX_ROUTE_EXPERTS 768

/*
 * Routing: top-k expert choice, expert histogram, offsets and the stable expert-sorted permutation.
 * Replaces torch.topk as used by the reference's MoE test
 * (kernels/triton/inference/col_major_moe_gemm/test_moe_gemm.py:54-57) and the grouping of the external
 * moe_align_block_size op (semantics: kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:141-166),
 * without its padding.
 *   logits   device, fp32 [T, E]
 *   ids      device out, int32 [T, k]: the k largest entries of each row, descending, ties to the lower id
 *   perm     device out, int32 [T*k]: flat positions p = token*k + j grouped by ascending expert, stable;
 *            the source token of sorted row i is perm[i] / k
 *   m_sizes  device out, int32 [E]: rows per expert (the m_sizes argument of the grouped GEMMs)
 *   offsets  device out, int32 [E+1] or NULL: exclusive prefix sum of m_sizes
 *            (dev/triton_groupGEMM/groupgemm.py:159-165)
 * moe_gg_route_group does the grouping for ids chosen elsewhere (flat_ids int32 [n]; ids outside [0, E) are
 * dropped). E <= MOE_GG_MAX_ROUTE_EXPERTS.
 */
int moe_gg_route_topk(const float* logits, int64_t T, int E, int k, int32_t* ids, int32_t* perm, int32_t* m_sizes,
                      int32_t* offsets, void* stream);
int moe_gg_route_group(const int32_t* flat_ids, int64_t n, int E, int32_t* perm, int32_t* m_sizes, int32_t* offsets,
                       void* stream);
/* The padded form of that grouping, with the outputs of the reference's moe_align_block_size
 * (kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:138-180; worked example :157-165), from the perm and
 * m_sizes that moe_gg_route_group / moe_gg_route_topk wrote:
 *   sorted_ids   device out, int32 [n + E * (block_size - 1)]: expert e's entries of perm, padded with the value n up
 *                to a multiple of block_size; entries beyond the padded total are n as well
 *   expert_ids   device out, int32 [n + E]: the expert of every block of block_size entries; -1 beyond the last block
 *                (the reference leaves those uninitialised)
 *   num_post_pad device out, int32 [1]: the padded total */
int moe_gg_align_block_size(const int32_t* perm, const int32_t* m_sizes, int E, int64_t n, int block_size,
                            int32_t* sorted_ids, int32_t* expert_ids, int32_t* num_post_pad, void* stream);
/* out[i, :] = x[perm[i] / k, :] for i < n; rows of row_bytes bytes (multiple of 16), x and out 16-byte aligned;
 * x has src_rows rows. n_valid (device, int32 [1], may be null) is the number of leading entries of perm that are in
 * use, e.g. offsets + E of moe_gg_route_group when ids were dropped. An output row whose position is at or beyond
 * *n_valid, or whose perm entry names no row of x (negative, or perm[i] / k >= src_rows), is written as zeros and
 * nothing is read for it. (The x[sorted_token_ids // top_k] gather of the reference's kernel,
 * kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:63-69, with its token_mask.) */
int moe_gg_gather_rows(const void* x, const int32_t* perm, int k, void* out, int64_t n, int64_t row_bytes,
                       int64_t src_rows, const int32_t* n_valid, void* stream);

/*
 * Backward pass of the bf16 grouped GEMM. Replaces grouped_gemm_backward
 * (kernels/MoE/group_GEMM/triton/tgroup_gemm_backwards.py:382-590; eager form
 * kernels/MoE/group_GEMM/triton/testing/pytorch_reference_backwards.py:165-197):
 *   grad_x[rows of g, :] = dY_g @ w[g]            grad_w[g*N : (g+1)*N, :] = dY_g^T @ x[rows of g, :]
 * where dY_g = grad_out[rows of g, g*N : (g+1)*N] for grad_layout = MOE_GG_OUT_BLOCK (the reference: grad_out is
 * [M, N*G]) and grad_out[rows of g, 0 : N] for MOE_GG_OUT_MN. fp32 accumulation, bf16 results.
 *   grad_out device bf16, leading dimension ld_go; x device [M, K]; w device [G*N, K]; m_sizes device int32 [G];
 *   grad_x device out [M, K]: rows >= sum(m_sizes) are not written; grad_w device out [G*N, K]: fully written
 *   (zeros for an expert without rows).
 *   workspace: device scratch of at least moe_gg_grouped_gemm_backward_workspace(...) bytes, 256-byte aligned,
 *   owned by the caller (the library never allocates); it holds w^T and the transposed, zero-padded copies of
 *   grad_out and x that make every operand contiguous along its reduction dimension. Large calls read the
 *   operands as stored and leave the workspace untouched.
 * Requires N % 4 == 0 and K % 4 == 0; N % 64 == 0 for the fast grad_x kernels.
 */
size_t moe_gg_grouped_gemm_backward_workspace(int G, int64_t M, int N, int K, int grad_layout);
int moe_gg_grouped_gemm_backward_bf16(const void* grad_out, int64_t ld_go, int grad_layout, const void* x, const void* w,
                                      const int32_t* m_sizes, int G, int64_t M, int N, int K, void* grad_x, void* grad_w,
                                      void* workspace, size_t workspace_bytes, void* stream);

/*
 * The same backward pass for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc). No counterpart in the reference. It takes no workspace: the
 * transposed copies go into an array of MOE_GG_STATIC_SCRATCH_BYTES bytes that is part of the library's device
 * image (every GPU the library runs on holds its own copy until the process ends), and the call allocates and frees
 * nothing. Same arguments, results (bit for bit) and return codes as moe_gg_grouped_gemm_backward_bf16, plus
 * MOE_GG_EUNSUPPORTED when the call needs transposed copies and
 * moe_gg_grouped_gemm_backward_workspace(G, M, N, K, grad_layout) exceeds MOE_GG_STATIC_SCRATCH_BYTES (calls large
 * enough to read their operands as stored need no copies and are not limited).
 * All calls on one GPU share that GPU's array: calls that may overlap in time on one GPU (different streams or
 * threads) race and must be serialised by the caller; calls on one stream are ordered and safe. Nothing in the
 * array has to survive between calls, and every byte a call reads from it was written by that call.
 */
#define MOE_GG_STATIC_SCRATCH_BYTES (32 << 20)
int moe_gg_grouped_gemm_backward_bf16_static(const void* grad_out, int64_t ld_go, int grad_layout, const void* x,
                                             const void* w, const int32_t* m_sizes, int G, int64_t M, int N, int K,
                                             void* grad_x, void* grad_w, void* stream);

/*
 * First GEMM of a gated MoE layer with the activation fused into its epilogue. Replaces the pair
 * invoke_fused_moe_kernel(hidden_states, w1, ...) + ops.silu_and_mul
 * (kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:271-284):
 *   y[off_g + i, c] = silu(x[off_g + i] . w[g*2n + c]) * (x[off_g + i] . w[g*2n + n + c]),   c < n
 * x device [M, K] bf16 expert-sorted; w device [G*2n, K] bf16 (per expert n gate rows, then n up rows: the
 * reference's w1 layout); y device out [M, n] bf16 with leading dimension ldy. Both products are rounded to bf16
 * before the activation, so the result equals moe_gg_grouped_gemm_bf16 followed by moe_gg_silu_and_mul bit for
 * bit, without the [M, 2n] intermediate. Requires K % 64 == 0, n % 4 == 0, 2n*K < 2^31, 16-byte aligned x and w.
 */
int moe_gg_grouped_gemm_swiglu_bf16(const void* x, const void* w, void* y, const int32_t* m_sizes, int G, int64_t M,
                                    int n, int K, int64_t ldy, void* stream);
/* The same on IEEE half data. */
int moe_gg_grouped_gemm_swiglu_f16(const void* x, const void* w, void* y, const int32_t* m_sizes, int G, int64_t M,
                                   int n, int K, int64_t ldy, void* stream);

/*
 * The same product with the layer's row gather folded into the activation loads: row i of the expert-sorted order
 * is row perm[i] / k of the token matrix, as the reference's kernel reads A through sorted_token_ids
 * (kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:75-80, 93-96) instead of from a gathered copy.
 *   y[i, c] = silu(tokens[perm[i] / k] . w[g(i)*2n + c]) * (tokens[perm[i] / k] . w[g(i)*2n + n + c])
 * tokens device [T, K] (bf16, or fp16 with dtype = MOE_GG_DTYPE_FP16); perm device [M] int32 as moe_gg_route_group
 * writes it (entries of the first sum(m_sizes) positions are slots token * k + j < T * k; later ones are not read);
 * everything else as moe_gg_grouped_gemm_swiglu_bf16, whose result on moe_gg_gather_rows(tokens, perm, k) it equals
 * bit for bit. Requires in addition T * K * 2 < 2^31 (MOE_GG_EUNSUPPORTED otherwise: gather first). A perm entry
 * outside [0, T * k) cannot make the loads leave the token matrix (it is folded into range); the row it produces is
 * unspecified.
 */
int moe_gg_grouped_gemm_swiglu_gather(const void* tokens, int64_t T, const int32_t* perm, int k, const void* w, void* y,
                                      const int32_t* m_sizes, int G, int64_t M, int n, int K, int64_t ldy, int dtype,
                                      void* stream);

/*
 * Glue between the two grouped GEMMs of a whole MoE layer, as in the reference's fused_moe
 * (kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:222-296; oracle torch_moe,
 * kernels/triton/inference/col_major_moe_gemm/test_moe_gemm.py:16-30). All data bf16.
 *
 * moe_gg_silu_and_mul replaces ops.silu_and_mul (v0_moe_fused.py:284):
 *   out[r, c] = silu(in[r, c]) * in[r, n + c];  in device [rows, 2n], out device [rows, n], n % 8 == 0.
 * moe_gg_invert_perm: inv[perm[i]] = i for i < *n_valid (device int32, e.g. offsets + E of moe_gg_route_*;
 *   NULL = all n). inv is not written elsewhere: fill it with -1 first if expert ids may have been dropped.
 * moe_gg_combine_topk replaces the routed-weight multiply (MUL_ROUTED_WEIGHT, v0_moe_fused.py:122-126) and
 *   the sum over the k rows of a token (:291-296):
 *   out[t, :] = sum_j weights[t, j] * y[inv[t*k + j], :]   (fp32 accumulation, j ascending; inv entries
 *   outside [0, n_rows) contribute nothing). y device [n_rows, d], out device [T, d], d % 8 == 0;
 *   weights device [T, k], fp32 or bf16 (weights_dtype = MOE_GG_DTYPE_FP32 / MOE_GG_DTYPE_BF16).
 * The _f16 forms are the same on IEEE half data (and half or fp32 weights): the reference's layers also take fp16,
 * and its W4A16 MoE test runs in it (kernels/triton/inference/gptq/mixtral/test_dequant_moe_gemm.py:25-84).
 */
int moe_gg_silu_and_mul(const void* in, void* out, int64_t rows, int n, void* stream);
int moe_gg_silu_and_mul_f16(const void* in, void* out, int64_t rows, int n, void* stream);
int moe_gg_invert_perm(const int32_t* perm, int32_t* inv, int64_t n, const int32_t* n_valid, void* stream);
int moe_gg_combine_topk(const void* y, const int32_t* inv, const void* weights, int weights_dtype, void* out,
                        int64_t T, int k, int d, int64_t n_rows, void* stream);
int moe_gg_combine_topk_f16(const void* y, const int32_t* inv, const void* weights, int weights_dtype, void* out,
                            int64_t T, int k, int d, int64_t n_rows, void* stream);

/*
 * 1 x 128 group-wise fp8 e4m3fn quantiser. Replaces float8_groupwise_quantize
 * (kernels/triton/inference/fp8/float8_groupwise_quant.py:53-91): per 128 consecutive elements
 * s = max(amax|x|, 1e-12) / 448, q = clamp(x / s, -448, 448) -> e4m3fn (RNE).
 *   in  device, bf16 or fp32 (dtype), numel elements, numel % 128 == 0;  out device, numel bytes;
 *   scales device out, fp32 [numel / 128].
 */
int moe_gg_fp8_groupwise_quant(const void* in, int dtype, void* out, float* scales, int64_t numel, void* stream);

/*
 * 128 x 128 block fp8 e4m3fn quantiser for weight matrices: the weight side of the block-scaled grouped GEMM
 * (w / w_scale of moe_gg_grouped_gemm_fp8 with MOE_GG_SCALE_BLOCK128). Stands where the reference calls
 * quantize_fp8_block of the FBGEMM package (kernels/needs_perf_help/fp8_gemm_bench.py:16-21, not vendored);
 * the rule is the one of the in-tree 1 x 128 quantiser (float8_groupwise_quant.py:36-50) applied to a whole block:
 * s = max(amax|block|, 1e-12) / 448, q = clamp(w / s, -448, 448) -> e4m3fn (RNE).
 *   in  device [rows, K] row-major, bf16 or fp32 (dtype), rows % 128 == 0, K % 128 == 0, 16-byte aligned;
 *   out device [rows, K] bytes, 16-byte aligned;  scales device out, fp32 [rows / 128, K / 128].
 */
int moe_gg_fp8_block128_quant(const void* in, int dtype, void* out, float* scales, int64_t rows, int K, void* stream);

/*
 * Test / tuning hooks (no counterpart in the reference).
 * moe_gg_set_variant pins the kernel variant used by an op (-1 = automatic choice). The pin is one process-global
 * setting per op (an atomic int): it applies to every later call of that op from any thread, on any device and
 * stream, until it is set back. It is NOT thread-safe in the sense that matters to a caller: two threads that pin
 * different variants, or one thread that pins while another launches, see each other's setting, and a caller that
 * pins must restore -1 itself (also on its error paths). Production code never calls it; the automatic choice is
 * the supported mode.
 * moe_gg_host_enumerate_tiles runs the kernels' tile scheduler on the host: for a host copy of
 * m_sizes it writes, for every persistent workgroup in launch order, the tiles it would visit as
 * int32 quintuples (workgroup, group, tile_m, tile_n, first_row_of_group). Returns the number of
 * tiles written (<= max_tiles), or a negative error.
 */
#define MOE_GG_OP_GG_BF16 0
/* variants of MOE_GG_OP_GG_BF16 */
#define MOE_GG_GG_PINGPONG_256 0 /* 256x256 tiles, two wave groups alternating load / MFMA phases */
#define MOE_GG_GG_TILED_256 1    /* 256x256 tiles, all waves in step */
#define MOE_GG_GG_TILED_128 2    /* 128x128 tiles */
#define MOE_GG_GG_TILED_64 3     /* 64x128 tiles */
#define MOE_GG_GG_GENERIC 4      /* one thread per output element, any shape / alignment */
#define MOE_GG_GG_DECODE 5       /* small-M path: weights streamed once, split-K inside the workgroup */
#define MOE_GG_GG_TILED_256_W4 6 /* 256x256 tiles on four waves of 128x128 outputs each (never chosen automatically) */
#define MOE_GG_GG_FOURWAVE_256 7 /* the ping-pong kernel's tiles, tile order and slab stream on four waves of 128x128
                                    outputs each, loads and LDS reads placed behind single MFMAs (never chosen
                                    automatically); while pinned, moe_gg_grouped_gemm_swiglu_bf16 / _f16 run their
                                    four-wave form too */
#define MOE_GG_GG_FOURWAVE_TALL 8 /* the same kernel with tiles of up to 256 + 32 rows: an expert's last full row tile
                                     takes along up to 32 rows behind it, which otherwise are a low tile that streams
                                     the expert's weight tile a second time (never chosen automatically; SiLU-and-mul
                                     entry points as for 7; host enumerators: MOE_GG_ORDER_TALL_TILES) */
#define MOE_GG_OP_GG_FP8 1
/* variants of MOE_GG_OP_GG_FP8 */
#define MOE_GG_FP8_TILED_128 0       /* 128x128 tiles for every expert */
#define MOE_GG_FP8_STREAM_PINGPONG 1 /* experts with <= 64 rows: streaming split-K kernel; others: 256x256 ping-pong */
#define MOE_GG_FP8_STREAM_TILED 2    /* experts with <= 64 rows: streaming split-K kernel; others: 128x128 tiles */
#define MOE_GG_FP8_PINGPONG 3        /* 256x256 ping-pong kernel for every expert */
#define MOE_GG_OP_TILE_ORDER 2
/* variants of MOE_GG_OP_TILE_ORDER: tile order of the forward 256x256 ping-pong kernels (bf16, f16, fp8, the fused
 * SiLU-and-mul GEMM, grad_x of the backward pass) and of the host enumerators below. -1 means TWO_LISTS: the
 * split-tail order is opt-in until a timed run on the hardware has shown what it is worth. */
#define MOE_GG_ORDER_TWO_LISTS 0   /* long tiles, then low tiles; last round cut by its fill alone */
#define MOE_GG_ORDER_SPLIT_TAILS 1 /* + a tall expert's last full tile and few rows become two half tiles; row
                                      pieces of the last round chosen with the second list in view */
#define MOE_GG_ORDER_TALL_TILES 2  /* host enumerators only: the lists of MOE_GG_GG_FOURWAVE_TALL (the kernels take
                                      this value as TWO_LISTS) */
#define MOE_GG_OP_W4A16 3
/* variants of MOE_GG_OP_W4A16 (bits, group size 128 and 16-bit output only; -1 and 0 are the default kernels) */
#define MOE_GG_W4_ONE_PASS 1 /* 33-64 rows per expert: one pass of four activation fragments on four waves instead of
                                two passes of two fragments on eight (the weights are read and unpacked once) */
#define MOE_GG_W4_WARMUP 2   /* up to 16 rows per expert: two extra waves per workgroup request the workgroup's weight
                                lines ahead of the consumer waves; lanes of activation rows that do not exist issue
                                no loads */
#define MOE_GG_W4_STAGED 4   /* activations reach a wave through its own LDS area: loads of 4 rows x 256 contiguous bytes,
                                written to LDS and read back as MFMA fragments, instead of fragment loads of
                                16 rows x 64 bytes */
int moe_gg_set_variant(int op, int variant);
int moe_gg_host_enumerate_tiles(const int32_t* m_sizes_host, int G, int64_t M, int N, int block_m,
                                int block_n, int num_workgroups, int xcds, int32_t* out,
                                int max_tiles);
/* The same for the 256 x 256 ping-pong kernels (block_m must be 256), which keep two tile lists (long tiles; low
 * tiles and, with MOE_GG_ORDER_SPLIT_TAILS pinned, the two half tiles that replace the last full tile + few rows of
 * a tall group), give every workgroup
 * its tiles of the second list spread between its long ones, and cut the long tiles of a sparsely filled last
 * round into row pieces. Six int32 per tile here: (workgroup,
 * group, first row inside the group, rows, first column, columns), for each workgroup in the order in which it
 * computes them; a piece may have 0 rows, and the columns may reach beyond N. With MOE_GG_ORDER_TALL_TILES pinned the
 * lists are those of MOE_GG_GG_FOURWAVE_TALL: rows may be up to 256 + 32. The tile decode is the kernels' own code
 * (compiled for the host). */
int moe_gg_host_enumerate_tiles_two_lists(const int32_t* m_sizes_host, int G, int64_t M, int N, int block_m,
                                          int block_n, int num_workgroups, int xcds, int32_t* out,
                                          int max_tiles);
/* Into how many row pieces (1, 2 or 4) the ping-pong kernels cut the long tiles of their last round when the long
 * list has n_long tiles, the second list n_low and the launch num_workgroups workgroups, in the tile order that is
 * in force (n_low only matters to MOE_GG_ORDER_SPLIT_TAILS). */
int moe_gg_host_tail_pieces(int n_long, int n_low, int num_workgroups);

/* bf16 forward, automatic kernel choice with 256 x 256 tiles: 1 if for these (host) m_sizes the low tiles (an
 * expert's rows beyond its last full 256-row tile, when fewer than 128 and the expert has at least two full tiles
 * or no other tile) are computed by the small-M kernel instead of the ping-pong kernel, 0 if not; the tile order
 * above then holds without its low tiles. Only calls with at most 32 experts and K >= 8192 (K a multiple of 128)
 * launch the second kernel. Both kernels take this decision on the device; this is its host mirror
 * (num_workgroups as for the enumerators: the CU count rounded down to a multiple of the XCD count). */
int moe_gg_host_tails_apart(const int32_t* m_sizes_host, int G, int64_t M, int N, int K, int num_workgroups);

#ifdef __cplusplus
}
#endif
#endif /* MOE_GG_H */
