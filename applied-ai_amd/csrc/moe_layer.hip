// Element-wise and index kernels that turn the grouped GEMMs into a whole MoE layer.
//
// The layer follows the reference's fused_moe (kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:222-296):
//   gather rows by expert -> GEMM with w1 -> SiLU-and-mul (ops.silu_and_mul, :284) -> GEMM with w2 ->
//   multiply by the routed weight (MUL_ROUTED_WEIGHT, :122-126) and sum the top-k rows of each token (:291-296).
// Its oracle is torch_moe (kernels/triton/inference/col_major_moe_gemm/test_moe_gemm.py:16-30).
// All three kernels are HBM-bound byte movers: 16-byte accesses, a row per workgroup (or a grid-stride
// loop), no LDS.
#include "common.h"
#include "kernels.h"

namespace {

DEVINL float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
DEVINL float bf16_hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xFFFF0000u); }
// The two 16-bit floats of a dword, and back (round to nearest even); F16: IEEE half, else bf16.
template <bool F16> DEVINL float lo16(uint32_t w) {
  return F16 ? (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xFFFFu)) : bf16_lo(w);
}
template <bool F16> DEVINL float hi16(uint32_t w) {
  return F16 ? (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16)) : bf16_hi(w);
}
template <bool F16> DEVINL uint32_t pack16x2(float a, float b) {
  if (!F16) return pack_bf16x2(a, b);
  return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)a) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)b) << 16);
}

// out[r, c] = silu(in[r, c]) * in[r, n + c], in [rows, 2n], out [rows, n], both bf16 or both fp16, n % 8 == 0.
// silu(v) = v / (1 + exp(-v)) evaluated in fp32; one rounding to the 16-bit type at the end.
template <bool F16>
__global__ __launch_bounds__(256) void silu_and_mul_kernel(const u32x4_t* __restrict__ in, u32x4_t* __restrict__ out,
                                                           int64_t rows, int n8) {
  const int64_t total = rows * n8;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = idx / n8;
    const int c = (int)(idx - r * n8);
    const u32x4_t g = in[r * (2 * n8) + c];
    const u32x4_t u = in[r * (2 * n8) + n8 + c];
    u32x4_t o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float g0 = lo16<F16>(g[e]), g1 = hi16<F16>(g[e]);
      const float a0 = g0 / (1.f + __expf(-g0)) * lo16<F16>(u[e]);
      const float a1 = g1 / (1.f + __expf(-g1)) * hi16<F16>(u[e]);
      o[e] = pack16x2<F16>(a0, a1);
    }
    out[r * n8 + c] = o;
  }
}

// inv[perm[i]] = i for i < *n_valid (all n if n_valid is null): where the flat position token * k + j sits
// in the expert-sorted row order. Positions whose expert id was dropped by the grouping keep what inv held.
__global__ __launch_bounds__(256) void invert_perm_kernel(const int32_t* __restrict__ perm, int32_t* __restrict__ inv, int n,
                                                          const int32_t* __restrict__ n_valid) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const int lim = n_valid ? min(*n_valid, n) : n;
  if (i < lim) {
    const int p = perm[i];
    if (p >= 0 && p < n) inv[p] = i;
  }
}

// out[t, :] = sum_j weight[t, j] * y[inv[t * k + j], :], fp32 accumulation in the order j = 0 .. k-1,
// 16-bit out. One workgroup per token; d % 8 == 0. F16: y and out are fp16, else bf16. W16: the weights have that
// 16-bit type too, else they are fp32.
template <bool W16, bool F16>
__global__ __launch_bounds__(256) void combine_topk_kernel(const u32x4_t* __restrict__ y, const int32_t* __restrict__ inv,
                                                           const void* __restrict__ weights, u32x4_t* __restrict__ out,
                                                           int k, int d8, int n_rows) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < d8; c += blockDim.x) {
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    for (int j = 0; j < k; ++j) {
      const int row = inv[(int64_t)t * k + j];
      if (row < 0 || row >= n_rows) continue;
      const float w = W16 ? lo16<F16>((uint32_t)((const uint16_t*)weights)[(int64_t)t * k + j])
                          : ((const float*)weights)[(int64_t)t * k + j];
      const u32x4_t v = y[(int64_t)row * d8 + c];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[2 * e] += w * lo16<F16>(v[e]);
        acc[2 * e + 1] += w * hi16<F16>(v[e]);
      }
    }
    u32x4_t o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = pack16x2<F16>(acc[2 * e], acc[2 * e + 1]);
    out[(int64_t)t * d8 + c] = o;
  }
}

}  // namespace

hipError_t silu_and_mul_launch(const void* in, void* out, int64_t rows, int n, bool fp16, hipStream_t stream) {
  if (rows == 0 || n == 0) return hipSuccess;
  const int64_t total = rows * (n / 8);
  const int blocks = (int)(total / 256 + 1 < 256 * 32 ? total / 256 + 1 : 256 * 32);
  if (fp16) hipLaunchKernelGGL(silu_and_mul_kernel<true>, dim3(blocks), dim3(256), 0, stream, (const u32x4_t*)in, (u32x4_t*)out, rows, n / 8);
  else hipLaunchKernelGGL(silu_and_mul_kernel<false>, dim3(blocks), dim3(256), 0, stream, (const u32x4_t*)in, (u32x4_t*)out, rows, n / 8);
  return hipGetLastError();
}

hipError_t invert_perm_launch(const int32_t* perm, int32_t* inv, int n, const int32_t* n_valid, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(invert_perm_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, perm, inv, n, n_valid);
  return hipGetLastError();
}

hipError_t combine_topk_launch(const void* y, const int32_t* inv, const void* weights, bool weights_16bit, bool fp16,
                               void* out, int T, int k, int d, int n_rows, hipStream_t stream) {
  if (T == 0 || d == 0) return hipSuccess;
  const u32x4_t* yp = (const u32x4_t*)y;
  u32x4_t* op = (u32x4_t*)out;
  const dim3 grid(T), block(256);
  if (fp16 && weights_16bit) hipLaunchKernelGGL((combine_topk_kernel<true, true>), grid, block, 0, stream, yp, inv, weights, op, k, d / 8, n_rows);
  else if (fp16) hipLaunchKernelGGL((combine_topk_kernel<false, true>), grid, block, 0, stream, yp, inv, weights, op, k, d / 8, n_rows);
  else if (weights_16bit) hipLaunchKernelGGL((combine_topk_kernel<true, false>), grid, block, 0, stream, yp, inv, weights, op, k, d / 8, n_rows);
  else hipLaunchKernelGGL((combine_topk_kernel<false, false>), grid, block, 0, stream, yp, inv, weights, op, k, d / 8, n_rows);
  return hipGetLastError();
}
