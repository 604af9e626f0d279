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

// out[r, c] = silu(in[r, c]) * in[r, n + c], in [rows, 2n] bf16, out [rows, n] bf16, n % 8 == 0.
// silu(v) = v / (1 + exp(-v)) evaluated in fp32; one rounding to bf16 at the end.
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
      const float g0 = bf16_lo(g[e]), g1 = bf16_hi(g[e]);
      const float a0 = g0 / (1.f + __expf(-g0)) * bf16_lo(u[e]);
      const float a1 = g1 / (1.f + __expf(-g1)) * bf16_hi(u[e]);
      o[e] = pack_bf16x2(a0, a1);
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
// bf16 out. One workgroup per token; d % 8 == 0. WBF16: weights are bf16, else fp32.
template <bool WBF16>
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
      const float w = WBF16 ? __builtin_bit_cast(float, (uint32_t)((const uint16_t*)weights)[(int64_t)t * k + j] << 16)
                            : ((const float*)weights)[(int64_t)t * k + j];
      const u32x4_t v = y[(int64_t)row * d8 + c];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[2 * e] += w * bf16_lo(v[e]);
        acc[2 * e + 1] += w * bf16_hi(v[e]);
      }
    }
    u32x4_t o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = pack_bf16x2(acc[2 * e], acc[2 * e + 1]);
    out[(int64_t)t * d8 + c] = o;
  }
}

}  // namespace

hipError_t silu_and_mul_launch(const void* in, void* out, int64_t rows, int n, hipStream_t stream) {
  if (rows == 0 || n == 0) return hipSuccess;
  const int64_t total = rows * (n / 8);
  const int blocks = (int)(total / 256 + 1 < 256 * 32 ? total / 256 + 1 : 256 * 32);
  hipLaunchKernelGGL(silu_and_mul_kernel, dim3(blocks), dim3(256), 0, stream, (const u32x4_t*)in, (u32x4_t*)out, rows, n / 8);
  return hipGetLastError();
}

hipError_t invert_perm_launch(const int32_t* perm, int32_t* inv, int n, const int32_t* n_valid, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(invert_perm_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, perm, inv, n, n_valid);
  return hipGetLastError();
}

hipError_t combine_topk_launch(const void* y, const int32_t* inv, const void* weights, bool weights_bf16, void* out,
                               int T, int k, int d, int n_rows, hipStream_t stream) {
  if (T == 0 || d == 0) return hipSuccess;
  if (weights_bf16)
    hipLaunchKernelGGL(combine_topk_kernel<true>, dim3(T), dim3(256), 0, stream, (const u32x4_t*)y, inv, weights, (u32x4_t*)out, k, d / 8, n_rows);
  else
    hipLaunchKernelGGL(combine_topk_kernel<false>, dim3(T), dim3(256), 0, stream, (const u32x4_t*)y, inv, weights, (u32x4_t*)out, k, d / 8, n_rows);
  return hipGetLastError();
}
