// 1 x 128 group-wise fp8 (OCP e4m3fn) activation quantiser for gfx950.
//
// Replaces _float8_groupwise_quant_kernel / float8_groupwise_quantize
// (kernels/triton/inference/fp8/float8_groupwise_quant.py:20-50, 53-91): per group of 128 consecutive
// elements  s = max(amax|x|, 1e-12) / 448,  q = clamp(x / s, -448, 448) -> e4m3fn (round to nearest even);
// q and s are stored, s as fp32 [..., K/128]. One wave per group, two elements per lane; the fp32
// division is the correctly rounded one, so the result is bit-identical to the CPU oracle.
// Also the 128 x 128 block form of the same rule for weight matrices (one scale per block), the weight side of
// the block-scaled fp8 grouped GEMM.
#include "common.h"
#include "kernels.h"

namespace {

template <bool BF16_IN>
__global__ __launch_bounds__(256) void fp8_groupwise_quant_kernel(const void* __restrict__ in, uint8_t* __restrict__ out,
                                                                 float* __restrict__ scales, int64_t groups) {
  const int lane = threadIdx.x & 63;
  const int64_t g = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (g >= groups) return;
  float a, b;
  if (BF16_IN) {
    const uint32_t v = ((const uint32_t*)in)[g * 64 + lane];
    a = __builtin_bit_cast(float, v << 16);
    b = __builtin_bit_cast(float, v & 0xFFFF0000u);
  } else {
    const float2 v = ((const float2*)in)[g * 64 + lane];
    a = v.x;
    b = v.y;
  }
  float amax = fmaxf(fabsf(a), fabsf(b));
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) amax = fmaxf(amax, __shfl_xor(amax, d, 64));
  const float s = fmaxf(amax, 1e-12f) / 448.0f;
  const float ya = fminf(fmaxf(a / s, -448.0f), 448.0f);
  const float yb = fminf(fmaxf(b / s, -448.0f), 448.0f);
  const int packed = __builtin_amdgcn_cvt_pk_fp8_f32(ya, yb, 0, false);
  ((uint16_t*)out)[g * 64 + lane] = (uint16_t)(packed & 0xFFFF);
  if (lane == 0) scales[g] = s;
}

// 128 x 128 block quantiser for a [rows, K] weight matrix (rows and K multiples of 128): one workgroup per block,
// thread t owns 64 consecutive elements of block row t / 2. Same scale and clamp rule as the 1 x 128 quantiser.
template <bool BF16_IN>
__global__ __launch_bounds__(256) void fp8_block128_quant_kernel(const void* __restrict__ in, uint8_t* __restrict__ out,
                                                                float* __restrict__ scales, int K) {
  __shared__ float wave_max[4];
  const int kb = blockIdx.x, rb = blockIdx.y;
  const int t = threadIdx.x;
  const int64_t elem0 = ((int64_t)rb * 128 + (t >> 1)) * K + (int64_t)kb * 128 + (t & 1) * 64;
  float v[64];
  if (BF16_IN) {
    const u32x4_t* src = (const u32x4_t*)((const uint16_t*)in + elem0);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const u32x4_t q = src[i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[i * 8 + 2 * j] = __builtin_bit_cast(float, q[j] << 16);
        v[i * 8 + 2 * j + 1] = __builtin_bit_cast(float, q[j] & 0xFFFF0000u);
      }
    }
  } else {
    const f32x4_t* src = (const f32x4_t*)((const float*)in + elem0);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const f32x4_t q = src[i];
#pragma unroll
      for (int j = 0; j < 4; ++j) v[i * 4 + j] = q[j];
    }
  }
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < 64; ++i) amax = fmaxf(amax, fabsf(v[i]));
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) amax = fmaxf(amax, __shfl_xor(amax, d, 64));
  if ((t & 63) == 0) wave_max[t >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
  const float s = fmaxf(amax, 1e-12f) / 448.0f;
  u32x4_t* dst = (u32x4_t*)(out + elem0);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    u32x4_t o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float* e = v + i * 16 + j * 4;
      int w = __builtin_amdgcn_cvt_pk_fp8_f32(fminf(fmaxf(e[0] / s, -448.0f), 448.0f),
                                              fminf(fmaxf(e[1] / s, -448.0f), 448.0f), 0, false);
      w = __builtin_amdgcn_cvt_pk_fp8_f32(fminf(fmaxf(e[2] / s, -448.0f), 448.0f),
                                          fminf(fmaxf(e[3] / s, -448.0f), 448.0f), w, true);
      o[j] = (uint32_t)w;
    }
    dst[i] = o;
  }
  if (t == 0) scales[(int64_t)rb * gridDim.x + kb] = s;
}

}  // namespace

hipError_t fp8_block128_quant_launch(const void* in, bool bf16_in, void* out, float* scales, int64_t rows, int K,
                                     hipStream_t stream) {
  if (rows == 0 || K == 0) return hipSuccess;
  const dim3 grid((unsigned)(K / 128), (unsigned)(rows / 128));
  if (bf16_in) hipLaunchKernelGGL(fp8_block128_quant_kernel<true>, grid, dim3(256), 0, stream, in, (uint8_t*)out, scales, K);
  else hipLaunchKernelGGL(fp8_block128_quant_kernel<false>, grid, dim3(256), 0, stream, in, (uint8_t*)out, scales, K);
  return hipGetLastError();
}

hipError_t fp8_groupwise_quant_launch(const void* in, bool bf16_in, void* out, float* scales, int64_t groups,
                                      hipStream_t stream) {
  if (groups == 0) return hipSuccess;
  const unsigned grid = (unsigned)((groups + 3) / 4);
  if (bf16_in) hipLaunchKernelGGL(fp8_groupwise_quant_kernel<true>, dim3(grid), dim3(256), 0, stream, in, (uint8_t*)out, scales, groups);
  else hipLaunchKernelGGL(fp8_groupwise_quant_kernel<false>, dim3(grid), dim3(256), 0, stream, in, (uint8_t*)out, scales, groups);
  return hipGetLastError();
}
