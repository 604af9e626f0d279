// 1 x 128 group-wise fp8 (OCP e4m3fn) activation quantiser for gfx950.
//
// Replaces _float8_groupwise_quant_kernel / float8_groupwise_quantize
// (kernels/triton/inference/fp8/float8_groupwise_quant.py:20-50, 53-91): per group of 128 consecutive
// elements  s = max(amax|x|, 1e-12) / 448,  q = clamp(x / s, -448, 448) -> e4m3fn (round to nearest even);
// q and s are stored, s as fp32 [..., K/128]. One wave per group, two elements per lane; the fp32
// division is the correctly rounded one, so the result is bit-identical to the CPU oracle.
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

}  // namespace

hipError_t fp8_groupwise_quant_launch(const void* in, bool bf16_in, void* out, float* scales, int64_t groups,
                                      hipStream_t stream) {
  if (groups == 0) return hipSuccess;
  const unsigned grid = (unsigned)((groups + 3) / 4);
  if (bf16_in) hipLaunchKernelGGL(fp8_groupwise_quant_kernel<true>, dim3(grid), dim3(256), 0, stream, in, (uint8_t*)out, scales, groups);
  else hipLaunchKernelGGL(fp8_groupwise_quant_kernel<false>, dim3(grid), dim3(256), 0, stream, in, (uint8_t*)out, scales, groups);
  return hipGetLastError();
}
