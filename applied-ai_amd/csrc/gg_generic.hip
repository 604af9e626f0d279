// Shape-agnostic grouped GEMM for inputs the tiled kernels do not take (K not a multiple of 64,
// unaligned pointers or leading dimensions). One workgroup computes 256 columns of one output row
// with plain fp32 FMAs; meant for small edge-case shapes, not for throughput.
#include "common.h"
#include "kernels.h"

namespace {

__global__ __launch_bounds__(256) void gg_bf16_generic(GgParams p) {
  __shared__ int s_g, s_row0, s_rows;
  const int m = blockIdx.x;
  if (threadIdx.x == 0) {
    // Serial walk of the offset table (dev/triton_groupGEMM/groupgemm.py:159-165).
    int64_t r = 0;
    int g_found = -1, row0 = 0, rows = 0;
    for (int g = 0; g < p.G; ++g) {
      int mg = p.m_sizes[g];
      if (mg < 0) mg = 0;
      if ((int64_t)mg > (int64_t)p.M - r) mg = (int)((int64_t)p.M - r);
      if (m >= r && m < r + mg) { g_found = g; row0 = (int)r; rows = mg; break; }
      r += mg;
    }
    s_g = g_found; s_row0 = row0; s_rows = rows;
  }
  __syncthreads();
  const int g = s_g;
  if (g < 0) return;  // row beyond sum(m_sizes): left untouched
  const int n = blockIdx.y * 256 + threadIdx.x;
  if (n >= p.N) return;
  const uint16_t* xr = (const uint16_t*)p.x + (int64_t)m * p.K;
  const uint16_t* wr = (const uint16_t*)p.w + ((int64_t)g * p.N + n) * p.K;
  uint16_t* yo = (uint16_t*)p.y + (int64_t)m * p.ldy + (int64_t)g * p.col_block + n;
  float acc = 0.f;
  if (p.fp16) {
    for (int k = 0; k < p.K; ++k) acc = __builtin_fmaf(f32_of_16<true>(xr[k]), f32_of_16<true>(wr[k]), acc);
    *yo = cvt_16<true>(acc);
  } else {
    for (int k = 0; k < p.K; ++k) acc = __builtin_fmaf(f32_of_16<false>(xr[k]), f32_of_16<false>(wr[k]), acc);
    *yo = cvt_16<false>(acc);
  }
}

}  // namespace

hipError_t gg_bf16_generic_launch(const GgParams& p, hipStream_t stream) {
  if (p.M == 0 || p.N == 0) return hipSuccess;
  dim3 grid(p.M, (p.N + 255) / 256);
  hipLaunchKernelGGL(gg_bf16_generic, grid, dim3(256), 0, stream, p);
  return hipGetLastError();
}
