// Small-expert fp8 (OCP e4m3) grouped GEMM for gfx950: weights streamed once, split-K inside the workgroup.
//
// Same contract as the tiled kernel of gg_fp8.hip (row-wise scales: dev/triton_groupGEMM/groupgemm.py:269-404;
// block scales: 1 x 128 activation scales of kernels/triton/inference/fp8/float8_groupwise_quant.py:53-91 and
// 128 x 128 weight scales), for experts with at most 16 * MF rows. With a few rows per expert the time is the
// time to stream the expert's weights from HBM once, and a tiled kernel that walks K in 128-byte columns
// of a few LDS stages cannot keep enough bytes in flight; here nothing is staged:
//
// Grid (N / (16 * NF), G). A workgroup owns 16 * NF weight rows of one expert and all of the expert's rows;
// its four waves split K four ways. A wave loads weight and activation fragments straight from global
// memory into the operand layout of v_mfma_f32_16x16x128_f8f6f4 with DEPTH K steps of loads in flight.
// Inside a 128-byte K step lane l takes bytes 16 q .. 16 q + 15 and 64 + 16 q .. 64 + 16 q + 15 of row l % 16
// (q = l / 16) for both operands, so every load instruction reads whole 64-byte half lines. In block mode
// the step's result is scaled by x_scale[m, kb] * w_scale[n / 128, kb] and added to the accumulator; in
// row-wise mode the scales are applied once at the end. The four partial sums are added through LDS in a
// fixed order (deterministic). Experts with no rows or with more than max_rows rows exit at once; the tiled
// kernel, launched beside this one, skips exactly the experts handled here.
#include "common.h"
#include "kernels.h"
#include "gg_tables.h"

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(int)))) int i32x8_t;

template <int MODE, int NF, int MF, int DEPTH>
__global__ __launch_bounds__(256) void gg_fp8_stream(GgParams p, int max_rows) {
  constexpr int WAVES = 4;
  constexpr int RP = MF >= 2 ? 2 : 1;          // the reduction runs in RP passes over MF / RP activation fragments,
  constexpr int MFP = MF / RP;                 // which keeps the LDS footprint at 32 KB and three workgroups per CU
  __shared__ __attribute__((aligned(16))) float red[WAVES][NF * MFP][256];
  __shared__ int s_g, s_row0, s_rows;
  __shared__ int32_t row_off[MOE_GG_MAX_GROUPS + 1];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int K = p.K, N = p.N;
  const int KB = K / 128;

  // Grid row blockIdx.y takes the blockIdx.y-th expert with 1 .. max_rows rows: the workgroups without work are
  // then the last ones of the launch (scattered among the others they make the dispatcher fill the CUs unevenly).
  build_row_offsets(p.m_sizes, p.G, p.M, row_off);
  if (wave == 0) {
    const int gi = nth_group(p.G, blockIdx.y, [&](int i) {
      const int r = row_off[i + 1] - row_off[i];
      return r > 0 && r <= max_rows;
    });
    if (lane == 0) {
      s_g = gi;
      s_row0 = gi < 0 ? 0 : row_off[gi];
      s_rows = gi < 0 ? 0 : row_off[gi + 1] - row_off[gi];
    }
  }
  __syncthreads();
  const int g = __builtin_amdgcn_readfirstlane(s_g);
  const int row0 = __builtin_amdgcn_readfirstlane(s_row0);
  const int rows = __builtin_amdgcn_readfirstlane(s_rows);
  if (g < 0 || rows == 0) return;
  const int nmf = (rows + 15) >> 4;  // activation fragments in use (<= MF)

  const int n0 = blockIdx.x * (16 * NF);
  const int fr = lane & 15, fq = lane >> 4;
  const int ks = wave * KB / WAVES, ke = (wave + 1) * KB / WAVES;  // K steps of this wave
  const int steps = ke - ks;

  const char* wbase = (const char*)p.w + ((int64_t)g * N + n0) * K + (int64_t)ks * 128 + fq * 16;
  const char* xbase = (const char*)p.x + (int64_t)row0 * K + (int64_t)ks * 128 + fq * 16;
  int64_t woff[NF], xoff[MF];
#pragma unroll
  for (int j = 0; j < NF; ++j) woff[j] = (int64_t)min(j * 16 + fr, N - n0 - 1) * K;
#pragma unroll
  for (int i = 0; i < MF; ++i) xoff[i] = (int64_t)min(i * 16 + fr, rows - 1) * K;
  // Block mode: lane's activation scale row per fragment; the weight scale is uniform over the workgroup
  // (16 * NF divides 128, so the workgroup's columns lie in one 128-row scale block).
  const float* xsc[MF];
  const float* wsc = nullptr;
  if (MODE == 1) {
#pragma unroll
    for (int i = 0; i < MF; ++i) xsc[i] = p.x_scale + (int64_t)(row0 + min(i * 16 + fr, rows - 1)) * KB + ks;
    wsc = p.w_scale + (((int64_t)g * N + n0) / 128) * KB + ks;
  }

  f32x4_t acc[NF][MF];
#pragma unroll
  for (int j = 0; j < NF; ++j)
#pragma unroll
    for (int i = 0; i < MF; ++i) acc[j][i] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  u32x4_t wlo[DEPTH][NF], whi[DEPTH][NF], xlo[DEPTH][MF], xhi[DEPTH][MF];
  float sc[DEPTH][MF];
  auto load = [&](int d, int t) {
#pragma unroll
    for (int j = 0; j < NF; ++j) {
      wlo[d][j] = *(const u32x4_t*)(wbase + woff[j] + t * 128);
      whi[d][j] = *(const u32x4_t*)(wbase + woff[j] + t * 128 + 64);
    }
#pragma unroll
    for (int i = 0; i < MF; ++i) {
      if (i < nmf) {
        xlo[d][i] = *(const u32x4_t*)(xbase + xoff[i] + t * 128);
        xhi[d][i] = *(const u32x4_t*)(xbase + xoff[i] + t * 128 + 64);
        if (MODE == 1) sc[d][i] = xsc[i][t] * wsc[t];
      }
    }
  };
  auto cat = [](const u32x4_t& lo, const u32x4_t& hi) {
    return i32x8_t{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
  };
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (d < steps) load(d, d);
  for (int t0 = 0; t0 < steps; t0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (t0 + d < steps) {
#pragma unroll
        for (int i = 0; i < MF; ++i) {
          if (i < nmf) {
            const i32x8_t xf = cat(xlo[d][i], xhi[d][i]);
#pragma unroll
            for (int j = 0; j < NF; ++j) {
              const i32x8_t wf = cat(wlo[d][j], whi[d][j]);
              if (MODE == 1) {
                const f32x4_t z = {0.f, 0.f, 0.f, 0.f};
                const f32x4_t r = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf, z, 0, 0, 0, 0, 0, 0);
                acc[j][i] += r * sc[d][i];
              } else {
                acc[j][i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf, acc[j][i], 0, 0, 0, 0, 0, 0);
              }
            }
          }
        }
        if (t0 + d + DEPTH < steps) load(d, t0 + d + DEPTH);
      }
    }
  }

  // Split-K reduction through LDS, then scales (row-wise mode) and the store: lane holds y[m][n .. n+3],
  // m = i * 16 + lane % 16, n = n0 + j * 16 + 4 * (lane / 16).
#pragma unroll
  for (int rp = 0; rp < RP; ++rp) {
    if (rp * MFP >= nmf) break;
    if (rp) __syncthreads();
#pragma unroll
    for (int j = 0; j < NF; ++j)
#pragma unroll
      for (int i = 0; i < MFP; ++i) *(f32x4_t*)&red[wave][j * MFP + i][lane * 4] = acc[j][rp * MFP + i];
    __syncthreads();
    for (int f = wave; f < NF * MFP; f += WAVES) {
      const int j = f / MFP, i = rp * MFP + f % MFP;
      const int m = i * 16 + fr;
      if (m >= rows) continue;
      f32x4_t v = *(const f32x4_t*)&red[0][f][lane * 4];
#pragma unroll
      for (int w2 = 1; w2 < WAVES; ++w2) v += *(const f32x4_t*)&red[w2][f][lane * 4];
      const int n = n0 + j * 16 + fq * 4;
      if (MODE == 0) {
        const float am = p.x_scale[row0 + m];
        const float* bs = p.w_scale + (int64_t)g * N;
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = v[r] * am * bs[min(n + r, N - 1)];
      }
      bf16_t* yrow = (bf16_t*)p.y + (int64_t)(row0 + m) * p.ldy + (int64_t)g * p.col_block;
      if (p.vec_store && n + 3 < N) {
        u32x2_t o;
        o[0] = pack_bf16x2(v[0], v[1]);
        o[1] = pack_bf16x2(v[2], v[3]);
        *(u32x2_t*)(yrow + n) = o;
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r < N) yrow[n + r] = (bf16_t)v[r];
      }
    }
  }
}

template <int MODE, int NF, int MF, int DEPTH>
hipError_t launch(const GgParams& p, hipStream_t stream) {
  dim3 grid((p.N + 16 * NF - 1) / (16 * NF), p.G);
  hipLaunchKernelGGL((gg_fp8_stream<MODE, NF, MF, DEPTH>), grid, dim3(256), 0, stream, p, 16 * MF);
  return hipGetLastError();
}

}  // namespace

int gg_fp8_stream_max_rows() { return 64; }

// One K step of loads in flight per wave and three workgroups per CU measured best (more steps in flight
// cost registers, hence resident waves, and were slower).
hipError_t gg_fp8_stream_launch(const GgParams& p, int scale_mode, hipStream_t stream) {
  if (scale_mode == 0) return launch<0, 4, 4, 1>(p, stream);
  return launch<1, 4, 4, 1>(p, stream);
}
