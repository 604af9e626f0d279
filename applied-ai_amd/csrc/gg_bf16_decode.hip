// Small-M ("decode") bf16 grouped GEMM for gfx950: split-K inside the workgroup, weights streamed once.
//
// Same contract as the reference's _kernel_grouped_gemm (dev/triton_groupGEMM/groupgemm.py:130-254):
// y[off_g : off_g + m_g, :] = x[off_g : ...] @ w[g]^T, but built for m_g of a few rows per expert,
// where the time is the time to stream the active experts' weights from HBM once. The split-K
// decode configurations of the reference's fused-MoE kernels are the model
// (kernels/triton/inference/col_major_moe_gemm/v1_moe_fused.py:297-312).
//
// Grid: (N / (16 * NF), G). A workgroup owns 16 * NF weight rows of one expert and all of the
// expert's (<= 16 * MF per pass) activation rows; its four waves split K four ways. Each wave loads
// its weight fragments straight from global memory into the MFMA "A" operand layout (lane l holds
// row l % 16, 16 bytes of K chunk l / 16 -> two consecutive K steps consume one 128-byte line per
// row) with DEPTH K steps of loads in flight. The loads of the two K steps that share a line are issued
// back to back (PAIR): issued a step apart, the second one mostly finds the line already evicted from the
// 32 KB vector L1 (the waves of a CU keep far more lines in flight than that) and fetches it again, which
// costs 15-20 % of the streaming rate. The fragments are multiplied with the activation fragments
// ("B" operand, L2-resident) by v_mfma_f32_16x16x32_bf16, and the four partial accumulators are
// summed through LDS (fixed order: deterministic) before the bf16 store. Grid row y works on the y-th
// expert with m_g > 0; the rows of the grid beyond the number of such experts exit at once, so the
// weights of an expert without rows are never touched.
#include "common.h"
#include "kernels.h"
#include "tile_sched.h"
#include "gg_tables.h"

namespace {

// TAIL: the kernel computes the low tiles that the 256 x 256 ping-pong kernel of the same call leaves out
// (p.tails_apart, moe_gg_tails_apart): of every expert the rows beyond its last full 256-row tile.
template <int NF, int MF, int WAVES, int DEPTH, bool PAIR, bool TAIL = false, bool F16 = false>
__global__ __launch_bounds__(64 * WAVES) void gg_bf16_decode(GgParams p) {
  __shared__ __attribute__((aligned(16))) float red[WAVES][NF * MF][256];
  __shared__ int s_g, s_row0, s_rows;
  __shared__ int32_t row_off[MOE_GG_MAX_GROUPS + 1];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int K = p.K, N = p.N;

  // Grid row blockIdx.y takes the blockIdx.y-th expert that has rows to compute, not expert blockIdx.y: the
  // workgroups without work are then the last ones of the launch. Scattered among the others they leave at once
  // and the dispatcher fills their places unevenly: with every second expert empty the working workgroups ended
  // up on part of the CUs only (123 us against 88 us for the same four experts next to each other).
  build_row_offsets(p.m_sizes, p.G, p.M, row_off);
  if (wave == 0) {
    bool apart = false;
    if (TAIL) {
      // The ping-pong kernel's own tables and counts, so that both take the same decision.
      long long n_long = 0, n_low = 0, passes = 0;
      for (int i = lane; i < p.G; i += 64) {
        const int r = row_off[i + 1] - row_off[i];
        n_long += moe_gg_long_row_tiles(r, 256);
        n_low += moe_gg_low_row_tiles(r, 256);
        passes += moe_gg_low_passes(r, 256);
      }
#pragma unroll
      for (int d = 32; d >= 1; d >>= 1) {
        n_long += __shfl_xor(n_long, d, 64);
        n_low += __shfl_xor(n_low, d, 64);
        passes += __shfl_xor(passes, d, 64);
      }
      const int ntn = moe_gg_cdiv(N, 256);
      apart = moe_gg_tails_apart((int)(n_long * ntn), (int)(n_low * ntn), passes * ntn, p.tails_apart);
    }
    const int g = nth_group(p.G, blockIdx.y, [&](int i) {
      const int r = row_off[i + 1] - row_off[i];
      return TAIL ? apart && moe_gg_low_row_tiles(r, 256) > 0 : r > 0;
    });
    if (lane == 0) {
      const int r = g < 0 ? 0 : row_off[g + 1] - row_off[g];
      s_g = g;
      s_row0 = g < 0 ? 0 : row_off[g] + (TAIL ? r / 256 * 256 : 0);
      s_rows = TAIL ? r % 256 : r;
    }
  }
  __syncthreads();
  const int g = s_g, row0 = s_row0, rows = s_rows;
  if (g < 0 || rows == 0) return;

  const int n0 = blockIdx.x * (16 * NF);
  const int fr = lane & 15, fq = lane >> 4;
  constexpr int H = PAIR ? 2 : 1;      // K steps (of 32) per load group
  constexpr int DP = DEPTH / H;        // load groups in flight
  const int kw = K / WAVES;            // K range of this wave
  const int steps = kw / (32 * H);     // load groups of this wave
  const bf16_t* wbase = (const bf16_t*)p.w + ((int64_t)g * N + n0) * K + wave * kw + fq * 8;
  const bf16_t* xbase = (const bf16_t*)p.x + (int64_t)row0 * K + wave * kw + fq * 8;
  int64_t woff[NF];
#pragma unroll
  for (int j = 0; j < NF; ++j) woff[j] = (int64_t)min(j * 16 + fr, N - n0 - 1) * K;

  for (int mb = 0; mb < rows; mb += 16 * MF) {  // one pass unless the expert has more than 16 * MF rows
    int64_t xoff[MF];
#pragma unroll
    for (int i = 0; i < MF; ++i) xoff[i] = (int64_t)min(mb + i * 16 + fr, rows - 1) * K;

    f32x4_t acc[NF][MF];
#pragma unroll
    for (int j = 0; j < NF; ++j)
#pragma unroll
      for (int i = 0; i < MF; ++i) acc[j][i] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    bf16x8_t wb[DP][H][NF], xb[DP][H][MF];
    auto load = [&](int d, int t) {
#pragma unroll
      for (int j = 0; j < NF; ++j)
#pragma unroll
        for (int h = 0; h < H; ++h) wb[d][h][j] = *(const bf16x8_t*)(wbase + woff[j] + (H * t + h) * 32);
#pragma unroll
      for (int i = 0; i < MF; ++i)
#pragma unroll
        for (int h = 0; h < H; ++h) xb[d][h][i] = *(const bf16x8_t*)(xbase + xoff[i] + (H * t + h) * 32);
    };
#pragma unroll
    for (int d = 0; d < DP; ++d)
      if (d < steps) load(d, d);
    for (int t0 = 0; t0 < steps; t0 += DP) {
#pragma unroll
      for (int d = 0; d < DP; ++d) {
        if (t0 + d < steps) {
#pragma unroll
          for (int h = 0; h < H; ++h)
#pragma unroll
            for (int j = 0; j < NF; ++j)
#pragma unroll
              for (int i = 0; i < MF; ++i)
                acc[j][i] = mfma_16x16x32<F16>(__builtin_bit_cast(u32x4_t, wb[d][h][j]), __builtin_bit_cast(u32x4_t, xb[d][h][i]), acc[j][i]);
          if (t0 + d + DP < steps) load(d, t0 + d + DP);
        }
      }
    }

    // Split-K reduction through LDS, then the store: lane holds y[m][n .. n+3] for
    // m = mb + i * 16 + lane % 16, n = n0 + j * 16 + 4 * (lane / 16).
#pragma unroll
    for (int j = 0; j < NF; ++j)
#pragma unroll
      for (int i = 0; i < MF; ++i) *(f32x4_t*)&red[wave][j * MF + i][lane * 4] = acc[j][i];
    __syncthreads();
    for (int f = wave; f < NF * MF; f += WAVES) {
      f32x4_t v = *(const f32x4_t*)&red[0][f][lane * 4];
#pragma unroll
      for (int w2 = 1; w2 < WAVES; ++w2) v += *(const f32x4_t*)&red[w2][f][lane * 4];
      const int j = f / MF, i = f % MF;
      const int m = mb + i * 16 + fr;
      const int n = n0 + j * 16 + fq * 4;
      if (m < rows) {
        bf16_t* yrow = (bf16_t*)p.y + (int64_t)(row0 + m) * p.ldy + (int64_t)g * p.col_block;
        if (p.vec_store && n + 3 < N) {
          u32x2_t o;
          o[0] = pack_16x2<F16>(v[0], v[1]);
          o[1] = pack_16x2<F16>(v[2], v[3]);
          *(u32x2_t*)(yrow + n) = o;
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (n + r < N) ((uint16_t*)yrow)[n + r] = cvt_16<F16>(v[r]);
        }
      }
    }
    __syncthreads();
  }
}

template <int NF, int MF, int DEPTH>
hipError_t launch(const GgParams& p, hipStream_t stream) {
  dim3 grid((p.N + 16 * NF - 1) / (16 * NF), p.G);
  if (p.fp16) {
    if (p.K % 256 == 0) hipLaunchKernelGGL((gg_bf16_decode<NF, MF, 4, DEPTH, true, false, true>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((gg_bf16_decode<NF, MF, 4, DEPTH, false, false, true>), grid, dim3(256), 0, stream, p);
  } else if (p.K % 256 == 0) hipLaunchKernelGGL((gg_bf16_decode<NF, MF, 4, DEPTH, true>), grid, dim3(256), 0, stream, p);
  else hipLaunchKernelGGL((gg_bf16_decode<NF, MF, 4, DEPTH, false>), grid, dim3(256), 0, stream, p);
  return hipGetLastError();
}

}  // namespace

// nf: 16-row weight fragments per wave (2 or 4); mf: 16-row activation fragments per pass (1, 2, 4).
hipError_t gg_bf16_decode_tails_launch(const GgParams& p, hipStream_t stream) {
  static_assert(MOE_GG_TAIL_PASS_ROWS == 32, "two activation fragments per pass");
  dim3 grid((p.N + 31) / 32, p.G);
  if (p.fp16) {
    if (p.K % 256 == 0) hipLaunchKernelGGL((gg_bf16_decode<2, 2, 4, 8, true, true, true>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((gg_bf16_decode<2, 2, 4, 8, false, true, true>), grid, dim3(256), 0, stream, p);
  } else if (p.K % 256 == 0) hipLaunchKernelGGL((gg_bf16_decode<2, 2, 4, 8, true, true>), grid, dim3(256), 0, stream, p);
  else hipLaunchKernelGGL((gg_bf16_decode<2, 2, 4, 8, false, true>), grid, dim3(256), 0, stream, p);
  return hipGetLastError();
}

hipError_t gg_bf16_decode_launch(const GgParams& p, int nf, int mf, hipStream_t stream) {
  if (nf == 2 && mf == 1) return launch<2, 1, 8>(p, stream);
  if (nf == 4 && mf == 1) return launch<4, 1, 4>(p, stream);
  if (nf == 2 && mf == 2) return launch<2, 2, 8>(p, stream);
  if (nf == 4 && mf == 2) return launch<4, 2, 4>(p, stream);
  if (nf == 2 && mf == 4) return launch<2, 4, 4>(p, stream);
  return hipErrorInvalidValue;
}
