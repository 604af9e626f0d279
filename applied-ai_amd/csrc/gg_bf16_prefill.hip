// Persistent bf16 grouped GEMM for gfx950: y[off_g : off_g + m_g, :] = x[off_g : ...] @ w[g]^T.
//
// Replaces the reference's _kernel_grouped_gemm (dev/triton_groupGEMM/groupgemm.py:130-254).
// One workgroup per CU walks the tile list of tile_sched.h. Per tile, BM x 64 (activations) and
// BN x 64 (weights) bf16 slabs are staged through double-buffered, XOR-swizzled LDS with 128-bit
// global loads, and consumed by v_mfma_f32_16x16x32_bf16. The weight fragment is the MFMA "A"
// operand and the activation fragment the "B" operand, so a lane ends up holding four consecutive
// output columns of one output row and the epilogue stores 8 bytes per lane.
#include "common.h"
#include "gg_tables.h"
#include "kernels.h"

namespace {

template <int BM_, int BN_, int WM_, int WN_>
struct Cfg {
  static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_;
  static constexpr int NT = 64 * WM * WN;       // threads per workgroup
  static constexpr int FM = BM / 16 / WM;       // activation fragments per wave
  static constexpr int FN = BN / 16 / WN;       // weight fragments per wave
  static constexpr int XL = BM * 8 / NT;        // 16-byte chunks of the x slab per thread
  static constexpr int WL = BN * 8 / NT;        // 16-byte chunks of the w slab per thread
  static constexpr int X_BYTES = BM * 128;
  static constexpr int W_BYTES = BN * 128;
  static constexpr int STAGE = X_BYTES + W_BYTES;
  static_assert((NT / 8) % 16 == 0, "row step of the loader must keep the swizzle phase");
  static_assert(BM % (16 * WM) == 0 && BN % (16 * WN) == 0, "tile must split evenly over waves");
};

template <class C>
__global__ __launch_bounds__(C::NT) void gg_bf16_persistent(GgParams p) {
  __shared__ __attribute__((aligned(16))) char lds[2 * C::STAGE];
  __shared__ int32_t row_off[MOE_GG_MAX_GROUPS + 1];
  __shared__ int32_t tile_off[MOE_GG_MAX_GROUPS + 1];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave % C::WM;
  const int wn = wave / C::WM;
  const int K = p.K, N = p.N;
  const int n_tiles_n = moe_gg_cdiv(N, C::BN);

  build_group_tables(p.m_sizes, p.G, p.M, C::BM, n_tiles_n, row_off, tile_off);
  const int total = tile_off[p.G];
  const int KT = K / 64;

  // Loader geometry: chunk id = i * NT + tid -> (row, 16-byte chunk of the 128-byte row).
  const int ld_row = tid >> 3, ld_c = tid & 7;
  const int ld_lds = lds_swizzle_off(ld_row, ld_c);
  // Fragment reads: row = frag * 16 + lane % 16, chunk = kk * 4 + lane / 16.
  const int fr = lane & 15, fq = lane >> 4;
  const int rd0 = fr * 128 + ((fq ^ (fr >> 1)) << 4);  // kk = 0; kk = 1 is rd0 ^ 64

  const bf16_t* __restrict__ xp = (const bf16_t*)p.x;
  const bf16_t* __restrict__ wp = (const bf16_t*)p.w;
  bf16_t* __restrict__ yp = (bf16_t*)p.y;

  for (int round = 0; round * (int)gridDim.x < total; ++round) {
    const int L = moe_gg_tile_of(blockIdx.x, gridDim.x, p.xcds, round);
    if (L >= total) continue;
    const MoeGgTile t = moe_gg_decode_tile(row_off, tile_off, p.G, L, C::BM);
    const int m0 = t.tm * C::BM;
    const int rows_valid = min(t.rows - m0, C::BM);
    const int n0 = t.tn * C::BN;
    const int cols_valid = min(N - n0, C::BN);

    const bf16_t* xg = xp + (int64_t)(t.row0 + m0) * K + ld_c * 8;
    const bf16_t* wg = wp + ((int64_t)t.g * N + n0) * K + ld_c * 8;
    int xoff[C::XL], woff[C::WL];
#pragma unroll
    for (int i = 0; i < C::XL; ++i) xoff[i] = min(ld_row + i * (C::NT / 8), rows_valid - 1) * K;
#pragma unroll
    for (int i = 0; i < C::WL; ++i) woff[i] = min(ld_row + i * (C::NT / 8), cols_valid - 1) * K;

    u32x4_t xr[C::XL], wr[C::WL];
    auto gload = [&](int kt) {
#pragma unroll
      for (int i = 0; i < C::XL; ++i) xr[i] = *(const u32x4_t*)(xg + xoff[i] + kt * 64);
#pragma unroll
      for (int i = 0; i < C::WL; ++i) wr[i] = *(const u32x4_t*)(wg + woff[i] + kt * 64);
    };
    auto lstore = [&](int buf) {
      char* xs = lds + buf * C::STAGE + ld_lds;
      char* ws = xs + C::X_BYTES;
#pragma unroll
      for (int i = 0; i < C::XL; ++i) *(u32x4_t*)(xs + i * (C::NT / 8) * 128) = xr[i];
#pragma unroll
      for (int i = 0; i < C::WL; ++i) *(u32x4_t*)(ws + i * (C::NT / 8) * 128) = wr[i];
    };

    f32x4_t acc[C::FN][C::FM];
#pragma unroll
    for (int j = 0; j < C::FN; ++j)
#pragma unroll
      for (int i = 0; i < C::FM; ++i) acc[j][i] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    gload(0);
    lstore(0);
    __syncthreads();

    for (int kt = 0; kt < KT; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < KT) gload(kt + 1);
      const char* xs = lds + cur * C::STAGE + wm * (C::FM * 16 * 128);
      const char* ws = lds + cur * C::STAGE + C::X_BYTES + wn * (C::FN * 16 * 128);
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const int ro = kk ? (rd0 ^ 64) : rd0;
        bf16x8_t wf[C::FN], xf[C::FM];
#pragma unroll
        for (int j = 0; j < C::FN; ++j) wf[j] = *(const bf16x8_t*)(ws + j * 2048 + ro);
#pragma unroll
        for (int i = 0; i < C::FM; ++i) xf[i] = *(const bf16x8_t*)(xs + i * 2048 + ro);
#pragma unroll
        for (int j = 0; j < C::FN; ++j)
#pragma unroll
          for (int i = 0; i < C::FM; ++i)
            acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j], xf[i], acc[j][i], 0, 0, 0);
      }
      if (kt + 1 < KT) lstore(cur ^ 1);
      __syncthreads();
    }

    // Epilogue: lane holds y[m][n .. n+3] for m = frag_m * 16 + lane % 16, n = frag_n * 16 + 4 * (lane / 16).
    bf16_t* yg = yp + (int64_t)(t.row0 + m0) * p.ldy + (int64_t)t.g * p.col_block + n0;
    const bool vec_ok = p.vec_store;
#pragma unroll
    for (int i = 0; i < C::FM; ++i) {
      const int m = (wm * C::FM + i) * 16 + fr;
      if (m < rows_valid) {
        bf16_t* yrow = yg + (int64_t)m * p.ldy;
#pragma unroll
        for (int j = 0; j < C::FN; ++j) {
          const int n = (wn * C::FN + j) * 16 + fq * 4;
          const f32x4_t v = acc[j][i];
          if (vec_ok && n + 3 < cols_valid) {
            u32x2_t o;
            o[0] = pack_bf16x2(v[0], v[1]);
            o[1] = pack_bf16x2(v[2], v[3]);
            *(u32x2_t*)(yrow + n) = o;
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (n + r < cols_valid) yrow[n + r] = (bf16_t)v[r];
          }
        }
      }
    }
  }
}

template <class C>
hipError_t launch(const GgParams& p, int num_wg, hipStream_t stream) {
  hipLaunchKernelGGL(gg_bf16_persistent<C>, dim3(num_wg), dim3(C::NT), 0, stream, p);
  return hipGetLastError();
}

}  // namespace

hipError_t gg_bf16_prefill_launch(const GgParams& p, int variant, int num_wg, hipStream_t stream) {
  switch (variant) {
    case 0: return launch<Cfg<256, 256, 2, 2>>(p, num_wg, stream);
    case 1: return launch<Cfg<256, 256, 2, 4>>(p, num_wg, stream);
    case 2: return launch<Cfg<128, 256, 2, 2>>(p, num_wg, stream);
    case 3: return launch<Cfg<128, 128, 2, 2>>(p, num_wg, stream);
    case 4: return launch<Cfg<256, 128, 2, 2>>(p, num_wg, stream);
    default: return hipErrorInvalidValue;
  }
}

int gg_bf16_prefill_block_m(int variant) {
  switch (variant) {
    case 0: case 1: case 4: return 256;
    case 2: case 3: return 128;
    default: return 0;
  }
}
