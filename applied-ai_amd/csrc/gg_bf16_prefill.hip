// Persistent bf16 grouped GEMM for gfx950: y[off_g : off_g + m_g, :] = x[off_g : ...] @ w[g]^T.
//
// Replaces the reference's _kernel_grouped_gemm (dev/triton_groupGEMM/groupgemm.py:130-254).
// One workgroup per CU walks the tile list of tile_sched.h. Per tile, BM x 64 (activations) and
// BN x 64 (weights) bf16 slabs are brought into double-buffered, XOR-swizzled LDS by
// global_load_lds_dwordx4 (no VGPR staging) and consumed by v_mfma_f32_16x16x32_bf16.
// The weight fragment is the MFMA "A" operand and the activation fragment the "B" operand, so a
// lane ends up holding four consecutive output columns of one output row and the epilogue stores
// 8 bytes per lane.
//
// K loop (one barrier per 64-wide K step): the fragments of the two 32-wide halves of a K step live
// in two register sets F0/F1. While the MFMAs of one half run, the ds_reads of the next half are in
// flight; the barrier in the middle of the step both publishes slab kt+1 and frees slab kt's buffer,
// into which the loads of slab kt+2 are issued at once.
//
// This is the general tiled kernel (tile shapes 256x256, 128x128 and 64x128); the 256x256 ping-pong
// kernel in gg_bf16_pp.hip is preferred when a launch has enough 256x256 tiles to fill the chip.
#include "common.h"
#include "gg_tables.h"
#include "kernels.h"

namespace {

template <int BM_, int BN_, int WM_, int WN_>
struct Cfg {
  static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_;
  static constexpr int NT = 64 * WM * WN;  // threads per workgroup
  static constexpr int NW = NT / 64;
  static constexpr int FM = BM / 16 / WM;  // activation fragments per wave
  static constexpr int FN = BN / 16 / WN;  // weight fragments per wave
  static constexpr int XI = BM / 8 / NW;   // slab-load instructions per wave (8 rows each), x
  static constexpr int WI = BN / 8 / NW;   // same, w
  static constexpr int X_BYTES = BM * 128;
  static constexpr int W_BYTES = BN * 128;
  static constexpr int STAGE = X_BYTES + W_BYTES;
  static constexpr int NLOAD = XI + WI;
  static_assert(NW % 2 == 0, "swizzle phase of a wave's rows relies on an even wave count");
  static_assert(BM % (16 * WM) == 0 && BN % (16 * WN) == 0, "tile must split evenly over waves");
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "slab rows must split evenly over waves");
};

// 64 lanes x 16 B from global memory straight into LDS: lane l's 16 bytes land at lds_addr + 16 l.
// Issued from inline assembly so that the compiler does not serialise the in-flight slab against
// the LDS reads of the slab being consumed; completion is tracked by hand with vmcnt.
DEVINL void dma16(const void* sbase, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n"
               :
               : "s"(lds_addr), "v"(voff), "s"(sbase)
               : "memory");
}
template <int N>
DEVINL void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// WGRAD = false: the forward product above. WGRAD = true: the weight gradient of the same layer,
//   dW[g][n][k] = sum over the rows m of expert g of dY[m][n] * X[m][k]
// (kernels/MoE/group_GEMM/triton/tgroup_gemm_backwards.py:202-375; eager form testing/pytorch_reference_backwards.py:165-197),
// as the same tiled product on transposed operands: p.x = dY^T [N, ldm] and p.w = X^T [K, ldm], both with the rows of
// expert g in columns pad_off[g] .. pad_off[g] + roundup(m_g, 64) - 1 (zero padded), so the reduction of expert g
// is a whole number of 64-wide steps. Every expert has the same ceil(N / BM) * ceil(K / BN) tiles; an expert
// without rows gets zeros. p.N = rows of dW per expert (N), p.K = columns (K), p.M = ldm, p.y = dW [G * N, K].
template <class C, bool WGRAD, bool F16 = false>
__global__ __launch_bounds__(C::NT) void gg_bf16_persistent(GgParams p) {
  __shared__ __attribute__((aligned(1024))) char lds[2 * C::STAGE];
  __shared__ int32_t row_off[MOE_GG_MAX_GROUPS + 1];
  __shared__ int32_t tile_off[MOE_GG_MAX_GROUPS + 1];
  constexpr int NW = C::NW;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % C::WM;
  const int wn = wave / C::WM;
  const int K = p.K, N = p.N;
  const int n_tiles_n = moe_gg_cdiv(WGRAD ? K : N, C::BN);
  const int tiles_per_group = moe_gg_cdiv(N, C::BM) * n_tiles_n;  // WGRAD only

  // WGRAD: tile_off counts 64-row blocks per expert, i.e. pad_off[g] = 64 * tile_off[g]; rows are bounded by
  // the number of gradient rows (p.skip_rows carries it, p.M is the padded leading dimension).
  if (WGRAD) build_group_tables(p.m_sizes, p.G, p.skip_rows, 64, 1, row_off, tile_off, 0, 1);
  else build_group_tables(p.m_sizes, p.G, p.M, C::BM, n_tiles_n, row_off, tile_off);
  const int total = WGRAD ? p.G * tiles_per_group : tile_off[p.G];
  const uint32_t pitch = WGRAD ? (uint32_t)p.M * 2u : (uint32_t)K * 2u;  // bytes between operand rows

  // Slab-load geometry: instruction i of wave w fills rows (i * NW + w) * 8 + lane / 8; the lane's
  // physical 16-byte slot is lane % 8 and must hold logical chunk slot ^ ((row >> 1) & 7).
  const int d_r = lane >> 3;
  const int d_c = (lane & 7) ^ (((wave & 1) << 2) | (lane >> 4));
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  const uint32_t lds_wave = lds_base + wave * 1024;

  // Fragment reads: row = frag * 16 + lane % 16, chunk = kk * 4 + lane / 16 (swizzled).
  const int fr = lane & 15, fq = lane >> 4;
  const int rd0 = fr * 128 + ((fq ^ (fr >> 1)) << 4);  // kk = 0; kk = 1 is rd0 ^ 64

  const char* xp = (const char*)p.x;
  const char* wp = (const char*)p.w;
  bf16_t* __restrict__ yp = (bf16_t*)p.y;

  for (int round = 0; round * (int)gridDim.x < total; ++round) {
    const int L = moe_gg_tile_of(blockIdx.x, gridDim.x, p.xcds, round);
    if (L >= total) continue;
    MoeGgTile t;
    int KT;
    const char *xg, *wg;
    if (WGRAD) {
      t.g = L / tiles_per_group;
      const int rem = L - t.g * tiles_per_group;
      t.tm = rem % moe_gg_cdiv(N, C::BM);   // tile along the rows of dW (n)
      t.tn = rem / moe_gg_cdiv(N, C::BM);   // tile along its columns (k)
      t.row0 = 0;
      t.rows = N;
      KT = tile_off[t.g + 1] - tile_off[t.g];
      const int64_t col0 = (int64_t)tile_off[t.g] * 128;  // byte offset of the expert's padded columns
      xg = xp + (int64_t)(t.tm * C::BM) * pitch + col0;
      wg = wp + (int64_t)(t.tn * C::BN) * pitch + col0;
    } else {
      t = moe_gg_decode_tile(row_off, tile_off, p.G, L, C::BM);
      KT = K / 64;
      xg = xp + (int64_t)(t.row0 + t.tm * C::BM) * pitch;
      wg = wp + ((int64_t)t.g * N + t.tn * C::BN) * pitch;
    }
    const int m0 = t.tm * C::BM;
    const int rows_valid = min(t.rows - m0, C::BM);
    const int n0 = t.tn * C::BN;
    const int cols_valid = min((WGRAD ? K : N) - n0, C::BN);

    uint32_t xoff[C::XI], woff[C::WI];
#pragma unroll
    for (int i = 0; i < C::XI; ++i)
      xoff[i] = (uint32_t)min((i * NW + wave) * 8 + d_r, rows_valid - 1) * pitch + d_c * 16;
#pragma unroll
    for (int i = 0; i < C::WI; ++i)
      woff[i] = (uint32_t)min((i * NW + wave) * 8 + d_r, cols_valid - 1) * pitch + d_c * 16;

    auto dma = [&](int kt, int buf) {
      const char* xs = xg + kt * 128;
      const char* ws = wg + kt * 128;
      const uint32_t lb = lds_wave + buf * C::STAGE;
#pragma unroll
      for (int i = 0; i < C::XI; ++i) dma16(xs, xoff[i], lb + i * NW * 1024);
#pragma unroll
      for (int i = 0; i < C::WI; ++i) dma16(ws, woff[i], lb + C::X_BYTES + i * NW * 1024);
    };
    f32x4_t acc[C::FN][C::FM];
#pragma unroll
    for (int j = 0; j < C::FN; ++j)
#pragma unroll
      for (int i = 0; i < C::FM; ++i) acc[j][i] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    bf16x8_t wf0[C::FN], xf0[C::FM], wf1[C::FN], xf1[C::FM];
    auto read_frags = [&](int buf, int kk, bf16x8_t (&wf)[C::FN], bf16x8_t (&xf)[C::FM]) {
      const char* xs = lds + buf * C::STAGE + wm * (C::FM * 16 * 128);
      const char* ws = lds + buf * C::STAGE + C::X_BYTES + wn * (C::FN * 16 * 128);
      const int ro = kk ? (rd0 ^ 64) : rd0;
#pragma unroll
      for (int j = 0; j < C::FN; ++j) wf[j] = *(const bf16x8_t*)(ws + j * 2048 + ro);
#pragma unroll
      for (int i = 0; i < C::FM; ++i) xf[i] = *(const bf16x8_t*)(xs + i * 2048 + ro);
    };
    auto mma = [&](bf16x8_t (&wf)[C::FN], bf16x8_t (&xf)[C::FM]) {
#pragma unroll
      for (int j = 0; j < C::FN; ++j)
#pragma unroll
        for (int i = 0; i < C::FM; ++i)
          acc[j][i] = mfma_16x16x32<F16>(__builtin_bit_cast(u32x4_t, wf[j]), __builtin_bit_cast(u32x4_t, xf[i]), acc[j][i]);
    };
    // Ask the scheduler to spread the fragment reads of the next half over the MFMAs of this one.
    auto interleave = [&]() {
      constexpr int NR = C::FN + C::FM, NM = C::FN * C::FM;
      constexpr int PER = NM / NR > 0 ? NM / NR : 1;
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, NM - PER * NR > 0 ? NM - PER * NR : 0, 0);
    };

    // Prologue: slabs 0 and 1 in flight, F0 <- (slab 0, half 0).
    dma(0, 0);
    if (KT > 1) dma(1, 1);
    if (KT > 1) wait_vmcnt<C::NLOAD>(); else wait_vmcnt<0>();
    __syncthreads();
    read_frags(0, 0, wf0, xf0);

    if constexpr (C::NW == 4 && C::FM == 8 && C::FN == 8) {
      // Four waves of 128 x 128 outputs: a wave is alone on its SIMD, so nothing else fills the issue slots an
      // instruction block without MFMAs leaves empty. The order is therefore written out, one MFMA at a time
      // (64 per 32-wide half step; an MFMA occupies the matrix pipe for four issue slots, so up to three other
      // instructions fit behind each): the 16 fragment reads of the next half step and, in a K step's second half,
      // the 16 slab loads of the step after next each follow an MFMA, and a scheduling barrier after every such pair
      // keeps the compiler from collecting them into blocks. Same loads, reads, waits and barrier as the loop below.
      auto read_one = [&](int buf, int kk, int r, bf16x8_t (&wf)[C::FN], bf16x8_t (&xf)[C::FM]) {
        // read r of a half step's 16: the activation fragments first (the first eight MFMAs use all of them)
        const char* xs = lds + buf * C::STAGE + wm * (C::FM * 16 * 128);
        const char* ws = lds + buf * C::STAGE + C::X_BYTES + wn * (C::FN * 16 * 128);
        const int ro = kk ? (rd0 ^ 64) : rd0;
        if (r < C::FM) xf[r] = *(const bf16x8_t*)(xs + r * 2048 + ro);
        else wf[r - C::FM] = *(const bf16x8_t*)(ws + (r - C::FM) * 2048 + ro);
      };
      // Load r of a slab's 16 of this wave (x rows first). `keep` is all ones, or zero for the loads behind the tile's
      // last slab: there is one loop body for every K step (no branch around a load: a lone wave pays for every
      // branch), so the last two steps issue their loads too, with every lane's offset zero (one line per
      // instruction, of slab KT - 1) and into the buffer that nobody reads again in this tile.
      auto dma_one = [&](int kt, int buf, int r, uint32_t keep) {
        const uint32_t lb = lds_wave + buf * C::STAGE;
        if (r < C::XI) dma16(xg + kt * 128, xoff[r] & keep, lb + r * NW * 1024);
        else dma16(wg + kt * 128, woff[r - C::XI] & keep, lb + C::X_BYTES + (r - C::XI) * NW * 1024);
      };
      for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        // First half: MFMAs on F0, F1 <- (slab kt, half 1), one read behind every fourth MFMA.
#pragma unroll
        for (int u = 0; u < 64; ++u) {
          const int j = u >> 3, i = u & 7;
          acc[j][i] = mfma_16x16x32<F16>(__builtin_bit_cast(u32x4_t, wf0[j]), __builtin_bit_cast(u32x4_t, xf0[i]), acc[j][i]);
          if ((u & 3) == 0) read_one(cur, 1, u >> 2, wf1, xf1);
          __builtin_amdgcn_sched_barrier(0);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this wave has read all of slab kt
        wait_vmcnt<0>();                                     // this wave's share of slab kt+1 has landed
        __syncthreads();
        // Second half: MFMAs on F1; slab kt+2 into the buffer slab kt left, one load behind every second MFMA of the
        // first 32 (a K step and a half ahead of the wait that covers it), then F0 <- (slab kt+1, half 0; behind the
        // last slab these reads return stale data that nothing uses).
        const uint32_t keep = kt + 2 < KT ? ~0u : 0u;
        const int kt2 = min(kt + 2, KT - 1);
#pragma unroll
        for (int u = 0; u < 64; ++u) {
          const int j = u >> 3, i = u & 7;
          acc[j][i] = mfma_16x16x32<F16>(__builtin_bit_cast(u32x4_t, wf1[j]), __builtin_bit_cast(u32x4_t, xf1[i]), acc[j][i]);
          if (u < 32 && (u & 1) == 0) dma_one(kt2, cur, u >> 1, keep);
          else if (u >= 32 && (u & 1) == 0) read_one(cur ^ 1, 0, (u - 32) >> 1, wf0, xf0);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    } else {
    for (int kt = 0; kt < KT; ++kt) {
      const int cur = kt & 1;
      read_frags(cur, 1, wf1, xf1);
      mma(wf0, xf0);
      interleave();
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this wave has read all of slab kt
      wait_vmcnt<0>();                                     // this wave's share of slab kt+1 has landed
      __syncthreads();
      if (kt + 2 < KT) dma(kt + 2, cur);
      __builtin_amdgcn_sched_barrier(0);
      if (kt + 1 < KT) read_frags(cur ^ 1, 0, wf0, xf0);
      mma(wf1, xf1);
      interleave();
      __builtin_amdgcn_sched_barrier(0);
    }
    }
    // All LDS reads of this tile were consumed by the MFMAs above; the next tile's prologue may
    // overwrite both buffers only after every wave got here.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    // Epilogue: lane holds y[m][n .. n+3] for m = frag_m * 16 + lane % 16, n = frag_n * 16 + 4 * (lane / 16).
    bf16_t* yg = WGRAD ? yp + ((int64_t)t.g * N + m0) * p.ldy + n0
                       : yp + (int64_t)(t.row0 + m0) * p.ldy + (int64_t)t.g * p.col_block + n0;
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
            o[0] = pack_16x2<F16>(v[0], v[1]);
            o[1] = pack_16x2<F16>(v[2], v[3]);
            *(u32x2_t*)(yrow + n) = o;
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (n + r < cols_valid) ((uint16_t*)yrow)[n + r] = cvt_16<F16>(v[r]);
          }
        }
      }
    }
  }
}

template <class C, bool WGRAD = false>
hipError_t launch(const GgParams& p, int num_wg, hipStream_t stream) {
  if (!WGRAD && p.fp16) hipLaunchKernelGGL((gg_bf16_persistent<C, false, true>), dim3(num_wg), dim3(C::NT), 0, stream, p);
  else hipLaunchKernelGGL((gg_bf16_persistent<C, WGRAD>), dim3(num_wg), dim3(C::NT), 0, stream, p);
  return hipGetLastError();
}

}  // namespace

hipError_t gg_bf16_tiled_launch(const GgParams& p, int block_m, int num_wg, hipStream_t stream) {
  switch (block_m) {
    case 256: return launch<Cfg<256, 256, 2, 4>>(p, num_wg, stream);
    // The same tile on four waves, 128 x 128 outputs each: accumulators in AGPRs, a third fewer LDS bytes per MFMA.
    case GG_TILED_256_FOUR_WAVES: return launch<Cfg<256, 256, 2, 2>>(p, num_wg, stream);
    case 128: return launch<Cfg<128, 128, 2, 2>>(p, num_wg, stream);
    case 64: return launch<Cfg<64, 128, 2, 2>>(p, num_wg, stream);
    default: return hipErrorInvalidValue;
  }
}

int gg_bf16_tiled_block_n(int block_m) { return (block_m == 256 || block_m == GG_TILED_256_FOUR_WAVES) ? 256 : 128; }

hipError_t gg_bf16_wgrad_launch(const GgParams& p, int block, int num_wg, hipStream_t stream) {
  if (block == 256) return launch<Cfg<256, 256, 2, 4>, true>(p, num_wg, stream);
  return launch<Cfg<128, 128, 2, 2>, true>(p, num_wg, stream);
}
