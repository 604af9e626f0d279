// Persistent fp8 (OCP e4m3) grouped GEMM for gfx950 with row-wise or block scales; bf16 output.
//
// Row-wise mode replaces _kernel_grouped_gemm_fp8_rowwise / grouped_gemm_fp8_rowwise
// (dev/triton_groupGEMM/groupgemm.py:269-404, 524-531): y = (x @ w_g^T) * x_scale[m] * w_scale[g*N + n],
// the scales applied once in the epilogue (groupgemm.py:374-384).
// Block mode extends it to per-1x128 activation scales x_scale[M, K/128] (the layout produced by
// kernels/triton/inference/fp8/float8_groupwise_quant.py:53-91) and per-128x128 weight scales
// w_scale[G*N/128, K/128]: every 128-wide K block is one MFMA whose result is scaled by
// x_scale[m, kb] * w_scale[(g*N + n)/128, kb] before it is added to the fp32 accumulator.
//
// Tiles are 128 x 128, one 256-thread workgroup per CU (one wave per SIMD, so a wave may use all 512
// registers). A K stage is 128 bytes = 128 fp8 values per row; NS = 4 stages of XOR-swizzled LDS are
// filled by global_load_lds_dwordx4 three stages ahead of their use (this path is bound by streaming
// every active expert's weights once, so the depth of the load queue matters more than anything).
// In block mode the stage's 128 activation scales and its weight scale travel with the slab into the
// same LDS stage. A stage is consumed by one v_mfma_f32_16x16x128_f8f6f4 per fragment pair (weight
// fragment = "A" operand, so a lane holds four consecutive output columns); the fragments of stage
// kt+1 are read from LDS while the MFMAs of stage kt run.
#include "common.h"
#include "gg_tables.h"
#include "kernels.h"

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(int)))) int i32x8_t;

constexpr int BM = 128, BN = 128;
constexpr int NW = 4, NT = 64 * NW;
constexpr int WM = 2;
constexpr int FM = 4, FN = 4;
constexpr int XI = BM / 8 / NW, WI = BN / 8 / NW;  // slab-load instructions per wave and slab
constexpr int NS = 4;                              // LDS stages
constexpr int X_BYTES = BM * 128;
constexpr int SLAB = (BM + BN) * 128;
constexpr int STAGE = SLAB + 1024;                 // + 512 B of activation scales + 2 x 256 B of weight scale

DEVINL void dma16(const void* sbase, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n"
               :
               : "s"(lds_addr), "v"(voff), "s"(sbase)
               : "memory");
}
DEVINL void dma4(const void* sbase, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2\n"
               :
               : "s"(lds_addr), "v"(voff), "s"(sbase)
               : "memory");
}
template <int N>
DEVINL void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
DEVINL int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
DEVINL const char* uni_ptr(const char* q) {
  const uint64_t v = (uint64_t)q;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (const char*)(((uint64_t)hi << 32) | lo);
}

template <int MODE>  // 0 = row-wise scales, 1 = 1x128 / 128x128 block scales
__global__ __launch_bounds__(NT) void gg_fp8_persistent(GgParams p) {
  __shared__ __attribute__((aligned(1024))) char lds[NS * STAGE];
  __shared__ int32_t row_off[MOE_GG_MAX_GROUPS + 1];
  __shared__ int32_t tile_off[MOE_GG_MAX_GROUPS + 1];
  constexpr int NL = XI + WI + (MODE == 1 ? 1 : 0);  // vector-memory instructions per wave and stage

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;
  const int K = p.K, N = p.N;  // K in elements = bytes
  const int n_tiles_n = moe_gg_cdiv(N, BN);

  build_group_tables(p.m_sizes, p.G, p.M, BM, n_tiles_n, row_off, tile_off, p.skip_rows);
  const int total = uni(tile_off[p.G]);
  const int KT = K / 128;

  const int d_r = lane >> 3;
  const uint32_t d_c16 = (uint32_t)(((lane & 7) ^ (((wave & 1) << 2) | (lane >> 4))) << 4);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;

  // Fragment reads: row = frag * 16 + lane % 16, 32 bytes = chunks 2q and 2q+1 of the row (q = lane / 16).
  const int fr = lane & 15, fq = lane >> 4;
  const int swz = (fr >> 1) & 7;
  const int rdA = fr * 128 + (((2 * fq) ^ swz) << 4);
  const int rdB = fr * 128 + (((2 * fq + 1) ^ swz) << 4);

  const char* xp = (const char*)p.x;
  const char* wp = (const char*)p.w;
  bf16_t* __restrict__ yp = (bf16_t*)p.y;

  for (int round = 0; round * (int)gridDim.x < total; ++round) {
    const int L = moe_gg_tile_of(blockIdx.x, gridDim.x, p.xcds, round);
    if (L >= total) continue;
    MoeGgTile t = moe_gg_decode_tile(row_off, tile_off, p.G, L, BM);
    t.g = uni(t.g); t.tm = uni(t.tm); t.tn = uni(t.tn); t.row0 = uni(t.row0); t.rows = uni(t.rows);
    const int m0 = t.tm * BM, n0 = t.tn * BN;
    const int rows_valid = min(t.rows - m0, BM);
    const int cols_valid = min(N - n0, BN);

    const char* xg = uni_ptr(xp + (int64_t)(t.row0 + m0) * K);
    const char* wg = uni_ptr(wp + ((int64_t)t.g * N + n0) * K);
    uint32_t xoff[XI], woff[WI];
#pragma unroll
    for (int i = 0; i < XI; ++i)
      xoff[i] = (uint32_t)min((i * NW + wave) * 8 + d_r, rows_valid - 1) * (uint32_t)K + d_c16;
#pragma unroll
    for (int i = 0; i < WI; ++i)
      woff[i] = (uint32_t)min((i * NW + wave) * 8 + d_r, cols_valid - 1) * (uint32_t)K + d_c16;
    // Block-mode scales of a stage: waves 0, 1 fetch the 128 activation scales (one row per lane), waves
    // 2, 3 each fetch the single weight scale of the tile's 128 x 128 block (every lane the same dword).
    const char* sc_base = nullptr;
    uint32_t sc_off = 0;
    if (MODE == 1) {
      const int KB = KT;
      if (wave < 2) {
        sc_base = uni_ptr((const char*)(p.x_scale + (int64_t)(t.row0 + m0) * KB));
        sc_off = (uint32_t)min(wave * 64 + lane, rows_valid - 1) * (uint32_t)(KB * 4);
      } else {
        sc_base = uni_ptr((const char*)(p.w_scale + ((int64_t)t.g * N + n0) / 128 * KB));
        sc_off = 0;
      }
    }
    // Issue the loads of K stage kt (clamped: past the end the last slab is re-read into a dead buffer,
    // which keeps the number of loads in flight - and with it the vmcnt bookkeeping - uniform).
    auto dma = [&](int kt) {
      const uint32_t lb = lds_base + (kt % NS) * STAGE;
      const int kc = min(kt, KT - 1);
#pragma unroll
      for (int i = 0; i < XI; ++i) dma16(xg + kc * 128, xoff[i], lb + (i * NW + wave) * 1024);
#pragma unroll
      for (int i = 0; i < WI; ++i) dma16(wg + kc * 128, woff[i], lb + X_BYTES + (i * NW + wave) * 1024);
      if (MODE == 1) dma4(sc_base + kc * 4, sc_off, lb + SLAB + wave * 256);
    };

    f32x4_t acc[FN][FM];
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int i = 0; i < FM; ++i) acc[j][i] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    i32x8_t wf[2][FN], xf[2][FM];
    float sc[2][FM];
    auto read_frags = [&](int kt, int b) {
      const char* st = lds + (kt % NS) * STAGE;
      const char* xs = st + wm * 2048;
      const char* ws = st + X_BYTES + wn * (FN * 2048);
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        const u32x4_t lo = *(const u32x4_t*)(ws + j * 2048 + rdA);
        const u32x4_t hi = *(const u32x4_t*)(ws + j * 2048 + rdB);
        wf[b][j] = i32x8_t{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
      }
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        const u32x4_t lo = *(const u32x4_t*)(xs + i * (WM * 2048) + rdA);
        const u32x4_t hi = *(const u32x4_t*)(xs + i * (WM * 2048) + rdB);
        xf[b][i] = i32x8_t{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
      }
      if (MODE == 1) {
        const float* s = (const float*)(st + SLAB);
        const float sw = s[128];
#pragma unroll
        for (int i = 0; i < FM; ++i) sc[b][i] = s[(i * WM + wm) * 16 + fr] * sw;
      }
    };
    auto mma = [&](int b) {
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int i = 0; i < FM; ++i) {
          if (MODE == 1) {
            const f32x4_t z = {0.f, 0.f, 0.f, 0.f};
            const f32x4_t d = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[b][j], xf[b][i], z, 0, 0, 0, 0, 0, 0);
            acc[j][i] += d * sc[b][i];
          } else {
            acc[j][i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[b][j], xf[b][i], acc[j][i], 0, 0, 0, 0, 0, 0);
          }
        }
    };
    // One K stage: publish slab kt+1, refill the buffer slab kt has just left, read the fragments of
    // kt+1 into register set b^1 while the MFMAs of stage kt (register set b) run.
    auto stage = [&](int kt, int b) {
      wait_vm<(NS - 2) * NL>();  // own share of slab kt+1; slabs kt+2 .. kt+NS-1 may still be in flight
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // own fragment reads of slab kt have returned
      __syncthreads();           // everyone's share of slab kt+1; and nobody reads slab kt's buffer any more
      dma(kt + NS);
      __builtin_amdgcn_sched_barrier(0);
      if (kt + 1 < KT) read_frags(kt + 1, b ^ 1);
      mma(b);
      __builtin_amdgcn_sched_barrier(0);
    };

#pragma unroll
    for (int s = 0; s < NS; ++s) dma(s);
    wait_vm<(NS - 1) * NL>();
    __syncthreads();
    read_frags(0, 0);
    int kt = 0;
    for (; kt + 1 < KT; kt += 2) {
      stage(kt, 0);
      stage(kt + 1, 1);
    }
    if (kt < KT) stage(kt, 0);
    wait_vm<0>();
    __syncthreads();  // trailing loads have landed and all fragment reads are done before the next tile

    // Epilogue: lane holds y[m][n .. n+3], m = (i * WM + wm) * 16 + lane % 16, n = (wn * FN + j) * 16 + 4 * (lane / 16).
    bf16_t* yg = yp + (int64_t)(t.row0 + m0) * p.ldy + (int64_t)t.g * p.col_block + n0;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      const int m = (i * WM + wm) * 16 + fr;
      if (m < rows_valid) {
        bf16_t* yrow = yg + (int64_t)m * p.ldy;
        const float am = MODE == 0 ? p.x_scale[t.row0 + m0 + m] : 1.f;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          const int n = (wn * FN + j) * 16 + fq * 4;
          f32x4_t v = acc[j][i];
          if (MODE == 0) {
            const float* bs = p.w_scale + (int64_t)t.g * N + n0;
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = v[r] * am * bs[min(n + r, cols_valid - 1)];
          }
          if (p.vec_store && n + 3 < cols_valid) {
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

}  // namespace

hipError_t gg_fp8_launch(const GgParams& p, int scale_mode, int num_wg, hipStream_t stream) {
  if (scale_mode == 0) hipLaunchKernelGGL(gg_fp8_persistent<0>, dim3(num_wg), dim3(NT), 0, stream, p);
  else hipLaunchKernelGGL(gg_fp8_persistent<1>, dim3(num_wg), dim3(NT), 0, stream, p);
  return hipGetLastError();
}
