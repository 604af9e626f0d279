// Persistent bf16 grouped GEMM for gfx950, "ping-pong" schedule.
//
// Replaces the reference's _kernel_grouped_gemm (dev/triton_groupGEMM/groupgemm.py:130-254):
// y[off_g : off_g + m_g, :] = x[off_g : ...] @ w[g]^T with fp32 accumulation and bf16 output.
//
// One 512-thread workgroup per CU walks the tile list of tile_sched.h; a tile is 256 x 256 outputs.
// Per 64-wide K step a 256 x 64 activation slab and a 256 x 64 weight slab (32 KB each) are written
// into one of two XOR-swizzled LDS stages by global_load_lds_dwordx4 (no VGPR staging) and consumed
// by v_mfma_f32_16x16x32_bf16. The weight fragment is the MFMA "A" operand and the activation
// fragment the "B" operand, so a lane ends up holding four consecutive output columns of one output
// row and the epilogue stores 8 bytes per lane.
//
// The eight waves form two groups of four (one wave of each group per SIMD). Every K step has a
// load phase L (all 24 fragment reads of the step into registers) and a compute phase C (64 MFMAs).
// The groups run half a step apart: while one group's waves own the matrix pipes, the other group's
// waves read LDS and issue the slab loads, and a workgroup barrier swaps the roles:
//
//   phase:   2s      2s+1    2s+2    2s+3
//   group 0: L(s)    C(s)    L(s+1)  C(s+1)
//   group 1: C(s-1)  L(s)    C(s)    L(s+1)
//
// Stage s & 1 is free once both groups finished L(s) (end of phase 2s+1); the loads of slab s+2 are
// issued in phase 2s+2 (group 0 at the start of L(s+1), group 1 spread over C(s)) and each wave
// waits for its own share before the barrier that ends phase 2s+3. The slab sequence runs straight
// through tile boundaries, so the first slabs of the next tile are in flight during the epilogue.
#include "common.h"
#include "gg_tables.h"
#include "kernels.h"

namespace {

constexpr int BM = 256, BN = 256;
constexpr int NW = 8, NT = 64 * NW;
constexpr int WM = 2;            // wave = wm + 2 * wn; group = wave >> 2
constexpr int FM = 8, FN = 4;    // 16-row activation / weight fragments per wave
constexpr int XI = BM / 8 / NW;  // slab-load instructions per wave and slab (8 rows each)
constexpr int WI = BN / 8 / NW;
constexpr int X_BYTES = BM * 128;
constexpr int STAGE = (BM + BN) * 128;

// 64 lanes x 16 B from global memory straight into LDS: lane l's 16 bytes land at lds_addr + 16 l.
// Issued from inline assembly so that the compiler does not serialise the in-flight slab against
// the LDS reads of the slab being consumed; completion is tracked by hand with vmcnt.
DEVINL void dma16(const void* sbase, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n"
               :
               : "s"(lds_addr), "v"(voff), "s"(sbase)
               : "memory");
}
// Values read from the LDS tables are the same in every lane; tell the compiler so (SGPRs).
DEVINL int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
DEVINL const char* uni_ptr(const char* q) {
  const uint64_t v = (uint64_t)q;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (const char*)(((uint64_t)hi << 32) | lo);
}
DEVINL MoeGgTile uni_tile(MoeGgTile t) {
  t.g = uni(t.g); t.tm = uni(t.tm); t.tn = uni(t.tn); t.row0 = uni(t.row0); t.rows = uni(t.rows);
  return t;
}
// One dword per lane; used to pull 64 different cache lines towards L2 ahead of time.
DEVINL void dma4(const void* sbase, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2\n"
               :
               : "s"(lds_addr), "v"(voff), "s"(sbase)
               : "memory");
}
template <int N>
DEVINL void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
DEVINL void wait_vm0() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
DEVINL void wait_lgkm0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

__device__ long long g_ts[256];
#define TS(i) do { if (DBG >= 1 && blockIdx.x == 0 && (tid == 0 || tid == 256)) g_ts[(tid >> 8) * 128 + (i)] = wall_clock64(); } while (0)

template <int DBG, int PFD, int NPF_ = 1>
__global__ __launch_bounds__(NT) void gg_bf16_pingpong(GgParams p) {
  __shared__ __attribute__((aligned(1024))) char lds[2 * STAGE];
  __shared__ __attribute__((aligned(256))) char pf_sink[NW * 256];
  constexpr int NPF = PFD > 0 ? NPF_ : 0;  // prefetch instructions per wave and slab
  __shared__ int32_t row_off[MOE_GG_MAX_GROUPS + 1];
  __shared__ int32_t tile_off[MOE_GG_MAX_GROUPS + 1];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1;
  const int wn = wave >> 1;
  const int grp = wave >> 2;
  const int K = p.K, N = p.N;
  const int n_tiles_n = moe_gg_cdiv(N, BN);
  TS(0);
  build_group_tables(p.m_sizes, p.G, p.M, BM, n_tiles_n, row_off, tile_off);
  TS(1);
  const int total = uni(tile_off[p.G]);
  const int KT = K / 64;
  const int nwg = gridDim.x;

  // Tiles of this workgroup: rounds 0 .. n_my - 1 (tile ids grow with the round).
  int n_my = 0;
  while (n_my * nwg < total && moe_gg_tile_of(blockIdx.x, nwg, p.xcds, n_my) < total) ++n_my;
  if (n_my == 0) return;

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

  // K rotation (experiment): decorrelate the K offsets different workgroups touch at the same time
  const int rot = DBG == 6 ? (int)(blockIdx.x % 8) * (KT / 8) : DBG == 7 ? (int)((blockIdx.x * 11) % KT) : DBG == 8 ? (int)((blockIdx.x % 8) * (KT / 8) + ((blockIdx.x / 8) % 4)) % KT : 0;
  // ---- slab-load cursor: runs ahead of the compute cursor, straight through tile boundaries ----
  const char* xg_d = xp;
  const char* wg_d = wp;
  uint32_t xoff_d[XI], woff_d[WI];
  int d_round = 0, d_kt = 0, d_step = 0;
  // Prefetch: thread tid touches one line of slab row tid (x rows for waves 0-3, w rows for waves 4-7).
  const uint32_t sink = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)pf_sink + wave * 256;
  const char* pf_base = xp;
  uint32_t pf_off = 0;
  auto dma_setup = [&](int round) {
    if (round >= n_my) return;  // past the last tile: keep re-loading the last tile (never read)
    const MoeGgTile t = uni_tile(moe_gg_decode_tile(row_off, tile_off, p.G, moe_gg_tile_of(blockIdx.x, nwg, p.xcds, round), BM));
    const int m0 = t.tm * BM, n0 = t.tn * BN;
    const int rows_valid = min(t.rows - m0, BM), cols_valid = min(N - n0, BN);
    xg_d = uni_ptr(xp + (int64_t)(t.row0 + m0) * K * 2);
    wg_d = uni_ptr(wp + ((int64_t)t.g * N + n0) * K * 2);
    if (DBG == 3) { xg_d = xp; wg_d = wp; }
#pragma unroll
    for (int i = 0; i < XI; ++i)
      xoff_d[i] = (uint32_t)min((i * NW + wave) * 8 + d_r, rows_valid - 1) * (uint32_t)(K * 2) + d_c * 16;
#pragma unroll
    for (int i = 0; i < WI; ++i)
      woff_d[i] = (uint32_t)min((i * NW + wave) * 8 + d_r, cols_valid - 1) * (uint32_t)(K * 2) + d_c * 16;
    pf_base = grp == 0 ? xg_d : wg_d;
    pf_off = (uint32_t)min(tid & 255, (grp == 0 ? rows_valid : cols_valid) - 1) * (uint32_t)(K * 2);
  };
  // Instruction idx (0 .. XI + WI - 1) of the cursor's slab; the last one advances the cursor.
  auto dma_one = [&](int idx) {
    if ((DBG == 2 || DBG == 4 || DBG == 5) && d_step >= 2) return;
    const uint32_t lb = lds_wave + (d_step & 1) * STAGE;
    int kq = DBG == 3 ? (d_kt & 15) : d_kt;
    if (DBG >= 6) { kq += rot; if (kq >= KT) kq -= KT; }
    if (idx < XI) dma16(xg_d + kq * 128, xoff_d[idx], lb + idx * NW * 1024);
    else dma16(wg_d + kq * 128, woff_d[idx - XI], lb + X_BYTES + (idx - XI) * NW * 1024);
    if (idx == XI + WI - 1) {
#pragma unroll
      for (int q = 0; q < NPF; ++q) dma4(pf_base + min(d_kt + PFD, KT - 1) * 128 + q * (128 / (NPF ? NPF : 1)), pf_off, sink);
      ++d_step;
      if (++d_kt == KT) {
        d_kt = 0;
        dma_setup(++d_round);
      }
    }
  };
  auto dma_all = [&]() {
#pragma unroll
    for (int i = 0; i < XI + WI; ++i) dma_one(i);
  };

  dma_setup(0);
  dma_all();  // slab 0 -> stage 0
  wait_vm0();
  __syncthreads();
  if (grp == 1) {  // stagger: group 1 runs one phase behind group 0
    dma_all();     // slab 1 (group 0 issues its share at the start of L(0))
    __syncthreads();
  }

  TS(2);
  long long st_vm = 0, st_b1 = 0, st_b2 = 0, st_L = 0, st_C = 0, tq = 0;
#define TQ() (DBG >= 1 ? wall_clock64() : 0)
  int step = 0;
  for (int r = 0; r < n_my; ++r) {
    TS(3 + r * 3);
    const MoeGgTile t = uni_tile(moe_gg_decode_tile(row_off, tile_off, p.G, moe_gg_tile_of(blockIdx.x, nwg, p.xcds, r), BM));
    const int m0 = t.tm * BM, n0 = t.tn * BN;
    const int rows_valid = min(t.rows - m0, BM);
    const int cols_valid = min(N - n0, BN);
    // Activation fragment i of this wave covers tile rows (i * WM + wm) * 16 .. + 15, so a partial
    // tile's rows spread evenly over both wave rows; nf = fragments with at least one valid row.
    const int nfrag_tile = (rows_valid + 15) >> 4;
    const int nf = max(0, (nfrag_tile - wm + 1) >> 1);

    f32x4_t acc[FN][FM];
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int i = 0; i < FM; ++i) acc[j][i] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    for (int kt = 0; kt < KT; ++kt, ++step) {
      // ---------------- L phase ----------------
      tq = TQ();
      if (grp == 0) dma_all();  // slab step + 1
      const char* xs = lds + (step & 1) * STAGE + wm * 2048;
      const char* ws = lds + (step & 1) * STAGE + X_BYTES + wn * (FN * 2048);
      bf16x8_t wf[2][FN], xf[2][FM];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        if (DBG == 4 && step > 0) continue;
        if (DBG == 5 && step > 0 && kk == 1) continue;
        const int ro = kk ? (rd0 ^ 64) : rd0;
#pragma unroll
        for (int j = 0; j < FN; ++j) wf[kk][j] = *(const bf16x8_t*)(ws + j * 2048 + ro);
#pragma unroll
        for (int i = 0; i < FM; ++i) xf[kk][i] = *(const bf16x8_t*)(xs + i * (WM * 2048) + ro);
      }
      __builtin_amdgcn_sched_barrier(0);
      wait_lgkm0();                // all of slab `step` is in this wave's registers
      { long long t = TQ(); st_L += t - tq; tq = t; }
      if (grp == 1) wait_vm<NPF>();  // own share of slab step + 1 (issued during the previous C phase)
      { long long t = TQ(); st_vm += t - tq; tq = t; }
      __syncthreads();
      { long long t = TQ(); st_b1 += t - tq; tq = t; }
      // ---------------- C phase ----------------
      __builtin_amdgcn_s_setprio(1);
      if (DBG >= 1 || nf == FM) {
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
          for (int j = 0; j < FN; ++j) {
#pragma unroll
            for (int i = 0; i < FM; ++i)
              acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[kk][j], xf[kk][i], acc[j][i], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (grp == 1) dma_one(kk * FN + j);  // slab step + 2, one instruction per 8 MFMAs
            __builtin_amdgcn_sched_barrier(0);
          }
      } else {
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
          for (int j = 0; j < FN; ++j) {
#pragma unroll
            for (int i = 0; i < FM; ++i)
              if (i < nf)
                acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[kk][j], xf[kk][i], acc[j][i], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (grp == 1) dma_one(kk * FN + j);
            __builtin_amdgcn_sched_barrier(0);
          }
      }
      __builtin_amdgcn_s_setprio(0);
      { long long t = TQ(); st_C += t - tq; tq = t; }
      if (grp == 0) wait_vm<NPF>();  // own share of slab step + 1 (issued at the start of this step's L phase)
      { long long t = TQ(); st_vm += t - tq; tq = t; }
      __syncthreads();
      { long long t = TQ(); st_b2 += t - tq; tq = t; }
    }

    TS(4 + r * 3);
    // Epilogue: lane holds y[m][n .. n+3] for m = (i * WM + wm) * 16 + lane % 16,
    // n = (wn * FN + j) * 16 + 4 * (lane / 16).
    bf16_t* yg = yp + (int64_t)(t.row0 + m0) * p.ldy + (int64_t)t.g * p.col_block + n0;
    const bool vec_ok = p.vec_store;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      const int m = (i * WM + wm) * 16 + fr;
      if (m < rows_valid) {
        bf16_t* yrow = yg + (int64_t)m * p.ldy;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          const int n = (wn * FN + j) * 16 + fq * 4;
          const f32x4_t v = acc[j][i];
          if (vec_ok && n + 3 < cols_valid) {
            u32x2_t o;
            o[0] = pack_bf16x2(v[0], v[1]);
            o[1] = pack_bf16x2(v[2], v[3]);
            *(u32x2_t*)(yrow + n) = o;
          } else {
#pragma unroll
            for (int rr = 0; rr < 4; ++rr)
              if (n + rr < cols_valid) yrow[n + rr] = (bf16_t)v[rr];
          }
        }
      }
    }
  }
  TS(3 + n_my * 3);
  if (DBG >= 1 && blockIdx.x == 0 && (tid == 0 || tid == 256)) {
    long long* o = g_ts + (tid >> 8) * 128 + 100;
    o[0] = st_L; o[1] = st_vm; o[2] = st_b1; o[3] = st_C; o[4] = st_b2; o[5] = step;
  }
  if (grp == 0) __syncthreads();  // pairs with group 1's last barrier
  wait_vm0();                     // trailing (never read) slab loads must land before the LDS is released
}

}  // namespace

void gg_debug_read_ts(long long* out) { (void)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_ts), sizeof(long long) * 256); }

hipError_t gg_bf16_pingpong_launch(const GgParams& p, int variant, int num_wg, hipStream_t stream) {
  switch (variant) {
    case 0: hipLaunchKernelGGL((gg_bf16_pingpong<0, 0>), dim3(num_wg), dim3(NT), 0, stream, p); break;
    case 1: hipLaunchKernelGGL((gg_bf16_pingpong<1, 0>), dim3(num_wg), dim3(NT), 0, stream, p); break;
    case 2: hipLaunchKernelGGL((gg_bf16_pingpong<2, 0>), dim3(num_wg), dim3(NT), 0, stream, p); break;
    case 3: hipLaunchKernelGGL((gg_bf16_pingpong<3, 0>), dim3(num_wg), dim3(NT), 0, stream, p); break;
    case 4: hipLaunchKernelGGL((gg_bf16_pingpong<4, 0>), dim3(num_wg), dim3(NT), 0, stream, p); break;
    case 5: hipLaunchKernelGGL((gg_bf16_pingpong<5, 0>), dim3(num_wg), dim3(NT), 0, stream, p); break;
    case 10: hipLaunchKernelGGL((gg_bf16_pingpong<6, 0>), dim3(num_wg), dim3(NT), 0, stream, p); break;
    case 11: hipLaunchKernelGGL((gg_bf16_pingpong<7, 0>), dim3(num_wg), dim3(NT), 0, stream, p); break;
    case 12: hipLaunchKernelGGL((gg_bf16_pingpong<8, 0>), dim3(num_wg), dim3(NT), 0, stream, p); break;
    case 13: hipLaunchKernelGGL((gg_bf16_pingpong<1, 3, 2>), dim3(num_wg), dim3(NT), 0, stream, p); break;
    case 14: hipLaunchKernelGGL((gg_bf16_pingpong<1, 3, 4>), dim3(num_wg), dim3(NT), 0, stream, p); break;
    case 6: hipLaunchKernelGGL((gg_bf16_pingpong<1, 2>), dim3(num_wg), dim3(NT), 0, stream, p); break;
    case 7: hipLaunchKernelGGL((gg_bf16_pingpong<1, 3>), dim3(num_wg), dim3(NT), 0, stream, p); break;
    case 8: hipLaunchKernelGGL((gg_bf16_pingpong<1, 4>), dim3(num_wg), dim3(NT), 0, stream, p); break;
    case 9: hipLaunchKernelGGL((gg_bf16_pingpong<1, 6>), dim3(num_wg), dim3(NT), 0, stream, p); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}
