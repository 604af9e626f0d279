// Persistent grouped GEMM for gfx950, "ping-pong" schedule; bf16 or fp8 (OCP e4m3) operands, bf16 output.
//
// bf16: replaces the reference's _kernel_grouped_gemm (dev/triton_groupGEMM/groupgemm.py:130-254):
// y[off_g : off_g + m_g, :] = x[off_g : ...] @ w[g]^T with fp32 accumulation and bf16 output.
// fp8, row-wise scales: _kernel_grouped_gemm_fp8_rowwise (groupgemm.py:269-404), scales applied in the
// epilogue (groupgemm.py:374-384). fp8, block scales: 1 x 128 activation scales as produced by
// kernels/triton/inference/fp8/float8_groupwise_quant.py:53-91 and 128 x 128 weight scales; a K step is
// one 128-wide scale block whose MFMA result is multiplied by x_scale[m, kb] * w_scale[n / 128, kb]
// before it is added to the accumulator.
//
// One 512-thread workgroup per CU walks the tile list of tile_sched.h; a tile is 256 x 256 outputs.
// Per K step of 128 bytes per row (64 bf16 or 128 fp8 values) a 256-row activation slab and a 256-row
// weight slab (32 KB each) are written into one of two XOR-swizzled LDS stages by
// global_load_lds_dwordx4 (no VGPR staging) and consumed by v_mfma_f32_16x16x32_bf16 (two per fragment
// pair and step) or v_mfma_f32_16x16x128_f8f6f4 (one; its 32-byte operand is the lane's two 16-byte
// reads, the same for both operands, so the order of k inside the step does not matter). The weight
// fragment is the MFMA "A" operand and the activation fragment the "B" operand, so a lane ends up
// holding four consecutive output columns of one output row and the epilogue stores 8 bytes per lane.
//
// The eight waves form two groups of four (one wave of each group per SIMD); group 0 owns weight
// rows 0-127 of the tile (W0), group 1 rows 128-255 (W1), both use all activation rows (X).
// Every K step s has a load phase L(s) (all 24 fragment reads of the step into registers, plus all
// slab-load instructions) and a compute phase C(s) (the MFMAs, nothing else). The groups run half a
// step apart, so that the matrix pipes always have exactly one wave per SIMD feeding them while
// the other wave does the memory work; a workgroup barrier swaps the roles:
//
//   phase:   2s          2s+1        2s+2        2s+3
//   group 0: L(s)        C(s)        L(s+1)      C(s+1)
//   group 1: C(s-1)      L(s)        C(s)        L(s+1)
//
// Which stage regions are free when decides who loads what:
//   X(s) is read in phases 2s and 2s+1, W0(s) only in 2s (group 0), W1(s) only in 2s+1 (group 1).
//   group 0 in L(s)  [phase 2s]   issues X(s+1)  -> stage (s+1)&1, free since phase 2s-1 (32 KB);
//   group 1 in L(s)  [phase 2s+1] issues W1(s+1) -> stage (s+1)&1, free since phase 2s-1,
//                                    and W0(s+2) -> stage s&1, free since phase 2s (32 KB together).
// Both load phases so put the same 32 KB through the CU's vector-memory path. Each group waits for its own
// loads at the end of the compute phase that follows. The slab sequence runs straight through tile
// boundaries, so the next tile's first slabs are in flight during the epilogue.
// Block scales of step s+1 (256 activation scales, the tile's two weight-block scales) travel with
// group 0's loads into a small per-stage LDS area.
#include <type_traits>

#include "common.h"
#include "gg_tables.h"
#include "kernels.h"

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(int)))) int i32x8_t;

constexpr int BM = 256, BN = 256;
constexpr int NW = 8, NT = 64 * NW;
constexpr int WM = 2;            // wave = wm + 2 * wn; group = wave >> 2 = wn >> 1
constexpr int FM = 8, FN = 4;    // 16-row activation / weight fragments per wave
constexpr int X_BYTES = BM * 128;
constexpr int STAGE = (BM + BN) * 128;
constexpr int TALL_BYTES = MOE_GG_TALL_ROWS * 128;  // per stage: the slab rows of a tall tile's rows 256 .. 287 (four-wave kernel)
constexpr int SCALE_BYTES = 2048;  // per stage: 256 activation scales, then 4 x 256 B of weight-block scales

// Operand kinds.
// OP_BF16_WGRAD: the weight gradient of the bf16 layer, dW[g][n][k] = sum over the rows m of expert g of
// dY[m][n] * X[m][k] (kernels/MoE/group_GEMM/triton/tgroup_gemm_backwards.py:202-375), as the same product on
// transposed operands: p.x = dY^T [N, ldm], p.w = X^T [K, ldm], the rows of expert g zero-padded to whole
// 64-column blocks (at least one), so the reduction of a tile is a whole number of K steps that depends on
// its expert. Every expert has the same ceil(N / 256) * ceil(K / 256) tiles. p.M = ldm, p.skip_rows = number
// of gradient rows, p.y = dW [G * N, K].
// OP_BF16_SWIGLU: the first GEMM of a gated MoE layer with SiLU-and-mul in the epilogue
// (kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:271-284: GEMM with w1 [E, 2n, K], then
// ops.silu_and_mul): y[m][c] = silu(x[m] . w[g][c]) * (x[m] . w[g][n + c]), y is [M, n]. The layout of w is the
// reference's (gate rows 0 .. n-1, up rows n .. 2n-1 of every expert); a tile takes 128 gate rows and the 128 up
// rows of the same output columns, placed in LDS so that every wave holds the gate and the up value of its own
// 32 output columns: weight-tile row 64 wn + 32 h + c (h = 0 gate, 1 up) is output column 32 wn + c.
// Both products are rounded to bf16 before the activation, as they are when the GEMM output is stored first.
// p.N = 2n.
// OP_BF16_NT: the product with weights that are NOT stored along the reduction, y[m][c] = sum_r x[m][r] * w[g][r][c]
// with w [G * R, C] row-major (p.K = R, p.N = C): the input gradient of the layer, dX = dY w, read from the
// forward weights as they are (kernels/MoE/group_GEMM/triton/tgroup_gemm_backwards.py:27-199 reads a transposed
// copy). A K step's weight slab is 64 rows r of 256 columns; each half (128 columns, 256-byte rows) is written
// into its LDS region row by row and read with ds_read_b64_tr_b16, which hands lane l of a 16-lane group column
// l of a 4-row block: two such reads give the lane the eight consecutive r of its column that the MFMA wants.
// Rows of 256 bytes cover all LDS banks, so the 32-byte column blocks are XOR-swizzled with
// (r & 3) | ((r >> 3) & 1) << 2: the 16 rows one instruction touches then fall on 8 different bank groups twice
// (512 bytes per instruction: the minimum).
// OP_BF16_WGRAD_DIRECT: the weight gradient read from dY [M, ldx] and X [M, K] as stored: both operands have the
// reduction index (the row m) as their slow dimension, so both slabs are 64 rows by 256 columns in the layout of
// OP_BF16_NT and both fragment kinds come from transposing reads. A tile reduces over the rows of its expert:
// max(1, ceil(m_g / 64)) K steps; rows beyond the expert's last one re-read that row (the loads stay inside the
// tensors), and group 0 overwrites them with zeros in the dY slab once it has landed, so they add nothing.
// OP_F16, OP_F16_SWIGLU: OP_BF16 / OP_BF16_SWIGLU on IEEE half data (the same kernels with the f16 MFMA and half
// conversions in the epilogue).
// OP_BF16_SWIGLU_GATHER, OP_F16_SWIGLU_GATHER: the SWIGLU kernels reading their activation rows through the layer's
// row permutation: row i of the expert-sorted order is row perm[i] / k of the token matrix p.x (the gather of
// fused_moe folded into the slab loads; the reference's kernel reads A through sorted_token_ids in the same way,
// kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:75-80). Per tile a loading lane keeps the byte
// offsets of its eight rows; a K step's loads add only the chunk offset.
constexpr int OP_BF16 = 0, OP_FP8_ROW = 1, OP_FP8_BLOCK = 2, OP_BF16_WGRAD = 3, OP_BF16_SWIGLU = 4, OP_BF16_NT = 5,
              OP_BF16_WGRAD_DIRECT = 6, OP_F16 = 7, OP_F16_SWIGLU = 8, OP_BF16_SWIGLU_GATHER = 9, OP_F16_SWIGLU_GATHER = 10;
constexpr bool op_gather(int op) { return op == OP_BF16_SWIGLU_GATHER || op == OP_F16_SWIGLU_GATHER; }
constexpr bool op_swiglu(int op) { return op == OP_BF16_SWIGLU || op == OP_F16_SWIGLU || op_gather(op); }
constexpr bool op_f16(int op) { return op == OP_F16 || op == OP_F16_SWIGLU || op == OP_F16_SWIGLU_GATHER; }
typedef short i16x4_t __attribute__((ext_vector_type(4)));

// 64 lanes x 16 B (or 4 B) from global memory straight into LDS: lane l's bytes land at lds_addr + 16 l
// (4 l). Issued from inline assembly so that the compiler does not serialise the in-flight slab against
// the LDS reads of the slab being consumed; completion is tracked by hand with vmcnt.
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
DEVINL void wait_lgkm0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

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

// a * b + c for a, b < 2^24 (row index and row pitch in bytes): one full-rate VALU instruction where the 32-bit
// multiply takes a quarter-rate one. The partner wave's MFMAs share the VALU issue port with these.
// (Written as an instruction: from the plain expression the compiler may still pick the 64-bit multiply-add.)
DEVINL uint32_t mad24(uint32_t a, uint32_t b, uint32_t c) {
  uint32_t d;
  asm("v_mad_u32_u24 %0, %1, %2, %3" : "=v"(d) : "v"(a), "s"(b), "v"(c));
  return d;
}

struct Shared {
  const int32_t* row_off;
  const int32_t* tile_off;   // forward: prefix of the long tiles; WGRAD: prefix of the padded 64-column blocks
  const int32_t* part_off;   // forward: prefix of the low tiles (one row of tiles per group at most)
  const int32_t* seq_tab;    // the workgroup's tiles in the order it computes them: (group, row tile | column tile << 16)
  char* lds;
  int n_my;       // tiles of this workgroup (<= MOE_GG_SEQ_CAP, the launcher's duty)
};

// Slab-load cursor of one wave: which slab (tile round, K step) its next load instructions fetch.
struct Cursor {
  const char* xg;   // activation rows of the tile, K offset 0
  const char* wg;   // weight rows of the tile
  const char* xsg;  // block mode: activation scales of the tile's first row, K block 0
  const char* wsg;  // block mode: weight scales of the tile's first 128-column block, K block 0
  int x_last;       // last valid activation row of the tile (rows beyond it re-read this one)
  int w_last;       // last valid weight row of the tile
  int ws_second;    // block mode: byte offset of the second column block's scales (0 if there is none)
  int KT;           // K steps of the cursor's tile
  int rows_g;       // WGRAD_DIRECT: rows of the tile's expert (its reduction length)
  int round, kt, step;
};

template <int GRP, int OP>
DEVINL void run_group(const GgParams& p, const Shared& sh) {
  constexpr bool FP8 = OP == OP_FP8_ROW || OP == OP_FP8_BLOCK;
  constexpr bool F16 = op_f16(OP);
  constexpr bool BLOCK = OP == OP_FP8_BLOCK;
  constexpr bool WGRAD = OP == OP_BF16_WGRAD;
  constexpr bool SWIGLU = op_swiglu(OP);
  constexpr bool GATHER = op_gather(OP);
  constexpr bool WG2 = OP == OP_BF16_WGRAD_DIRECT;
  constexpr bool WNT = OP == OP_BF16_NT || WG2;  // weight slab: 64 reduction rows by 256 columns (transposing reads)
  constexpr int TILE_COLS = SWIGLU ? BN / 2 : BN;  // output columns of a tile
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1;
  const int wn = wave >> 1;
  const int gw = wave & 3;  // wave index inside its group
  const int N = p.N;
  const uint32_t KROW = WGRAD ? (uint32_t)p.M * 2u : (uint32_t)p.K * (FP8 ? 1u : 2u);  // bytes per operand row
  const int KT_fwd = (int)((uint32_t)p.K * (FP8 ? 1u : 2u) / 128u);  // K steps of every forward tile
  const int NCOLS = (WGRAD || WG2) ? p.K : (SWIGLU ? N / 2 : N);      // output columns of a group
  // Bytes between rows of the x operand: the two backward kernels read the output gradient with its own leading
  // dimension and, for the [M, N * G] layout, at the expert's column block.
  const uint32_t XPITCH = (WG2 || OP == OP_BF16_NT) ? (uint32_t)p.ldx * 2u : KROW;
  const int nwg = gridDim.x;
  // Tile of a round. Forward: rows of x / rows of w[g]. WGRAD: rows of dY^T (n) / rows of X^T (k), both at the
  // column offset of the expert's padded block; t.row0 = first row of the expert's block of dW, t.rows = N.
  // m0, h: first row inside the group, rows (a whole tile or a row piece of one); n0, nc: first column, columns
  struct TileRef { MoeGgTile t; int KT, rows_g, m0, h, n0, nc; int64_t xoff, woff; };
  // The workgroup's own sequence (moe_gg_seq_round): its long tiles in round order with its low tiles spread
  // evenly between them, at a phase that differs between XCDs, so that memory-bound low tiles and compute-bound
  // long tiles run side by side on the chip, while the workgroups of one XCD take theirs together and stay in
  // step. Tile ids: long tiles 0 .. n_long - 1, then the low tiles.
  auto tile_ref = [&](int seq) {
    TileRef r;
    // Decoded in the prologue: group | rows << 16 | columns / 32 << 26, first row / 64 | first column / 32 << 16.
    const int gh = uni(sh.seq_tab[2 * seq]);
    const int mn = uni(sh.seq_tab[2 * seq + 1]);
    const int g = gh & 0xFFFF;
    r.h = (gh >> 16) & 0x3FF;
    r.nc = (int)((uint32_t)gh >> 26) * 32;
    r.m0 = (mn & 0xFFFF) * 64;
    r.n0 = (int)((uint32_t)mn >> 16) * 32;
    r.t.g = g; r.t.tm = 0; r.t.tn = 0;
    r.rows_g = 0;
    if (WG2) {
      // Output: rows tm * 256 .. of the expert's block of dW (n), columns tn * 256 .. (k). Operands: the expert's
      // rows of dY at columns g * x_col_block + tm * 256 .., and of X at columns tn * 256 ...
      int row0 = uni(sh.row_off[g]);
      r.rows_g = uni(sh.row_off[g + 1]) - row0;
      if (r.rows_g == 0) row0 = min(row0, p.M - 1);  // an expert without rows: one K step of zeros, loads in bounds
      r.t.row0 = g * N; r.t.rows = N;
      r.KT = max(1, moe_gg_cdiv(r.rows_g, 64));
      r.xoff = (int64_t)row0 * XPITCH + ((int64_t)g * p.x_col_block + r.m0) * 2;
      r.woff = (int64_t)row0 * (int64_t)p.K * 2 + (int64_t)r.n0 * 2;
    } else if (WGRAD) {
      r.t.row0 = g * N; r.t.rows = N;
      const int b0 = uni(sh.tile_off[g]);
      r.KT = uni(sh.tile_off[g + 1]) - b0;
      r.xoff = (int64_t)r.m0 * KROW + (int64_t)b0 * 128;
      r.woff = (int64_t)r.n0 * KROW + (int64_t)b0 * 128;
    } else {
      r.t.row0 = uni(sh.row_off[g]);
      r.t.rows = uni(sh.row_off[g + 1]) - r.t.row0;
      r.KT = KT_fwd;
      r.xoff = GATHER ? 0 : (int64_t)(r.t.row0 + r.m0) * XPITCH + (OP == OP_BF16_NT ? (int64_t)g * p.x_col_block * 2 : 0);
      if (WNT) r.woff = ((int64_t)g * p.K * N + r.n0) * 2;  // w[g][0][n0]
      else r.woff = ((int64_t)g * N + r.n0) * KROW;
    }
    return r;
  };

  // Slab-load geometry: an instruction fills 8 rows (1 KB of LDS); lane -> row lane / 8, physical
  // 16-byte slot lane % 8, which must hold logical chunk slot ^ ((row >> 1) & 7). Inside a group the
  // 8-row blocks are dealt round-robin to the four waves, so the block parity is gw & 1.
  const int d_r = lane >> 3;
  const uint32_t d_c16 = (uint32_t)(((lane & 7) ^ (((gw & 1) << 2) | (lane >> 4))) << 4);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)sh.lds;
  const uint32_t lds_scale = lds_base + 2 * STAGE;

  // Fragment reads: row = frag * 16 + lane % 16, chunk = kk * 4 + lane / 16 (swizzled).
  const int fr = lane & 15, fq = lane >> 4;
  const int rd0 = fr * 128 + ((fq ^ (fr >> 1)) << 4);  // kk = 0; kk = 1 is rd0 ^ 64

  const char* xp = (const char*)p.x;
  const char* wp = (const char*)p.w;
  bf16_t* __restrict__ yp = (bf16_t*)p.y;

  Cursor c;
  uint32_t gather_off[8];  // GATHER, group 0: byte offset in p.x of the lane's row of its block idx * 4 + gw, idx = 0 .. 7
  auto cursor_tile = [&](int round) {
    c.round = round;
    if (round >= sh.n_my) return;  // past the last tile: keep re-loading the last tile (never read)
    const TileRef tr = tile_ref(round);
    const MoeGgTile& t = tr.t;
    const int m0 = tr.m0, n0 = tr.n0;
    c.KT = tr.KT;
    c.rows_g = tr.rows_g;
    c.x_last = max(tr.h, 1) - 1;  // (a piece without rows loads row 0 and stores nothing)
    c.w_last = max(min(NCOLS - n0, tr.nc), 1) - 1;  // SWIGLU: last valid output column of the tile
    c.xg = uni_ptr(xp + tr.xoff);
    c.wg = uni_ptr(wp + tr.woff);
    if (GATHER && GRP == 0) {
      // The sorted rows t.row0 + m0 .. of this tile, looked up once per tile; rows beyond the tile's last one repeat
      // it, as the plain kernel re-reads it. An entry that names no slot of the token matrix (a caller's corrupt
      // perm) is folded into range, so that the loads stay inside p.x whatever perm holds.
      const int32_t* pp = p.gather_perm + t.row0 + m0;
#pragma unroll
      for (int idx = 0; idx < 8; ++idx) {
        const uint32_t slot = (uint32_t)pp[min((idx * 4 + gw) * 8 + d_r, c.x_last)];
        gather_off[idx] = min(slot / (uint32_t)p.gather_k, (uint32_t)p.gather_rows - 1u) * XPITCH;
      }
    }
    if (BLOCK) {
      c.xsg = uni_ptr((const char*)(p.x_scale + (int64_t)(t.row0 + m0) * KT_fwd));
      c.wsg = uni_ptr((const char*)(p.w_scale + (((int64_t)t.g * N + n0) / 128) * KT_fwd));
      c.ws_second = n0 + 128 < N ? KT_fwd * 4 : 0;
    }
  };
  auto cursor_next = [&]() {
    ++c.step;
    if (++c.kt == c.KT) {
      c.kt = 0;
      cursor_tile(c.round + 1);
    }
  };
  // Block b (8 rows) of the cursor slab's activation / weight rows.
  // WGRAD_DIRECT: what group 0 has to zero in the slab it loaded last: rows zf_valid .. 63 of stage zf_stage.
  int zf_valid = 64, zf_stage = 0;
  auto dma_x = [&](int b) {
    if (WG2) {
      // As the weight slab of OP_BF16_NT (see dma_w): block b = rows 4 (b & 15) .. + 3 of the slab's 64 rows of
      // dY, column half b >> 4. Rows beyond the expert's last one re-read it.
      const int bb = b & 15;
      const uint32_t sw = (uint32_t)((lane >> 4) | (((bb >> 1) & 1) << 2));
      const uint32_t chunk = (uint32_t)min((int)(((b >> 4) << 4) + ((lane & 15) ^ (sw << 1))), c.x_last >> 3);
      const int rlast = max(c.rows_g - 1 - c.kt * 64, 0);
      const uint32_t off = mad24((uint32_t)min(bb * 4 + (lane >> 4), rlast), XPITCH, chunk << 4);
      dma16(c.xg + (int64_t)c.kt * (64 * (int64_t)XPITCH), off, lds_base + (c.step & 1) * STAGE + b * 1024);
      return;
    }
    if (b * 8 > c.x_last) return;  // block entirely below the tile's last row: its fragments are never used
    const uint32_t off = GATHER ? gather_off[b >> 2] + d_c16 : mad24((uint32_t)min(b * 8 + d_r, c.x_last), XPITCH, d_c16);
    dma16(c.xg + c.kt * 128, off, lds_base + (c.step & 1) * STAGE + b * 1024);
  };
  // Weight rows: of the cursor slab, or (prev) of the slab before it, whose state group 1 keeps in wp_*.
  const char* wp_wg = nullptr;
  int wp_last = 0, wp_kt = 0, wp_step = 0;
  const uint32_t WROW = (uint32_t)(WG2 ? p.K : N) * 2u;  // slab layouts of OP_BF16_NT: bytes per weight row
  int wp_rows_g = 0;
  auto dma_w = [&](int b, bool prev) {
    const int w_last = prev ? wp_last : c.w_last;
    if (WNT) {
      // Block b: rows 4 (b & 15) .. + 3 of the slab's 64, column half b >> 4; lane -> row lane / 16, physical
      // 16-byte slot lane % 16, which holds logical chunk slot ^ (swizzle(row) << 1). Chunks beyond the last
      // valid column re-read that one (their columns are never stored).
      const int bb = b & 15;
      const uint32_t sw = (uint32_t)((lane >> 4) | (((bb >> 1) & 1) << 2));
      const uint32_t chunk = (uint32_t)min((int)(((b >> 4) << 4) + ((lane & 15) ^ (sw << 1))), w_last >> 3);
      int r = bb * 4 + (lane >> 4);
      if (WG2) r = min(r, max((prev ? wp_rows_g : c.rows_g) - 1 - (prev ? wp_kt : c.kt) * 64, 0));
      const uint32_t off = mad24((uint32_t)r, WROW, chunk << 4);
      dma16((prev ? wp_wg : c.wg) + (int64_t)(prev ? wp_kt : c.kt) * (64 * (int64_t)WROW), off,
            lds_base + ((prev ? wp_step : c.step) & 1) * STAGE + X_BYTES + b * 1024);
      return;
    }
    uint32_t row;
    if (SWIGLU) row = (uint32_t)min((b >> 3) * 32 + (b & 3) * 8 + d_r, w_last) + (((b >> 2) & 1) ? (uint32_t)NCOLS : 0u);
    else row = (uint32_t)min(b * 8 + d_r, w_last);
    const uint32_t off = mad24(row, KROW, d_c16);
    dma16((prev ? wp_wg : c.wg) + (prev ? wp_kt : c.kt) * 128, off,
          lds_base + ((prev ? wp_step : c.step) & 1) * STAGE + X_BYTES + b * 1024);
  };
  auto keep_prev = [&]() { wp_wg = c.wg; wp_last = c.w_last; wp_kt = c.kt; wp_step = c.step; wp_rows_g = c.rows_g; };
  // WGRAD_DIRECT, group 0, after its loads have landed: zero the rows of the dY slab that lie beyond the expert's
  // last row (only the last K step of a tile has any). Every wave clears the blocks it loaded itself.
  auto zero_fill = [&]() {
    if (!WG2 || GRP != 0) return;
    if (zf_valid < 64) {
#pragma unroll
      for (int idx = 0; idx < 8; ++idx) {
        const int b = idx * 4 + gw;
        if ((b & 15) * 4 + (lane >> 4) >= zf_valid)
          *(u32x4_t*)(sh.lds + zf_stage * STAGE + b * 1024 + lane * 16) = u32x4_t{0u, 0u, 0u, 0u};
      }
      wait_lgkm0();
    }
  };
  // Block scales of the cursor slab: wave gw of group 0 fetches the activation scales of rows
  // 64 gw .. 64 gw + 63 (one per lane) and a private copy of the two weight-block scales (lanes 0-31 the
  // first column block, lanes 32-63 the second).
  auto dma_xscale = [&]() {
    const uint32_t off = (uint32_t)min(gw * 64 + lane, c.x_last) * (uint32_t)(KT_fwd * 4);
    dma4(c.xsg + c.kt * 4, off, lds_scale + (c.step & 1) * SCALE_BYTES + gw * 256);
  };
  auto dma_wscale = [&]() {
    const uint32_t off = lane < 32 ? 0u : (uint32_t)c.ws_second;
    dma4(c.wsg + c.kt * 4, off, lds_scale + (c.step & 1) * SCALE_BYTES + 1024 + gw * 256);
  };
  // Load instruction idx of this wave in a load phase; the last one advances the cursor. Both groups issue
  // 8 slab instructions per wave and phase:
  // Group 0 (cursor = slab s + 1): 8 activation blocks (idx 0-7); block mode: the scales (8, 9).
  // Group 1 (cursor = slab s + 2): 4 blocks of W1 of the slab before the cursor (idx 0-3), 4 blocks of W0 of the
  // cursor slab (idx 4-7).
  constexpr int NDMA = GRP == 0 ? (BLOCK ? 10 : 8) : 8;
  auto dma_one = [&](int idx) {
    if (GRP == 0) {
      if (idx < 8) dma_x(idx * 4 + gw);
      else if (idx == 8) dma_xscale();
      else dma_wscale();
    } else {
      if (idx < 4) dma_w(16 + idx * 4 + gw, true);
      else dma_w((idx - 4) * 4 + gw, false);
    }
    if (idx == NDMA - 1) {
      if (GRP == 1) keep_prev();
      if (WG2 && GRP == 0) {
        zf_valid = c.kt == c.KT - 1 ? c.rows_g - c.kt * 64 : 64;
        zf_stage = c.step & 1;
      }
      cursor_next();
    }
  };

  // Prologue: slab 0 of the first tile (group 0 the activations and scales, group 1 all weight rows), then the
  // stagger: group 1 runs one phase behind group 0 and sends W0(1) now; W1(1) and W0(2) follow in its L(0).
  c.kt = 0; c.step = 0;
  cursor_tile(0);
  if (GRP == 0) {
#pragma unroll
    for (int i = 0; i < NDMA; ++i) dma_one(i);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_w(i * 4 + gw, false);
    cursor_next();
  }
  wait_vm<0>();
  zero_fill();
  __syncthreads();
  if (GRP == 1) {
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_w(i * 4 + gw, false);
    keep_prev();
    cursor_next();
    __syncthreads();
  }

  int step = 0;
  for (int r = 0; r < sh.n_my; ++r) {
    wave_whole();  // the lanes left the epilogue's masked store blocks at different points
    const TileRef tr = tile_ref(r);
    const MoeGgTile& t = tr.t;
    const int KT = tr.KT;
    const int m0 = tr.m0, n0 = tr.n0;
    const int rows_valid = tr.h;
    const int cols_valid = min(NCOLS - n0, tr.nc);
    // Activation fragments of this wave that hold at least one valid row (fragments are dealt
    // alternately to wm = 0 / 1, so a short tile shortens every wave's C phase alike).
    const int nfm = min(FM, max(0, ((rows_valid + 15) / 16 - wm + WM - 1) / WM));

    // The tile body exists twice: for full-height tiles (all MFMAs of a step, no branches) and for
    // short tiles, which skip the MFMAs of activation fragments that hold no valid row. Each copy has
    // its own accumulators, so the two K loops do not have to agree on a register assignment.
    auto do_tile = [&](auto short_tag) {
      constexpr bool SHORT = decltype(short_tag)::value;
      f32x4_t acc[FN][FM];
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int i = 0; i < FM; ++i) acc[j][i] = f32x4_t{0.f, 0.f, 0.f, 0.f};

      for (int kt = 0; kt < KT; ++kt, ++step) {
        // ---------------- L phase: 24 fragment reads interleaved with this wave's slab loads ----------------
        // Activation fragment i covers tile rows (i * WM + wm) * 16 .. + 15; weight fragment j covers
        // tile columns (wn * FN + j) * 16 .. + 15.
        const char* xs = sh.lds + (step & 1) * STAGE + wm * 2048;
        const char* ws = sh.lds + (step & 1) * STAGE + X_BYTES + wn * (FN * 2048);
        u32x4_t wf[2][FN], xf[2][FM];
        // OP_BF16_NT: the lane's address inside the wave's column half for fragment f: row block of its k quarter, row
        // lane % 16 / 4 of a 4-row block, swizzled 32-byte column block, 8-byte piece lane % 4.
        // The swizzle term of the lane (bits 5-7) is folded into one per-step base; a fragment's column block is an
        // XOR on those bits. The base passes through an empty asm so that the addresses are formed here, per step,
        // and not kept in registers across the K loop.
        const int tr_ti = (lane & 15) >> 2, tr_ts = tr_ti | ((fq & 1) << 2);
        uint32_t tr_base = lds_base + (uint32_t)((step & 1) * STAGE + fq * 2048 + tr_ti * 256 + (tr_ts << 5) + (lane & 3) * 8);
        asm volatile("" : "+v"(tr_base));
        auto wt_addr = [&](int f) {
          return (tr_base ^ (uint32_t)((((wn & 1) << 2) + f) << 5)) + (uint32_t)(X_BYTES + (wn >> 1) * 16384);
        };
        // WGRAD_DIRECT: the same for activation fragment i: tile row block 2 i + wm = column block (2 i + wm) % 8 of
        // half i / 4 of the dY slab.
        auto xt_addr = [&](int i) {
          return (tr_base ^ (uint32_t)((((i & 3) << 1) + wm) << 5)) + (uint32_t)((i >> 2) * 16384);
        };
        auto tr_pair = [&](uint32_t a) {
          typedef __attribute__((address_space(3))) i16x4_t* lds_i16x4_ptr;
          const i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)(uintptr_t)a);
          const i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)(uintptr_t)(a + 1024));
          const u32x2_t l2 = __builtin_bit_cast(u32x2_t, lo), h2 = __builtin_bit_cast(u32x2_t, hi);
          return u32x4_t{l2[0], l2[1], h2[0], h2[1]};
        };
        int issued = 0;
#pragma unroll
        for (int q = 0; q < 24; ++q) {
          // spread the NDMA load instructions evenly over the 24 reads
          if (issued < NDMA && q * NDMA >= issued * 24) {
            __builtin_amdgcn_sched_barrier(0);
            dma_one(issued);
            ++issued;
            if (issued < NDMA && q * NDMA >= issued * 24) { dma_one(issued); ++issued; }
            __builtin_amdgcn_sched_barrier(0);
          }
          const int kk = q / 12, f = q % 12;
          const int ro = kk ? (rd0 ^ 64) : rd0;
          if (f < FN && WNT) wf[kk][f] = tr_pair(wt_addr(f) + kk * 8192);
          else if (f < FN) wf[kk][f] = *(const u32x4_t*)(ws + f * 2048 + ro);
          else if (WG2) xf[kk][f - FN] = tr_pair(xt_addr(f - FN) + kk * 8192);
          else xf[kk][f - FN] = *(const u32x4_t*)(xs + (f - FN) * (WM * 2048) + ro);
        }
        float sc[FM];
        if (BLOCK) {
          const float* sl = (const float*)(sh.lds + 2 * STAGE + (step & 1) * SCALE_BYTES);
          const float sw = sl[256 + (wn >> 1) * 32];  // the wave's 64 columns lie in column block wn / 2 of the tile's two
#pragma unroll
          for (int i = 0; i < FM; ++i) sc[i] = sl[(i * WM + wm) * 16 + fr] * sw;
        }
        __builtin_amdgcn_sched_barrier(0);
        wait_lgkm0();  // all of slab `step` is in this wave's registers
        if (GRP == 1) wait_vm<NDMA>();  // first step: W0(1) of the prologue has landed; later nothing older is left
        __syncthreads();
        // ---------------- C phase: MFMAs only ----------------
        // (No s_setprio here: with the computing wave at raised priority the kernels ran 0.5-2 % slower.)
        // bf16: one of the two MFMAs (K half kk) of fragment pair (j, i); fp8: its single MFMA.
        auto mma = [&](int j, int i, int kk) {
          if (!FP8) {
            acc[j][i] = mfma_16x16x32<F16>(wf[kk][j], xf[kk][i], acc[j][i]);
          } else {
            const i32x8_t a = {(int)wf[0][j][0], (int)wf[0][j][1], (int)wf[0][j][2], (int)wf[0][j][3],
                               (int)wf[1][j][0], (int)wf[1][j][1], (int)wf[1][j][2], (int)wf[1][j][3]};
            const i32x8_t b = {(int)xf[0][i][0], (int)xf[0][i][1], (int)xf[0][i][2], (int)xf[0][i][3],
                               (int)xf[1][i][0], (int)xf[1][i][1], (int)xf[1][i][2], (int)xf[1][i][3]};
            if (BLOCK) {
              const f32x4_t z = {0.f, 0.f, 0.f, 0.f};
              const f32x4_t d = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, z, 0, 0, 0, 0, 0, 0);
              acc[j][i] += d * sc[i];
            } else {
              acc[j][i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[j][i], 0, 0, 0, 0, 0, 0);
            }
          }
        };
        constexpr int NKK = FP8 ? 1 : 2;
        if (!SHORT) {
#pragma unroll
          for (int kk = 0; kk < NKK; ++kk)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
              for (int i = 0; i < FM; ++i) mma(j, i, kk);
        } else {
#pragma unroll
          for (int i = 0; i < FM; ++i) {
            if (i < nfm) {
#pragma unroll
              for (int kk = 0; kk < NKK; ++kk)
#pragma unroll
                for (int j = 0; j < FN; ++j) mma(j, i, kk);
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        // Group 0: X(step + 1), issued in this step's load phase, is read in the next phase. Group 1: of its loads of
        // this step's load phase only W1(step + 1), issued first, is read that soon; the four W0(step + 2) loads may
        // stay in flight until the end of its next load phase (the wait there leaves only that phase's own loads).
        if (GRP == 0) wait_vm<0>(); else wait_vm<4>();
        zero_fill();
        __syncthreads();
      }

      // Epilogue: lane holds y[m][n .. n+3] for m = (i * WM + wm) * 16 + lane % 16,
      // n = (wn * FN + j) * 16 + 4 * (lane / 16). Addresses are a per-fragment uniform base plus one
      // 32-bit lane offset. The lane indices pass through an empty asm so that the address arithmetic
      // is redone here for every tile instead of being hoisted out of the tile loop, where it would
      // occupy (and spill) registers during the K loop.
      bf16_t* yg = yp + (int64_t)(t.row0 + m0) * p.ldy + ((WGRAD || WG2) ? 0 : (int64_t)t.g * p.col_block) + n0;
      int er = fr, eq = fq;
      asm volatile("" : "+v"(er), "+v"(eq));
      // Row-wise fp8 scales (groupgemm.py:374-384): y *= x_scale[m] * w_scale[g * N + n].
      const float* xrow_scale = OP == OP_FP8_ROW ? p.x_scale + t.row0 + m0 : nullptr;
      const float* wcol_scale = OP == OP_FP8_ROW ? p.w_scale + (int64_t)t.g * N + n0 : nullptr;
      if (SWIGLU) {
        // acc[j][i], j = 0, 1: gate of output columns 32 wn + 16 j + 4 eq .. + 3; acc[j + 2][i]: up of the same columns.
#pragma unroll
        for (int i = 0; i < FM; ++i) {
          const int m = (i * WM + wm) * 16 + er;
          if (m < rows_valid) {
            bf16_t* yrow = yg + (int64_t)m * p.ldy;
            u32x2_t q[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const f32x4_t gv = acc[j][i], uv = acc[j + 2][i];
              // both products rounded to the 16-bit type first, as they are when the GEMM output is stored
              const uint32_t g01 = pack_16x2<F16>(gv[0], gv[1]), g23 = pack_16x2<F16>(gv[2], gv[3]);
              const uint32_t u01 = pack_16x2<F16>(uv[0], uv[1]), u23 = pack_16x2<F16>(uv[2], uv[3]);
              const float g[4] = {f32_of_16<F16>((uint16_t)g01), f32_of_16<F16>((uint16_t)(g01 >> 16)),
                                  f32_of_16<F16>((uint16_t)g23), f32_of_16<F16>((uint16_t)(g23 >> 16))};
              const float u[4] = {f32_of_16<F16>((uint16_t)u01), f32_of_16<F16>((uint16_t)(u01 >> 16)),
                                  f32_of_16<F16>((uint16_t)u23), f32_of_16<F16>((uint16_t)(u23 >> 16))};
              float o[4];
#pragma unroll
              for (int rr = 0; rr < 4; ++rr) o[rr] = g[rr] / (1.f + __expf(-g[rr])) * u[rr];
              q[j][0] = pack_16x2<F16>(o[0], o[1]);
              q[j][1] = pack_16x2<F16>(o[2], o[3]);
            }
            if (p.vec_store == 2 && cols_valid == TILE_COLS) {
              // 16-byte stores: lanes l and l ^ 16 trade halves as in the plain epilogue below.
              const bool odd = eq & 1;
              const uint32_t r0 = (uint32_t)__builtin_amdgcn_ds_swizzle((int)(odd ? q[0][0] : q[1][0]), 0x401F);
              const uint32_t r1 = (uint32_t)__builtin_amdgcn_ds_swizzle((int)(odd ? q[0][1] : q[1][1]), 0x401F);
              u32x4_t o4;
              if (odd) o4 = u32x4_t{r0, r1, q[1][0], q[1][1]}; else o4 = u32x4_t{q[0][0], q[0][1], r0, r1};
              *(u32x4_t*)(yrow + wn * 32 + eq * 4 + (odd ? 16 - 4 : 0)) = o4;
            } else {
#pragma unroll
              for (int j = 0; j < 2; ++j) {
                const int n = wn * 32 + j * 16 + eq * 4;
                if (p.vec_store && n + 3 < cols_valid) {
                  *(u32x2_t*)(yrow + n) = q[j];
                } else {
#pragma unroll
                  for (int rr = 0; rr < 4; ++rr)
                    if (n + rr < cols_valid) {
                      const uint32_t w2 = q[j][rr >> 1];
                      ((uint16_t*)yrow)[n + rr] = (uint16_t)((rr & 1) ? (w2 >> 16) : (w2 & 0xFFFFu));
                    }
                }
              }
            }
          }
        }
      } else if (p.vec_store && cols_valid == BN && p.ldy < (1 << 24)) {
        const uint32_t voff = (uint32_t)er * (uint32_t)p.ldy + (uint32_t)(wn * FN * 16 + eq * 4);
        f32x4_t bs[FN];
        if (OP == OP_FP8_ROW) {
#pragma unroll
          for (int j = 0; j < FN; ++j) bs[j] = *(const f32x4_t*)(wcol_scale + (wn * FN + j) * 16 + eq * 4);
        }
#pragma unroll
        for (int i = 0; i < FM; ++i) {
          const int mrow = (i * WM + wm) * 16;
          bf16_t* ybase = yg + (int64_t)mrow * p.ldy;  // uniform
          if (mrow + er < rows_valid) {
            float am = 1.f;
            if (OP == OP_FP8_ROW) am = xrow_scale[mrow + er];
            if (p.vec_store == 2) {
            // Lanes l and l ^ 16 (column quarters 2q, 2q + 1 of the same row) trade halves so that each stores 16
            // bytes: the even one columns 8 q' .. + 7 of fragment j, the odd one those of fragment j + 1.
#pragma unroll
            for (int j = 0; j < FN; j += 2) {
              f32x4_t v0 = acc[j][i], v1 = acc[j + 1][i];
              if (OP == OP_FP8_ROW) { v0 = v0 * am * bs[j]; v1 = v1 * am * bs[j + 1]; }
              const uint32_t a0 = pack_16x2<F16>(v0[0], v0[1]), a1 = pack_16x2<F16>(v0[2], v0[3]);
              const uint32_t b0 = pack_16x2<F16>(v1[0], v1[1]), b1 = pack_16x2<F16>(v1[2], v1[3]);
              const bool odd = eq & 1;
              const uint32_t s0 = odd ? a0 : b0, s1 = odd ? a1 : b1;   // what the partner stores
              const uint32_t r0 = (uint32_t)__builtin_amdgcn_ds_swizzle((int)s0, 0x401F);  // lane ^ 16
              const uint32_t r1 = (uint32_t)__builtin_amdgcn_ds_swizzle((int)s1, 0x401F);
              u32x4_t o;
              if (odd) o = u32x4_t{r0, r1, b0, b1}; else o = u32x4_t{a0, a1, r0, r1};
              // even: fragment j, columns 16 j + 4 eq .. + 7; odd: fragment j + 1, columns 16 (j + 1) + 4 (eq - 1) ..
              *(u32x4_t*)(ybase + voff + (odd ? (j + 1) * 16 - 4 : j * 16)) = o;
            }
            } else {
#pragma unroll
            for (int j = 0; j < FN; ++j) {
              f32x4_t v = acc[j][i];
              if (OP == OP_FP8_ROW) v = v * am * bs[j];
              u32x2_t o;
              o[0] = pack_16x2<F16>(v[0], v[1]);
              o[1] = pack_16x2<F16>(v[2], v[3]);
              *(u32x2_t*)(ybase + voff + j * 16) = o;
            }
            }
          }
        }
      } else {
#pragma unroll
        for (int i = 0; i < FM; ++i) {
          const int m = (i * WM + wm) * 16 + er;
          if (m < rows_valid) {
            bf16_t* yrow = yg + (int64_t)m * p.ldy;
            float am = 1.f;
            if (OP == OP_FP8_ROW) am = xrow_scale[m];
#pragma unroll
            for (int j = 0; j < FN; ++j) {
              const int n = (wn * FN + j) * 16 + eq * 4;
              const f32x4_t v = acc[j][i];
#pragma unroll
              for (int rr = 0; rr < 4; ++rr)
                if (n + rr < cols_valid) {
                  float o = v[rr];
                  if (OP == OP_FP8_ROW) o = o * am * wcol_scale[n + rr];
                  ((uint16_t*)yrow)[n + rr] = cvt_16<F16>(o);
                }
            }
          }
        }
      }
    };
    if (nfm == FM) do_tile(std::false_type{});
    else do_tile(std::true_type{});
  }
  if (GRP == 0) __syncthreads();  // pairs with group 1's last barrier
  wait_vm<0>();                   // trailing (never read) slab loads must land before the LDS is released
}


// ---- Four waves, 128 x 128 outputs each ------------------------------------------------------------------------
// The same 256 x 256 tile, LDS stages, slab loads and tile order on a workgroup of four waves, one per SIMD. Wave
// (wm, wn) owns the activation fragments i = 0 .. 7 of tile rows (2 i + wm) * 16 .. + 15 and the weight fragments
// j = 0 .. 7 of tile columns (8 wn + j) * 16 .. + 15: 64 accumulators of four registers (all 256 accumulation
// registers), and per 32-wide half step 16 fragment reads feed 64 MFMAs where a wave of the eight-wave kernel reads
// 12 for 32: a third fewer LDS bytes per MFMA. A wave alone on its SIMD has nobody to fill the issue slots that an
// instruction block without MFMAs leaves empty, so the order is written out one MFMA at a time (an MFMA holds the
// matrix pipe for four issue slots: up to three other instructions fit behind it). Each half of a K step is two
// blocks of 32 MFMAs: first those of the activation fragments 0 .. 3, which carry the other instructions, then those
// of fragments 4 .. 7, which one uniform branch skips for a tile of at most 128 rows (low tiles, row pieces). First
// half: the 16 reads of the second half's fragments follow every second MFMA of the first block; then the wave
// waits for its reads and for its loads of the next slab, and the workgroup's one barrier per K step publishes that
// slab and frees the buffer of the present one. Second half: behind the MFMAs of the first block alternate the 16
// loads of the slab after next (into that buffer, more than a K step ahead of the wait that covers them) and the 16
// reads of the next step's first half. A scheduling barrier after every such pair keeps the compiler from
// collecting reads or loads into blocks. The slab stream runs through tile boundaries (the loads
// and the reads for a tile's first step are issued in the last step of the tile before, and land during its
// epilogue); behind the last tile the loads are still issued, with every lane's offset zero (one line per
// instruction) into a buffer nobody reads again: one loop body, no branch around a load.
constexpr int W4_NW = 4, W4_NT = 64 * W4_NW, W4_FM = 8, W4_FN = 8;

// TALL: tiles of up to BM + MOE_GG_TALL_ROWS rows (moe_gg_tall_tail: the few rows behind a group's last full row tile
// ride along with that tile instead of streaming the weight tile a second time as a low tile). A wave then has a ninth
// activation fragment, tile rows 256 + 16 wm .. + 15: its slab rows live in a 4 KB area per stage behind the two
// stages (one more load instruction per wave and slab, issued only for tall tiles), its fragment reads are issued for
// every tile (they cost two reads per K step and spare the loop a second condition), and its eight MFMAs per half step
// form a third block that one uniform branch skips for tiles of at most 256 rows.
template <int OP, bool TALL = false>
DEVINL void run_fourwave(const GgParams& p, const Shared& sh) {
  static_assert(OP == OP_BF16 || OP == OP_F16 || OP == OP_BF16_SWIGLU || OP == OP_F16_SWIGLU,
                "forward product on 16-bit floats, plain or with SiLU-and-mul in the epilogue");
  constexpr bool F16 = op_f16(OP);
  constexpr bool SWIGLU = op_swiglu(OP);
  constexpr int FMW = W4_FM, FNW = W4_FN;
  constexpr int FMA = FMW + (TALL ? 1 : 0);  // activation fragments a wave holds accumulators for
  constexpr int TILE_COLS = SWIGLU ? BN / 2 : BN;  // output columns of a tile
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;
  const int N = p.N;
  const int NCOLS = SWIGLU ? N / 2 : N;      // output columns of a group
  const uint32_t KROW = (uint32_t)p.K * 2u;  // bytes per operand row
  const int KT = (int)(KROW / 128u);         // K steps of every tile

  struct Tile { int g, row0, m0, h, n0, nc; };
  auto tile_at = [&](int seq) {
    // As decoded in the prologue: group | rows << 16 | columns / 32 << 26, first row / 64 | first column / 32 << 16.
    const int gh = uni(sh.seq_tab[2 * seq]), mn = uni(sh.seq_tab[2 * seq + 1]);
    Tile t;
    t.g = gh & 0xFFFF;
    t.h = (gh >> 16) & 0x3FF;
    t.nc = (int)((uint32_t)gh >> 26) * 32;
    t.m0 = (mn & 0xFFFF) * 64;
    t.n0 = (int)((uint32_t)mn >> 16) * 32;
    t.row0 = uni(sh.row_off[t.g]);
    return t;
  };

  // Slab loads: an instruction fills 8 rows (1 KB of LDS): lane -> row lane / 8, physical 16-byte slot lane % 8, which
  // must hold logical chunk slot ^ ((row >> 1) & 7). Instruction r of wave w fills the 8-row block 4 r + w.
  const int d_r = lane >> 3;
  const uint32_t d_c16 = (uint32_t)(((lane & 7) ^ (((wave & 1) << 2) | (lane >> 4))) << 4);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)sh.lds;
  // Fragment reads: row = fragment * 16 + lane % 16, chunk = half * 4 + lane / 16 (swizzled).
  const int fr = lane & 15, fq = lane >> 4;
  const int rd0 = fr * 128 + ((fq ^ (fr >> 1)) << 4);  // first half; the second is rd0 ^ 64

  const char* xp = (const char*)p.x;
  const char* wp = (const char*)p.w;
  bf16_t* __restrict__ yp = (bf16_t*)p.y;

  // Load cursor: the slab (tile of the sequence, K step) that the next 16 load instructions of this wave fetch.
  const char* c_xg = xp;
  const char* c_wg = wp;
  uint32_t c_xoff[8], c_woff[8];
  uint32_t c_xoff_tall = 0;  // TALL: the wave's 8 rows of tile rows 256 .. 287
  bool c_tall = false;       // TALL: the cursor's tile has such rows
  uint32_t c_keep = ~0u;  // zero behind the last tile
  int c_seq = 0, c_kt = 0;
  auto cursor_tile = [&](int seq) {
    c_seq = seq;
    c_kt = 0;
    if (seq >= sh.n_my) {  // behind the last tile: the pointers stay at the last tile's (in bounds), offsets zero
      c_keep = 0u;
      c_tall = false;
      return;
    }
    const Tile t = tile_at(seq);
    // w_last: last valid weight row of the tile; SWIGLU: last valid output column (a gate row and an up row each)
    const int x_last = max(t.h, 1) - 1, w_last = max(min(NCOLS - t.n0, t.nc), 1) - 1;
    if constexpr (TALL) {
      c_tall = t.h > BM;
      c_xoff_tall = (uint32_t)min(BM + wave * 8 + d_r, x_last) * KROW + d_c16;
    }
    c_xg = uni_ptr(xp + (int64_t)(t.row0 + t.m0) * KROW);
    c_wg = uni_ptr(wp + ((int64_t)t.g * N + t.n0) * KROW);
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      // rows beyond the tile's last one re-read it (the loads stay inside the tensors)
      const int b = r * W4_NW + wave;  // 8-row block of the slab
      c_xoff[r] = (uint32_t)min(b * 8 + d_r, x_last) * KROW + d_c16;
      // SWIGLU: LDS weight row 128 wn + 64 h + c (h = 0 gate, 1 up) holds output column 64 wn + c of the tile, so that
      // a wave has the gate and the up value of its own 64 columns: block b -> wn = b >> 4, h = (b >> 3) & 1.
      const uint32_t wrow = SWIGLU ? (uint32_t)min((b >> 4) * 64 + (b & 7) * 8 + d_r, w_last) + (((b >> 3) & 1) ? (uint32_t)NCOLS : 0u)
                                   : (uint32_t)min(b * 8 + d_r, w_last);
      c_woff[r] = wrow * KROW + d_c16;
    }
  };
  auto cursor_next = [&]() {
    if (c_keep != 0u && ++c_kt == KT) cursor_tile(c_seq + 1);
  };
  auto load_one = [&](int r, int buf) {  // load r of the cursor slab's 16 (activation rows first) into stage buf
    const uint32_t lb = lds_base + buf * STAGE + wave * 1024;
    if (r < 8) dma16(c_xg + c_kt * 128, c_xoff[r] & c_keep, lb + r * W4_NW * 1024);
    else dma16(c_wg + c_kt * 128, c_woff[r - 8] & c_keep, lb + X_BYTES + (r - 8) * W4_NW * 1024);
  };
  // TALL: the seventeenth load of a slab, rows 256 + 8 wave .. + 7 into the stage's extra area (tall tiles only)
  auto load_tall = [&](int buf) {
    if (c_tall) dma16(c_xg + c_kt * 128, c_xoff_tall, lds_base + 2 * STAGE + buf * TALL_BYTES + wave * 1024);
  };

  bf16x8_t wf0[FNW], xf0[FMA], wf1[FNW], xf1[FMA];
  auto read_one = [&](int buf, int half, int r, bf16x8_t (&wf)[FNW], bf16x8_t (&xf)[FMA]) {
    // read r of a half step's 16: the activation fragments first (the first eight MFMAs use all of them)
    const char* st = sh.lds + buf * STAGE;
    const int ro = half ? (rd0 ^ 64) : rd0;
    if (r < FMW) xf[r] = *(const bf16x8_t*)(st + (r * 2 + wm) * 2048 + ro);
    else wf[r - FMW] = *(const bf16x8_t*)(st + X_BYTES + (wn * FNW + r - FMW) * 2048 + ro);
  };
  // TALL: fragment 8 (tile rows 256 + 16 wm .. + 15) of a half step, from the stage's extra area
  auto read_tall = [&](int buf, int half, bf16x8_t (&xf)[FMA]) {
    xf[FMA - 1] = *(const bf16x8_t*)(sh.lds + 2 * STAGE + buf * TALL_BYTES + wm * 2048 + (half ? (rd0 ^ 64) : rd0));
  };

  f32x4_t acc[FNW][FMA];
  // TALL: the ninth fragment's 32 accumulation registers do not fit the AGPRs, which the other 256 fill, and the
  // compiler selects one form of MFMA for the whole function (AGPR accumulators: it would copy these 32 registers into
  // spare AGPRs and back around every MFMA). So their MFMAs are written out with VGPR accumulators. The compiler does
  // not know the instruction, i.e. it tracks the operands (it waits for the LDS reads behind a and b) but inserts none
  // of the wait states an MFMA result needs before another kind of instruction reads it: a dependent MFMA on the same
  // accumulator follows 72 MFMAs later at the earliest (no wait needed), and the epilogue's first read is kept 32
  // issue slots away by the s_nops behind the K loop.
  auto mfma_vgpr = [&](const bf16x8_t& a, const bf16x8_t& b, f32x4_t& c) {
    if constexpr (F16) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    else asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  };

  // Stream start: slabs 0 and 1 in flight, first fragments read.
  cursor_tile(0);
#pragma unroll
  for (int r = 0; r < 16; ++r) load_one(r, 0);
  if constexpr (TALL) load_tall(0);
  cursor_next();
#pragma unroll
  for (int r = 0; r < 16; ++r) load_one(r, 1);
  if constexpr (TALL) load_tall(1);
  cursor_next();
  wait_vm<16>();  // slab 0 (loads return in order; TALL: 16 or 17 are behind it, so at least slab 0 has landed)
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 16; ++r) read_one(0, 0, r, wf0, xf0);
  if constexpr (TALL) read_tall(0, 0, xf0);

  int step = 0;  // K steps done, over all tiles: slab `step` sits in stage step & 1
  for (int seq = 0; seq < sh.n_my; ++seq) {
    // The lanes of a wave leave the epilogue's row-masked store blocks at different points and are together again
    // here (no instruction; it also keeps the compiler from moving memory operations across the tile boundary).
    __builtin_amdgcn_wave_barrier();
    const Tile t = tile_at(seq);
#pragma unroll
    for (int j = 0; j < FNW; ++j)
#pragma unroll
      for (int i = 0; i < FMA; ++i) acc[j][i] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // Activation fragments of this wave that hold rows of the tile: i with (2 i + wm) * 16 < t.h. A tile of at most
    // 128 rows (low tile, row piece) has none beyond i = 3: the MFMAs of fragments 4 .. 7 form a block of their own
    // in each half step, behind the block that carries the reads and loads, and one uniform branch skips it.
    const bool upper = (moe_gg_cdiv(t.h, 16) - wm + 1) / 2 > 4;
    const bool tall = TALL && t.h > BM;  // the ninth fragment has rows (for wm = 1: if more than 16)
    for (int kt = 0; kt < KT; ++kt, ++step) {
      const int cur = step & 1;
      // First half: MFMAs on (wf0, xf0); (wf1, xf1) <- second half of the slab, one read behind every second MFMA of
      // the first block.
#pragma unroll
      for (int u = 0; u < 32; ++u) {
        const int j = u >> 2, i = u & 3;
        acc[j][i] = mfma_16x16x32<F16>(__builtin_bit_cast(u32x4_t, wf0[j]), __builtin_bit_cast(u32x4_t, xf0[i]), acc[j][i]);
        if ((u & 1) == 0) read_one(cur, 1, u >> 1, wf1, xf1);
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (TALL) {
        read_tall(cur, 1, xf1);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (upper) {
#pragma unroll
        for (int u = 0; u < 32; ++u) {
          const int j = u >> 2, i = 4 + (u & 3);
          acc[j][i] = mfma_16x16x32<F16>(__builtin_bit_cast(u32x4_t, wf0[j]), __builtin_bit_cast(u32x4_t, xf0[i]), acc[j][i]);
        }
      }
      if constexpr (TALL) {
        __builtin_amdgcn_sched_barrier(0);
        if (tall) {
#pragma unroll
          for (int j = 0; j < FNW; ++j) mfma_vgpr(wf0[j], xf0[FMA - 1], acc[j][FMA - 1]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      wait_lgkm0();   // this wave has read all it needs of the slab
      wait_vm<0>();   // its share of the next slab has landed
      __syncthreads();
      // Second half: MFMAs on (wf1, xf1); behind the MFMAs of the first block, alternately, one of the 16 loads of the
      // slab after next (into the stage that is free now; more than a K step ahead of the wait that covers them) and
      // one of the 16 reads (wf0, xf0) <- first half of the next slab.
#pragma unroll
      for (int u = 0; u < 32; ++u) {
        const int j = u >> 2, i = u & 3;
        acc[j][i] = mfma_16x16x32<F16>(__builtin_bit_cast(u32x4_t, wf1[j]), __builtin_bit_cast(u32x4_t, xf1[i]), acc[j][i]);
        __builtin_amdgcn_sched_barrier(0);           // the MFMA first, then what rides in its shadow
        if ((u & 1) == 0) load_one(u >> 1, cur);   // five instructions with its offset mask and M0 write
        else read_one(cur ^ 1, 0, u >> 1, wf0, xf0);   // one: three per MFMA on average, the slots an MFMA leaves
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (TALL) {
        load_tall(cur);
        read_tall(cur ^ 1, 0, xf0);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (upper) {
#pragma unroll
        for (int u = 0; u < 32; ++u) {
          const int j = u >> 2, i = 4 + (u & 3);
          acc[j][i] = mfma_16x16x32<F16>(__builtin_bit_cast(u32x4_t, wf1[j]), __builtin_bit_cast(u32x4_t, xf1[i]), acc[j][i]);
        }
      }
      if constexpr (TALL) {
        __builtin_amdgcn_sched_barrier(0);
        if (tall) {
#pragma unroll
          for (int j = 0; j < FNW; ++j) mfma_vgpr(wf1[j], xf1[FMA - 1], acc[j][FMA - 1]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      cursor_next();
    }
    if constexpr (TALL) {
      // The results of the last hand-written MFMAs must not be read before they are written (see mfma_vgpr). The
      // accumulators are operands of the statement, so that no instruction that reads one can be moved in front of it.
      if (tall)
        asm volatile("s_nop 15\n\ts_nop 15"
                     : "+v"(acc[0][FMA - 1]), "+v"(acc[1][FMA - 1]), "+v"(acc[2][FMA - 1]), "+v"(acc[3][FMA - 1]),
                       "+v"(acc[4][FMA - 1]), "+v"(acc[5][FMA - 1]), "+v"(acc[6][FMA - 1]), "+v"(acc[7][FMA - 1]));
    }

    // Epilogue: lane holds y[m][n .. n + 3] for m = (2 i + wm) * 16 + lane % 16, n = (8 wn + j) * 16 + 4 (lane / 16).
    const int rows_valid = t.h, cols_valid = min(NCOLS - t.n0, t.nc);
    bf16_t* yg = yp + (int64_t)(t.row0 + t.m0) * p.ldy + (int64_t)t.g * p.col_block + t.n0;
    if constexpr (SWIGLU) {
      // acc[j][i], j = 0 .. 3: gate of output columns 64 wn + 16 j + 4 fq .. + 3; acc[j + 4][i]: up of the same columns.
#pragma unroll
      for (int i = 0; i < FMA; ++i) {
        const int m = (i * 2 + wm) * 16 + fr;
        if (m < rows_valid) {
          bf16_t* yrow = yg + (int64_t)m * p.ldy;
          u32x2_t q[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const f32x4_t gv = acc[j][i], uv = acc[j + 4][i];
            // both products rounded to the 16-bit type first, as they are when the GEMM output is stored
            const uint32_t g01 = pack_16x2<F16>(gv[0], gv[1]), g23 = pack_16x2<F16>(gv[2], gv[3]);
            const uint32_t u01 = pack_16x2<F16>(uv[0], uv[1]), u23 = pack_16x2<F16>(uv[2], uv[3]);
            const float g[4] = {f32_of_16<F16>((uint16_t)g01), f32_of_16<F16>((uint16_t)(g01 >> 16)),
                                f32_of_16<F16>((uint16_t)g23), f32_of_16<F16>((uint16_t)(g23 >> 16))};
            const float u[4] = {f32_of_16<F16>((uint16_t)u01), f32_of_16<F16>((uint16_t)(u01 >> 16)),
                                f32_of_16<F16>((uint16_t)u23), f32_of_16<F16>((uint16_t)(u23 >> 16))};
            float o[4];
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) o[rr] = g[rr] / (1.f + __expf(-g[rr])) * u[rr];
            q[j][0] = pack_16x2<F16>(o[0], o[1]);
            q[j][1] = pack_16x2<F16>(o[2], o[3]);
          }
          if (p.vec_store == 2 && cols_valid == TILE_COLS) {
            // 16-byte stores: lanes l and l ^ 16 trade halves as in the plain epilogue below.
            const bool odd = fq & 1;
#pragma unroll
            for (int j = 0; j < 4; j += 2) {
              const uint32_t r0 = (uint32_t)__builtin_amdgcn_ds_swizzle((int)(odd ? q[j][0] : q[j + 1][0]), 0x401F);
              const uint32_t r1 = (uint32_t)__builtin_amdgcn_ds_swizzle((int)(odd ? q[j][1] : q[j + 1][1]), 0x401F);
              u32x4_t o4;
              if (odd) o4 = u32x4_t{r0, r1, q[j + 1][0], q[j + 1][1]}; else o4 = u32x4_t{q[j][0], q[j][1], r0, r1};
              *(u32x4_t*)(yrow + wn * 64 + j * 16 + fq * 4 + (odd ? 16 - 4 : 0)) = o4;
            }
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int n = wn * 64 + j * 16 + fq * 4;
              if (p.vec_store && n + 3 < cols_valid) {
                *(u32x2_t*)(yrow + n) = q[j];
              } else {
#pragma unroll
                for (int rr = 0; rr < 4; ++rr)
                  if (n + rr < cols_valid) {
                    const uint32_t w2 = q[j][rr >> 1];
                    ((uint16_t*)yrow)[n + rr] = (uint16_t)((rr & 1) ? (w2 >> 16) : (w2 & 0xFFFFu));
                  }
              }
            }
          }
        }
      }
    } else if (p.vec_store && cols_valid == BN && p.ldy < (1 << 24)) {
      const uint32_t voff = (uint32_t)fr * (uint32_t)p.ldy + (uint32_t)(wn * FNW * 16 + fq * 4);
#pragma unroll
      for (int i = 0; i < FMA; ++i) {
        const int mrow = (i * 2 + wm) * 16;
        bf16_t* ybase = yg + (int64_t)mrow * p.ldy;  // uniform
        if (mrow + fr < rows_valid) {
          if (p.vec_store == 2) {
            // Lanes l and l ^ 16 (column quarters 2 q, 2 q + 1 of the same row) trade halves so that each stores 16
            // bytes: the even one columns 8 q' .. + 7 of fragment j, the odd one those of fragment j + 1.
#pragma unroll
            for (int j = 0; j < FNW; j += 2) {
              const f32x4_t v0 = acc[j][i], v1 = acc[j + 1][i];
              const uint32_t a0 = pack_16x2<F16>(v0[0], v0[1]), a1 = pack_16x2<F16>(v0[2], v0[3]);
              const uint32_t b0 = pack_16x2<F16>(v1[0], v1[1]), b1 = pack_16x2<F16>(v1[2], v1[3]);
              const bool odd = fq & 1;
              const uint32_t s0 = odd ? a0 : b0, s1 = odd ? a1 : b1;   // what the partner stores
              const uint32_t r0 = (uint32_t)__builtin_amdgcn_ds_swizzle((int)s0, 0x401F);  // lane ^ 16
              const uint32_t r1 = (uint32_t)__builtin_amdgcn_ds_swizzle((int)s1, 0x401F);
              u32x4_t o;
              if (odd) o = u32x4_t{r0, r1, b0, b1}; else o = u32x4_t{a0, a1, r0, r1};
              *(u32x4_t*)(ybase + voff + (odd ? (j + 1) * 16 - 4 : j * 16)) = o;
            }
          } else {
#pragma unroll
            for (int j = 0; j < FNW; ++j) {
              const f32x4_t v = acc[j][i];
              u32x2_t o;
              o[0] = pack_16x2<F16>(v[0], v[1]);
              o[1] = pack_16x2<F16>(v[2], v[3]);
              *(u32x2_t*)(ybase + voff + j * 16) = o;
            }
          }
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < FMA; ++i) {
        const int m = (i * 2 + wm) * 16 + fr;
        if (m < rows_valid) {
          bf16_t* yrow = yg + (int64_t)m * p.ldy;
#pragma unroll
          for (int j = 0; j < FNW; ++j) {
            const int n = (wn * FNW + j) * 16 + fq * 4;
            const f32x4_t v = acc[j][i];
#pragma unroll
            for (int rr = 0; rr < 4; ++rr)
              if (n + rr < cols_valid) ((uint16_t*)yrow)[n + rr] = cvt_16<F16>(v[rr]);
          }
        }
      }
    }
  }
  wait_vm<0>();  // the trailing (never read) slab loads must land before the LDS is released
}

// FOURWAVE: the workgroup is four waves running run_fourwave (one wave per SIMD, 128 x 128 outputs each) instead of the
// two groups of four above; tables, tile order and LDS stages are the same.
template <int OP, bool FOURWAVE = false, bool TALL = false, bool LISTS2 = FOURWAVE || op_gather(OP)>
DEVINL void pingpong_body(const GgParams& p) {
  static_assert(!TALL || FOURWAVE, "tall tiles are the four-wave kernel's");
  static_assert(LISTS2 || (!FOURWAVE && !TALL && !op_gather(OP)), "the first prologue knows the eight-wave kernels without a row gather");
  constexpr int NTB = FOURWAVE ? W4_NT : NT;  // threads of the workgroup
  __shared__ __attribute__((aligned(1024))) char lds[2 * STAGE + (OP == OP_FP8_BLOCK ? 2 * SCALE_BYTES : 0) + (TALL ? 2 * TALL_BYTES : 0)];
  __shared__ int32_t row_off[MOE_GG_MAX_GROUPS + 1];
  __shared__ int32_t tile_off[MOE_GG_MAX_GROUPS + 1];
  __shared__ int32_t part_off[MOE_GG_MAX_GROUPS + 1];
  __shared__ int32_t seq_tab[2 * MOE_GG_SEQ_CAP];
  static_assert(2 * MOE_GG_SEQ_CAP >= MOE_GG_MAX_GROUPS + 1, "seq_tab doubles as a prefix table below");

  int n_my = 0;
  if constexpr (!LISTS2) {
    // The lists, sequence and tile decode of the kernels that run by default, kept word for word as they last ran on a
    // GPU (the two-list order; row pieces of the last round by its fill alone).
    int total, total_low = 0;
    if (OP == OP_BF16_WGRAD_DIRECT) {
      build_row_offsets(p.m_sizes, p.G, p.M, row_off);
      total = p.G * moe_gg_cdiv(p.N, BM) * moe_gg_cdiv(p.K, BN);
    } else if (OP == OP_BF16_WGRAD) {
      // tile_off counts the 64-column blocks of the padded operands (at least one per expert).
      build_group_tables(p.m_sizes, p.G, p.skip_rows, 64, 1, row_off, tile_off, 0, 1);
      total = p.G * moe_gg_cdiv(p.N, BM) * moe_gg_cdiv(p.K, BN);
    } else {
      const int ntn = op_swiglu(OP) ? moe_gg_cdiv(p.N / 2, BN / 2) : moe_gg_cdiv(p.N, BN);
      const int skip = p.skip_rows;
      build_row_offsets(p.m_sizes, p.G, p.M, row_off);
      build_tile_prefix(row_off, p.G, tile_off, [&](int rows) { return rows > skip ? moe_gg_long_row_tiles(rows, BM) * ntn : 0; });
      build_tile_prefix(row_off, p.G, part_off, [&](int rows) { return rows > skip ? moe_gg_low_row_tiles(rows, BM) * ntn : 0; });
      total_low = uni(part_off[p.G]);
      total = uni(tile_off[p.G]);
      if ((OP == OP_BF16 || OP == OP_F16) && p.tails_apart) {
        // Few low tiles that would open a round of their own are computed by the small-M kernel of the same call.
        build_tile_prefix(row_off, p.G, seq_tab, [&](int rows) { return moe_gg_low_passes(rows, BM) * ntn; });
        if (moe_gg_tails_apart(total, total_low, uni(seq_tab[p.G]), p.tails_apart)) total_low = 0;
        __syncthreads();  // seq_tab is rewritten below
      }
    }
    const int nwg = gridDim.x;
    // Tiles of this workgroup in each list: rounds 0 .. n - 1 (tile ids grow with the round).
    // (Forward kernels: the long tiles of a sparsely filled last round are cut into row pieces, moe_gg_tail_pieces.)
    const bool fwd = OP != OP_BF16_WGRAD && OP != OP_BF16_WGRAD_DIRECT;
    const int tail_s = fwd ? moe_gg_tail_pieces(total, nwg) : 1;
    const int tail_first = fwd ? moe_gg_tail_first(total, nwg) : total;
    const int long_ids = fwd ? moe_gg_long_ids(total, nwg) : total;
    const int low_ids = total_low;
    int n_long = 0, n_low = 0;
    while (n_long * nwg < long_ids && moe_gg_tile_of(blockIdx.x, nwg, p.xcds, n_long) < long_ids) ++n_long;
    while ((n_long + n_low) * nwg < long_ids + low_ids && moe_gg_tile_of(blockIdx.x, nwg, p.xcds, n_long + n_low) < long_ids + low_ids)
      ++n_low;
    if (n_long + n_low == 0) return;
    // The sequence of this workgroup (moe_gg_seq_round), decoded once into a table: the arithmetic runs per thread
    // here; in the K loop it would occupy scalar registers that the loop needs.
    // Tile ids: the long tiles of all groups (group, then column tile, then row tile), then the low tiles (group,
    // column tile; see moe_gg_long_row_tiles), dealt to the workgroups round-robin: every workgroup gets the same
    // number (+- 1) of long tiles, and the low tiles go on where the long ones stopped.
    n_my = min(n_long + n_low, MOE_GG_SEQ_CAP);
    const int phase = moe_gg_low_phase(blockIdx.x, p.xcds);
    for (int i = threadIdx.x; i < n_my; i += NT) {
      int L = moe_gg_tile_of(blockIdx.x, nwg, p.xcds, moe_gg_seq_round(i, n_long + n_low, n_low, phase));
      constexpr int TC = op_swiglu(OP) ? BN / 2 : BN;  // output columns of a tile
      int g, m0, h, n0, nc = TC;  // group, first row inside the group, rows, first column, columns
      if (OP == OP_BF16_WGRAD || OP == OP_BF16_WGRAD_DIRECT) {
        // Tiles of an expert in bands of four column tiles, column tile fastest inside a band: the 32 tiles an XCD
        // works on at a time are 8 row tiles x 4 column tiles, which share 8 + 4 operand slabs per K step (with the
        // row tile fastest they were 32 + 1: 3 % slower at the Mixtral shape, the reads from the fabric bound it).
        const int ntm = moe_gg_cdiv(p.N, BM), ntn = moe_gg_cdiv(p.K, BN), tpg = ntm * ntn;
        g = L / tpg;
        const int rem = L - g * tpg;
        const int band = rem / (4 * ntm), idx = rem - band * (4 * ntm);
        const int wb = min(4, ntn - band * 4);  // column tiles of this band
        const int tm = idx / wb;
        n0 = (band * 4 + idx - tm * wb) * BN;
        m0 = tm * BM;
        h = min(p.N - m0, BM);
      } else if (L < long_ids) {
        int piece = 0;
        if (L >= tail_first) {  // a piece of a tile of the last round
          piece = (L - tail_first) % tail_s;
          L = tail_first + (L - tail_first) / tail_s;
        }
        g = moe_gg_find_group(tile_off, p.G, L);
        const int idx = L - tile_off[g];
        const int rows = row_off[g + 1] - row_off[g];
        const int nf = moe_gg_long_row_tiles(rows, BM);
        const int tn = idx / nf;
        n0 = tn * TC;
        m0 = (idx - tn * nf) * BM;
        h = min(rows - m0, BM);
        if (tail_s > 1 && L >= tail_first) {
          int off;
          moe_gg_piece_rows(h, tail_s, piece, &off, &h);
          if (h > 0) m0 += off;  // a piece without rows keeps the tile's first row: its loads must stay in bounds
        }
      } else {
        // Low tiles. (Cutting few low tiles into column pieces for more workgroups was measured: no gain, a low
        // tile is bound by the per-step cost of the K loop, not by the bytes it streams.)
        const int Lp = L - long_ids;
        g = moe_gg_find_group(part_off, p.G, Lp);
        const int tn = Lp - part_off[g];
        n0 = tn * TC;
        const int rows = row_off[g + 1] - row_off[g];
        m0 = rows / BM * BM;
        h = rows - m0;
      }
      seq_tab[2 * i] = g | (h << 16) | ((nc / 32) << 26);
      seq_tab[2 * i + 1] = (m0 / 64) | ((n0 / 32) << 16);
    }
  } else {
    // The same with the selectable orders: split tails (p.split_tails), tall tiles (TALL); one decode function shared
    // with the host mirror. Also the prologue of the kernels that came with it (four waves, row gather).
    int total, total_low = 0;
    // Forward lists with p.split_tails: tall groups with a few rows beyond their last full tile get two half tiles for
    // their last rows (moe_gg_split_tail), unless the small-M kernel of the same call takes the low tiles.
    bool split = p.split_tails != 0;
    bool apart = false;  // the low tiles are the small-M kernel's
    if (OP == OP_BF16_WGRAD_DIRECT) {
      build_row_offsets(p.m_sizes, p.G, p.M, row_off);
      total = p.G * moe_gg_cdiv(p.N, BM) * moe_gg_cdiv(p.K, BN);
    } else if (OP == OP_BF16_WGRAD) {
      // tile_off counts the 64-column blocks of the padded operands (at least one per expert).
      build_group_tables(p.m_sizes, p.G, p.skip_rows, 64, 1, row_off, tile_off, 0, 1);
      total = p.G * moe_gg_cdiv(p.N, BM) * moe_gg_cdiv(p.K, BN);
    } else {
      const int ntn = op_swiglu(OP) ? moe_gg_cdiv(p.N / 2, BN / 2) : moe_gg_cdiv(p.N, BN);
      const int skip = p.skip_rows;
      build_row_offsets(p.m_sizes, p.G, p.M, row_off);
      if ((OP == OP_BF16 || OP == OP_F16) && p.tails_apart) {
        // Few low tiles that would open a round of their own are computed by the small-M kernel of the same call,
        // which takes the same decision from the same counts (the lists without split tails).
        build_tile_prefix(row_off, p.G, tile_off, [&](int rows) { return rows > skip ? moe_gg_long_row_tiles(rows, BM) * ntn : 0; });
        build_tile_prefix(row_off, p.G, part_off, [&](int rows) { return rows > skip ? moe_gg_low_row_tiles(rows, BM) * ntn : 0; });
        build_tile_prefix(row_off, p.G, seq_tab, [&](int rows) { return moe_gg_low_passes(rows, BM) * ntn; });
        apart = moe_gg_tails_apart(uni(tile_off[p.G]), uni(part_off[p.G]), uni(seq_tab[p.G]), p.tails_apart);
        if (apart) split = false;
        __syncthreads();  // the tables are rewritten below
      }
      if constexpr (TALL) {
        split = false;  // the lists of moe_gg_tall_tail
        build_tile_prefix(row_off, p.G, tile_off, [&](int rows) { return rows > skip ? moe_gg_long_row_tiles_tall(rows, BM) * ntn : 0; });
        build_tile_prefix(row_off, p.G, part_off, [&](int rows) { return rows > skip ? moe_gg_low_row_tiles_tall(rows, BM) * ntn : 0; });
      } else {
      build_tile_prefix(row_off, p.G, tile_off, [&](int rows) { return rows > skip ? moe_gg_long_row_tiles2(rows, BM, split) * ntn : 0; });
      build_tile_prefix(row_off, p.G, part_off, [&](int rows) { return rows > skip ? moe_gg_low_row_tiles2(rows, BM, split) * ntn : 0; });
      }
      total_low = apart ? 0 : uni(part_off[p.G]);
      total = uni(tile_off[p.G]);
    }
    const int nwg = gridDim.x;
    // Tiles of this workgroup in each list: rounds 0 .. n - 1 (tile ids grow with the round).
    // (Forward kernels: the long tiles of a sparsely filled last round are cut into row pieces: by the fill of that
    // round alone (moe_gg_tail_pieces), or, with p.split_tails, as many as make the busiest workgroup's load smallest
    // with the second list dealt behind them, moe_gg_tail_pieces_low.)
    const bool fwd = OP != OP_BF16_WGRAD && OP != OP_BF16_WGRAD_DIRECT;
    const int tail_s = !fwd ? 1 : (p.split_tails && !TALL) ? moe_gg_tail_pieces_low(total, total_low, nwg) : moe_gg_tail_pieces(total, nwg);
    const int tail_first = moe_gg_tail_first_s(total, nwg, tail_s);
    const int long_ids = moe_gg_long_ids_s(total, nwg, tail_s);
    const int low_ids = total_low;
    int n_long = 0, n_low = 0;
    while (n_long * nwg < long_ids && moe_gg_tile_of(blockIdx.x, nwg, p.xcds, n_long) < long_ids) ++n_long;
    while ((n_long + n_low) * nwg < long_ids + low_ids && moe_gg_tile_of(blockIdx.x, nwg, p.xcds, n_long + n_low) < long_ids + low_ids)
      ++n_low;
    if (n_long + n_low == 0) return;
    // The sequence of this workgroup (moe_gg_seq_round), decoded once into a table: the arithmetic runs per thread
    // here; in the K loop it would occupy scalar registers that the loop needs.
    // Tile ids: the long tiles of all groups (group, then column tile, then row tile), then the second list (group,
    // column tile, then the group's low tile or its two half tiles; see moe_gg_long_row_tiles, moe_gg_split_tail),
    // dealt to the workgroups round-robin: every workgroup gets the same number (+- 1) of long tiles, and the second
    // list goes on where the long ones stopped.
    n_my = min(n_long + n_low, MOE_GG_SEQ_CAP);
    const int phase = moe_gg_low_phase(blockIdx.x, p.xcds);
    for (int i = threadIdx.x; i < n_my; i += NTB) {
      int L = moe_gg_tile_of(blockIdx.x, nwg, p.xcds, moe_gg_seq_round(i, n_long + n_low, n_low, phase));
      constexpr int TC = op_swiglu(OP) ? BN / 2 : BN;  // output columns of a tile
      int g, m0, h, n0, nc = TC;  // group, first row inside the group, rows, first column, columns
      if (OP == OP_BF16_WGRAD || OP == OP_BF16_WGRAD_DIRECT) {
        // Tiles of an expert in bands of four column tiles, column tile fastest inside a band: the 32 tiles an XCD
        // works on at a time are 8 row tiles x 4 column tiles, which share 8 + 4 operand slabs per K step (with the
        // row tile fastest they were 32 + 1: 3 % slower at the Mixtral shape, the reads from the fabric bound it).
        const int ntm = moe_gg_cdiv(p.N, BM), ntn = moe_gg_cdiv(p.K, BN), tpg = ntm * ntn;
        g = L / tpg;
        const int rem = L - g * tpg;
        const int band = rem / (4 * ntm), idx = rem - band * (4 * ntm);
        const int wb = min(4, ntn - band * 4);  // column tiles of this band
        const int tm = idx / wb;
        n0 = (band * 4 + idx - tm * wb) * BN;
        m0 = tm * BM;
        h = min(p.N - m0, BM);
      } else {
        // Long tiles (the last round cut into row pieces when it is sparsely filled), then the second list.
        // (Cutting few low tiles into column pieces for more workgroups was measured: no gain, a low tile is bound
        // by the per-step cost of the K loop, not by the bytes it streams.)
        MoeGgListTile lt;
        if constexpr (TALL) lt = moe_gg_two_list_decode_tall(row_off, tile_off, part_off, p.G, L, long_ids, tail_first, tail_s, BM, TC);
        else lt = moe_gg_two_list_decode(row_off, tile_off, part_off, p.G, L, long_ids, tail_first, tail_s, BM, TC, split);
        g = lt.g; m0 = lt.m0; h = lt.h; n0 = lt.n0;
      }
      seq_tab[2 * i] = g | (h << 16) | ((nc / 32) << 26);
      seq_tab[2 * i + 1] = (m0 / 64) | ((n0 / 32) << 16);
    }
  }
  __syncthreads();

  Shared sh{row_off, tile_off, part_off, seq_tab, lds, n_my};
  if constexpr (FOURWAVE) {
    run_fourwave<OP, TALL>(p, sh);
  } else {
    const int grp = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 8));
    if (grp == 0) run_group<0, OP>(p, sh);
    else run_group<1, OP>(p, sh);
  }
}

__global__ __launch_bounds__(NT) void gg_bf16_pingpong(GgParams p) { pingpong_body<OP_BF16>(p); }
__global__ __launch_bounds__(NT) void gg_f16_pingpong(GgParams p) { pingpong_body<OP_F16>(p); }
__global__ __launch_bounds__(W4_NT) void gg_bf16_fourwave(GgParams p) { pingpong_body<OP_BF16, true>(p); }
__global__ __launch_bounds__(W4_NT) void gg_f16_fourwave(GgParams p) { pingpong_body<OP_F16, true>(p); }
__global__ __launch_bounds__(W4_NT) void gg_bf16_fourwave_swiglu(GgParams p) { pingpong_body<OP_BF16_SWIGLU, true>(p); }
__global__ __launch_bounds__(W4_NT) void gg_f16_fourwave_swiglu(GgParams p) { pingpong_body<OP_F16_SWIGLU, true>(p); }
__global__ __launch_bounds__(W4_NT) void gg_bf16_fourwave_tall(GgParams p) { pingpong_body<OP_BF16, true, true>(p); }
__global__ __launch_bounds__(W4_NT) void gg_f16_fourwave_tall(GgParams p) { pingpong_body<OP_F16, true, true>(p); }
__global__ __launch_bounds__(W4_NT) void gg_bf16_fourwave_tall_swiglu(GgParams p) { pingpong_body<OP_BF16_SWIGLU, true, true>(p); }
__global__ __launch_bounds__(W4_NT) void gg_f16_fourwave_tall_swiglu(GgParams p) { pingpong_body<OP_F16_SWIGLU, true, true>(p); }
__global__ __launch_bounds__(NT) void gg_bf16_pingpong_wgrad(GgParams p) { pingpong_body<OP_BF16_WGRAD>(p); }
__global__ __launch_bounds__(NT) void gg_bf16_pingpong_swiglu(GgParams p) { pingpong_body<OP_BF16_SWIGLU>(p); }
__global__ __launch_bounds__(NT) void gg_f16_pingpong_swiglu(GgParams p) { pingpong_body<OP_F16_SWIGLU>(p); }
__global__ __launch_bounds__(NT) void gg_bf16_pingpong_swiglu_gather(GgParams p) { pingpong_body<OP_BF16_SWIGLU_GATHER>(p); }
__global__ __launch_bounds__(NT) void gg_f16_pingpong_swiglu_gather(GgParams p) { pingpong_body<OP_F16_SWIGLU_GATHER>(p); }
__global__ __launch_bounds__(NT) void gg_bf16_pingpong_nt(GgParams p) { pingpong_body<OP_BF16_NT>(p); }
__global__ __launch_bounds__(NT) void gg_bf16_pingpong_wgrad_direct(GgParams p) { pingpong_body<OP_BF16_WGRAD_DIRECT>(p); }
__global__ __launch_bounds__(NT) void gg_fp8_pingpong_rowwise(GgParams p) { pingpong_body<OP_FP8_ROW>(p); }
__global__ __launch_bounds__(NT) void gg_fp8_pingpong_block(GgParams p) { pingpong_body<OP_FP8_BLOCK>(p); }
// The forward eight-wave kernels behind the second prologue, for the split-tail order (p.split_tails): the K loops are
// the same source as above.
__global__ __launch_bounds__(NT) void gg_bf16_pingpong_split(GgParams p) { pingpong_body<OP_BF16, false, false, true>(p); }
__global__ __launch_bounds__(NT) void gg_f16_pingpong_split(GgParams p) { pingpong_body<OP_F16, false, false, true>(p); }
__global__ __launch_bounds__(NT) void gg_bf16_pingpong_swiglu_split(GgParams p) { pingpong_body<OP_BF16_SWIGLU, false, false, true>(p); }
__global__ __launch_bounds__(NT) void gg_f16_pingpong_swiglu_split(GgParams p) { pingpong_body<OP_F16_SWIGLU, false, false, true>(p); }
__global__ __launch_bounds__(NT) void gg_bf16_pingpong_nt_split(GgParams p) { pingpong_body<OP_BF16_NT, false, false, true>(p); }
__global__ __launch_bounds__(NT) void gg_fp8_pingpong_rowwise_split(GgParams p) { pingpong_body<OP_FP8_ROW, false, false, true>(p); }
__global__ __launch_bounds__(NT) void gg_fp8_pingpong_block_split(GgParams p) { pingpong_body<OP_FP8_BLOCK, false, false, true>(p); }

}  // namespace

hipError_t gg_bf16_pingpong_launch(const GgParams& p, int num_wg, hipStream_t stream) {
  if (p.split_tails) {
    if (p.fp16) hipLaunchKernelGGL(gg_f16_pingpong_split, dim3(num_wg), dim3(NT), 0, stream, p);
    else hipLaunchKernelGGL(gg_bf16_pingpong_split, dim3(num_wg), dim3(NT), 0, stream, p);
  } else if (p.fp16) hipLaunchKernelGGL(gg_f16_pingpong, dim3(num_wg), dim3(NT), 0, stream, p);
  else hipLaunchKernelGGL(gg_bf16_pingpong, dim3(num_wg), dim3(NT), 0, stream, p);
  return hipGetLastError();
}

hipError_t gg_bf16_fourwave_launch(const GgParams& p, bool tall, int num_wg, hipStream_t stream) {
  if (tall) {
    if (p.fp16) hipLaunchKernelGGL(gg_f16_fourwave_tall, dim3(num_wg), dim3(W4_NT), 0, stream, p);
    else hipLaunchKernelGGL(gg_bf16_fourwave_tall, dim3(num_wg), dim3(W4_NT), 0, stream, p);
  } else if (p.fp16) hipLaunchKernelGGL(gg_f16_fourwave, dim3(num_wg), dim3(W4_NT), 0, stream, p);
  else hipLaunchKernelGGL(gg_bf16_fourwave, dim3(num_wg), dim3(W4_NT), 0, stream, p);
  return hipGetLastError();
}

hipError_t gg_bf16_fourwave_swiglu_launch(const GgParams& p, bool tall, int num_wg, hipStream_t stream) {
  if (tall) {
    if (p.fp16) hipLaunchKernelGGL(gg_f16_fourwave_tall_swiglu, dim3(num_wg), dim3(W4_NT), 0, stream, p);
    else hipLaunchKernelGGL(gg_bf16_fourwave_tall_swiglu, dim3(num_wg), dim3(W4_NT), 0, stream, p);
  } else if (p.fp16) hipLaunchKernelGGL(gg_f16_fourwave_swiglu, dim3(num_wg), dim3(W4_NT), 0, stream, p);
  else hipLaunchKernelGGL(gg_bf16_fourwave_swiglu, dim3(num_wg), dim3(W4_NT), 0, stream, p);
  return hipGetLastError();
}

hipError_t gg_bf16_pingpong_wgrad_launch(const GgParams& p, int num_wg, hipStream_t stream) {
  hipLaunchKernelGGL(gg_bf16_pingpong_wgrad, dim3(num_wg), dim3(NT), 0, stream, p);
  return hipGetLastError();
}

hipError_t gg_bf16_pingpong_swiglu_launch(const GgParams& p, int num_wg, hipStream_t stream) {
  if (p.gather_perm) {
    if (p.fp16) hipLaunchKernelGGL(gg_f16_pingpong_swiglu_gather, dim3(num_wg), dim3(NT), 0, stream, p);
    else hipLaunchKernelGGL(gg_bf16_pingpong_swiglu_gather, dim3(num_wg), dim3(NT), 0, stream, p);
  } else if (p.split_tails) {
    if (p.fp16) hipLaunchKernelGGL(gg_f16_pingpong_swiglu_split, dim3(num_wg), dim3(NT), 0, stream, p);
    else hipLaunchKernelGGL(gg_bf16_pingpong_swiglu_split, dim3(num_wg), dim3(NT), 0, stream, p);
  } else if (p.fp16) hipLaunchKernelGGL(gg_f16_pingpong_swiglu, dim3(num_wg), dim3(NT), 0, stream, p);
  else hipLaunchKernelGGL(gg_bf16_pingpong_swiglu, dim3(num_wg), dim3(NT), 0, stream, p);
  return hipGetLastError();
}

hipError_t gg_bf16_pingpong_nt_launch(const GgParams& p, int num_wg, hipStream_t stream) {
  if (p.split_tails) hipLaunchKernelGGL(gg_bf16_pingpong_nt_split, dim3(num_wg), dim3(NT), 0, stream, p);
  else hipLaunchKernelGGL(gg_bf16_pingpong_nt, dim3(num_wg), dim3(NT), 0, stream, p);
  return hipGetLastError();
}

hipError_t gg_bf16_pingpong_wgrad_direct_launch(const GgParams& p, int num_wg, hipStream_t stream) {
  hipLaunchKernelGGL(gg_bf16_pingpong_wgrad_direct, dim3(num_wg), dim3(NT), 0, stream, p);
  return hipGetLastError();
}

hipError_t gg_fp8_pingpong_launch(const GgParams& p, int scale_mode, int num_wg, hipStream_t stream) {
  if (p.split_tails) {
    if (scale_mode == 0) hipLaunchKernelGGL(gg_fp8_pingpong_rowwise_split, dim3(num_wg), dim3(NT), 0, stream, p);
    else hipLaunchKernelGGL(gg_fp8_pingpong_block_split, dim3(num_wg), dim3(NT), 0, stream, p);
  } else if (scale_mode == 0) hipLaunchKernelGGL(gg_fp8_pingpong_rowwise, dim3(num_wg), dim3(NT), 0, stream, p);
  else hipLaunchKernelGGL(gg_fp8_pingpong_block, dim3(num_wg), dim3(NT), 0, stream, p);
  return hipGetLastError();
}
