// W4A16 split-K dequant GEMM for gfx950: c[M, N] = a[M, K] @ dequant(qweight, scales, qzeros).
//
// Replaces matmul_split_k / matmul_split_k_kernel
// (kernels/triton/inference/gptq/splitk_dequant_gemm.py:91-141, 23-89). Data layout as there:
//   qweight [K/8, N] int32, nibble j of a word = row 8*i + j            (:56, :76)
//   scales  [K/group, N] (same 16-bit float type as a)
//   qzeros  [K/group, N/8] int32, nibble j of a word = column 8*i + j   (:57, :70)
//   w(k, n) = (q(k, n) - (z(g, n) + zero_offset)) * s(g, n),  g = k / group   (:73-77)
//
// A workgroup of eight waves owns 64 output columns; the waves split K by quantisation group
// (wave w takes groups w, w+8, ...: the interleaved K split of the reference, :45,80-81) and their
// partial sums are added through LDS in a fixed order, so no atomics, no zero-initialised output and
// bit-identical results run to run.
//
// Per 32-wide K step a lane loads one dwordx4 of qweight: 4 adjacent columns x 8 consecutive k.
// Word j becomes the MFMA "A" fragment of column n0 + 4*(lane%16) + j without any arithmetic:
// ((word >> 4t) & 0x000F000F) | MAGIC puts nibble t in the low and nibble t+4 in the high half of a
// dword as the floats BIAS + q (BIAS = 128 for bf16, 1024 for fp16, exact). The activation fragment is
// permuted to the same k order (0,4,1,5,2,6,3,7). One extra MFMA per step with an all-ones A fragment
// gives S = sum_k x[k]; after each group the lane folds scale and zero point in fp32:
//   total += s * (acc_group - (BIAS + z + zero_offset) * S).
// With the four words of a lane feeding four MFMAs, a lane ends up with 16 consecutive output
// columns of one output row.
//
// Quantised output (QOUT kernels, W4Params::cq != nullptr): a workgroup does two adjacent 64-column blocks one
// after the other and, instead of storing 16-bit values, quantises each row's 128 results to fp8 e4m3fn with one
// fp32 scale - float8_groupwise_quantize (kernels/triton/inference/fp8/float8_groupwise_quant.py:20-50) applied to
// the 16-bit result, bit for bit, without the round trip of that result through memory.
#include "common.h"
#include "gg_tables.h"
#include "kernels.h"

namespace {

template <bool FP16>
struct Elem;
template <>
struct Elem<false> {  // bf16
  static constexpr uint32_t MAGIC = 0x43004300u;  // 128.0 | 128.0
  static constexpr uint32_t ONES = 0x3F803F80u;
  static constexpr float BIAS = 128.f;
  static DEVINL f32x4_t mfma(u32x4_t a, u32x4_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
  static DEVINL float to_f32(uint16_t h) { return __builtin_bit_cast(float, (uint32_t)h << 16); }
  static DEVINL uint16_t from_f32(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
};
template <>
struct Elem<true> {  // fp16
  static constexpr uint32_t MAGIC = 0x64006400u;  // 1024.0 | 1024.0
  static constexpr uint32_t ONES = 0x3C003C00u;
  static constexpr float BIAS = 1024.f;
  static DEVINL f32x4_t mfma(u32x4_t a, u32x4_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
  static DEVINL float to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
  static DEVINL uint16_t from_f32(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }
};

// What one workgroup works on: the whole problem (dense call), or one expert of a grouped call
// (rows row0 .. row0 + M - 1 of a and c, and that expert's slice of the stacked weights).
struct W4View {
  const uint16_t* a;
  const int32_t* qweight;
  const uint16_t* scales;
  const int32_t* qzeros;
  uint16_t* c;
  int M;
  uint8_t* cq;    // QOUT: [M, N] e4m3fn
  float* cscale;  // QOUT: [M, N/128]
};

// Must be called by every thread of the workgroup (it contains a barrier in grouped mode).
DEVINL W4View w4_view(const W4Params& p) {
  W4View v{(const uint16_t*)p.a, p.qweight, (const uint16_t*)p.scales, p.qzeros, (uint16_t*)p.c, p.M, (uint8_t*)p.cq, p.cscale};
  if (p.m_sizes == nullptr) return v;
  // Grid row blockIdx.y takes the blockIdx.y-th expert that has rows (the workgroups without work are then the last
  // ones of the launch; scattered among the others they make the dispatcher fill the CUs unevenly).
  __shared__ int s_g, s_row0, s_rows;
  if (threadIdx.x < 64) {
    const int l = threadIdx.x, per = (p.G + 63) >> 6, g0 = l * per, want = blockIdx.y;
    auto rows_of = [&](int i) {
      const int m = p.m_sizes[i];
      return m < 0 ? 0 : (m > p.M ? p.M : m);
    };
    long long s = 0;
    int c = 0, m_first = 0;  // m_first: rows of the lane's first expert (its only one when G <= 64)
    for (int i = 0; i < per; ++i)
      if (g0 + i < p.G) {
        const int m = rows_of(g0 + i);
        if (i == 0) m_first = m;
        s += m;
        c += m > 0;
      }
    long long run = wave_incl_scan_i64(s) - s;
    int incl = c;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d, 64);
      if (l >= d) incl += up;
    }
    const bool here = want >= incl - c && want < incl;  // true in one lane at most
    if (__ballot(here) == 0) {
      if (l == 0) s_g = -1;
    } else if (here) {
      int k = want - (incl - c);
      for (int i = 0; i < per; ++i) {
        const int m = i == 0 ? m_first : (g0 + i < p.G ? rows_of(g0 + i) : 0);
        if (m > 0 && k-- == 0) {
          const long long r0 = run > p.M ? p.M : run;
          s_g = g0 + i;
          s_row0 = (int)r0;
          s_rows = (long long)m > p.M - r0 ? (int)(p.M - r0) : m;
          break;
        }
        run += m;
      }
    }
  }
  __syncthreads();
  const int g = s_g;
  if (g < 0) {
    v.M = 0;
    return v;
  }
  const int row0 = s_row0;
  const int ngroups = p.K / p.group_size;
  v.M = s_rows;
  v.a += (int64_t)row0 * p.K;
  if (v.c) v.c += (int64_t)row0 * p.N;
  if (v.cq) {
    v.cq += (int64_t)row0 * p.N;
    v.cscale += (int64_t)row0 * (p.N / 128);
  }
  v.qweight += (int64_t)g * (p.K / 8) * p.N;
  v.scales += (int64_t)g * ngroups * p.N;
  v.qzeros += (int64_t)g * ngroups * (p.N / 8);
  return v;
}

// Sum the waves' partial results of rows mb .. mb + 16 MF - 1 x columns n0 .. n0 + 63 (red[wave][i][m_local * 64 +
// col]) in a fixed order and store them. A wave takes one row per pass, a lane one column. QOUT: column block 0
// (cb = 0) only keeps its values, rounded to the 16-bit type; column block 1 then has each row's 128 values in one
// wave (two per lane) and quantises them as fp8_groupwise_quant_kernel (quant.hip) does.
template <bool FP16, bool QOUT, int MF, int NW>
DEVINL void w4_reduce_store(const float (&red)[NW][MF][16 * 64], const W4View& v, int N, int mb, int n0, int cb,
                            float (&keep)[16 * MF / NW]) {
  using E = Elem<FP16>;
  static_assert(16 % NW == 0, "one row per wave and pass: 16 MF rows in 16 MF / NW passes");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rows_here = min(v.M - mb, 16 * MF);
#pragma unroll
  for (int k = 0; k < 16 * MF / NW; ++k) {
    const int ml = wave + NW * k;
    if (ml >= rows_here) continue;  // the same for all lanes of a wave
    const int i = ml / 16, rem = (ml % 16) * 64 + lane;
    float sum = red[0][i][rem];
#pragma unroll
    for (int w2 = 1; w2 < NW; ++w2) sum += red[w2][i][rem];
    const uint16_t h = E::from_f32(sum);
    if (!QOUT) {
      if (n0 + lane < N) v.c[(int64_t)(mb + ml) * N + n0 + lane] = h;
    } else if (cb == 0) {
      keep[k] = E::to_f32(h);
    } else {
      const float a = keep[k], b = E::to_f32(h);
      float amax = fmaxf(fabsf(a), fabsf(b));
#pragma unroll
      for (int d = 32; d >= 1; d >>= 1) amax = fmaxf(amax, __shfl_xor(amax, d, 64));
      const float s = fmaxf(amax, 1e-12f) / 448.0f;
      const float ya = fminf(fmaxf(a / s, -448.0f), 448.0f);
      const float yb = fminf(fmaxf(b / s, -448.0f), 448.0f);
      const int packed = __builtin_amdgcn_cvt_pk_fp8_f32(ya, yb, 0, false);
      uint8_t* q = v.cq + (int64_t)(mb + ml) * N + (n0 - 64) + lane;
      q[0] = (uint8_t)(packed & 0xFF);
      q[64] = (uint8_t)((packed >> 8) & 0xFF);
      if (lane == 0) v.cscale[(int64_t)(mb + ml) * (N / 128) + (n0 - 64) / 128] = s;
    }
  }
}

constexpr int WAVES = 8;
constexpr int DEPTH = 8;  // K steps of qweight loads in flight per wave

// 64 lanes x 4 B from global memory straight into LDS (lane l's dword lands at lds_addr + 4 l): a load without a
// register destination, used where only the request matters. Completion is tracked by hand with vmcnt.
DEVINL void dma4(const void* sbase, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2\n"
               :
               : "s"(lds_addr), "v"(voff), "s"(sbase)
               : "memory");
}
template <int N>
DEVINL void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
DEVINL const char* uni_ptr(const char* q) {
  const uint64_t v = (uint64_t)q;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (const char*)(((uint64_t)hi << 32) | lo);
}

// Any group size that is a multiple of 32; scales / zeros are loaded where they are used.
template <bool FP16, int MF, bool QOUT>
__global__ __launch_bounds__(64 * WAVES) void w4a16_splitk_anygroup(W4Params p) {
  using E = Elem<FP16>;
  __shared__ __attribute__((aligned(16))) float red[WAVES][MF][64 * 16];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int fr = lane & 15, fq = lane >> 4;
  const uint32_t nib_mask = 0x000F000Fu, magic = E::MAGIC;  // the two constants of the nibble unpack
  const W4View v = w4_view(p);
  const int N = p.N, K = p.K, M = v.M;
  constexpr int CB = QOUT ? 2 : 1;                 // 64-column blocks per workgroup
  const int spg = p.group_size / 32;               // K steps per quantisation group
  const int ngroups = K / p.group_size;
  const int my_groups = ngroups > wave ? (ngroups - wave + WAVES - 1) / WAVES : 0;
  const int steps = my_groups * spg;               // K steps of this wave

  // step t of this wave -> absolute K step
  auto kstep = [&](int t) { return ((t / spg) * WAVES + wave) * spg + t % spg; };

  float keep[16 * MF / WAVES];
  for (int mb = 0; mb < M; mb += 16 * MF)
  for (int cb = 0; cb < CB; ++cb) {
    const int n0 = (blockIdx.x * CB + cb) * 64;
    // qweight: lane reads words of columns n0 + 4*fr .. + 3 (clamped at the right edge), k-word row 4*step + fq
    const int wcol = min(n0 + 4 * fr, N - 4);
    const int32_t* qw = v.qweight + wcol;
    // output / scale columns of this lane: n0 + 16*fq + 0..15
    const int ocol = n0 + 16 * fq;
    const int ocol_c = min(ocol, N - 16 >= 0 ? N - 16 : 0);
    const uint16_t* arow[MF];
#pragma unroll
    for (int i = 0; i < MF; ++i) arow[i] = v.a + (int64_t)min(mb + i * 16 + fr, M - 1) * K + fq * 8;

    f32x4_t total[MF][4];  // [m fragment][j]: rows n-local 4*ii + j ... see epilogue
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) total[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    u32x4_t wb[DEPTH];
    auto loadw = [&](int d, int t) { wb[d] = *(const u32x4_t*)(qw + (int64_t)(kstep(t) * 4 + fq) * N); };
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
      if (d < steps) loadw(d, d);

    f32x4_t accg[MF][4], accs[MF];
    for (int t0 = 0; t0 < steps; t0 += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int t = t0 + d;
        if (t < steps) {
          if (t % spg == 0) {
#pragma unroll
            for (int i = 0; i < MF; ++i) {
#pragma unroll
              for (int j = 0; j < 4; ++j) accg[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
              accs[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            }
          }
          const int ks = kstep(t);
          // activation fragments, permuted to the k order the nibble unpack produces
          u32x4_t xb[MF];
#pragma unroll
          for (int i = 0; i < MF; ++i) {
            const u32x4_t xv = *(const u32x4_t*)(arow[i] + ks * 32);
            xb[i][0] = __builtin_amdgcn_perm(xv[2], xv[0], 0x05040100u);  // k 0, 4
            xb[i][1] = __builtin_amdgcn_perm(xv[2], xv[0], 0x07060302u);  // k 1, 5
            xb[i][2] = __builtin_amdgcn_perm(xv[3], xv[1], 0x05040100u);  // k 2, 6
            xb[i][3] = __builtin_amdgcn_perm(xv[3], xv[1], 0x07060302u);  // k 3, 7
          }
          const u32x4_t w4 = wb[d];
          if (t + DEPTH < steps) loadw(d, t + DEPTH);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            u32x4_t af;
#pragma unroll
            for (int e = 0; e < 4; ++e) af[e] = ((w4[j] >> (4 * e)) & nib_mask) | magic;
#pragma unroll
            for (int i = 0; i < MF; ++i) accg[i][j] = E::mfma(af, xb[i], accg[i][j]);
          }
          const u32x4_t ones = {E::ONES, E::ONES, E::ONES, E::ONES};
#pragma unroll
          for (int i = 0; i < MF; ++i) accs[i] = E::mfma(ones, xb[i], accs[i]);

          if (t % spg == spg - 1) {
            // fold scale and zero point of this group: lane's columns are ocol + 4*ii + j
            const int g = ks / spg;
            const u32x4_t s0 = *(const u32x4_t*)(v.scales + (int64_t)g * N + ocol_c);
            const u32x4_t s1 = *(const u32x4_t*)(v.scales + (int64_t)g * N + ocol_c + 8);
            const u32x2_t zw = *(const u32x2_t*)(v.qzeros + (int64_t)g * (N / 8) + ocol_c / 8);
#pragma unroll
            for (int ii = 0; ii < 4; ++ii)
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                const int c = 4 * ii + j;  // column offset inside the lane's 16
                const uint32_t sw = c < 8 ? s0[c >> 1] : s1[(c - 8) >> 1];
                const float s = E::to_f32((uint16_t)((c & 1) ? (sw >> 16) : (sw & 0xFFFFu)));
                const uint32_t z = (zw[c >> 3] >> (4 * (c & 7))) & 0xFu;
                const float zz = E::BIAS + (float)(int)(z + (uint32_t)p.zero_offset);
#pragma unroll
                for (int i = 0; i < MF; ++i) total[i][j][ii] += s * (accg[i][j][ii] - zz * accs[i][ii]);
              }
          }
        }
      }
    }

    // Cross-wave (split-K) reduction, fixed order. red[wave][i][(m_local * 64) + col_local]
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int ii = 0; ii < 4; ++ii) red[wave][i][fr * 64 + 16 * fq + 4 * ii + j] = total[i][j][ii];
    __syncthreads();
    w4_reduce_store<FP16, QOUT, MF, WAVES>(red, v, N, mb, n0, cb, keep);
    __syncthreads();
  }
}

// group_size == 128 (four K steps per group). Every load - qweight, activations, scales, zeros - is
// issued GA groups ahead of its use and consumed in issue order, because vector memory loads return in
// order: a late-issued small load would otherwise wait for all the weight loads queued before it.
//
// Operand roles are the other way round than in the kernel above: the activation fragment is the MFMA
// "A" operand and the unpacked weights the "B" operand, so a lane ends up with output rows
// 4 * (lane / 16) + r of the four adjacent columns n0 + 4 * (lane % 16) + j of its own qweight words. It
// then needs just four scales and four zero points per group (one 8-byte and one 4-byte load), and the
// fold costs a quarter of the vector instructions of the 16-columns-per-lane layout.
//
// WARM > 0: the workgroup has WARM more waves that compute nothing. They request one dword of every 128-byte line
// of the workgroup's weight strip (64 columns = two lines per k-word row), in K order, as fast as the memory system
// takes the requests, so that the consumer waves, whose queues are a group deep, find their lines in the L2 or on
// the way there: a launch of this size is bound by how early its bytes are requested, not by bandwidth. The
// requests are loads into a scrap LDS area (no register destination). With WARM the consumer lanes of activation
// rows beyond M also issue no loads (their fragment is zero) instead of re-reading the last row.
//
// STAGE: the activations of a quantisation group (16 MF rows x 256 bytes) reach the wave through its own LDS area
// instead of as fragment loads. A fragment load takes 64 bytes of each of 16 rows (16 half lines per instruction, the
// rows a whole K apart), and every workgroup of the launch pulls the same few rows out of the L2 that way: measured
// 4.5 us per 16 rows, several times what the bytes cost. Staged, a load instruction takes 4 rows x 256 contiguous
// bytes (8 whole lines), the same number of instructions and registers; the pieces are written to LDS when the group's
// turn comes (16-byte chunks XOR-swizzled with the row, so that the fragment reads spread over all banks) and read
// back as the MFMA fragments. The area is the wave's own: no barrier, the LDS queue of a wave is in order.
template <bool FP16, int MF, int GA, int NWAVES, bool QOUT, int WARM = 0, bool STAGE = false>  // GA = groups kept in flight
__global__ __launch_bounds__(64 * (NWAVES + WARM)) void w4a16_splitk_g128(W4Params p) {
  using E = Elem<FP16>;
  constexpr int SPG = 4, D = SPG * GA;
  constexpr bool MASK = WARM > 0;
  static_assert(!STAGE || GA == 1, "the staged form keeps one group in flight");
  __shared__ __attribute__((aligned(16))) float red[NWAVES][MF][16 * 64];
  __shared__ __attribute__((aligned(256))) uint32_t scrap[WARM > 0 ? WARM : 1][64];
  __shared__ __attribute__((aligned(16))) u32x4_t stage[STAGE ? NWAVES : 1][STAGE ? 16 * MF : 1][16];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int fr = lane & 15, fq = lane >> 4;
  // The two constants of the nibble unpack. In the selectable forms (one pass, warm-up waves, staged activations) they
  // live in registers, the mask in a scalar and the exponent pattern in a vector one, hidden from constant folding:
  // mask-and-or is then one v_and_or_b32, which takes no literal and one scalar operand; with literals, as in the
  // kernels that run by default, it is an and and an or.
  uint32_t nib_mask = 0x000F000Fu, magic = E::MAGIC;
  if constexpr (WARM > 0 || STAGE || MF == 4) {
    asm volatile("" : "+s"(nib_mask));
    asm volatile("" : "+v"(magic));
  }
  const W4View v = w4_view(p);
  const int N = p.N, K = p.K, M = v.M;
  constexpr int CB = QOUT ? 2 : 1;                      // 64-column blocks per workgroup
  const int ngroups = K / 128;
  const int my_groups = ngroups > wave ? (ngroups - wave + NWAVES - 1) / NWAVES : 0;
  const int steps = my_groups * SPG;
  auto kstep = [&](int t) { return ((t / SPG) * NWAVES + wave) * SPG + t % SPG; };

  const int zshift = 16 * (fr & 1);                     // the lane's four zero nibbles inside the word

  // One pass = 16 MF rows x one 64-column block over the whole K. The first loads of the next pass are issued
  // before the cross-wave reduction of the current one, so the load queue does not run dry between passes.
  const int passes = (M + 16 * MF - 1) / (16 * MF) * CB;
  if (passes == 0) return;  // an expert without rows (the same for the whole workgroup)
  if (WARM > 0 && wave >= NWAVES) {
    // A warm-up wave: lines 2 r and 2 r + 1 are the two halves of k-word row r of the strip (256 bytes at
    // qweight[r][n0]); the WARM waves take blocks of 64 lines in turn. The last block repeats its last line.
    const int ww = __builtin_amdgcn_readfirstlane(wave) - NWAVES;  // the same in every lane: scalar registers below
    const uint32_t scrap_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint32_t*)scrap[ww];
    const int lines = (K / 8) * 2;
    for (int cb = 0; cb < CB; ++cb) {
      const char* base = uni_ptr((const char*)(v.qweight + (blockIdx.x * CB + cb) * 64));
      for (int l0 = ww * 64; l0 < lines; l0 += WARM * 64) {
        const int line = min(l0 + lane, lines - 1);
        dma4(base, (uint32_t)(line >> 1) * (uint32_t)N * 4u + (uint32_t)(line & 1) * 128u, scrap_addr);
      }
    }
    wait_vm<0>();
    for (int pass = 0; pass < passes; ++pass) {  // the barriers of the consumer waves' passes
      __syncthreads();
      __syncthreads();
    }
    return;
  }
  const int32_t* qw;        // k-word row 4 * step + fq, columns n0 + 4 fr .. + 3
  const uint16_t* sc;
  const int32_t* zp;
  const uint16_t* arow[MF];
  bool row_ok[MF];          // MASK: the lane's row of fragment i exists
  // STAGE: piece q (0 .. 4 MF - 1) of a group is rows 4 q + lane / 16 of the pass, 16-byte chunk lane % 16.
  const int sr = lane >> 4, sc16 = lane & 15;
  const uint16_t* srow = nullptr;  // row sr of the pass, chunk sc16, K offset 0
  int srows = 0;                   // rows of the pass that exist
  auto setup = [&](int pass) {
    const int mb = pass / CB * (16 * MF), n0 = (blockIdx.x * CB + pass % CB) * 64;
    qw = v.qweight + n0 + 4 * fr;
    sc = v.scales + n0 + 4 * fr;
    zp = v.qzeros + (n0 + 4 * fr) / 8;
#pragma unroll
    for (int i = 0; i < MF; ++i) {
      arow[i] = v.a + (int64_t)min(mb + i * 16 + fr, M - 1) * K + fq * 8;
      row_ok[i] = mb + i * 16 + fr < M;
    }
    if constexpr (STAGE) {
      srow = v.a + (int64_t)(mb + sr) * K + sc16 * 8;
      srows = M - mb;
    }
  };
  u32x4_t wb[D], xr[D][MF];
  u32x2_t sg[GA];
  uint32_t zg[GA];
  // STAGE: all pieces of the wave's group gi (the gi-th of its own) into xr; rows that do not exist are zero.
  auto load_pieces = [&](int gi) {
    const int64_t koff = ((int64_t)gi * NWAVES + wave) * 128;  // first k of the group
#pragma unroll
    for (int q = 0; q < 4 * MF; ++q) {
      xr[q / MF][q % MF] = u32x4_t{0u, 0u, 0u, 0u};
      if (4 * q + sr < srows) xr[q / MF][q % MF] = *(const u32x4_t*)(srow + (int64_t)(4 * q) * K + koff);
    }
  };
  auto load_step = [&](int d, int t) {
    const int ks = kstep(t);
    wb[d] = *(const u32x4_t*)(qw + (int64_t)(ks * 4 + fq) * N);
    if constexpr (!STAGE) {  // staged: the activations come group by group (load_pieces)
#pragma unroll
      for (int i = 0; i < MF; ++i) {
        if (MASK) {
          xr[d][i] = u32x4_t{0u, 0u, 0u, 0u};
          if (row_ok[i]) xr[d][i] = *(const u32x4_t*)(arow[i] + ks * 32);
        } else {
          xr[d][i] = *(const u32x4_t*)(arow[i] + ks * 32);
        }
      }
    }
  };
  auto load_group = [&](int q, int gi) {  // gi = index among this wave's groups
    const int64_t g = (int64_t)gi * NWAVES + wave;
    sg[q] = *(const u32x2_t*)(sc + g * N);
    zg[q] = (uint32_t)zp[g * (N / 8)];
  };
  auto first_loads = [&]() {
#pragma unroll
    for (int q = 0; q < GA; ++q) {
#pragma unroll
      for (int e = 0; e < SPG; ++e)
        if (q * SPG + e < steps) load_step(q * SPG + e, q * SPG + e);
      if (q < my_groups) load_group(q, q);
      if constexpr (STAGE) {
        if (q < my_groups) load_pieces(q);
      }
    }
  };
  setup(0);
  first_loads();

  float keep[16 * MF / NWAVES];
  for (int pass = 0; pass < passes; ++pass) {
    const int mb = pass / CB * (16 * MF), cb = pass % CB, n0 = (blockIdx.x * CB + cb) * 64;
    f32x4_t total[MF][4];  // [row fragment i][column j]: rows mb + 16 i + 4 fq + r
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) total[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    for (int g0 = 0; g0 < my_groups; g0 += GA) {
#pragma unroll
      for (int q = 0; q < GA; ++q) {
        const int gi = g0 + q;  // index among this wave's groups; its loads sit in ring slots q * SPG .. + 3
        if (gi < my_groups) {
          const bool more = gi + GA < my_groups;
          f32x4_t accg[MF][4], accs[MF];
#pragma unroll
          for (int i = 0; i < MF; ++i) {
#pragma unroll
            for (int j = 0; j < 4; ++j) accg[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            accs[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
          }
          if constexpr (STAGE) {
            // The group's pieces from registers into the wave's LDS area (row 4 p + sr, chunk sc16 at slot
            // sc16 ^ (row % 16)), then the registers take the next group's. The lanes of a wave read what other
            // lanes of it wrote: LDS serves a wave's accesses in order, and the two wave barriers keep the compiler
            // from moving the reads of one group and the writes of the next across each other.
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int pc = 0; pc < 4 * MF; ++pc) stage[wave][4 * pc + sr][sc16 ^ ((4 * pc + sr) & 15)] = xr[pc / MF][pc % MF];
            __builtin_amdgcn_wave_barrier();
            if (more) load_pieces(gi + GA);
          }
#pragma unroll
          for (int e = 0; e < SPG; ++e) {
            const int d = q * SPG + e;
            u32x4_t xb[MF];
#pragma unroll
            for (int i = 0; i < MF; ++i) {
              // fragment i of step e: row 16 i + fr, k chunk 4 e + fq of the group
              u32x4_t xv;
              if constexpr (STAGE) xv = stage[wave][16 * i + fr][(4 * e + fq) ^ fr];
              else xv = xr[d][i];
              xb[i][0] = __builtin_amdgcn_perm(xv[2], xv[0], 0x05040100u);  // k 0, 4
              xb[i][1] = __builtin_amdgcn_perm(xv[2], xv[0], 0x07060302u);  // k 1, 5
              xb[i][2] = __builtin_amdgcn_perm(xv[3], xv[1], 0x05040100u);  // k 2, 6
              xb[i][3] = __builtin_amdgcn_perm(xv[3], xv[1], 0x07060302u);  // k 3, 7
            }
            const u32x4_t w4 = wb[d];
            // Refill two K steps at a time: their activation fragments are the two halves of the same 128-byte
            // lines, and issued back to back the second load still finds the line in the vector L1.
            if (more && (e & 1)) { load_step(d - 1, (gi + GA) * SPG + e - 1); load_step(d, (gi + GA) * SPG + e); }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              u32x4_t bf;
#pragma unroll
              for (int e2 = 0; e2 < 4; ++e2) bf[e2] = ((w4[j] >> (4 * e2)) & nib_mask) | magic;
#pragma unroll
              for (int i = 0; i < MF; ++i) accg[i][j] = E::mfma(xb[i], bf, accg[i][j]);
            }
            const u32x4_t ones = {E::ONES, E::ONES, E::ONES, E::ONES};
#pragma unroll
            for (int i = 0; i < MF; ++i) accs[i] = E::mfma(xb[i], ones, accs[i]);
          }
          const u32x2_t sq = sg[q];
          const uint32_t zq = zg[q] >> zshift;
          if (more) load_group(q, gi + GA);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const uint32_t sw = sq[j >> 1];
            const float s = E::to_f32((uint16_t)((j & 1) ? (sw >> 16) : (sw & 0xFFFFu)));
            const uint32_t z = (zq >> (4 * j)) & 0xFu;
            const float zz = E::BIAS + (float)(int)(z + (uint32_t)p.zero_offset);
#pragma unroll
            for (int i = 0; i < MF; ++i) total[i][j] += s * (accg[i][j] - zz * accs[i]);
          }
        }
      }
    }

    if (pass + 1 < passes) {
      setup(pass + 1);
      first_loads();
    }
    // Cross-wave (split-K) reduction in a fixed order: red[wave][i][m_local * 64 + col_local].
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        *(f32x4_t*)&red[wave][i][(4 * fq + r) * 64 + 4 * fr] = f32x4_t{total[i][0][r], total[i][1][r], total[i][2][r], total[i][3][r]};
    __syncthreads();
    w4_reduce_store<FP16, QOUT, MF, NWAVES>(red, v, N, mb, n0, cb, keep);
    __syncthreads();
  }
}

template <bool FP16, bool QOUT>
hipError_t launch(const W4Params& p, int variant, hipStream_t stream) {
  // Grouped call: one grid row per expert; the kernel variant follows the average rows per expert (an
  // expert with more rows than one pass covers is done in several passes over its weights).
  // (fp8 output: 128 columns per workgroup, N % 128 == 0 checked by the caller.)
  dim3 grid(QOUT ? p.N / 128 : (p.N + 63) / 64, p.m_sizes ? p.G : 1), block(64 * WAVES);
  const int M = p.m_sizes ? (p.M + p.G - 1) / p.G : p.M;
  if constexpr (!QOUT) {
    // Selectable variants (MOE_GG_OP_W4A16), group size 128: never chosen by default. The warm-up waves go with the
    // one-fragment kernel only: ten waves leave a wave 168 registers, which the two-fragment kernel (232) does not
    // fit, and the four-fragment kernel needs a four-wave workgroup for its 430. Bit 4: activations staged through LDS.
    constexpr int WARM = 2;
    const bool one_pass = (variant & 1) && M > 32, warm = (variant & 2) && M <= 16, staged = (variant & 4) != 0;
    if (p.group_size == 128 && (one_pass || warm || staged)) {
      if (one_pass) {
        if (staged) hipLaunchKernelGGL((w4a16_splitk_g128<FP16, 4, 1, 4, false, 0, true>), grid, dim3(64 * 4), 0, stream, p);
        else hipLaunchKernelGGL((w4a16_splitk_g128<FP16, 4, 1, 4, false>), grid, dim3(64 * 4), 0, stream, p);
      } else if (M <= 16) {
        if (warm && staged) hipLaunchKernelGGL((w4a16_splitk_g128<FP16, 1, 1, WAVES, false, WARM, true>), grid, dim3(64 * (WAVES + WARM)), 0, stream, p);
        else if (warm) hipLaunchKernelGGL((w4a16_splitk_g128<FP16, 1, 1, WAVES, false, WARM>), grid, dim3(64 * (WAVES + WARM)), 0, stream, p);
        else hipLaunchKernelGGL((w4a16_splitk_g128<FP16, 1, 1, WAVES, false, 0, true>), grid, block, 0, stream, p);
      } else {
        hipLaunchKernelGGL((w4a16_splitk_g128<FP16, 2, 1, WAVES, false, 0, true>), grid, block, 0, stream, p);
      }
      return hipGetLastError();
    }
  }
  // Group size 128: one activation fragment per pass for M <= 16, two for more rows (32 rows per pass over the
  // weights; four fragments do not fit the registers), all loads issued one group ahead (deeper queues and
  // more waves measured slower). Other group sizes: up to four activation fragments per pass (two with fp8
  // output, whose kept values of the first column block need registers too).
  if (M <= 16 && p.group_size == 128) hipLaunchKernelGGL((w4a16_splitk_g128<FP16, 1, 1, WAVES, QOUT>), grid, block, 0, stream, p);
  else if (p.group_size == 128) hipLaunchKernelGGL((w4a16_splitk_g128<FP16, 2, 1, WAVES, QOUT>), grid, block, 0, stream, p);
  else if (M <= 16) hipLaunchKernelGGL((w4a16_splitk_anygroup<FP16, 1, QOUT>), grid, block, 0, stream, p);
  else if (M <= 32 || QOUT) hipLaunchKernelGGL((w4a16_splitk_anygroup<FP16, 2, QOUT>), grid, block, 0, stream, p);
  else if constexpr (!QOUT) hipLaunchKernelGGL((w4a16_splitk_anygroup<FP16, 4, false>), grid, block, 0, stream, p);
  return hipGetLastError();
}

}  // namespace

hipError_t w4a16_splitk_launch(const W4Params& p, bool fp16, int variant, hipStream_t stream) {
  if (p.cq) return fp16 ? launch<true, true>(p, variant, stream) : launch<false, true>(p, variant, stream);
  return fp16 ? launch<true, false>(p, variant, stream) : launch<false, false>(p, variant, stream);
}
