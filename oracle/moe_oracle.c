/*
 * moe_oracle.c - CPU restatement of the reference's MoE grouped-GEMM path.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing under oracle/ is part of the shipped library: only tests/,
 * __graft_entry__.smoke() and bench.py's cpu_baseline leg may load it, and only as the checker.
 *
 * Every function restates the algorithm of a reference file (paths relative to the reference
 * checkout) in plain scalar C with double-precision accumulation. Where each function is pinned
 * (known answers, closed forms, independent library routines) is listed per function; the tests
 * live in tests/test_oracle.py.
 *
 * Parity status:
 *   orc_offsets, orc_grouped_gemm, orc_route, orc_moe_align_block_size, orc_topk,
 *   orc_w4_dequant, orc_e4m3_*, orc_fp8_groupwise_quant, orc_grouped_gemm_fp8 (rowwise),
 *   orc_silu_and_mul, orc_fused_moe, orc_grouped_gemm_backward, orc_fp8_block_quant_weight: pinned.
 *   For orc_fp8_block_quant_weight (128x128 weight quantiser) the reference calls quantize_fp8_block of
 *   the FBGEMM package, which is not vendored and pinned to no version
 *   (kernels/needs_perf_help/fp8_gemm_bench.py:16-21); its published rule is per-block
 *   max(amax, 1e-12) against the e4m3 maximum 448 with a clamp to +-448, the rule of the in-tree
 *   1x128 quantiser, which this file applies to a whole block (scale stored as amax/448, codes from
 *   w / scale). Pinned by constructed blocks, index order, numpy/torch routines and agreement with
 *   the 1x128 quantiser where both must coincide.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

float orc_round_bf16(float f);

/* ---- offsets: exclusive prefix sum of m_sizes --------------------------------------------------
 * dev/triton_groupGEMM/groupgemm.py:159-165 (running M_start/M_end offsets) and the host form in
 * kernels/MoE/group_GEMM/triton/tgroup_gemm_backwards.py:471-477 (group_offsets[G+1]).
 * Pinned by: fixed m_sizes cases of the reference tests ([25,50,25], [4,4], [32]*4, [1024,1024],
 * 20 groups of 52/51) and numpy.cumsum. */
void orc_offsets(const int32_t* m_sizes, int G, int32_t* offsets) {
  int32_t run = 0;
  for (int g = 0; g < G; ++g) {
    offsets[g] = run;
    run += m_sizes[g];
  }
  offsets[G] = run;
}

/* ---- grouped GEMM: y[off_g + i, cb*g + n] = sum_k x[off_g + i, k] * w[g*N + n, k] ---------------
 * The per-group oracle loop of dev/triton_groupGEMM/testing/unit_tests.py:49-55 and
 * base_testing.py:125-131; with col_block = N it is the [M, N*G] block layout of
 * kernels/MoE/group_GEMM/triton/testing/fast_verification.py:83-96. Rows >= sum(m_sizes) and, in
 * block layout, the other experts' columns are not written.
 * Pinned by: G = 1 equals a dense matmul (numpy float64), brute-force 8x8x8 (unit_tests.py:136-149),
 * group-permutation invariance, torch.matmul per group. */
void orc_grouped_gemm(const float* x, const float* w, const int32_t* m_sizes, int G, int64_t M, int N,
                      int K, float* y, int64_t ldy, int col_block) {
  int64_t off = 0;
  for (int g = 0; g < G; ++g) {
    int64_t m = m_sizes[g];
    if (m > 0) {
#pragma omp parallel for schedule(static)
      for (int64_t i = 0; i < m; ++i) {
        const float* xr = x + (off + i) * K;
        float* yr = y + (off + i) * ldy + (int64_t)g * col_block;
        for (int n = 0; n < N; ++n) {
          const float* wr = w + ((int64_t)g * N + n) * K;
          double acc = 0.0;
          for (int k = 0; k < K; ++k) acc += (double)xr[k] * (double)wr[k];
          yr[n] = (float)acc;
        }
      }
      off += m;
    }
  }
  (void)M;
}

/* ---- backward of the grouped GEMM ---------------------------------------------------------------
 * kernels/MoE/group_GEMM/triton/testing/pytorch_reference_backwards.py:165-197 (per expert
 * grad_x[rows] = dY_g @ w[g], grad_w[g] = dY_g^T @ x[rows]; outputs start from zeros) which is what
 * grouped_gemm_backward (tgroup_gemm_backwards.py:382-590) computes. dY_g = go[rows of g, g*col_block .. + N).
 * Pinned by: torch.autograd through the per-expert forward loop of fast_verification.py:83-99,
 * G = 1 equals the dense dY @ w and dY^T @ x (numpy float64), and the adjoint identity
 * <dY, forward(x, w)> = <grad_x, x> = <grad_w, w>. */
void orc_grouped_gemm_backward(const float* go, int64_t ld_go, int col_block, const float* x, const float* w,
                               const int32_t* m_sizes, int G, int64_t M, int N, int K, float* grad_x,
                               float* grad_w) {
  memset(grad_x, 0, sizeof(float) * (size_t)M * K);
  memset(grad_w, 0, sizeof(float) * (size_t)G * N * K);
  int64_t off = 0;
  for (int g = 0; g < G; ++g) {
    int64_t m = m_sizes[g];
    if (m <= 0) continue;
    const float* dy = go + off * ld_go + (int64_t)g * col_block;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i)
      for (int k = 0; k < K; ++k) {
        double acc = 0.0;
        for (int n = 0; n < N; ++n) acc += (double)dy[i * ld_go + n] * (double)w[((int64_t)g * N + n) * K + k];
        grad_x[(off + i) * K + k] = (float)acc;
      }
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n)
      for (int k = 0; k < K; ++k) {
        double acc = 0.0;
        for (int64_t i = 0; i < m; ++i) acc += (double)dy[i * ld_go + n] * (double)x[(off + i) * K + k];
        grad_w[((int64_t)g * N + n) * K + k] = (float)acc;
      }
    off += m;
  }
}

/* ---- top-k routing ------------------------------------------------------------------------------
 * topk_ids = torch.topk(score, k) as used by the reference's MoE test
 * (kernels/triton/inference/col_major_moe_gemm/test_moe_gemm.py:54-57): the k largest entries of
 * each row in descending order. Ties (which torch leaves unspecified) go to the lower expert index.
 * Pinned by: numpy stable argsort of the negated row, and torch.topk on tie-free inputs. */
void orc_topk(const float* logits, int64_t T, int E, int k, int32_t* ids) {
  uint8_t* taken = (uint8_t*)malloc((size_t)E);
  for (int64_t t = 0; t < T; ++t) {
    const float* row = logits + t * E;
    memset(taken, 0, (size_t)E);
    for (int j = 0; j < k; ++j) {
      int best = -1;
      for (int e = 0; e < E; ++e) {
        if (taken[e]) continue;
        if (best < 0 || row[e] > row[best]) best = e;
      }
      taken[best] = 1;
      ids[t * k + j] = best;
    }
  }
  free(taken);
}

/* ---- expert grouping ----------------------------------------------------------------------------
 * flat = topk_ids.reshape(-1); rows are grouped by ascending expert, and inside an expert keep the
 * order of their flat index (a stable sort). This is the grouping of the reference's oracle mask
 * loop (test_moe_gemm.py:24-29) and of moe_align_block_size
 * (kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:141-166).
 * Outputs: perm[n] (flat indices in sorted order; the source token is perm[i] / k), m_sizes[E].
 * An id outside [0, E) (a masked slot, e.g. -1) belongs to no expert: it is counted nowhere, its
 * position appears nowhere in perm, and the sum(m_sizes) .. n-1 tail of perm is -1 (the reference's
 * kernel masks such slots out through token_mask, v0_moe_fused.py:63-66).
 * Pinned by: the docstring known answer of v0_moe_fused.py:157-165 (through
 * orc_moe_align_block_size below), numpy stable argsort and bincount (over the valid positions
 * when ids are masked). */
void orc_route(const int32_t* flat_ids, int64_t n, int E, int32_t* perm, int32_t* m_sizes) {
  int64_t* cursor = (int64_t*)calloc((size_t)E + 1, sizeof(int64_t));
  memset(m_sizes, 0, sizeof(int32_t) * (size_t)E);
  for (int64_t i = 0; i < n; ++i)
    if (flat_ids[i] >= 0 && flat_ids[i] < E) m_sizes[flat_ids[i]]++;
  int64_t run = 0;
  for (int e = 0; e < E; ++e) {
    cursor[e] = run;
    run += m_sizes[e];
  }
  for (int64_t i = 0; i < n; ++i)
    if (flat_ids[i] >= 0 && flat_ids[i] < E) perm[cursor[flat_ids[i]]++] = (int32_t)i;
  for (int64_t i = run; i < n; ++i) perm[i] = -1;
  free(cursor);
}

/* Padded form of the same grouping, exactly as the docstring of moe_align_block_size describes it
 * (v0_moe_fused.py:141-166): each expert's run is padded with the value n up to a multiple of
 * block_size; expert_ids holds the expert of every block. Exists so that the docstring's worked
 * example can pin orc_route's ordering. sorted_ids must hold n + E*(block_size-1) entries. */
void orc_moe_align_block_size(const int32_t* flat_ids, int64_t n, int E, int block_size,
                              int32_t* sorted_ids, int32_t* expert_ids, int32_t* num_post_pad) {
  int32_t* perm = (int32_t*)malloc(sizeof(int32_t) * (size_t)(n > 0 ? n : 1));
  int32_t* cnt = (int32_t*)malloc(sizeof(int32_t) * (size_t)E);
  orc_route(flat_ids, n, E, perm, cnt);
  int64_t o = 0, src = 0, blk = 0;
  for (int e = 0; e < E; ++e) {
    int padded = (cnt[e] + block_size - 1) / block_size * block_size;
    for (int i = 0; i < padded; ++i) sorted_ids[o++] = i < cnt[e] ? perm[src + i] : (int32_t)n;
    for (int b = 0; b < padded / block_size; ++b) expert_ids[blk++] = e;
    src += cnt[e];
  }
  *num_post_pad = (int32_t)o;
  free(perm);
  free(cnt);
}

/* ---- W4A16 dequantisation -----------------------------------------------------------------------
 * kernels/triton/inference/gptq/splitk_dequant_gemm.py:56-77:
 *   q(k, n) = (qweight[k / 8, n] >> 4 * (k % 8)) & 0xF        (8 nibbles along K, LSB = lowest k)
 *   z(g, n) = (qzeros[g, n / 8] >> 4 * (n % 8)) & 0xF         (8 nibbles along N), g = k / group
 *   w(k, n) = q * s(g, n) - (z + zero_offset) * s(g, n)
 * zero_offset = 1 is the reference's (AutoGPTQ v1) convention at :73-74; 0 gives (q - z) * s.
 * Pinned by: brute force on K=128, N=8 with an independent numpy bit-twiddling unpack; the all-equal
 * case q == z + zero_offset -> 0; q = 15, z = 0 -> 15 s. */
void orc_w4_dequant(const int32_t* qweight, const float* scales, const int32_t* qzeros, int K, int N,
                    int group_size, int zero_offset, float* w_out) {
  const int zcols = N / 8;
  for (int k = 0; k < K; ++k) {
    int g = k / group_size;
    for (int n = 0; n < N; ++n) {
      uint32_t qw = (uint32_t)qweight[(int64_t)(k / 8) * N + n];
      uint32_t zw = (uint32_t)qzeros[(int64_t)g * zcols + n / 8];
      int q = (int)((qw >> (4 * (k % 8))) & 0xFu);
      int z = (int)((zw >> (4 * (n % 8))) & 0xFu) + zero_offset;
      float s = scales[(int64_t)g * N + n];
      w_out[(int64_t)k * N + n] = (float)q * s - (float)z * s;
    }
  }
}

/* c[M, N] = a[M, K] @ w[K, N] with the dequantised weights (the dense product the reference's
 * split-K kernel accumulates with atomics, splitk_dequant_gemm.py:60-89). */
void orc_w4a16_gemm(const float* a, const int32_t* qweight, const float* scales, const int32_t* qzeros,
                    int M, int N, int K, int group_size, int zero_offset, float* c) {
  float* w = (float*)malloc(sizeof(float) * (size_t)K * (size_t)N);
  orc_w4_dequant(qweight, scales, qzeros, K, N, group_size, zero_offset, w);
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m) {
    double* acc = (double*)calloc((size_t)N, sizeof(double));
    for (int k = 0; k < K; ++k) {
      double av = a[(int64_t)m * K + k];
      const float* wr = w + (int64_t)k * N;
      for (int n = 0; n < N; ++n) acc[n] += av * (double)wr[n];
    }
    for (int n = 0; n < N; ++n) c[(int64_t)m * N + n] = (float)acc[n];
    free(acc);
  }
  free(w);
}

/* ---- fp8 e4m3fn (OCP: bias 7, no infinities, 0x7F/0xFF = NaN, max 448) ----------------------------
 * The element type the reference quantises to (float8_groupwise_quant.py:83, torch.float8_e4m3fn).
 * Pinned by: all 256 codes against torch's float8_e4m3fn -> float32 cast; encode against torch's
 * float32 -> float8_e4m3fn cast on random and boundary values. */
float orc_e4m3_to_f32(uint8_t v) {
  int sign = v >> 7, e = (v >> 3) & 0xF, m = v & 7;
  float r;
  if (e == 0xF && m == 7) return NAN;
  if (e == 0) r = ldexpf((float)m, -9);               /* subnormal: m / 8 * 2^-6 */
  else r = ldexpf(1.0f + (float)m / 8.0f, e - 7);
  return sign ? -r : r;
}

/* Round-to-nearest-even, saturating to +-448 (callers clamp first, as the reference does). */
uint8_t orc_f32_to_e4m3(float f) {
  if (isnan(f)) return 0x7F;
  uint8_t sign = signbit(f) ? 0x80 : 0;
  float a = fabsf(f);
  if (a >= 448.0f) return sign | 0x7E;
  if (a < ldexpf(1.0f, -10)) return sign;             /* below half the smallest subnormal */
  int e;
  (void)frexpf(a, &e);                                /* a = fr * 2^e, fr in [0.5, 1) */
  int exp = e - 1;                                    /* a = 1.x * 2^exp */
  if (exp < -6) exp = -6;                             /* subnormal range shares 2^-6 spacing / 8 */
  float q = ldexpf(a, 3 - exp);                       /* in units of the spacing: 8..16 (or 0..8) */
  float rq = nearbyintf(q);                           /* default rounding mode: nearest even */
  int iq = (int)rq;
  int biased = exp + 7;
  if (exp == -6 && iq < 8) return sign | (uint8_t)iq; /* subnormal */
  if (iq == 16) { iq = 8; biased += 1; }
  if (biased > 15 || (biased == 15 && iq - 8 > 6)) return sign | 0x7E;
  return sign | (uint8_t)(biased << 3) | (uint8_t)(iq - 8);
}

/* ---- 1 x block group-wise activation quantiser --------------------------------------------------
 * kernels/triton/inference/fp8/float8_groupwise_quant.py:36-50: per group of `block` consecutive
 * elements: s = max(amax|x|, 1e-12) / 448; q = clamp(x / s, -448, 448) -> e4m3fn; scale stored.
 * Pinned by: closed form on constructed groups (amax element maps to code 0x7E, zero group gives
 * s = 1e-12/448 and all-zero codes), round trip |q*s - x| <= s * 2^-4 * |q|. */
void orc_fp8_groupwise_quant(const float* x, int64_t numel, int block, uint8_t* q, float* scales) {
  int64_t groups = numel / block;
#pragma omp parallel for schedule(static)
  for (int64_t gi = 0; gi < groups; ++gi) {
    const float* xg = x + gi * block;
    float amax = 0.0f;
    for (int i = 0; i < block; ++i) amax = fmaxf(amax, fabsf(xg[i]));
    float s = fmaxf(amax, 1e-12f) / 448.0f;
    for (int i = 0; i < block; ++i) {
      float y = xg[i] / s;
      y = fminf(fmaxf(y, -448.0f), 448.0f);
      q[gi * block + i] = orc_f32_to_e4m3(y);
    }
    scales[gi] = s;
  }
}

/* 128 x 128 block quantiser for a [rows, K] weight matrix: one scale per (rows/128, K/128) block,
 * same scale and clamp rule as above (see the file header for its source).
 * Pinned by: a spike per block on a 2 x 3 grid of blocks (scale = |spike|/448 at [row block, K block],
 * code 0x7E / 0xFE at the spike, all-zero block -> 1e-12/448 and zero codes), numpy
 * reshape(rb,128,kb,128).max for the scales with torch's e4m3 cast for the codes, equality with
 * orc_fp8_groupwise_quant when every row of a block holds the block's amax, power-of-two equivariance. */
void orc_fp8_block_quant_weight(const float* w, int64_t rows, int K, int block, uint8_t* q, float* scales) {
  int64_t rb = rows / block;
  int kb = K / block;
  for (int64_t bi = 0; bi < rb; ++bi)
    for (int bj = 0; bj < kb; ++bj) {
      float amax = 0.0f;
      for (int i = 0; i < block; ++i)
        for (int j = 0; j < block; ++j) amax = fmaxf(amax, fabsf(w[(bi * block + i) * K + bj * block + j]));
      float s = fmaxf(amax, 1e-12f) / 448.0f;
      for (int i = 0; i < block; ++i)
        for (int j = 0; j < block; ++j) {
          int64_t idx = (bi * block + i) * K + bj * block + j;
          float y = fminf(fmaxf(w[idx] / s, -448.0f), 448.0f);
          q[idx] = orc_f32_to_e4m3(y);
        }
      scales[bi * kb + bj] = s;
    }
}

/* ---- fp8 grouped GEMM ---------------------------------------------------------------------------
 * scale_mode 0 (row-wise): y = (xq @ wq^T) * x_scale[m] * w_scale[g*N + n], the epilogue of
 * dev/triton_groupGEMM/groupgemm.py:374-384 and the oracle of testing/base_testing.py:83-88.
 * scale_mode 1 (block): x_scale is [M, K/128], w_scale is [G*N/128, K/128]; every 128-wide K block
 * is scaled by x_scale[m, kb] * w_scale[(g*N + n)/128, kb] before it is summed (dequantise, then the
 * bf16 oracle above).
 * Pinned by: all scales = 1 reduces to orc_grouped_gemm on the decoded values; row-wise closed form
 * of base_testing.py:83-88 evaluated with torch in float64. */
void orc_grouped_gemm_fp8(const uint8_t* xq, const uint8_t* wq, const float* x_scale, const float* w_scale,
                          int scale_mode, const int32_t* m_sizes, int G, int64_t M, int N, int K,
                          float* y, int64_t ldy, int col_block) {
  static float lut[256];
  for (int i = 0; i < 256; ++i) lut[i] = orc_e4m3_to_f32((uint8_t)i);
  const int kb = K / 128;
  int64_t off = 0;
  for (int g = 0; g < G; ++g) {
    int64_t m = m_sizes[g];
    if (m <= 0) continue;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i) {
      const uint8_t* xr = xq + (off + i) * K;
      float* yr = y + (off + i) * ldy + (int64_t)g * col_block;
      for (int n = 0; n < N; ++n) {
        const int64_t wrow = (int64_t)g * N + n;
        const uint8_t* wr = wq + wrow * K;
        double acc = 0.0;
        if (scale_mode == 0) {
          for (int k = 0; k < K; ++k) acc += (double)lut[xr[k]] * (double)lut[wr[k]];
          acc *= (double)x_scale[off + i];
          acc *= (double)w_scale[wrow];
        } else {
          for (int b = 0; b < kb; ++b) {
            double part = 0.0;
            for (int k = b * 128; k < (b + 1) * 128; ++k) part += (double)lut[xr[k]] * (double)lut[wr[k]];
            acc += part * (double)x_scale[(off + i) * kb + b] * (double)w_scale[(wrow / 128) * kb + b];
          }
        }
        yr[n] = (float)acc;
      }
    }
    off += m;
  }
  (void)M;
}

/* fp32 -> bf16 -> fp32 with round-to-nearest-even; the rounding of the final store of the GEMM
 * kernels (the reference casts the fp32 accumulator to the output dtype, groupgemm.py:244).
 * Pinned by: torch's float32 -> bfloat16 cast. */
float orc_round_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return f; /* NaN */
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7FFFu + lsb;
  u &= 0xFFFF0000u;
  float r;
  memcpy(&r, &u, 4);
  return r;
}

/* ---- SiLU-and-mul ------------------------------------------------------------------------------
 * ops.silu_and_mul as used by kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:284 and
 * SiluAndMul in test_moe_gemm.py:29: out[r, c] = silu(in[r, c]) * in[r, n + c], silu(v) = v / (1 + e^-v).
 * Pinned by: torch.nn.functional.silu on the CPU and the closed-form values silu(0) = 0,
 * silu(v) - silu(-v) = v. */
void orc_silu_and_mul(const float* in, int64_t rows, int n, float* out) {
  for (int64_t r = 0; r < rows; ++r)
    for (int c = 0; c < n; ++c) {
      double g = in[r * 2 * n + c], u = in[r * 2 * n + n + c];
      out[r * n + c] = (float)(g / (1.0 + exp(-g)) * u);
    }
}

/* ---- whole MoE layer ----------------------------------------------------------------------------
 * torch_moe of kernels/triton/inference/col_major_moe_gemm/test_moe_gemm.py:16-30:
 *   out[t] = sum_j topk_weight[t, j] * ( silu_and_mul(a[t] @ w1[e]^T) @ w2[e]^T ),  e = topk_ids[t, j].
 * a [T, K], w1 [E, 2n, K], w2 [E, d, n], out [T, d]; double accumulation. With round_intermediate != 0
 * the two intermediate activations and the second product are rounded to bf16 where the layer stores
 * them (the reference stores them in the activation dtype: intermediate_cache1..3, v0_moe_fused.py:266-274).
 * Ids outside [0, E) contribute nothing.
 * Pinned by: a torch float64 restatement with library matmuls on random inputs, and the special cases
 * k = 1 with weight 1 (one expert's MLP) and w2 = 0 (zero output). */
void orc_fused_moe(const float* a, const float* w1, const float* w2, const float* topk_weight,
                   const int32_t* topk_ids, int64_t T, int K, int E, int n, int d, int k, int round_intermediate,
                   float* out) {
  float* h1 = (float*)malloc(sizeof(float) * 2 * (size_t)n);
  float* h2 = (float*)malloc(sizeof(float) * (size_t)n);
  for (int64_t t = 0; t < T; ++t) {
    for (int c = 0; c < d; ++c) out[t * d + c] = 0.f;
    double* accum = (double*)calloc((size_t)d, sizeof(double));
    for (int j = 0; j < k; ++j) {
      int e = topk_ids[t * k + j];
      if (e < 0 || e >= E) continue;
      const float* w1e = w1 + (size_t)e * 2 * n * K;
      const float* w2e = w2 + (size_t)e * d * n;
      for (int c = 0; c < 2 * n; ++c) {
        double s = 0.0;
        for (int q = 0; q < K; ++q) s += (double)a[t * K + q] * (double)w1e[(size_t)c * K + q];
        h1[c] = round_intermediate ? orc_round_bf16((float)s) : (float)s;
      }
      orc_silu_and_mul(h1, 1, n, h2);
      if (round_intermediate)
        for (int c = 0; c < n; ++c) h2[c] = orc_round_bf16(h2[c]);
      for (int c = 0; c < d; ++c) {
        double s = 0.0;
        for (int q = 0; q < n; ++q) s += (double)h2[q] * (double)w2e[(size_t)c * n + q];
        float y = round_intermediate ? orc_round_bf16((float)s) : (float)s;
        accum[c] += (double)topk_weight[t * k + j] * (double)y;
      }
    }
    for (int c = 0; c < d; ++c) out[t * d + c] = (float)accum[c];
    free(accum);
  }
  free(h1);
  free(h2);
}
