// Token -> expert routing for the grouped GEMM: top-k, expert histogram, offsets, stable grouping, gather.
//
// Replaces what the reference's MoE tests do with torch.topk
// (kernels/triton/inference/col_major_moe_gemm/test_moe_gemm.py:54-57) and the external
// moe_align_block_size op whose semantics are given in
// kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:141-166 (without its padding):
//   ids      = top-k expert ids per token, descending score, ties to the lower expert id
//   flat     = ids.reshape(-1)                       (position p = token * k + j)
//   perm     = stable argsort(flat)                  (rows grouped by ascending expert)
//   m_sizes  = bincount(flat, minlength = E)
//   offsets  = exclusive prefix sum of m_sizes       (groupgemm.py:159-165 / tgroup_gemm_backwards.py:471-477)
//   x_sorted = x[perm // k]
// All of it is integer / index work and bit-exact against the CPU oracle.
#include "common.h"
#include "gg_tables.h"
#include "kernels.h"

namespace {

// ---- top-k: one wave per token; lane l holds experts l, l + 64, ... -------------------------------
constexpr int TOPK_MAX_PER_LANE = 16;  // E <= 1024

__global__ __launch_bounds__(256) void route_topk_kernel(const float* __restrict__ logits, int T, int E, int k,
                                                         int32_t* __restrict__ ids) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;
  const float* row = logits + (int64_t)t * E;
  float v[TOPK_MAX_PER_LANE];
#pragma unroll
  for (int i = 0; i < TOPK_MAX_PER_LANE; ++i) {
    const int e = lane + 64 * i;
    v[i] = e < E ? row[e] : -__builtin_inff();
  }
  uint32_t taken = 0;
  for (int j = 0; j < k; ++j) {
    // local best: larger value wins, equal values keep the lower expert id (lower i)
    float bv = -__builtin_inff();
    int be = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < TOPK_MAX_PER_LANE; ++i) {
      const int e = lane + 64 * i;
      const bool ok = e < E && !((taken >> i) & 1u);
      if (ok && (be == 0x7fffffff || v[i] > bv)) { bv = v[i]; be = e; }
    }
    // wave arg-max with the same tie rule
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
      const float ov = __shfl_xor(bv, d, 64);
      const int oe = __shfl_xor(be, d, 64);
      const bool other = oe != 0x7fffffff && (be == 0x7fffffff || ov > bv || (ov == bv && oe < be));
      if (other) { bv = ov; be = oe; }
    }
    if (lane == 0) ids[(int64_t)t * k + j] = be;
    if ((be & 63) == lane) taken |= 1u << (be >> 6);
  }
}

// ---- stable grouping by expert: a single workgroup of 16 waves --------------------------------------
// Wave w owns the contiguous segment [w * seg, (w + 1) * seg) of the flat id list.
//  1. per-wave expert histograms in LDS;
//  2. per expert: exclusive prefix over the waves (-> start of each wave's run inside the expert) and total;
//  3. exclusive prefix over experts -> offsets;
//  4. every wave walks its segment 64 entries at a time in order: lanes holding the same expert are found
//     with one ballot per id bit, ranked by lane position, and placed after the entries counted so far.
constexpr int GROUP_WAVES = 16;

__global__ __launch_bounds__(64 * GROUP_WAVES) void route_group_kernel(const int32_t* __restrict__ flat, int n, int E,
                                                                        int32_t* __restrict__ perm,
                                                                        int32_t* __restrict__ m_sizes,
                                                                        int32_t* __restrict__ offsets) {
  extern __shared__ int32_t sh[];          // [GROUP_WAVES][E] counters, then [E + 1] offsets
  int32_t* cnt = sh;
  int32_t* off = sh + GROUP_WAVES * E;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int seg = (n + GROUP_WAVES - 1) / GROUP_WAVES;
  const int lo = min(wave * seg, n), hi = min(lo + seg, n);

  for (int i = tid; i < GROUP_WAVES * E; i += blockDim.x) cnt[i] = 0;
  __syncthreads();
  for (int p = lo + lane; p < hi; p += 64) {
    const int e = flat[p];
    if (e >= 0 && e < E) atomicAdd(&cnt[wave * E + e], 1);
  }
  __syncthreads();
  for (int e = tid; e < E; e += blockDim.x) {
    int run = 0;
    for (int w = 0; w < GROUP_WAVES; ++w) {
      const int c = cnt[w * E + e];
      cnt[w * E + e] = run;
      run += c;
    }
    off[e + 1] = run;  // totals, turned into offsets below
    m_sizes[e] = run;
  }
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    off[0] = 0;
    for (int e = 0; e < E; ++e) {
      run += off[e + 1];
      off[e + 1] = run;
    }
  }
  __syncthreads();
  if (offsets)
    for (int e = tid; e <= E; e += blockDim.x) offsets[e] = off[e];

  int bits = 0;
  while ((1 << bits) < E) ++bits;
  for (int base = lo; base < hi; base += 64) {
    const int p = base + lane;
    const bool live = p < hi;
    int e = live ? flat[p] : -1;
    if (e < 0 || e >= E) e = -1;  // ids outside [0, E) are dropped (not written to perm)
    unsigned long long match = __ballot(e >= 0);
    for (int b = 0; b < bits; ++b) {
      const unsigned long long m = __ballot((e >> b) & 1);
      match &= ((e >> b) & 1) ? m : ~m;
    }
    if (e >= 0) {
      const int rank = __popcll(match & ((1ull << lane) - 1ull));
      const int leader = __ffsll((long long)match) - 1;
      int start = 0;
      if (lane == leader) {
        start = cnt[wave * E + e];
        cnt[wave * E + e] = start + __popcll(match);
      }
      start = __shfl(start, leader, 64);
      perm[off[e] + start + rank] = p;
    }
  }
  // Dropped ids leave sum(m_sizes) < n: the unused tail of perm is -1, never stale memory.
  for (int i = off[E] + tid; i < n; i += blockDim.x) perm[i] = -1;
}

// ---- gather: out[i] = x[perm[i] / k], rows of row_bytes (multiple of 16) ----------------------------
// Positions at or beyond *n_valid (when given) and entries of perm that name no row of x (negative, or
// perm[i] / k >= src_rows) read nothing: their output row is zeros.
__global__ __launch_bounds__(256) void gather_rows_kernel(const char* __restrict__ x, const int32_t* __restrict__ perm,
                                                          int k, char* __restrict__ out, int n, int64_t row_bytes,
                                                          int64_t src_rows, const int32_t* __restrict__ n_valid) {
  const int i = blockIdx.x;
  if (i >= n) return;
  const int32_t pi = perm[i];
  const int64_t src = pi / k;
  const bool ok = pi >= 0 && src < src_rows && (!n_valid || i < *n_valid);
  u32x4_t* d = (u32x4_t*)(out + (int64_t)i * row_bytes);
  if (!ok) {
    const u32x4_t z = {0u, 0u, 0u, 0u};
    for (int64_t c = threadIdx.x; c < row_bytes / 16; c += blockDim.x) d[c] = z;
    return;
  }
  const u32x4_t* s = (const u32x4_t*)(x + src * row_bytes);
  for (int64_t c = threadIdx.x; c < row_bytes / 16; c += blockDim.x) d[c] = s[c];
}

// Padded form of the grouping (moe_align_block_size, kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:138-180):
// expert e's run of perm padded with the value n up to a multiple of block_size. Every workgroup rebuilds the two
// prefix tables (rows, padded rows) from m_sizes in LDS; thread i then writes sorted_ids[i] and expert_ids[i].
__global__ __launch_bounds__(256) void align_block_size_kernel(const int32_t* __restrict__ perm,
                                                               const int32_t* __restrict__ m_sizes, int E, int n,
                                                               int block_size, int32_t* __restrict__ sorted_ids,
                                                               int n_sorted, int32_t* __restrict__ expert_ids,
                                                               int n_blocks_cap, int32_t* __restrict__ num_post_pad) {
  __shared__ int32_t row_off[MOE_GG_MAX_GROUPS + 1];
  __shared__ int32_t pad_off[MOE_GG_MAX_GROUPS + 1];
  build_row_offsets(m_sizes, E, n, row_off);
  build_tile_prefix(row_off, E, pad_off, [&](int rows) { return moe_gg_cdiv(rows, block_size) * block_size; });
  const int total = pad_off[E];
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i == 0) num_post_pad[0] = total;
  if (i < n_sorted) {
    int v = n;
    if (i < total) {
      const int e = moe_gg_find_group(pad_off, E, i);
      const int j = i - pad_off[e];
      if (j < row_off[e + 1] - row_off[e]) v = perm[row_off[e] + j];
    }
    sorted_ids[i] = v;
  }
  if (i < n_blocks_cap) {
    const long long first = (long long)i * block_size;
    expert_ids[i] = first < total ? moe_gg_find_group(pad_off, E, (int)first) : -1;
  }
}

}  // namespace

hipError_t route_topk_launch(const float* logits, int T, int E, int k, int32_t* ids, hipStream_t stream) {
  if (T == 0) return hipSuccess;
  hipLaunchKernelGGL(route_topk_kernel, dim3((T + 3) / 4), dim3(256), 0, stream, logits, T, E, k, ids);
  return hipGetLastError();
}

hipError_t route_group_launch(const int32_t* flat, int n, int E, int32_t* perm, int32_t* m_sizes, int32_t* offsets,
                              hipStream_t stream) {
  const size_t lds = sizeof(int32_t) * ((size_t)GROUP_WAVES * E + E + 1);
  hipLaunchKernelGGL(route_group_kernel, dim3(1), dim3(64 * GROUP_WAVES), lds, stream, flat, n, E, perm, m_sizes, offsets);
  return hipGetLastError();
}

hipError_t gather_rows_launch(const void* x, const int32_t* perm, int k, void* out, int n, int64_t row_bytes,
                              int64_t src_rows, const int32_t* n_valid, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(gather_rows_kernel, dim3(n), dim3(256), 0, stream, (const char*)x, perm, k, (char*)out, n, row_bytes,
                     src_rows, n_valid);
  return hipGetLastError();
}

hipError_t align_block_size_launch(const int32_t* perm, const int32_t* m_sizes, int E, int n, int block_size,
                                   int32_t* sorted_ids, int32_t* expert_ids, int32_t* num_post_pad,
                                   hipStream_t stream) {
  const int n_sorted = n + E * (block_size - 1), n_blocks_cap = n + E;
  const int threads = n_sorted > n_blocks_cap ? n_sorted : n_blocks_cap;
  hipLaunchKernelGGL(align_block_size_kernel, dim3((threads + 255) / 256), dim3(256), 0, stream, perm, m_sizes, E, n,
                     block_size, sorted_ids, n_sorted, expert_ids, n_blocks_cap, num_post_pad);
  return hipGetLastError();
}
