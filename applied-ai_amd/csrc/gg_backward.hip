// Operand preparation for the backward pass of the grouped GEMM
// (kernels/MoE/group_GEMM/triton/tgroup_gemm_backwards.py:382-590; eager form
// kernels/MoE/group_GEMM/triton/testing/pytorch_reference_backwards.py:165-197):
//   grad_x[rows of g] = dY[rows of g, cols of g] @ w[g]              -> forward kernel on (dY, w[g]^T)
//   grad_w[g]         = dY[rows of g, cols of g]^T @ x[rows of g]    -> tiled kernel on (dY^T, x^T), reduction over rows
// The MFMA kernels want both operands contiguous along the reduction dimension, so the backward pass first
// transposes: w[g] [N, K] -> [K, N] per expert, and dY / x [rows, C] -> [C, padded rows] with every expert's rows
// padded to a multiple of 64 with zeros (its reduction is then a whole number of K steps). 64 x 64 tiles through
// LDS, 8-byte global accesses; HBM-bound byte movers.
#include "common.h"
#include "gg_tables.h"
#include "kernels.h"

namespace {

constexpr int TT = 64;  // tile edge


// Reads tile[r][c] = src[(r0 + r) * src_pitch + c0 + c] for r < rvalid, c < cvalid (zeros elsewhere) and writes
// dst[(dst_row0 + c0 + c) * dst_pitch + q0 + r] for c < cvalid and r < rstore. 256 threads; 16-byte global accesses
// where the addresses allow, 2-byte accesses elsewhere. tile: 64 rows of 33 dwords (64 values + padding).
DEVINL void transpose_tile(const uint16_t* __restrict__ src, int64_t src_pitch, int64_t r0, int c0, int rvalid, int cvalid,
                           uint16_t* __restrict__ dst, int64_t dst_row0, int64_t dst_pitch, int64_t q0, int rstore,
                           uint32_t (*tile)[TT / 2 + 1]) {
  const int tid = threadIdx.x;
  const int tr = tid >> 3, ch = (tid & 7) * 8;
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int r = pass * 32 + tr;
    u32x4_t q = {0u, 0u, 0u, 0u};
    if (r < rvalid) {
      const uint16_t* s = src + (r0 + r) * src_pitch + c0 + ch;
      if (ch + 7 < cvalid && (((uintptr_t)s) & 15) == 0) {
        q = *(const u32x4_t*)s;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (ch + e < cvalid) q[e >> 1] |= (uint32_t)s[e] << (16 * (e & 1));
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) tile[r][(ch >> 1) + j] = q[j];
  }
  __syncthreads();
  const uint16_t* th = (const uint16_t*)&tile[0][0];
  constexpr int PH = TT + 2;   // pitch of the tile in 16-bit values
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int c = pass * 32 + tr;   // row of dst
    if (c < cvalid) {
      uint16_t* d = dst + (dst_row0 + c0 + c) * dst_pitch + q0 + ch;
      uint16_t a[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) a[e] = th[(ch + e) * PH + c];
      if (ch + 7 < rstore && (((uintptr_t)d) & 15) == 0) {
        u32x4_t q;
#pragma unroll
        for (int j = 0; j < 4; ++j) q[j] = (uint32_t)a[2 * j] | ((uint32_t)a[2 * j + 1] << 16);
        *(u32x4_t*)d = q;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (ch + e < rstore) d[e] = a[e];
      }
    }
  }
}

// Batched plain transpose: src [B, R, C] -> dst [B, C, R]. Grid (ceil(R / 64), ceil(C / 64), B).
__global__ __launch_bounds__(256) void transpose_batched_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                                int R, int C) {
  __shared__ uint32_t tile[TT][TT / 2 + 1];
  const int b = blockIdx.z;
  const int r0 = blockIdx.x * TT, c0 = blockIdx.y * TT;
  // The last row tile may be partial: the columns of dst beyond R must not be written.
  const int rvalid = min(TT, R - r0), cvalid = min(TT, C - c0);
  transpose_tile(src + (int64_t)b * R * C, C, r0, c0, rvalid, cvalid, dst + (int64_t)b * R * C, 0, R, r0, rvalid, tile);
}

// Per-expert padded transpose: src rows are expert-sorted; expert g owns rows row_off[g] .. + m_g - 1 and, in src,
// columns g * col_block .. + C - 1 (col_block = 0: the same C columns for every expert). dst [C, ldm]:
// dst[c][pad_off[g] + i] = src[row_off[g] + i][g * col_block + c] for i < m_g, zero for m_g <= i < max(64, roundup(m_g, 64)).
// Grid (upper bound on the number of 64-row blocks, ceil(C / 64)); blocks beyond the real count exit.
__global__ __launch_bounds__(256) void transpose_padded_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                               const int32_t* __restrict__ m_sizes, int G, int M, int C,
                                                               int64_t src_pitch, int col_block, int64_t ldm) {
  __shared__ uint32_t tile[TT][TT / 2 + 1];
  __shared__ int32_t row_off[MOE_GG_MAX_GROUPS + 1];
  __shared__ int32_t blk_off[MOE_GG_MAX_GROUPS + 1];
  build_group_tables(m_sizes, G, M, TT, 1, row_off, blk_off, 0, 1);  // an expert without rows owns one block of zeros
  const int L = blockIdx.x;
  if (L >= blk_off[G]) return;
  const int g = moe_gg_find_group(blk_off, G, L);
  const int rb = L - blk_off[g];
  const int rows = row_off[g + 1] - row_off[g];
  const int c0 = blockIdx.y * TT;
  transpose_tile(src + (int64_t)g * col_block, src_pitch, (int64_t)row_off[g] + rb * TT, c0, min(TT, rows - rb * TT),
                 min(TT, C - c0), dst, 0, ldm, (int64_t)L * TT, TT, tile);
}

// dst[row_off[g] + i][c] = src[row_off[g] + i][g * col_block + c]: the expert's own column block of a [M, C * G]
// gradient as a contiguous [M, C] matrix. Grid (64-row blocks as in the padded transpose, ceil(C / 512)).
// C % 8 == 0 and 16-byte aligned rows (8-byte accesses otherwise: C % 4 == 0).
constexpr int CC = 512;
__global__ __launch_bounds__(256) void compact_block_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                            const int32_t* __restrict__ m_sizes, int G, int M, int C,
                                                            int64_t src_pitch, int col_block, int wide) {
  __shared__ int32_t row_off[MOE_GG_MAX_GROUPS + 1];
  __shared__ int32_t blk_off[MOE_GG_MAX_GROUPS + 1];
  build_group_tables(m_sizes, G, M, TT, 1, row_off, blk_off);
  const int L = blockIdx.x;
  if (L >= blk_off[G]) return;
  const int g = moe_gg_find_group(blk_off, G, L);
  const int rb = L - blk_off[g];
  const int rows = row_off[g + 1] - row_off[g];
  const int rvalid = min(TT, rows - rb * TT);
  const int64_t r0 = (int64_t)row_off[g] + rb * TT;
  const int c0 = blockIdx.y * CC;
  const int cw = min(CC, C - c0);
  const uint16_t* s = src + (int64_t)g * col_block + c0;
  uint16_t* d = dst + c0;
  if (wide) {
    const int per = cw / 8;
    for (int idx = threadIdx.x; idx < rvalid * per; idx += blockDim.x) {
      const int r = idx / per, c = (idx - r * per) * 8;
      *(u32x4_t*)(d + (r0 + r) * C + c) = *(const u32x4_t*)(s + (r0 + r) * src_pitch + c);
    }
  } else {
    const int per = cw / 4;
    for (int idx = threadIdx.x; idx < rvalid * per; idx += blockDim.x) {
      const int r = idx / per, c = (idx - r * per) * 4;
      *(u32x2_t*)(d + (r0 + r) * C + c) = *(const u32x2_t*)(s + (r0 + r) * src_pitch + c);
    }
  }
}

}  // namespace

hipError_t compact_block_launch(const void* src, void* dst, const int32_t* m_sizes, int G, int M, int C, int64_t src_pitch,
                                int col_block, hipStream_t stream) {
  if (C == 0 || M == 0) return hipSuccess;
  const int wide = C % 8 == 0 && src_pitch % 8 == 0 && col_block % 8 == 0 && (((uintptr_t)src | (uintptr_t)dst) & 15) == 0;
  hipLaunchKernelGGL(compact_block_kernel, dim3(M / TT + G, (C + CC - 1) / CC), dim3(256), 0, stream, (const uint16_t*)src,
                     (uint16_t*)dst, m_sizes, G, M, C, src_pitch, col_block, wide);
  return hipGetLastError();
}

hipError_t transpose_batched_launch(const void* src, void* dst, int B, int R, int C, hipStream_t stream) {
  if (B == 0 || R == 0 || C == 0) return hipSuccess;
  hipLaunchKernelGGL(transpose_batched_kernel, dim3((R + TT - 1) / TT, (C + TT - 1) / TT, B), dim3(256), 0, stream,
                     (const uint16_t*)src, (uint16_t*)dst, R, C);
  return hipGetLastError();
}

hipError_t transpose_padded_launch(const void* src, void* dst, const int32_t* m_sizes, int G, int M, int C,
                                   int64_t src_pitch, int col_block, int64_t ldm, hipStream_t stream) {
  if (C == 0 || ldm == 0) return hipSuccess;
  const int blocks = M / TT + G;  // >= sum over experts of ceil(m_g / 64)
  hipLaunchKernelGGL(transpose_padded_kernel, dim3(blocks, (C + TT - 1) / TT), dim3(256), 0, stream, (const uint16_t*)src,
                     (uint16_t*)dst, m_sizes, G, M, C, src_pitch, col_block, ldm);
  return hipGetLastError();
}
