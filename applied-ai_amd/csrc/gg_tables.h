// In-kernel construction of the row-offset and tile-offset tables of tile_sched.h.
// One wavefront scans m_sizes with a shuffle prefix sum; the result is identical to
// moe_gg_build_tables (row offsets are min(prefix, M), which equals the serial clamped walk).
#pragma once
#include "common.h"
#include "tile_sched.h"

DEVINL long long wave_incl_scan_i64(long long x) {
  const int l = lane_id();
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    long long v = __shfl_up(x, d, 64);
    if (l >= d) x += v;
  }
  return x;
}

// The n-th group (counted from 0) for which has_work(g) holds, or -1 if there are fewer. Called by all 64 lanes of
// one wave; every lane gets the answer.
template <class F>
DEVINL int nth_group(int G, int n, F has_work) {
  const int l = lane_id(), per = (G + 63) >> 6, g0 = l * per;
  int c = 0;
  for (int i = 0; i < per; ++i)
    if (g0 + i < G && has_work(g0 + i)) ++c;
  int incl = c;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int v = __shfl_up(incl, d, 64);
    if (l >= d) incl += v;
  }
  int found = -1;
  if (n >= incl - c && n < incl) {
    int k = n - (incl - c);
    for (int i = 0; i < per && found < 0; ++i)
      if (g0 + i < G && has_work(g0 + i) && k-- == 0) found = g0 + i;
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) found = max(found, __shfl_xor(found, d, 64));
  return found;
}

// Must be called by every thread of the workgroup (it ends with a barrier).
// row_off: LDS array of G + 1 entries, G <= MOE_GG_MAX_GROUPS: row_off[g] = min(sum of the clamped sizes before g, M).
DEVINL void build_row_offsets(const int32_t* __restrict__ m_sizes, int G, int M, int32_t* row_off) {
  const int per = (G + 63) >> 6;
  if (wave_id() == 0) {
    const int g0 = lane_id() * per;
    long long s = 0;
    for (int i = 0; i < per; ++i) {
      int g = g0 + i;
      if (g < G) {
        int m = m_sizes[g];
        m = m < 0 ? 0 : (m > M ? M : m);
        s += m;
      }
    }
    long long run = wave_incl_scan_i64(s) - s;
    for (int i = 0; i < per; ++i) {
      int g = g0 + i;
      if (g < G) {
        row_off[g] = (int32_t)(run > M ? M : run);
        int m = m_sizes[g];
        m = m < 0 ? 0 : (m > M ? M : m);
        run += m;
      }
    }
    if (lane_id() == 63) row_off[G] = (int32_t)(run > M ? M : run);
  }
  __syncthreads();
}

// tile_off[g] = sum over the groups before g of tiles_of(rows of the group); G + 1 entries. Needs row_off
// complete (build_row_offsets); every thread of the workgroup must call it (it ends with a barrier).
template <class F>
DEVINL void build_tile_prefix(const int32_t* row_off, int G, int32_t* tile_off, F tiles_of) {
  const int per = (G + 63) >> 6;
  if (wave_id() == 0) {
    const int g0 = lane_id() * per;
    long long s = 0;
    for (int i = 0; i < per; ++i) {
      int g = g0 + i;
      if (g < G) s += tiles_of(row_off[g + 1] - row_off[g]);
    }
    long long run = wave_incl_scan_i64(s) - s;
    for (int i = 0; i < per; ++i) {
      int g = g0 + i;
      if (g < G) {
        tile_off[g] = (int32_t)run;
        run += tiles_of(row_off[g + 1] - row_off[g]);
      }
    }
    if (lane_id() == 63) tile_off[G] = (int32_t)run;
  }
  __syncthreads();
}

// Groups with at most skip_rows rows keep their rows in row_off but get no tiles (another kernel
// of the same call computes them). min_tiles: lower bound of every group's tile count (also of an empty group).
DEVINL void build_group_tables(const int32_t* __restrict__ m_sizes, int G, int M, int BM, int n_tiles_n,
                               int32_t* row_off, int32_t* tile_off, int skip_rows = 0, int min_tiles = 0) {
  build_row_offsets(m_sizes, G, M, row_off);
  build_tile_prefix(row_off, G, tile_off, [&](int rows) {
    return max(min_tiles, rows > skip_rows ? moe_gg_cdiv(rows, BM) * n_tiles_n : 0);
  });
}
