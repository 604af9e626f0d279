// Tile scheduler for the grouped GEMM: walks the m_sizes offset table.
//
// Restates the persistent tile walk of the reference kernel
// (dev/triton_groupGEMM/groupgemm.py:159-254): groups are visited in order, empty groups
// contribute no tiles, and inside a group the linear tile index runs M-fastest
// (tile_m = idx % num_m_tiles, tile_n = idx / num_m_tiles; groupgemm.py:190-191).
// Instead of every workgroup re-scanning all G sizes per tile, two exclusive prefix tables
// are built once per launch (row offsets = groupgemm.py:161-165's running M offset, and tile
// offsets) and a tile id is mapped to its group with a binary search.
//
// The same code compiles for the host (used by the scheduler tests) and the device.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define MOE_GG_HD __host__ __device__ inline
#else
#define MOE_GG_HD inline
#endif

struct MoeGgTile {
  int g;      // group (expert) index
  int tm;     // tile index along the group's rows
  int tn;     // tile index along N
  int row0;   // first row of the group in x / y
  int rows;   // number of rows of the group (m_sizes[g] after clamping)
};

// Rows a group may use: negative sizes count as empty and the running sum never passes M,
// so a corrupt m_sizes cannot make a kernel read or write out of bounds.
MOE_GG_HD int moe_gg_clamp_rows(int m, int64_t row0, int64_t M) {
  if (m < 0) m = 0;
  int64_t left = M - row0;
  if (left < 0) left = 0;
  return (int64_t)m > left ? (int)left : m;
}

MOE_GG_HD int moe_gg_cdiv(int a, int b) { return (a + b - 1) / b; }

// Serial construction of both tables; row_off and tile_off have G + 1 entries.
// Returns the total number of tiles.
MOE_GG_HD int moe_gg_build_tables(const int32_t* m_sizes, int G, int64_t M, int BM, int n_tiles_n,
                                  int32_t* row_off, int32_t* tile_off) {
  int64_t r = 0;
  int t = 0;
  for (int g = 0; g < G; ++g) {
    row_off[g] = (int32_t)r;
    tile_off[g] = t;
    int m = moe_gg_clamp_rows(m_sizes[g], r, M);
    r += m;
    t += moe_gg_cdiv(m, BM) * n_tiles_n;
  }
  row_off[G] = (int32_t)r;
  tile_off[G] = t;
  return t;
}

// Largest g with tile_off[g] <= L, skipping empty groups (their range is empty). L < tile_off[G].
MOE_GG_HD int moe_gg_find_group(const int32_t* tile_off, int G, int L) {
  int lo = 0, hi = G;  // invariant: tile_off[lo] <= L < tile_off[hi]
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (tile_off[mid] <= L) lo = mid; else hi = mid;
  }
  return lo;
}

MOE_GG_HD MoeGgTile moe_gg_decode_tile(const int32_t* row_off, const int32_t* tile_off, int G, int L,
                                       int BM) {
  MoeGgTile t;
  t.g = moe_gg_find_group(tile_off, G, L);
  t.row0 = row_off[t.g];
  t.rows = row_off[t.g + 1] - t.row0;
  int idx = L - tile_off[t.g];
  int nmt = moe_gg_cdiv(t.rows, BM);
  t.tm = idx % nmt;
  t.tn = idx / nmt;
  return t;
}

// Linear tile id handled by persistent workgroup `wg` (of `nwg`, a multiple of `xcds`) in round
// `round`. Workgroups are dealt to the chip's XCDs round-robin (wg % xcds), each XCD with a
// private L2; giving an XCD a contiguous run of nwg / xcds tile ids per round makes the
// workgroups that share an L2 also share weight and activation tiles.
MOE_GG_HD int moe_gg_tile_of(int wg, int nwg, int xcds, int round) {
  int per = nwg / xcds;
  return round * nwg + (wg % xcds) * per + wg / xcds;
}

// ---- Two-list order of the ping-pong kernel ---------------------------------------------------------
// Row tiles of a group that go into the list of long tiles. A tile of fewer than BM / 2 rows is a low tile
// (it streams its whole weight tile for a few rows: bound by memory, not by the matrix pipes) and goes into
// the second list when nothing is lost by taking it away from its neighbours: when it is the only row tile of
// its group, or the last one of a group with at least two full tiles before it. (Next to its full neighbours a
// low tile finds their weight slabs in the L2; away from them it reads them again, which only pays for tall
// groups, where the better balance is worth more than one more pass over the group's weights.)
MOE_GG_HD int moe_gg_long_row_tiles(int rows, int BM) {
  const int full = rows / BM, rem = rows - full * BM;
  if (full == 0) return rem >= BM / 2 ? 1 : 0;
  return full + ((rem >= BM / 2 || (rem > 0 && full < 2)) ? 1 : 0);
}
MOE_GG_HD int moe_gg_low_row_tiles(int rows, int BM) { return moe_gg_cdiv(rows, BM) - moe_gg_long_row_tiles(rows, BM); }

// A workgroup's own sequence of n_my tiles, n_low_my of them low: its long tiles in round order with its low
// tiles spread evenly between them. Returns the number of low tiles among the first i sequence positions;
// low tile j sits at position floor((j + phase / 256) * n_my / n_low_my), 0 <= phase < 256.
MOE_GG_HD int moe_gg_low_before(int i, int n_my, int n_low_my, int phase) {
  if (n_low_my == 0) return 0;
  const long long den = 256LL * n_my;
  const long long num = (long long)i * n_low_my * 256 - (long long)phase * n_my;
  const long long c = num <= 0 ? 0 : (num + den - 1) / den;
  return c < n_low_my ? (int)c : n_low_my;
}
// Phase of a workgroup: the same for all workgroups of an XCD (they take their low tiles together and stay in
// step), different between XCDs (memory-bound and compute-bound tiles then run side by side on the chip).
MOE_GG_HD int moe_gg_low_phase(int wg, int xcds) { return ((wg % xcds) * 256 + 128) / xcds; }

// Round (argument of moe_gg_tile_of over the concatenated list: long tiles, then low tiles) of sequence
// position seq. The kernel tabulates a workgroup's sequence, which may have at most MOE_GG_SEQ_CAP positions;
// moe_gg_two_list_fits tells a launcher, from the shape alone, whether that holds for every m_sizes.
#define MOE_GG_SEQ_CAP 1024
MOE_GG_HD int moe_gg_seq_round(int seq, int n_my, int n_low_my, int phase) {
  const int lb = moe_gg_low_before(seq, n_my, n_low_my, phase);
  const bool low = moe_gg_low_before(seq + 1, n_my, n_low_my, phase) > lb;
  return low ? (n_my - n_low_my) + lb : seq - lb;
}
// Upper bound of the tile count: sum of ceil(m_g / BM) <= M / BM + G row tiles, times the column tiles (a last
// round cut into pieces has at most num_wg ids). Row offsets inside a group are tabulated in units of 64 rows
// in 16 bits, column offsets in units of 32.
MOE_GG_HD bool moe_gg_two_list_fits(int64_t M, int G, int BM, int n_tiles_n, int num_wg) {
  return M < (1 << 22) && (int64_t)n_tiles_n * BM < (1 << 21) &&
         (M / BM + G) * (int64_t)n_tiles_n <= (int64_t)(MOE_GG_SEQ_CAP - 2) * num_wg;
}

// Tail split. With n_long long tiles on num_wg workgroups the last round holds n_long % num_wg tiles; when it is
// at most half full, each of its tiles is cut into 2 or 4 pieces of rows (multiples of 64) that different
// workgroups compute, so the round takes about a half or a quarter as long (a piece loads its whole weight tile
// but runs only its share of the MFMAs). Ids: 0 .. first - 1 whole tiles, then pieces: first + t * s + piece.
MOE_GG_HD int moe_gg_tail_pieces(int n_long, int num_wg) {
  const int tail = n_long % num_wg;
  if (tail == 0 || tail * 2 > num_wg) return 1;
  return tail * 4 <= num_wg ? 4 : 2;
}
MOE_GG_HD int moe_gg_tail_first(int n_long, int num_wg) {
  return moe_gg_tail_pieces(n_long, num_wg) == 1 ? n_long : n_long - n_long % num_wg;
}
MOE_GG_HD int moe_gg_long_ids(int n_long, int num_wg) {
  const int first = moe_gg_tail_first(n_long, num_wg);
  return first + (n_long - first) * moe_gg_tail_pieces(n_long, num_wg);
}
// Low tiles left to the small-M kernel. A low tile keeps its workgroup busy for all K steps at the pace of the
// loads (about half the time of a full tile) however few rows it has; when the low tiles are few and do not fit
// into the free workgroups of the last round of long tiles, they would add a round that most CUs sit out. The
// small-M kernel (32 rows per pass, every CU streaming) computes those rows faster as long as its passes re-read
// less than about 3/8 of a round's weight tiles. low_passes: sum over the low tiles of ceil(rows / 32).
#define MOE_GG_TAIL_PASS_ROWS 32
MOE_GG_HD int moe_gg_low_passes(int rows, int BM) {
  return moe_gg_low_row_tiles(rows, BM) * moe_gg_cdiv(rows % BM, MOE_GG_TAIL_PASS_ROWS);
}
MOE_GG_HD bool moe_gg_tails_apart(int n_long, int n_low, long long low_passes, int num_wg) {
  if (n_low <= 0 || low_passes * 8 > (long long)num_wg * 3) return false;
  const int used = moe_gg_long_ids(n_long, num_wg) % num_wg;
  return n_low > (used == 0 ? 0 : num_wg - used);
}

// Piece p of s of a tile with rv valid rows (BM = 256): first row and number of rows (0 if the tile is too low).
MOE_GG_HD void moe_gg_piece_rows(int rv, int s, int p, int* off, int* h) {
  const int per = 256 / s;
  *off = p * per;
  const int left = rv - *off;
  *h = left < 0 ? 0 : (left > per ? per : left);
}

// ---- Split tails -----------------------------------------------------------------------------------
// A tall group (at least two full row tiles) whose last rows are few (at most BM / 4) does not get a full tile plus a
// low tile of those few rows (1 + about 0.6 tile times, the low tile bound by its K steps' load latency, not by its
// rows), but two tiles of about half height: the last BM + rem rows are cut into BM / 2 and BM / 2 + rem rows
// (about 0.55 tile times each). Both go into the second list, next to each other, so that they run at the same time
// on one XCD and share their weight slabs in its L2. `split` switches the rule on; with it off the functions below
// are moe_gg_long_row_tiles / moe_gg_low_row_tiles (the lists of a launch whose low tiles go to the small-M kernel).
MOE_GG_HD bool moe_gg_split_tail(int rows, int BM) {
  const int full = rows / BM, rem = rows - full * BM;
  return full >= 2 && rem > 0 && rem * 4 <= BM;
}
MOE_GG_HD int moe_gg_long_row_tiles2(int rows, int BM, bool split) {
  return split && moe_gg_split_tail(rows, BM) ? rows / BM - 1 : moe_gg_long_row_tiles(rows, BM);
}
MOE_GG_HD int moe_gg_low_row_tiles2(int rows, int BM, bool split) {
  return split && moe_gg_split_tail(rows, BM) ? 2 : moe_gg_low_row_tiles(rows, BM);
}

// Row pieces of the last round of long tiles when a second list follows it: the ids after the last full round are
// P pieces of cost a (tail * s pieces of a tile, or the tail tiles themselves), then n_low tiles of the second list
// of cost b, dealt round-robin; s in {1, 2, 4} (s > 1 only if tail * s <= num_wg) is chosen for the smallest load of
// the busiest workgroup. Costs in hundredths of a full tile, from timings of row pieces and low tiles.
#define MOE_GG_COST_FULL 100
#define MOE_GG_COST_HALF 55
#define MOE_GG_COST_QUARTER 43
#define MOE_GG_COST_LOW 58
MOE_GG_HD int moe_gg_rr_max_load(int P, int a, int Q, int b, int n) {
  // load(w) = a * (P / n + (w < P % n)) + b * #{i < Q : (P + i) % n == w}; the maximum is at one of a few w.
  const int s0 = P % n;
  int best = 0;
  const int cand[5] = {0, s0, (s0 + n - 1) % n, (int)(((long long)P + Q - 1 + n) % n), (int)(((long long)P + Q) % n)};
  for (int c = 0; c < 5; ++c) {
    const int w = cand[c];
    const int d = (w - s0 + n) % n;
    const int low = Q > d ? (Q - d - 1) / n + 1 : 0;
    const int load = a * (P / n + (w < s0 ? 1 : 0)) + b * low;
    if (load > best) best = load;
  }
  return best;
}
MOE_GG_HD int moe_gg_tail_pieces_low(int n_long, int n_low, int num_wg) {
  const int tail = n_long % num_wg;
  if (tail == 0) return 1;
  int best_s = 1, best = moe_gg_rr_max_load(tail, MOE_GG_COST_FULL, n_low, MOE_GG_COST_LOW, num_wg);
  if (tail * 2 <= num_wg) {
    const int l2 = moe_gg_rr_max_load(tail * 2, MOE_GG_COST_HALF, n_low, MOE_GG_COST_LOW, num_wg);
    if (l2 < best) { best = l2; best_s = 2; }
  }
  if (tail * 4 <= num_wg) {
    const int l4 = moe_gg_rr_max_load(tail * 4, MOE_GG_COST_QUARTER, n_low, MOE_GG_COST_LOW, num_wg);
    if (l4 < best) { best = l4; best_s = 4; }
  }
  return best_s;
}
MOE_GG_HD int moe_gg_tail_first_s(int n_long, int num_wg, int s) { return s == 1 ? n_long : n_long - n_long % num_wg; }
MOE_GG_HD int moe_gg_long_ids_s(int n_long, int num_wg, int s) {
  const int first = moe_gg_tail_first_s(n_long, num_wg, s);
  return first + (n_long - first) * s;
}

// Tile or row piece with id L of the two-list order: ids 0 .. long_ids - 1 are the long tiles (group, then column
// tile, then row tile; the last round cut into tail_s pieces each from id tail_first on), the ids after them the
// second list (group, then column tile, then the group's one or two tiles). long_off / low_off: prefix tables of
// the tile counts of the two lists per group. The same code decodes on the device and in the host mirror. A tile
// never reaches beyond its group's rows, whatever the tables hold (h is cut, and m0 falls back to the group's
// first row): the kernels load from row m0 also when h is 0.
struct MoeGgListTile { int g, m0, h, n0; };
MOE_GG_HD MoeGgListTile moe_gg_two_list_decode(const int32_t* row_off, const int32_t* long_off, const int32_t* low_off,
                                               int G, int L, int long_ids, int tail_first, int tail_s, int BM, int TC,
                                               bool split) {
  MoeGgListTile t;
  int rows;
  if (L < long_ids) {
    int piece = 0;
    if (L >= tail_first) {  // a piece of a tile of the last round
      piece = (L - tail_first) % tail_s;
      L = tail_first + (L - tail_first) / tail_s;
    }
    t.g = moe_gg_find_group(long_off, G, L);
    const int idx = L - long_off[t.g];
    rows = row_off[t.g + 1] - row_off[t.g];
    int nf = moe_gg_long_row_tiles2(rows, BM, split);
    if (nf < 1) nf = 1;
    const int tn = idx / nf;
    t.n0 = tn * TC;
    t.m0 = (idx - tn * nf) * BM;
    t.h = rows - t.m0 < BM ? rows - t.m0 : BM;
    if (tail_s > 1 && L >= tail_first) {
      int off;
      moe_gg_piece_rows(t.h, tail_s, piece, &off, &t.h);
      if (t.h > 0) t.m0 += off;  // a piece without rows keeps the tile's first row: its loads must stay in bounds
    }
  } else {
    const int Lp = L - long_ids;
    t.g = moe_gg_find_group(low_off, G, Lp);
    rows = row_off[t.g + 1] - row_off[t.g];
    const int idx = Lp - low_off[t.g];
    if (split && moe_gg_split_tail(rows, BM)) {
      const int tn = idx >> 1, half = idx & 1;
      t.n0 = tn * TC;
      t.m0 = (rows / BM - 1) * BM + half * (BM / 2);
      t.h = half ? rows - t.m0 : BM / 2;
    } else {
      t.n0 = idx * TC;
      t.m0 = rows / BM * BM;
      t.h = rows - t.m0;
    }
  }
  if (t.h < 0) t.h = 0;
  if (t.m0 < 0 || t.m0 >= rows) { t.m0 = 0; t.h = 0; }
  if (t.m0 + t.h > rows) t.h = rows - t.m0;
  if (t.h > BM) t.h = BM;
  return t;
}

// ---- Tall tiles ------------------------------------------------------------------------------------
// Lists of a kernel whose tiles may hold up to BM + MOE_GG_TALL_ROWS rows: a group with at least one full row tile and
// at most MOE_GG_TALL_ROWS rows behind its last one gets no tile for those rows; its last full tile takes them along.
// (Such a tail would otherwise stream the group's whole weight tile a second time, for a few rows, in every column
// tile.) Everything else is the two-list order above without split tails.
#define MOE_GG_TALL_ROWS 32
MOE_GG_HD bool moe_gg_tall_tail(int rows, int BM) {
  const int full = rows / BM, rem = rows - full * BM;
  return full >= 1 && rem > 0 && rem <= MOE_GG_TALL_ROWS;
}
MOE_GG_HD int moe_gg_long_row_tiles_tall(int rows, int BM) {
  return moe_gg_tall_tail(rows, BM) ? rows / BM : moe_gg_long_row_tiles(rows, BM);
}
MOE_GG_HD int moe_gg_low_row_tiles_tall(int rows, int BM) {
  return moe_gg_tall_tail(rows, BM) ? 0 : moe_gg_low_row_tiles(rows, BM);
}
// moe_gg_two_list_decode for these lists: h may reach BM + MOE_GG_TALL_ROWS; of a tall tile cut into row pieces the
// last piece takes the extra rows.
MOE_GG_HD MoeGgListTile moe_gg_two_list_decode_tall(const int32_t* row_off, const int32_t* long_off, const int32_t* low_off,
                                                    int G, int L, int long_ids, int tail_first, int tail_s, int BM, int TC) {
  MoeGgListTile t;
  int rows;
  if (L < long_ids) {
    int piece = 0;
    if (L >= tail_first) {  // a piece of a tile of the last round
      piece = (L - tail_first) % tail_s;
      L = tail_first + (L - tail_first) / tail_s;
    }
    t.g = moe_gg_find_group(long_off, G, L);
    const int idx = L - long_off[t.g];
    rows = row_off[t.g + 1] - row_off[t.g];
    int nf = moe_gg_long_row_tiles_tall(rows, BM);
    if (nf < 1) nf = 1;
    const int tn = idx / nf;
    t.n0 = tn * TC;
    t.m0 = (idx - tn * nf) * BM;
    t.h = rows - t.m0 < BM ? rows - t.m0 : BM;
    if (moe_gg_tall_tail(rows, BM) && t.m0 + BM == rows / BM * BM) t.h = rows - t.m0;  // the last full tile and the tail
    if (tail_s > 1 && L >= tail_first) {
      const int rv = t.h;
      int off;
      moe_gg_piece_rows(rv < BM ? rv : BM, tail_s, piece, &off, &t.h);
      if (piece == tail_s - 1 && rv > BM) t.h += rv - BM;
      if (t.h > 0) t.m0 += off;  // a piece without rows keeps the tile's first row: its loads must stay in bounds
    }
  } else {
    const int Lp = L - long_ids;
    t.g = moe_gg_find_group(low_off, G, Lp);
    rows = row_off[t.g + 1] - row_off[t.g];
    t.n0 = (Lp - low_off[t.g]) * TC;
    t.m0 = rows / BM * BM;
    t.h = rows - t.m0;
  }
  if (t.h < 0) t.h = 0;
  if (t.m0 < 0 || t.m0 >= rows) { t.m0 = 0; t.h = 0; }
  if (t.m0 + t.h > rows) t.h = rows - t.m0;
  if (t.h > BM + MOE_GG_TALL_ROWS) t.h = BM + MOE_GG_TALL_ROWS;
  return t;
}

