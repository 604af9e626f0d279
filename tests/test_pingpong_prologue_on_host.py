"""The ping-pong kernels' prologue (which tiles a workgroup computes, in which order) run on the CPU: the statements
between two markers of applied-ai_amd/csrc/gg_pingpong.hip are compiled verbatim with g++ behind stand-ins for the
few device helpers they use (serial table builders, a loop over the thread ids), executed for every workgroup, and
compared with the host mirror of the C ABI (moe_gg_host_enumerate_tiles_two_lists) entry by entry, plus exact cover
where the mirror has no counterpart (launches whose low tiles go to the small-M kernel, fp8 launches that leave
small experts to the streaming kernel). What it cannot see is the K loop that consumes the table."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "applied-ai_amd", "csrc")
I32P = ctypes.POINTER(ctypes.c_int32)
CAP = 1 << 17

HARNESS_HEAD = r'''
#include <cstdio>
#include <cstdint>
#include <cstdlib>
#include <algorithm>
#include "tile_sched.h"
#define MOE_GG_MAX_GROUPS 1024
using std::min; using std::max;
constexpr int BM = 256, BN = 256, NT = 512, NTB = NT;
constexpr int OP_BF16 = 0, OP_FP8_ROW = 1, OP_FP8_BLOCK = 2, OP_BF16_WGRAD = 3, OP_BF16_SWIGLU = 4, OP_BF16_NT = 5,
              OP_BF16_WGRAD_DIRECT = 6, OP_F16 = 7, OP_F16_SWIGLU = 8, OP_BF16_SWIGLU_GATHER = 9, OP_F16_SWIGLU_GATHER = 10;
constexpr bool op_gather(int op) { return op == OP_BF16_SWIGLU_GATHER || op == OP_F16_SWIGLU_GATHER; }
constexpr bool op_swiglu(int op) { return op == OP_BF16_SWIGLU || op == OP_F16_SWIGLU || op_gather(op); }
struct GgParams { const int32_t* m_sizes; int G, M, N, K, skip_rows, tails_apart, xcds, split_tails; };
struct Dim { int x; };
static Dim blockIdx, threadIdx, gridDim;
static int uni(int v) { return v; }
static void __syncthreads() {}
static void build_row_offsets(const int32_t* m_sizes, int G, int M, int32_t* row_off) {
  long long run = 0;
  for (int g = 0; g < G; ++g) { row_off[g] = (int32_t)(run > M ? M : run); int m = m_sizes[g]; m = m < 0 ? 0 : (m > M ? M : m); run += m; }
  row_off[G] = (int32_t)(run > M ? M : run);
}
template <class F> static void build_tile_prefix(const int32_t* row_off, int G, int32_t* tile_off, F tiles_of) {
  long long run = 0;
  for (int g = 0; g < G; ++g) { tile_off[g] = (int32_t)run; run += tiles_of(row_off[g + 1] - row_off[g]); }
  tile_off[G] = (int32_t)run;
}
static void build_group_tables(const int32_t*, int, int, int, int, int32_t*, int32_t*, int, int) { abort(); }

template <int OP, bool TALL = false, bool LISTS2 = false>
static void prologue(const GgParams& p, int32_t* seq_out, int* n_my_out) {
  static int32_t row_off[MOE_GG_MAX_GROUPS + 1], tile_off[MOE_GG_MAX_GROUPS + 1], part_off[MOE_GG_MAX_GROUPS + 1];
  static int32_t seq_tab[2 * MOE_GG_SEQ_CAP];
  *n_my_out = 0;
  for (int tid = 0; tid < NT; ++tid) {  // every thread runs the whole prologue; its own table entries are kept
    threadIdx.x = tid;
'''
HARNESS_TAIL = r'''
    *n_my_out = n_my;
    for (int i = tid; i < n_my; i += NT) { seq_out[2 * i] = seq_tab[2 * i]; seq_out[2 * i + 1] = seq_tab[2 * i + 1]; }
  }
}

extern "C" int emu_prologue(int op, const int32_t* m_sizes, int G, int M, int N, int K, int skip_rows, int tails_apart,
                            int nwg, int xcds, int split_tails, int lists2, int32_t* out, int cap) {
  const bool tall = split_tails == 2;   // the four-wave kernel's lists with tiles of up to 256 + 32 rows
  GgParams p{m_sizes, G, M, N, K, skip_rows, tails_apart, xcds, tall ? 0 : split_tails};
  gridDim.x = nwg;
  static int32_t seq[2 * MOE_GG_SEQ_CAP];
  int written = 0;
  for (int wg = 0; wg < nwg; ++wg) {
    blockIdx.x = wg;
    int n_my = 0;
    // As the launchers choose: the first prologue for the kernels that run by default, the second one for the
    // split-tail order, the row gather and the four-wave kernels (lists2 = 1 forces it: those kernels also run the
    // plain two-list order through it).
    const bool second = lists2 || p.split_tails;
    if (op == OP_BF16 && tall) prologue<OP_BF16, true, true>(p, seq, &n_my);
    else if (op == OP_BF16_SWIGLU && tall) prologue<OP_BF16_SWIGLU, true, true>(p, seq, &n_my);
    else if (tall) return -1;
    else if (op == OP_BF16 && second) prologue<OP_BF16, false, true>(p, seq, &n_my);
    else if (op == OP_BF16) prologue<OP_BF16>(p, seq, &n_my);
    else if (op == OP_BF16_SWIGLU && second) prologue<OP_BF16_SWIGLU, false, true>(p, seq, &n_my);
    else if (op == OP_BF16_SWIGLU) prologue<OP_BF16_SWIGLU>(p, seq, &n_my);
    else if (op == OP_BF16_SWIGLU_GATHER) prologue<OP_BF16_SWIGLU_GATHER, false, true>(p, seq, &n_my);
    else if (op == OP_FP8_BLOCK && second) prologue<OP_FP8_BLOCK, false, true>(p, seq, &n_my);
    else if (op == OP_FP8_BLOCK) prologue<OP_FP8_BLOCK>(p, seq, &n_my);
    else return -1;
    for (int i = 0; i < n_my; ++i) {
      if (written >= cap) return written;
      const int gh = seq[2 * i], mn = seq[2 * i + 1];   // the decode of run_group's tile_ref
      int32_t* o = out + (size_t)written * 6;
      o[0] = wg; o[1] = gh & 0xFFFF; o[2] = (mn & 0xFFFF) * 64; o[3] = (gh >> 16) & 0x3FF;
      o[4] = (int)((uint32_t)mn >> 16) * 32; o[5] = (int)((uint32_t)gh >> 26) * 32;
      ++written;
    }
  }
  return written;
}
'''


@pytest.fixture(scope="module")
def emu(tmp_path_factory):
    src = open(os.path.join(CSRC, "gg_pingpong.hip")).read()
    begin = "  int n_my = 0;\n  if constexpr (!LISTS2) {\n"
    end = "  __syncthreads();\n\n  Shared sh{row_off"
    assert src.count(begin) == 1 and src.count(end) == 1, "markers of the prologue moved"
    body = src[src.index(begin):src.index(end)]      # both prologues: the default kernels' and the second one
    early = "    if (n_long + n_low == 0) return;"
    assert body.count(early) == 2
    body = body.replace(early, "    if (n_long + n_low == 0) { *n_my_out = 0; return; }")
    d = tmp_path_factory.mktemp("emu")
    cpp = d / "emu.cpp"
    cpp.write_text(HARNESS_HEAD + body + HARNESS_TAIL)
    so = d / "libemu.so"
    subprocess.run(["g++", "-O1", "-std=c++17", "-shared", "-fPIC", "-I", CSRC, "-o", str(so), str(cpp)], check=True)
    lib = ctypes.CDLL(str(so))
    lib.emu_prologue.restype = ctypes.c_int
    lib.emu_prologue.argtypes = [ctypes.c_int, I32P] + [ctypes.c_int] * 10 + [I32P, ctypes.c_int]
    return lib


@pytest.fixture(params=[0, 1], ids=["two_lists", "split_tails"])
def split(lib, request):
    """Tile order for one test: the host mirror is pinned to it, the device prologue gets it as p.split_tails."""
    assert lib.moe_gg_set_variant(2, request.param) == 0     # MOE_GG_OP_TILE_ORDER
    try:
        yield request.param
    finally:
        lib.moe_gg_set_variant(2, -1)


def device_tiles(emu, op, sizes, N, K, nwg, skip=0, tails=0, M=None, split=0, lists2=0):
    ms = np.ascontiguousarray(sizes, dtype=np.int32)
    out = np.zeros((CAP, 6), dtype=np.int32)
    n = emu.emu_prologue(op, ms.ctypes.data_as(I32P), len(ms), int(ms.sum()) if M is None else M, N, K, skip, tails, nwg, 8,
                         split, lists2, out.ctypes.data_as(I32P), CAP)
    assert 0 <= n < CAP
    return out[:n]


def host_tiles(lib, sizes, N, block_n, nwg):
    ms = np.ascontiguousarray(sizes, dtype=np.int32)
    out = np.zeros((CAP, 6), dtype=np.int32)
    n = lib.moe_gg_host_enumerate_tiles_two_lists(ms.ctypes.data_as(I32P), len(ms), int(ms.sum()), N, 256, block_n, nwg, 8,
                                                  out.ctypes.data_as(I32P), CAP)
    assert 0 <= n < CAP
    return out[:n]


def shape_sets():
    from applied_ai_amd import configs

    rng = np.random.default_rng(3)
    edge = [0, 1, 63, 64, 65, 127, 128, 129, 255, 256, 257, 319, 320, 321, 511, 512, 513, 576, 577, 640, 767, 768, 769, 832,
            833, 1039, 1048]
    cases = [([1012, 1039, 1048, 1036, 998, 1023, 1040, 996], 14336, 256), ([1012, 1039, 1048, 1036, 998, 1023, 1040, 996], 4096, 256),
             (configs.cfg5_routing()[3].tolist(), 4096, 256), ([530], 256, 8), ([1035, 1031, 991, 1008, 1011, 1033, 1067, 1016], 4096, 256)]
    for _ in range(120):
        G = int(rng.integers(1, 40))
        sizes = [int(rng.choice(edge)) if rng.random() < 0.6 else int(rng.integers(0, 1500)) for _ in range(G)]
        cases.append((sizes, int(rng.choice([64, 256, 300, 512, 1000, 2048, 4096])), int(rng.choice([8, 16, 64, 256, 304]))))
    return cases


def test_device_prologue_equals_the_host_mirror(emu, lib, split):
    for sizes, N, nwg in shape_sets():
        h = host_tiles(lib, sizes, N, 256, nwg)
        for lists2 in (0, 1):   # the default kernels' prologue and the second one (four-wave kernels run it in both orders)
            d = device_tiles(emu, 0, sizes, N, 4096, nwg, split=split, lists2=lists2).copy()
            assert h.shape == d.shape and (h == d).all(), ("bf16", sizes[:8], N, nwg, lists2)
        n_out = max(128, N // 2 // 128 * 128)       # fused gate/up kernel: p.N = 2 n, tiles of 128 output columns
        h = host_tiles(lib, sizes, n_out, 128, nwg)
        for op in (4, 9):   # the fused gate/up kernel and its form with the row gather
            d = device_tiles(emu, op, sizes, 2 * n_out, 4096, nwg, split=split)
            assert h.shape == d.shape and (h == d).all(), ("swiglu", op, sizes[:8], n_out, nwg)


def test_tall_tile_prologue_equals_the_host_mirror_and_covers_every_row_once(emu, lib):
    """The lists of the four-wave kernel with tall tiles (MOE_GG_GG_FOURWAVE_TALL; host mirror: MOE_GG_ORDER_TALL_TILES):
    an expert with 1 .. 32 rows behind its last full row tile has no tile for them, its last full tile is that much
    taller; of a tall tile cut into row pieces the last piece takes the extra rows."""
    assert lib.moe_gg_set_variant(2, 2) == 0
    try:
        tall_seen = 0
        for sizes, N, nwg in shape_sets():
            h = host_tiles(lib, sizes, N, 256, nwg)
            d = device_tiles(emu, 0, sizes, N, 4096, nwg, split=2)
            assert h.shape == d.shape and (h == d).all(), ("bf16", sizes[:8], N, nwg)
            c = [np.zeros((max(m, 0), -(-N // 256)), dtype=np.int32) for m in sizes]
            for wg, g, m0, hh, n0, nc in d.tolist():
                assert m0 % 64 == 0 and 0 <= hh <= 288 and m0 + hh <= sizes[g], (g, m0, hh)
                if hh > 256:
                    assert 0 < sizes[g] % 256 <= 32 and m0 + hh == sizes[g]
                    tall_seen += 1
                if hh:
                    c[g][m0:m0 + hh, n0 // 256] += 1
            assert all((x == 1).all() for x in c), (sizes[:8], N, nwg)
            for g, m in enumerate(sizes):     # no tile starts in the absorbed rows
                if m >= 256 and 0 < m % 256 <= 32:
                    assert not any(t[1] == g and t[2] >= m // 256 * 256 for t in d.tolist())
            n_out = max(128, N // 2 // 128 * 128)
            h = host_tiles(lib, sizes, n_out, 128, nwg)
            d = device_tiles(emu, 4, sizes, 2 * n_out, 4096, nwg, split=2)
            assert h.shape == d.shape and (h == d).all(), ("swiglu", sizes[:8], n_out, nwg)
        assert tall_seen > 100
    finally:
        lib.moe_gg_set_variant(2, -1)


def cover(tiles, sizes, N):
    c = [np.zeros((m, -(-N // 256)), dtype=np.int32) for m in sizes]
    for wg, g, m0, h, n0, nc in tiles.tolist():
        assert m0 % 64 == 0 and 0 <= n0 < N and m0 + h <= sizes[g] and (h == 0 or m0 < sizes[g]), (g, m0, h, n0)
        if h:
            c[g][m0:m0 + h, n0 // 256] += 1
    return c


def test_low_tiles_left_to_the_small_m_kernel_are_exactly_the_rows_it_computes(emu, lib, split):
    """p.tails_apart set (bf16, K >= 8192, few experts): when the decision (the host mirror's) is 'apart', the table
    holds every row up to each tall expert's last full tile and nothing of the few rows behind it; otherwise all rows."""
    for sizes, N in (([1012, 1039, 1048, 1036, 998, 1023, 1040, 996], 4096), ([1151] + [1024] * 6 + [897], 4096),
                     ([1124] * 4 + [1024] * 4, 4096), ([40, 2008, 2000, 2000, 2048, 0, 48, 48], 4096), ([1039, 700] + [0] * 6, 4096)):
        ms = np.ascontiguousarray(sizes, dtype=np.int32)
        apart = lib.moe_gg_host_tails_apart(ms.ctypes.data_as(I32P), len(ms), int(ms.sum()), N, 14336, 256)
        c = cover(device_tiles(emu, 0, sizes, N, 14336, 256, tails=256, split=split), sizes, N)
        for g, m in enumerate(sizes):
            full, rem = divmod(m, 256)
            low = 0 < rem < 128 and (full >= 2 or full == 0)
            keep = full * 256 if (apart and low) else m
            assert (c[g][:keep] == 1).all() and (c[g][keep:] == 0).all(), (sizes, g, apart)


def test_fp8_prologue_skips_the_streaming_kernels_experts(emu, lib, split):
    rng = np.random.default_rng(9)
    for _ in range(40):
        G = int(rng.integers(1, 60))
        sizes = [int(rng.integers(0, 90)) if rng.random() < 0.5 else int(rng.integers(0, 1400)) for _ in range(G)]
        N, nwg = int(rng.choice([128, 256, 512, 1024, 4096])), int(rng.choice([8, 64, 256]))
        for skip in (0, 64):
            c = cover(device_tiles(emu, 2, sizes, N, 7168, nwg, skip=skip, split=split), sizes, N)
            for g, m in enumerate(sizes):
                assert (c[g] == (0 if m <= skip else 1)).all(), (sizes[:6], g, m, skip)


def test_corrupt_sizes_are_clamped_in_the_prologue(emu, lib, split):
    # a negative entry counts as empty and the running sum is cut at M: no tile starts past its group's rows
    sizes = [300, -5, 700, 90]
    d = device_tiles(emu, 0, sizes, 512, 4096, 16, M=800, split=split)
    eff = [300, 0, 500, 0]
    c = [np.zeros((m, 2), dtype=np.int32) for m in eff]
    for wg, g, m0, h, n0, nc in d.tolist():
        assert eff[g] > 0 and m0 + h <= eff[g]
        if h:
            c[g][m0:m0 + h, n0 // 256] += 1
    assert all((x == 1).all() for x in c)
