// Driver of the data-race check of the emulated library (tests/emu, test infrastructure only): calls every entry point
// of include/moe_gg.h once or a few times on small shapes. Linked with the kernels compiled under ThreadSanitizer and
// emu_core.cpp built with EMU_TSAN, where every wave is a sanitizer fiber: a pair of accesses by two waves that no
// barrier orders, or by two workgroups of a launch, is reported whatever order the emulation runs them in. Results
// are not checked here (tests/test_emu_kernels.py does that); the exit status is the sanitizer's.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <utility>
#include <vector>

#include "../../include/moe_gg.h"

static uint32_t rng_state = 12345u;
static uint32_t rnd() { rng_state = rng_state * 1664525u + 1013904223u; return rng_state >> 8; }

template <class T> struct Buf {
  std::vector<T> v;
  explicit Buf(size_t n) : v(n + 64) {}
  T* p() { return v.data(); }
};
static Buf<uint16_t> bf16_small(size_t n) {  // bf16 integers -3 .. 3
  static const uint16_t code[7] = {0xC040, 0xC000, 0xBF80, 0x0000, 0x3F80, 0x4000, 0x4040};
  Buf<uint16_t> b(n);
  for (size_t i = 0; i < n; ++i) b.v[i] = code[rnd() % 7];
  return b;
}
static Buf<uint16_t> f16_small(size_t n) {
  static const uint16_t code[5] = {0xC000, 0xBC00, 0x0000, 0x3C00, 0x4000};
  Buf<uint16_t> b(n);
  for (size_t i = 0; i < n; ++i) b.v[i] = code[rnd() % 5];
  return b;
}
static Buf<uint8_t> fp8_codes(size_t n) {
  Buf<uint8_t> b(n);
  for (size_t i = 0; i < n; ++i) b.v[i] = (uint8_t)((0x30 + rnd() % 0x18) | ((rnd() & 1) << 7));
  return b;
}
static Buf<float> ones(size_t n) {
  Buf<float> b(n);
  for (size_t i = 0; i < n; ++i) b.v[i] = 1.0f;
  return b;
}
static Buf<int32_t> words(size_t n) {
  Buf<int32_t> b(n);
  for (size_t i = 0; i < n; ++i) b.v[i] = (int32_t)((rnd() << 8) ^ rnd());
  return b;
}

static int failures = 0;
static void check(int rc, const char* what) {
  std::printf("%-60s rc %d\n", what, rc);
  std::fflush(stdout);
  if (rc != 0) ++failures;
}

extern "C" int race_selftest(int kernel, int barrier);

// One grouped launch of the 256 x 256 ping-pong kernels (or the backward pass) on the given expert sizes.
static int one_shape(const char* op, int N, int K, int G, char** sizes) {
  Buf<int32_t> ms(G);
  int M = 0;
  for (int g = 0; g < G; ++g) M += (ms.v[g] = std::atoi(sizes[g]));
  Buf<uint16_t> y((size_t)M * N + 64);
  if (!std::strcmp(op, "fp8row") || !std::strcmp(op, "fp8block")) {
    const int mode = !std::strcmp(op, "fp8block");
    auto xq = fp8_codes((size_t)M * K), wq = fp8_codes((size_t)G * N * K);
    auto xs = ones((size_t)M * (K / 128) + 1), wsc = ones((size_t)G * N);
    moe_gg_set_variant(MOE_GG_OP_GG_FP8, MOE_GG_FP8_PINGPONG);
    check(moe_gg_grouped_gemm_fp8(xq.p(), wq.p(), y.p(), xs.p(), wsc.p(), mode, ms.p(), G, M, N, K, N, MOE_GG_OUT_MN, nullptr), op);
  } else if (!std::strcmp(op, "bwd")) {
    auto x = bf16_small((size_t)M * K), w = bf16_small((size_t)G * N * K), go = bf16_small((size_t)M * N);
    Buf<uint16_t> gx((size_t)M * K), gw((size_t)G * N * K);
    const size_t wsb = moe_gg_grouped_gemm_backward_workspace(G, M, N, K, 0);
    Buf<uint8_t> ws(wsb + 512);
    uint8_t* wsp = ws.p() + ((256 - ((uintptr_t)ws.p() & 255)) & 255);
    check(moe_gg_grouped_gemm_backward_bf16(go.p(), N, 0, x.p(), w.p(), ms.p(), G, M, N, K, gx.p(), gw.p(), wsp, wsb, nullptr), op);
  } else if (!std::strcmp(op, "swigluw4") || !std::strcmp(op, "swiglutall")) {  // the fused kernel on four waves (N = output columns n, w [G, 2 n, K])
    auto x = bf16_small((size_t)M * K), w = bf16_small((size_t)G * 2 * N * K);
    moe_gg_set_variant(MOE_GG_OP_GG_BF16, !std::strcmp(op, "swiglutall") ? MOE_GG_GG_FOURWAVE_TALL : MOE_GG_GG_FOURWAVE_256);
    check(moe_gg_grouped_gemm_swiglu_bf16(x.p(), w.p(), y.p(), ms.p(), G, M, N, K, N, nullptr), op);
    moe_gg_set_variant(MOE_GG_OP_GG_BF16, -1);
  } else if (!std::strcmp(op, "swiglu")) {
    auto x = bf16_small((size_t)M * K), w = bf16_small((size_t)G * 2 * N * K);
    check(moe_gg_grouped_gemm_swiglu_bf16(x.p(), w.p(), y.p(), ms.p(), G, M, N, K, N, nullptr), op);
  } else if (!std::strcmp(op, "gather")) {  // sorted row i = token row perm[i] / 2, perm a shuffle of the slots
    const int T = (M + 1) / 2;
    auto x = bf16_small((size_t)T * K), w = bf16_small((size_t)G * 2 * N * K);
    Buf<int32_t> perm(M);
    for (int i = 0; i < M; ++i) perm.v[i] = i;
    for (int i = M - 1; i > 0; --i) std::swap(perm.v[i], perm.v[rnd() % (i + 1)]);
    check(moe_gg_grouped_gemm_swiglu_gather(x.p(), T, perm.p(), 2, w.p(), y.p(), ms.p(), G, M, N, K, N, MOE_GG_DTYPE_BF16, nullptr), op);
  } else {
    const bool f16 = !std::strcmp(op, "f16") || !std::strcmp(op, "f16w4");
    const bool fourwave = !std::strcmp(op, "bf16w4") || !std::strcmp(op, "f16w4");
    const bool tall = !std::strcmp(op, "bf16tall");
    auto x = f16 ? f16_small((size_t)M * K) : bf16_small((size_t)M * K);
    auto w = f16 ? f16_small((size_t)G * N * K) : bf16_small((size_t)G * N * K);
    moe_gg_set_variant(MOE_GG_OP_GG_BF16, tall ? MOE_GG_GG_FOURWAVE_TALL : fourwave ? MOE_GG_GG_FOURWAVE_256 : MOE_GG_GG_PINGPONG_256);
    check((f16 ? moe_gg_grouped_gemm_f16 : moe_gg_grouped_gemm_bf16)(x.p(), w.p(), y.p(), ms.p(), G, M, N, K, N, MOE_GG_OUT_MN, nullptr), op);
  }
  return failures ? 1 : 0;
}

// race_check                       all entry points (exit status 0 unless the sanitizer reported something: then 66)
// race_check selftest K B          control kernel K (0: stores, 1: global->LDS load), B = 1 with / 0 without the barrier
// race_check shape OP N K m1 m2 .. one launch; OP = bf16 | f16 | bf16w4 | f16w4 | bf16tall | swiglu | swigluw4 | swiglutall |
//                                  gather | fp8row | fp8block | bwd
int main(int argc, char** argv) {
  // EMU_TILE_ORDER = 0 / 1: the ping-pong kernels' tile order for this run (MOE_GG_OP_TILE_ORDER)
  if (const char* order = std::getenv("EMU_TILE_ORDER")) moe_gg_set_variant(MOE_GG_OP_TILE_ORDER, std::atoi(order));
  if (argc == 4 && !std::strcmp(argv[1], "selftest")) {
    std::printf("sum %d\n", race_selftest(std::atoi(argv[2]), std::atoi(argv[3])));
    return 0;
  }
  if (argc >= 6 && !std::strcmp(argv[1], "shape")) return one_shape(argv[2], std::atoi(argv[3]), std::atoi(argv[4]), argc - 5, argv + 5);
  {
    const int sizes[] = {300, 0, 70, 530};
    const int G = 4, M = 900, N = 512, K = 256;
    Buf<int32_t> ms(G);
    std::memcpy(ms.p(), sizes, sizeof(sizes));
    auto x = bf16_small((size_t)M * K), w = bf16_small((size_t)G * N * K);
    Buf<uint16_t> y((size_t)M * N * G);
    for (int variant = -1; variant <= 8; ++variant) {
      moe_gg_set_variant(MOE_GG_OP_GG_BF16, variant);
      check(moe_gg_grouped_gemm_bf16(x.p(), w.p(), y.p(), ms.p(), G, M, N, K, N, MOE_GG_OUT_MN, nullptr), "grouped_gemm_bf16 (every variant)");
    }
    moe_gg_set_variant(MOE_GG_OP_GG_BF16, -1);
    check(moe_gg_grouped_gemm_bf16(x.p(), w.p(), y.p(), ms.p(), G, M, N, K, (int64_t)N * G, MOE_GG_OUT_BLOCK, nullptr), "grouped_gemm_bf16 [M, N G] layout");
    auto xh = f16_small((size_t)M * K), wh = f16_small((size_t)G * N * K);
    check(moe_gg_grouped_gemm_f16(xh.p(), wh.p(), y.p(), ms.p(), G, M, N, K, N, MOE_GG_OUT_MN, nullptr), "grouped_gemm_f16");
    const int n = 128;  // w as [G, 2 n, K]
    check(moe_gg_grouped_gemm_swiglu_bf16(x.p(), w.p(), y.p(), ms.p(), G, M, n, K, n, nullptr), "grouped_gemm_swiglu_bf16");
    check(moe_gg_grouped_gemm_swiglu_f16(xh.p(), wh.p(), y.p(), ms.p(), G, M, n, K, n, nullptr), "grouped_gemm_swiglu_f16");
    // backward: grad_out [M, N], workspace and static forms, then the [M, N G] layout
    auto go = bf16_small((size_t)M * N * G);
    Buf<uint16_t> gx((size_t)M * K), gw((size_t)G * N * K);
    const size_t wsb = moe_gg_grouped_gemm_backward_workspace(G, M, N, K, 1);
    Buf<uint8_t> ws(wsb + 512);
    uint8_t* wsp = ws.p() + ((256 - ((uintptr_t)ws.p() & 255)) & 255);
    check(moe_gg_grouped_gemm_backward_bf16(go.p(), N, 0, x.p(), w.p(), ms.p(), G, M, N, K, gx.p(), gw.p(), wsp, wsb, nullptr), "backward (workspace)");
    check(moe_gg_grouped_gemm_backward_bf16_static(go.p(), N, 0, x.p(), w.p(), ms.p(), G, M, N, K, gx.p(), gw.p(), nullptr), "backward (static scratch)");
    check(moe_gg_grouped_gemm_backward_bf16(go.p(), (int64_t)N * G, 1, x.p(), w.p(), ms.p(), G, M, N, K, gx.p(), gw.p(), wsp, wsb, nullptr), "backward ([M, N G] gradient)");
    const int Ns = 68, Ks = 36;  // not multiples of 64: the transposing path
    check(moe_gg_grouped_gemm_backward_bf16(go.p(), Ns, 0, x.p(), w.p(), ms.p(), G, M, Ns, Ks, gx.p(), gw.p(), wsp, wsb, nullptr), "backward (N = 68, K = 36)");
  }
  {
    const int sizes[] = {300, 0, 70, 30, 530};
    const int G = 5, M = 930, N = 256, K = 256;
    Buf<int32_t> ms(G);
    std::memcpy(ms.p(), sizes, sizeof(sizes));
    auto xq = fp8_codes((size_t)M * K), wq = fp8_codes((size_t)G * N * K);
    auto xs = ones((size_t)M * (K / 128)), wsc = ones((size_t)G * N);
    Buf<uint16_t> y((size_t)M * N);
    for (int mode = 0; mode < 2; ++mode)
      for (int variant = -1; variant <= 3; ++variant) {
        moe_gg_set_variant(MOE_GG_OP_GG_FP8, variant);
        check(moe_gg_grouped_gemm_fp8(xq.p(), wq.p(), y.p(), xs.p(), wsc.p(), mode, ms.p(), G, M, N, K, N, MOE_GG_OUT_MN, nullptr),
              mode ? "grouped_gemm_fp8 block scales (every variant)" : "grouped_gemm_fp8 row scales (every variant)");
      }
    moe_gg_set_variant(MOE_GG_OP_GG_FP8, -1);
  }
  {  // the bf16 launch pair that leaves low tiles to the small-M kernel
    const int G = 1, M = 520, N = 64, K = 8192;
    Buf<int32_t> ms(G);
    ms.v[0] = M;
    auto x = bf16_small((size_t)M * K), w = bf16_small((size_t)G * N * K);
    Buf<uint16_t> y((size_t)M * N);
    check(moe_gg_grouped_gemm_bf16(x.p(), w.p(), y.p(), ms.p(), G, M, N, K, N, MOE_GG_OUT_MN, nullptr), "grouped_gemm_bf16 K = 8192 (low tiles apart)");
  }
  {
    const int K = 512, N = 256, E = 4;
    auto qw = words((size_t)E * (K / 8) * N), qz = words((size_t)E * (K / 128) * (N / 8));
    Buf<uint16_t> sc((size_t)E * (K / 128) * N);
    for (auto& v : sc.v) v = 0x3C00;  // 1.0 as fp16, 0.0078 as bf16: both finite
    auto a = bf16_small((size_t)80 * K);
    Buf<uint16_t> c((size_t)80 * N);
    const int Ms[] = {1, 16, 33, 70};
    for (int variant = 0; variant <= 7; ++variant) {  // the default kernels, then the selectable ones
      moe_gg_set_variant(MOE_GG_OP_W4A16, variant);
      for (int M : Ms)
        check(moe_gg_w4a16_splitk(a.p(), qw.p(), sc.p(), qz.p(), c.p(), M, N, K, 128, 1, MOE_GG_DTYPE_BF16, nullptr), "w4a16_splitk (M = 1, 16, 33, 70; every variant)");
    }
    moe_gg_set_variant(MOE_GG_OP_W4A16, -1);
    check(moe_gg_w4a16_splitk(a.p(), qw.p(), sc.p(), qz.p(), c.p(), 20, N, K, 64, 0, MOE_GG_DTYPE_FP16, nullptr), "w4a16_splitk group 64 fp16");
    const int sizes[] = {3, 0, 40, 12};
    Buf<int32_t> ms(E);
    std::memcpy(ms.p(), sizes, sizeof(sizes));
    check(moe_gg_w4a16_grouped(a.p(), qw.p(), sc.p(), qz.p(), c.p(), ms.p(), E, 55, N, K, 128, 1, MOE_GG_DTYPE_BF16, nullptr), "w4a16_grouped");
    moe_gg_set_variant(MOE_GG_OP_W4A16, MOE_GG_W4_WARMUP);
    check(moe_gg_w4a16_grouped(a.p(), qw.p(), sc.p(), qz.p(), c.p(), ms.p(), E, 55, N, K, 128, 1, MOE_GG_DTYPE_BF16, nullptr), "w4a16_grouped with warm-up waves");
    moe_gg_set_variant(MOE_GG_OP_W4A16, -1);
    Buf<uint8_t> cq((size_t)80 * N);
    Buf<float> cs((size_t)80 * (N / 128));
    check(moe_gg_w4a16_grouped_fp8out(a.p(), qw.p(), sc.p(), qz.p(), cq.p(), cs.p(), ms.p(), E, 55, N, K, 128, 1, MOE_GG_DTYPE_BF16, nullptr), "w4a16_grouped_fp8out");
  }
  {
    const int T = 700, E = 60, k = 4, n = T * k;
    Buf<float> logits((size_t)T * E);
    for (auto& v : logits.v) v = (float)(rnd() % 1000) * 1e-3f;
    Buf<int32_t> ids(n), perm(n), ms(E), off(E + 1), inv(n), sorted((size_t)n + E * 15), eids(n + E), post(1);
    check(moe_gg_route_topk(logits.p(), T, E, k, ids.p(), perm.p(), ms.p(), off.p(), nullptr), "route_topk");
    for (int i = 0; i < n; i += 7) ids.v[i] = -1;  // masked slots
    check(moe_gg_route_group(ids.p(), n, E, perm.p(), ms.p(), off.p(), nullptr), "route_group (masked ids)");
    check(moe_gg_align_block_size(perm.p(), ms.p(), E, n, 16, sorted.p(), eids.p(), post.p(), nullptr), "align_block_size");
    auto x = bf16_small((size_t)T * 256);
    Buf<uint16_t> xs((size_t)n * 256), comb((size_t)T * 256);
    check(moe_gg_gather_rows(x.p(), perm.p(), k, xs.p(), n, 512, T, off.p() + E, nullptr), "gather_rows");
    check(moe_gg_invert_perm(perm.p(), inv.p(), n, off.p() + E, nullptr), "invert_perm");
    for (auto& v : inv.v) v = (int32_t)(rnd() % n);
    auto wt = ones((size_t)n);
    check(moe_gg_combine_topk(xs.p(), inv.p(), wt.p(), MOE_GG_DTYPE_FP32, comb.p(), T, k, 256, n, nullptr), "combine_topk");
    Buf<uint16_t> act((size_t)n * 128);
    check(moe_gg_silu_and_mul(xs.p(), act.p(), n, 128, nullptr), "silu_and_mul");
    Buf<uint8_t> q((size_t)n * 256);
    Buf<float> qs((size_t)n * 2);
    check(moe_gg_fp8_groupwise_quant(xs.p(), MOE_GG_DTYPE_BF16, q.p(), qs.p(), (int64_t)n * 256, nullptr), "fp8_groupwise_quant");
    check(moe_gg_fp8_block128_quant(xs.p(), MOE_GG_DTYPE_BF16, q.p(), qs.p(), 256, 256, nullptr), "fp8_block128_quant");
  }
  std::printf("calls that returned an error: %d\n", failures);
  return failures ? 1 : 0;
}
