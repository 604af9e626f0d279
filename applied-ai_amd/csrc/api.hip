// C-ABI layer of libmoe_gg.so: argument validation, kernel-variant choice, launches.
#include "../../include/moe_gg.h"
#include "kernels.h"
#include "tile_sched.h"

#include <atomic>
#include <mutex>

namespace {

struct DeviceInfo {
  int cus = 0;
  int xcds = 8;
  bool ok = false;
};

constexpr int kMaxDevices = 16;
DeviceInfo g_dev[kMaxDevices];
std::once_flag g_dev_once[kMaxDevices];
std::atomic<int> g_variant[8] = {{-1}, {-1}, {-1}, {-1}, {-1}, {-1}, {-1}, {-1}};

int current_device_info(const DeviceInfo** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return MOE_GG_EDEVICE;
  std::call_once(g_dev_once[dev], [dev]() {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return;
    g_dev[dev].cus = prop.multiProcessorCount;
    // Workgroups are dealt round-robin over the XCDs (MI355X: 8 XCDs x 32 CUs); a partitioned device reports fewer.
    int xccs = 0;
    if (hipDeviceGetAttribute(&xccs, hipDeviceAttributeNumberOfXccs, dev) != hipSuccess) {
      (void)hipGetLastError();  // not a launch error: do not leave it for the next hipGetLastError()
      xccs = 0;
    }
    g_dev[dev].xcds = (xccs >= 1 && xccs <= 16) ? xccs : 8;
    g_dev[dev].ok = prop.multiProcessorCount > 0;
  });
  if (!g_dev[dev].ok) return MOE_GG_EDEVICE;
  *out = &g_dev[dev];
  return MOE_GG_OK;
}

// Variant bits of the W4A16 kernels (MOE_GG_OP_W4A16): 0 unless pinned.
int w4_variant() {
  const int v = g_variant[MOE_GG_OP_W4A16].load();
  return v < 0 ? 0 : v & 7;
}

// Tile order of the forward ping-pong kernels (MOE_GG_OP_TILE_ORDER): the split-tail order only when it is pinned.
int split_tails_on() { return g_variant[MOE_GG_OP_TILE_ORDER].load() == MOE_GG_ORDER_SPLIT_TAILS ? 1 : 0; }

bool aligned(const void* p, size_t a) { return ((uintptr_t)p % a) == 0; }

// How wide the kernels may store row segments of y: 2 = 16 bytes, 1 = 8 bytes, 0 = element by element. col_step
// is the distance between the column offsets the call may add (N for the per-expert column blocks, else 0).
int vec_store_level(const void* y, int64_t ldy, int64_t col_step) {
  if (aligned(y, 16) && ldy % 8 == 0 && col_step % 8 == 0) return 2;
  if (aligned(y, 8) && ldy % 4 == 0 && col_step % 4 == 0) return 1;
  return 0;
}

// fp8: the dedicated small-M kernel (weights streamed straight into MFMA operands, split-K inside the workgroup)
// beats the ping-pong kernel only for a few rows per expert (measured: up to about 12) or when the launch has
// too few 256 x 256 tiles to give every CU several (few experts, narrow N); never above 40 rows per expert.
bool use_streaming_kernel(int64_t M, int G, int64_t ntn256, int num_wg) {
  if (M > (int64_t)G * 40) return false;
  return M <= (int64_t)G * 12 || (int64_t)G * ntn256 < 4 * (int64_t)num_wg;
}
// bf16: the small-M kernel streams weights at 5.8-6.0 TB/s with one or two activation fragments per pass (up
// to 24 rows per expert on average) and beats every tiled kernel there (measured for 8-64 experts, N and K of
// 2048-14336); with four fragments it falls behind them.
bool use_decode_kernel(int64_t M, int G) { return M <= (int64_t)G * 24; }

}  // namespace

// The ping-pong kernels form slab offsets with 24-bit multiplies: an operand row must be shorter than 16 MB.
constexpr int64_t PINGPONG_MAX_ROW_BYTES = 1 << 24;
// bf16 forward: largest expert count for which the small-M kernel is launched behind the ping-pong kernel for the
// low tiles (moe_gg_tails_apart).
constexpr int TAILS_APART_MAX_GROUPS = 32;
// ... and the shortest reduction: a round of low tiles costs about 0.9 us per 64-wide K step and the second launch
// 5-15 us also when it finds nothing to do, so below this K there is little to gain.
constexpr int TAILS_APART_MIN_K = 8192;

extern "C" {

int moe_gg_abi_version(void) { return MOE_GG_ABI_VERSION; }

const char* moe_gg_strerror(int code) {
  switch (code) {
    case MOE_GG_OK: return "success";
    case MOE_GG_EINVAL: return "invalid argument (null pointer, negative size or bad enum)";
    case MOE_GG_ESHAPE: return "inconsistent dimensions";
    case MOE_GG_EALIGN: return "pointer or leading dimension not sufficiently aligned";
    case MOE_GG_EUNSUPPORTED: return "request outside the supported range of the kernels";
    case MOE_GG_EDEVICE: return "no usable gfx950 device";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "unknown moe_gg error";
}

int moe_gg_set_variant(int op, int variant) {
  if (op < 0 || op >= 8) return MOE_GG_EINVAL;
  g_variant[op].store(variant);
  return MOE_GG_OK;
}

static int grouped_gemm_16(const void* x, const void* w, void* y, const int32_t* m_sizes, int G, int64_t M, int N, int K,
                           int64_t ldy, int out_layout, bool fp16, void* stream) {
  if (G < 0 || M < 0 || N < 0 || K < 0) return MOE_GG_EINVAL;
  if (out_layout != MOE_GG_OUT_MN && out_layout != MOE_GG_OUT_BLOCK) return MOE_GG_EINVAL;
  if (M > INT32_MAX || (int64_t)G * N > INT32_MAX || ldy > INT32_MAX) return MOE_GG_EUNSUPPORTED;
  const int64_t min_ld = out_layout == MOE_GG_OUT_BLOCK ? (int64_t)N * G : (int64_t)N;
  if (ldy < min_ld) return MOE_GG_ESHAPE;
  if (G == 0 || M == 0 || N == 0) return MOE_GG_OK;  // nothing to compute
  if (!x || !w || !y || !m_sizes) return MOE_GG_EINVAL;
  if (K == 0) return MOE_GG_ESHAPE;
  if (G > MOE_GG_MAX_GROUPS_ABI) return MOE_GG_EUNSUPPORTED;
  if (!aligned(m_sizes, 4) || !aligned(x, 2) || !aligned(w, 2) || !aligned(y, 2)) return MOE_GG_EALIGN;

  const DeviceInfo* di = nullptr;
  int rc = current_device_info(&di);
  if (rc != MOE_GG_OK) return rc;

  GgParams p{};
  p.x = x; p.w = w; p.y = y; p.m_sizes = m_sizes;
  p.G = G; p.M = (int)M; p.N = N; p.K = K;
  p.ldy = (int)ldy;
  p.col_block = out_layout == MOE_GG_OUT_BLOCK ? N : 0;
  p.vec_store = vec_store_level(y, ldy, N);
  p.xcds = di->xcds;
  p.fp16 = fp16 ? 1 : 0;
  p.split_tails = split_tails_on();

  hipStream_t s = (hipStream_t)stream;
  const bool tiled_ok = K % 64 == 0 && aligned(x, 16) && aligned(w, 16);
  int variant = g_variant[MOE_GG_OP_GG_BF16].load();
  if (!tiled_ok || variant == MOE_GG_GG_GENERIC) return (int)gg_bf16_generic_launch(p, s);

  int num_wg = di->cus - di->cus % p.xcds;
  if (num_wg <= 0) { num_wg = di->cus; p.xcds = 1; }
  const bool decode_ok = K % 128 == 0;
  const int64_t ntn256 = (N + 255) / 256;
  // The ping-pong kernel tabulates each workgroup's tile sequence and forms slab offsets with 24-bit multiplies.
  const bool pingpong_ok = K < PINGPONG_MAX_ROW_BYTES / 2 && moe_gg_two_list_fits(M, G, 256, (int)ntn256, num_wg);
  const bool automatic = variant < 0;
  if (variant < 0 && decode_ok && use_decode_kernel(M, G)) variant = MOE_GG_GG_DECODE;
  if (variant == MOE_GG_GG_DECODE) {
    if (!decode_ok) return MOE_GG_EUNSUPPORTED;
    const int64_t avg = (M + G - 1) / G;
    const int mf = avg <= 10 ? 1 : (avg <= 24 ? 2 : 4);
    int nf = ((int64_t)(N / 64) * G >= 4 * (int64_t)di->cus) ? 4 : 2;
    // One activation fragment per pass (up to 10 rows per expert on average): the narrow workgroups are 2-20 %
    // faster on every shape measured (8-256 experts, N and K of 2048-14336), also when there are many of them.
    if (mf == 4 || mf == 1) nf = 2;
    return (int)gg_bf16_decode_launch(p, nf, mf, s);
  }
  if (variant < 0) {
    // m_sizes lives on the device and is never copied back, so the tile shape is picked from a rough
    // count of 256 x 256 tiles (each expert adds about half a partial row tile). Measured over expert
    // counts 2 .. 256 and 128 .. 8192 rows: the ping-pong kernel wins whenever there are enough tiles
    // to occupy the CUs, also for experts of 16 .. 128 rows (short tiles skip most of their work and
    // the kernel then streams weights at 5 TB/s); smaller tiles only pay for small problems.
    // The ping-pong kernel from 0.4 tiles per CU on: it cuts the tiles of a sparse last round into row pieces, so
    // 100-190 tiles still occupy 256 CUs (measured over 4-32 experts, 256-1536 rows, N and K of 2048-8192: +35 to
    // +80 % over the 128-row tiles on most such shapes, -4 to -15 % on a few with K = 2048).
    const int64_t t256 = (M / 256 + (G + 1) / 2) * ntn256;
    if (t256 * 5 >= (int64_t)num_wg * 2 && pingpong_ok) variant = MOE_GG_GG_PINGPONG_256;
    else if (t256 * 4 >= (int64_t)num_wg * 3) variant = MOE_GG_GG_TILED_256;
    else if (t256 * 4 >= num_wg) variant = MOE_GG_GG_TILED_128;
    else variant = MOE_GG_GG_TILED_64;
  }
  switch (variant) {
    case MOE_GG_GG_PINGPONG_256: {
      if (!pingpong_ok) return MOE_GG_EUNSUPPORTED;
      // Automatic choice only: few low tiles that would take a round of their own go to the small-M kernel
      // (moe_gg_tails_apart, decided on the device by both kernels). Its grid has N / 32 workgroups per expert,
      // most of which leave at once: only worth launching for a few experts.
      const bool tails = automatic && decode_ok && G <= TAILS_APART_MAX_GROUPS && K >= TAILS_APART_MIN_K;
      p.tails_apart = tails ? num_wg : 0;
      const hipError_t e = gg_bf16_pingpong_launch(p, num_wg, s);
      if (e != hipSuccess || !tails) return (int)e;
      return (int)gg_bf16_decode_tails_launch(p, s);
    }
    case MOE_GG_GG_FOURWAVE_256:
    case MOE_GG_GG_FOURWAVE_TALL:
      if (!pingpong_ok) return MOE_GG_EUNSUPPORTED;
      return (int)gg_bf16_fourwave_launch(p, variant == MOE_GG_GG_FOURWAVE_TALL, num_wg, s);
    case MOE_GG_GG_TILED_256: return (int)gg_bf16_tiled_launch(p, 256, num_wg, s);
    case MOE_GG_GG_TILED_256_W4: return (int)gg_bf16_tiled_launch(p, GG_TILED_256_FOUR_WAVES, num_wg, s);
    case MOE_GG_GG_TILED_128: return (int)gg_bf16_tiled_launch(p, 128, num_wg, s);
    case MOE_GG_GG_TILED_64: return (int)gg_bf16_tiled_launch(p, 64, num_wg, s);
    default: return MOE_GG_EINVAL;
  }
}

int moe_gg_grouped_gemm_bf16(const void* x, const void* w, void* y, const int32_t* m_sizes, int G,
                             int64_t M, int N, int K, int64_t ldy, int out_layout, void* stream) {
  return grouped_gemm_16(x, w, y, m_sizes, G, M, N, K, ldy, out_layout, false, stream);
}

int moe_gg_grouped_gemm_f16(const void* x, const void* w, void* y, const int32_t* m_sizes, int G,
                            int64_t M, int N, int K, int64_t ldy, int out_layout, void* stream) {
  return grouped_gemm_16(x, w, y, m_sizes, G, M, N, K, ldy, out_layout, true, stream);
}

int moe_gg_grouped_gemm_fp8(const void* x, const void* w, void* y, const float* x_scale, const float* w_scale,
                            int scale_mode, const int32_t* m_sizes, int G, int64_t M, int N, int K,
                            int64_t ldy, int out_layout, void* stream) {
  if (G < 0 || M < 0 || N < 0 || K < 0) return MOE_GG_EINVAL;
  if (out_layout != MOE_GG_OUT_MN && out_layout != MOE_GG_OUT_BLOCK) return MOE_GG_EINVAL;
  if (scale_mode != MOE_GG_SCALE_ROWWISE && scale_mode != MOE_GG_SCALE_BLOCK128) return MOE_GG_EINVAL;
  if (M > INT32_MAX || (int64_t)G * N > INT32_MAX || ldy > INT32_MAX) return MOE_GG_EUNSUPPORTED;
  const int64_t min_ld = out_layout == MOE_GG_OUT_BLOCK ? (int64_t)N * G : (int64_t)N;
  if (ldy < min_ld) return MOE_GG_ESHAPE;
  if (G == 0 || M == 0 || N == 0) return MOE_GG_OK;
  if (!x || !w || !y || !m_sizes || !x_scale || !w_scale) return MOE_GG_EINVAL;
  if (K == 0) return MOE_GG_ESHAPE;
  if (G > MOE_GG_MAX_GROUPS_ABI) return MOE_GG_EUNSUPPORTED;
  if (K % 128 != 0 || (scale_mode == MOE_GG_SCALE_BLOCK128 && N % 128 != 0)) return MOE_GG_EUNSUPPORTED;
  if (K >= PINGPONG_MAX_ROW_BYTES) return MOE_GG_EUNSUPPORTED;
  if (!aligned(x, 16) || !aligned(w, 16) || !aligned(y, 2) || !aligned(x_scale, 4) || !aligned(w_scale, 4) ||
      !aligned(m_sizes, 4))
    return MOE_GG_EALIGN;
  const DeviceInfo* di = nullptr;
  int rc = current_device_info(&di);
  if (rc != MOE_GG_OK) return rc;
  GgParams p{};
  p.x = x; p.w = w; p.y = y; p.m_sizes = m_sizes; p.x_scale = x_scale; p.w_scale = w_scale;
  p.G = G; p.M = (int)M; p.N = N; p.K = K;
  p.ldy = (int)ldy;
  p.col_block = out_layout == MOE_GG_OUT_BLOCK ? N : 0;
  p.vec_store = vec_store_level(y, ldy, N);
  p.xcds = di->xcds;
  p.split_tails = split_tails_on();
  int num_wg = di->cus - di->cus % p.xcds;
  if (num_wg <= 0) { num_wg = di->cus; p.xcds = 1; }
  // A few rows per expert (see use_streaming_kernel): the experts with up to 64 rows go to the streaming
  // split-K kernel and the ping-pong kernel takes the rest; m_sizes stays on the device, so both are launched
  // and a workgroup whose expert belongs to the other kernel exits after reading m_sizes. Otherwise the
  // ping-pong kernel does everything.
  int variant = g_variant[MOE_GG_OP_GG_FP8].load();
  // The ping-pong kernel tabulates each workgroup's tile sequence: beyond its capacity the 128 x 128 kernel runs.
  const bool pingpong_ok = moe_gg_two_list_fits(M, G, 256, (N + 255) / 256, num_wg);
  if (variant < 0)
    variant = !pingpong_ok ? MOE_GG_FP8_TILED_128
              : use_streaming_kernel(M, G, (N + 255) / 256, num_wg) ? MOE_GG_FP8_STREAM_PINGPONG : MOE_GG_FP8_PINGPONG;
  else if (variant != MOE_GG_FP8_TILED_128 && variant != MOE_GG_FP8_STREAM_TILED && !pingpong_ok)
    return MOE_GG_EUNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
  if (variant == MOE_GG_FP8_TILED_128) return (int)gg_fp8_launch(p, scale_mode, num_wg, s);
  if (variant == MOE_GG_FP8_PINGPONG) return (int)gg_fp8_pingpong_launch(p, scale_mode, num_wg, s);
  if (variant != MOE_GG_FP8_STREAM_PINGPONG && variant != MOE_GG_FP8_STREAM_TILED) return MOE_GG_EINVAL;
  hipError_t e = gg_fp8_stream_launch(p, scale_mode, s);
  if (e != hipSuccess) return (int)e;
  p.skip_rows = gg_fp8_stream_max_rows();
  if (variant == MOE_GG_FP8_STREAM_TILED) return (int)gg_fp8_launch(p, scale_mode, num_wg, s);
  return (int)gg_fp8_pingpong_launch(p, scale_mode, num_wg, s);
}

int moe_gg_w4a16_splitk(const void* a, const int32_t* qweight, const void* scales, const int32_t* qzeros,
                        void* c, int M, int N, int K, int group_size, int zero_offset, int dtype,
                        void* stream) {
  if (M < 0 || N < 0 || K < 0 || group_size <= 0) return MOE_GG_EINVAL;
  if (zero_offset != 0 && zero_offset != 1) return MOE_GG_EINVAL;
  if (dtype != MOE_GG_DTYPE_BF16 && dtype != MOE_GG_DTYPE_FP16) return MOE_GG_EINVAL;
  if (M == 0 || N == 0) return MOE_GG_OK;
  if (!a || !qweight || !scales || !qzeros || !c) return MOE_GG_EINVAL;
  if (K == 0 || K % group_size != 0 || K % 8 != 0 || N % 8 != 0) return MOE_GG_ESHAPE;
  if (group_size % 32 != 0 || N % 64 != 0) return MOE_GG_EUNSUPPORTED;
  if (!aligned(a, 16) || !aligned(qweight, 16) || !aligned(scales, 16) || !aligned(qzeros, 8) || !aligned(c, 2))
    return MOE_GG_EALIGN;
  const DeviceInfo* di = nullptr;
  int rc = current_device_info(&di);
  if (rc != MOE_GG_OK) return rc;
  W4Params p{a, qweight, scales, qzeros, c, M, N, K, group_size, zero_offset};
  return (int)w4a16_splitk_launch(p, dtype == MOE_GG_DTYPE_FP16, w4_variant(), (hipStream_t)stream);
}

static int w4a16_grouped_any(const void* a, const int32_t* qweight, const void* scales, const int32_t* qzeros, void* c,
                            void* c_q, float* c_scale, bool fp8out, const int32_t* m_sizes, int G, int64_t M, int N,
                            int K, int group_size, int zero_offset, int dtype, void* stream) {
  if (G < 0 || M < 0 || N < 0 || K < 0 || group_size <= 0) return MOE_GG_EINVAL;
  if (zero_offset != 0 && zero_offset != 1) return MOE_GG_EINVAL;
  if (dtype != MOE_GG_DTYPE_BF16 && dtype != MOE_GG_DTYPE_FP16) return MOE_GG_EINVAL;
  if (G == 0 || M == 0 || N == 0) return MOE_GG_OK;
  if (!a || !qweight || !scales || !qzeros || !m_sizes) return MOE_GG_EINVAL;
  if (fp8out ? (!c_q || !c_scale) : !c) return MOE_GG_EINVAL;
  if (K == 0 || K % group_size != 0 || K % 8 != 0 || N % 8 != 0) return MOE_GG_ESHAPE;
  if (group_size % 32 != 0 || N % (fp8out ? 128 : 64) != 0 || G > 65535 || M > INT32_MAX) return MOE_GG_EUNSUPPORTED;
  if (!aligned(a, 16) || !aligned(qweight, 16) || !aligned(scales, 16) || !aligned(qzeros, 8) || !aligned(m_sizes, 4))
    return MOE_GG_EALIGN;
  if (fp8out ? !aligned(c_scale, 4) : !aligned(c, 2)) return MOE_GG_EALIGN;
  const DeviceInfo* di = nullptr;
  int rc = current_device_info(&di);
  if (rc != MOE_GG_OK) return rc;
  W4Params p{a, qweight, scales, qzeros, fp8out ? nullptr : c, (int)M, N, K, group_size, zero_offset, m_sizes, G};
  if (fp8out) {
    p.cq = c_q;
    p.cscale = c_scale;
  }
  return (int)w4a16_splitk_launch(p, dtype == MOE_GG_DTYPE_FP16, w4_variant(), (hipStream_t)stream);
}

int moe_gg_w4a16_grouped(const void* a, const int32_t* qweight, const void* scales, const int32_t* qzeros, void* c,
                         const int32_t* m_sizes, int G, int64_t M, int N, int K, int group_size, int zero_offset,
                         int dtype, void* stream) {
  return w4a16_grouped_any(a, qweight, scales, qzeros, c, nullptr, nullptr, false, m_sizes, G, M, N, K, group_size,
                           zero_offset, dtype, stream);
}

int moe_gg_w4a16_grouped_fp8out(const void* a, const int32_t* qweight, const void* scales, const int32_t* qzeros,
                                void* c_q, float* c_scale, const int32_t* m_sizes, int G, int64_t M, int N, int K,
                                int group_size, int zero_offset, int dtype, void* stream) {
  return w4a16_grouped_any(a, qweight, scales, qzeros, nullptr, c_q, c_scale, true, m_sizes, G, M, N, K, group_size,
                           zero_offset, dtype, stream);
}

int moe_gg_route_topk(const float* logits, int64_t T, int E, int k, int32_t* ids, int32_t* perm, int32_t* m_sizes,
                      int32_t* offsets, void* stream) {
  if (T < 0 || E <= 0 || k <= 0 || k > E) return MOE_GG_EINVAL;
  if (E > MOE_GG_MAX_ROUTE_EXPERTS || T * k > INT32_MAX) return MOE_GG_EUNSUPPORTED;
  if (!m_sizes || (T > 0 && (!logits || !ids || !perm))) return MOE_GG_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  hipError_t e = route_topk_launch(logits, (int)T, E, k, ids, s);
  if (e != hipSuccess) return (int)e;
  return (int)route_group_launch(ids, (int)(T * k), E, perm, m_sizes, offsets, s);
}

int moe_gg_route_group(const int32_t* flat_ids, int64_t n, int E, int32_t* perm, int32_t* m_sizes, int32_t* offsets,
                       void* stream) {
  if (n < 0 || E <= 0) return MOE_GG_EINVAL;
  if (E > MOE_GG_MAX_ROUTE_EXPERTS || n > INT32_MAX) return MOE_GG_EUNSUPPORTED;
  if (!m_sizes || (n > 0 && (!flat_ids || !perm))) return MOE_GG_EINVAL;
  return (int)route_group_launch(flat_ids, (int)n, E, perm, m_sizes, offsets, (hipStream_t)stream);
}

int moe_gg_align_block_size(const int32_t* perm, const int32_t* m_sizes, int E, int64_t n, int block_size,
                            int32_t* sorted_ids, int32_t* expert_ids, int32_t* num_post_pad, void* stream) {
  if (n < 0 || E <= 0 || block_size <= 0) return MOE_GG_EINVAL;
  if (E > MOE_GG_MAX_ROUTE_EXPERTS || n + (int64_t)E * block_size > INT32_MAX) return MOE_GG_EUNSUPPORTED;
  if (!m_sizes || !sorted_ids || !expert_ids || !num_post_pad || (n > 0 && !perm)) return MOE_GG_EINVAL;
  return (int)align_block_size_launch(perm, m_sizes, E, (int)n, block_size, sorted_ids, expert_ids, num_post_pad,
                                      (hipStream_t)stream);
}

int moe_gg_gather_rows(const void* x, const int32_t* perm, int k, void* out, int64_t n, int64_t row_bytes,
                       int64_t src_rows, const int32_t* n_valid, void* stream) {
  if (n < 0 || k <= 0 || row_bytes < 0 || src_rows < 0) return MOE_GG_EINVAL;
  if (n == 0 || row_bytes == 0) return MOE_GG_OK;
  if (!perm || !out || (src_rows > 0 && !x)) return MOE_GG_EINVAL;
  if (n > INT32_MAX) return MOE_GG_EUNSUPPORTED;
  if (row_bytes % 16 != 0 || !aligned(x, 16) || !aligned(out, 16)) return MOE_GG_EALIGN;
  if (n_valid && !aligned(n_valid, 4)) return MOE_GG_EALIGN;
  return (int)gather_rows_launch(x, perm, k, out, (int)n, row_bytes, src_rows, n_valid, (hipStream_t)stream);
}

// perm == nullptr: x is [M, K], the rows in expert-sorted order; else x is the token matrix [T, K] and sorted row i is
// its row perm[i] / k.
static int grouped_gemm_swiglu_16(const void* x, const void* w, void* y, const int32_t* m_sizes, int G, int64_t M, int n,
                                  int K, int64_t ldy, bool fp16, void* stream, const int32_t* perm = nullptr, int k = 1,
                                  int64_t T = 0) {
  if (G < 0 || M < 0 || n < 0 || K < 0) return MOE_GG_EINVAL;
  if (ldy < n) return MOE_GG_ESHAPE;
  if (G == 0 || M == 0 || n == 0) return MOE_GG_OK;
  if (!x || !w || !y || !m_sizes) return MOE_GG_EINVAL;
  if (perm) {
    if (k <= 0 || T <= 0) return MOE_GG_EINVAL;
    if (T * (int64_t)K * 2 >= INT32_MAX) return MOE_GG_EUNSUPPORTED;  // the loads add 32-bit byte offsets to the base
    if (!aligned(perm, 4)) return MOE_GG_EALIGN;
  }
  if (G > MOE_GG_MAX_GROUPS_ABI || M > INT32_MAX || ldy > INT32_MAX) return MOE_GG_EUNSUPPORTED;
  if (K == 0 || K % 64 != 0 || n % 4 != 0 || (int64_t)2 * n * K >= INT32_MAX || K >= PINGPONG_MAX_ROW_BYTES / 2 ||
      2 * (int64_t)n >= PINGPONG_MAX_ROW_BYTES)
    return MOE_GG_EUNSUPPORTED;
  if (!aligned(x, 16) || !aligned(w, 16) || !aligned(y, 2) || !aligned(m_sizes, 4)) return MOE_GG_EALIGN;
  const DeviceInfo* di = nullptr;
  int rc = current_device_info(&di);
  if (rc != MOE_GG_OK) return rc;
  GgParams p{};
  p.x = x; p.w = w; p.y = y; p.m_sizes = m_sizes;
  p.G = G; p.M = (int)M; p.N = 2 * n; p.K = K;
  p.ldy = (int)ldy;
  p.vec_store = vec_store_level(y, ldy, 0);
  p.xcds = di->xcds;
  int num_wg = di->cus - di->cus % p.xcds;
  if (num_wg <= 0) { num_wg = di->cus; p.xcds = 1; }
  if (!moe_gg_two_list_fits(M, G, 256, (n + 127) / 128, num_wg)) return MOE_GG_EUNSUPPORTED;
  p.fp16 = fp16 ? 1 : 0;
  p.split_tails = split_tails_on();
  p.gather_perm = perm;
  p.gather_k = k;
  p.gather_rows = (int)T;
  // The four-wave forms when one of them is pinned for the grouped GEMM (they have no row gather).
  const int pinned = g_variant[MOE_GG_OP_GG_BF16].load();
  if (!perm && (pinned == MOE_GG_GG_FOURWAVE_256 || pinned == MOE_GG_GG_FOURWAVE_TALL))
    return (int)gg_bf16_fourwave_swiglu_launch(p, pinned == MOE_GG_GG_FOURWAVE_TALL, num_wg, (hipStream_t)stream);
  return (int)gg_bf16_pingpong_swiglu_launch(p, num_wg, (hipStream_t)stream);
}

int moe_gg_grouped_gemm_swiglu_bf16(const void* x, const void* w, void* y, const int32_t* m_sizes, int G, int64_t M,
                                    int n, int K, int64_t ldy, void* stream) {
  return grouped_gemm_swiglu_16(x, w, y, m_sizes, G, M, n, K, ldy, false, stream);
}

int moe_gg_grouped_gemm_swiglu_f16(const void* x, const void* w, void* y, const int32_t* m_sizes, int G, int64_t M,
                                   int n, int K, int64_t ldy, void* stream) {
  return grouped_gemm_swiglu_16(x, w, y, m_sizes, G, M, n, K, ldy, true, stream);
}

int moe_gg_grouped_gemm_swiglu_gather(const void* tokens, int64_t T, const int32_t* perm, int k, const void* w, void* y,
                                      const int32_t* m_sizes, int G, int64_t M, int n, int K, int64_t ldy, int dtype,
                                      void* stream) {
  if (dtype != MOE_GG_DTYPE_BF16 && dtype != MOE_GG_DTYPE_FP16) return MOE_GG_EINVAL;
  if (T < 0 || k <= 0) return MOE_GG_EINVAL;
  if (M > 0 && G > 0 && n > 0 && (!perm || T == 0)) return MOE_GG_EINVAL;
  return grouped_gemm_swiglu_16(tokens, w, y, m_sizes, G, M, n, K, ldy, dtype == MOE_GG_DTYPE_FP16, stream, perm, k, T);
}

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }
// Leading dimension of the transposed operands: every expert padded to whole 64-row blocks.
static int64_t backward_ldm(int G, int64_t M) { return (M / 64 + G) * 64; }

size_t moe_gg_grouped_gemm_backward_workspace(int G, int64_t M, int N, int K, int grad_layout) {
  if (G <= 0 || M <= 0 || N <= 0 || K <= 0) return 0;
  const size_t ldm = (size_t)backward_ldm(G, M);
  size_t b = align256((size_t)G * N * K * 2) + align256((size_t)N * ldm * 2) + align256((size_t)K * ldm * 2);
  if (grad_layout == MOE_GG_OUT_BLOCK) b += align256((size_t)M * N * 2);
  return b;
}

// Scratch memory of moe_gg_grouped_gemm_backward_bf16_static: one array per device in the library's own image, so
// that entry point never allocates. Host code must not use the array's name as an address: the per-device address
// comes from hipGetSymbolAddress (static_scratch_ptr below).
static __device__ __align__(256) unsigned char scratch[MOE_GG_STATIC_SCRATCH_BYTES];

namespace {
void* g_scratch_ptr[kMaxDevices];
std::once_flag g_scratch_once[kMaxDevices];
hipError_t g_scratch_err[kMaxDevices];

// Address of `scratch` on the current device; looked up once per device with that device current.
int static_scratch_ptr(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return MOE_GG_EDEVICE;
  std::call_once(g_scratch_once[dev], [dev]() {
    void* p = nullptr;
    g_scratch_err[dev] = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    g_scratch_ptr[dev] = g_scratch_err[dev] == hipSuccess ? p : nullptr;
  });
  if (g_scratch_err[dev] != hipSuccess) return (int)g_scratch_err[dev];
  if (!g_scratch_ptr[dev]) return MOE_GG_EDEVICE;
  *out = g_scratch_ptr[dev];
  return MOE_GG_OK;
}
}  // namespace

// static_scratch: the workspace is the library's own array, looked up only when the call needs it, and a call
// whose transposed copies would not fit into it is refused.
static int backward_bf16_impl(const void* grad_out, int64_t ld_go, int grad_layout, const void* x, const void* w,
                              const int32_t* m_sizes, int G, int64_t M, int N, int K, void* grad_x, void* grad_w,
                              void* workspace, size_t workspace_bytes, bool static_scratch, void* stream) {
  if (G < 0 || M < 0 || N < 0 || K < 0) return MOE_GG_EINVAL;
  if (grad_layout != MOE_GG_OUT_MN && grad_layout != MOE_GG_OUT_BLOCK) return MOE_GG_EINVAL;
  const int64_t min_ld = grad_layout == MOE_GG_OUT_BLOCK ? (int64_t)N * G : (int64_t)N;
  if (ld_go < min_ld) return MOE_GG_ESHAPE;
  if (G == 0 || N == 0 || K == 0) return MOE_GG_OK;
  if (!grad_w || !m_sizes) return MOE_GG_EINVAL;
  if (M > 0 && (!grad_out || !x || !w || !grad_x)) return MOE_GG_EINVAL;
  if (G > MOE_GG_MAX_GROUPS_ABI || M > INT32_MAX - 64 * (int64_t)G || (int64_t)G * N > INT32_MAX || ld_go > INT32_MAX)
    return MOE_GG_EUNSUPPORTED;
  if (N % 4 != 0 || K % 4 != 0 || ld_go % 4 != 0) return MOE_GG_EUNSUPPORTED;
  // 32-bit byte offsets inside a 256-row operand tile of pitch 2 * ldm
  if (backward_ldm(G, M > 0 ? M : 1) > (1 << 22)) return MOE_GG_EUNSUPPORTED;
  if (grad_layout == MOE_GG_OUT_MN && ld_go != N) return MOE_GG_EUNSUPPORTED;
  const size_t ws_need = moe_gg_grouped_gemm_backward_workspace(G, M > 0 ? M : 1, N, K, grad_layout);
  if (!static_scratch && (!workspace || workspace_bytes < ws_need)) return MOE_GG_EINVAL;
  if (!aligned(grad_out, 16) || !aligned(x, 16) || !aligned(w, 16) || !aligned(grad_x, 16) || !aligned(grad_w, 16) ||
      !aligned(workspace, 256) || !aligned(m_sizes, 4))
    return MOE_GG_EALIGN;
  const DeviceInfo* di = nullptr;
  int rc = current_device_info(&di);
  if (rc != MOE_GG_OK) return rc;
  hipStream_t s = (hipStream_t)stream;
  const int64_t Mw = M > 0 ? M : 1;
  const int64_t ldm = backward_ldm(G, Mw);

  hipError_t e;
  int num_wg = di->cus - di->cus % di->xcds;
  int xcds = di->xcds;
  if (num_wg <= 0) { num_wg = di->cus; xcds = 1; }
  const int v = g_variant[MOE_GG_OP_GG_BF16].load();
  const int x_col_block = grad_layout == MOE_GG_OUT_BLOCK ? N : 0;
  // Both gradients can be computed from the operands as stored (ping-pong kernels with transposing LDS reads)
  // when there are enough 256 x 256 tiles (see below) and the row pitches allow 16-byte pieces; no workspace is
  // touched then.
  // Otherwise, or when a kernel variant is pinned, the operands are transposed into the workspace first.
  const bool direct_shapes = v < 0 && N % 8 == 0 && K % 8 == 0 && ld_go % 8 == 0 &&
                             ld_go < PINGPONG_MAX_ROW_BYTES / 2 && (int64_t)K < PINGPONG_MAX_ROW_BYTES / 2 &&
                             (int64_t)N < PINGPONG_MAX_ROW_BYTES / 2;
  // grad_x = dY [M, N] times w[g] [N, K]: from the operands as stored almost always: the other way transposes all
  // the weights first (254 -> 143 us at 8 experts x 32 rows, N = K = 4096); only calls of a few tiles are as fast
  // or faster through the small-tile forward kernels.
  const int64_t gx_ntn256 = (K + 255) / 256;
  const int64_t gx_t256 = (M / 256 + (G + 1) / 2) * gx_ntn256;
  const bool nt_ok = direct_shapes && N % 64 == 0 && moe_gg_two_list_fits(M, G, 256, (int)gx_ntn256, num_wg) &&
                     gx_t256 * 8 >= (int64_t)num_wg;
  // grad_w[g] = dY_g^T X_g.
  const int64_t t256 = (int64_t)G * ((N + 255) / 256) * ((K + 255) / 256);
  const bool pingpong_ok = t256 <= (int64_t)(MOE_GG_SEQ_CAP - 1) * num_wg;  // its per-workgroup tile table
  const bool gw_direct = M > 0 && direct_shapes && pingpong_ok && t256 * 4 >= (int64_t)num_wg * 3;
  if (static_scratch && !((nt_ok || M == 0) && gw_direct)) {
    // The call goes through transposed copies: they live in the library's own array.
    if (ws_need > (size_t)MOE_GG_STATIC_SCRATCH_BYTES) return MOE_GG_EUNSUPPORTED;
    rc = static_scratch_ptr(&workspace);
    if (rc != MOE_GG_OK) return rc;
  }
  char* ws = (char*)workspace;
  void* wt = ws;                      ws += align256((size_t)G * N * K * 2);
  void* dyt = ws;                     ws += align256((size_t)N * ldm * 2);
  void* xt = ws;                      ws += align256((size_t)K * ldm * 2);
  void* dyc = ws;
  if (M > 0) {
    if (nt_ok) {
      GgParams q{};
      q.x = grad_out; q.w = w; q.y = grad_x; q.m_sizes = m_sizes;
      q.G = G; q.M = (int)M; q.N = K; q.K = N;
      q.ldy = K;
      q.ldx = (int)ld_go; q.x_col_block = x_col_block;
      q.vec_store = vec_store_level(grad_x, K, 0);
      q.xcds = xcds;
      q.split_tails = split_tails_on();
      e = gg_bf16_pingpong_nt_launch(q, num_wg, s);
      if (e != hipSuccess) return (int)e;
    } else {
      // The forward kernels on (dY [M, N] dense, w^T [G*K, N]).
      const void* dy = grad_out;
      if (grad_layout == MOE_GG_OUT_BLOCK) {
        e = compact_block_launch(grad_out, dyc, m_sizes, G, (int)M, N, ld_go, N, s);
        if (e != hipSuccess) return (int)e;
        dy = dyc;
      }
      e = transpose_batched_launch(w, wt, G, N, K, s);
      if (e != hipSuccess) return (int)e;
      rc = moe_gg_grouped_gemm_bf16(dy, wt, grad_x, m_sizes, G, M, K, N, K, MOE_GG_OUT_MN, stream);
      if (rc != MOE_GG_OK) return rc;
    }
  }
  if (gw_direct) {
    GgParams q{};
    q.x = grad_out; q.w = x; q.y = grad_w; q.m_sizes = m_sizes;
    q.G = G; q.M = (int)M; q.N = N; q.K = K;
    q.ldy = K;
    q.ldx = (int)ld_go; q.x_col_block = x_col_block;
    q.vec_store = vec_store_level(grad_w, K, 0);
    q.xcds = xcds;
    return (int)gg_bf16_pingpong_wgrad_direct_launch(q, num_wg, s);
  }
  // dY^T and x^T with every expert padded to whole 64-row blocks. Also without any row (M = 0): nothing is read
  // then and every expert gets its one block of zeros, which makes grad_w all zeros below.
  e = transpose_padded_launch(grad_out, dyt, m_sizes, G, (int)M, N, ld_go, x_col_block, ldm, s);
  if (e != hipSuccess) return (int)e;
  e = transpose_padded_launch(x, xt, m_sizes, G, (int)M, K, K, 0, ldm, s);
  if (e != hipSuccess) return (int)e;
  GgParams p{};
  p.x = dyt; p.w = xt; p.y = grad_w; p.m_sizes = m_sizes;
  p.G = G; p.M = (int)ldm; p.N = N; p.K = K;
  p.ldy = K;
  p.col_block = 0;
  p.vec_store = vec_store_level(grad_w, K, 0);
  p.xcds = xcds;
  p.skip_rows = (int)M;
  if (v == MOE_GG_GG_TILED_256) return (int)gg_bf16_wgrad_launch(p, 256, num_wg, s);
  if (v == MOE_GG_GG_TILED_128) return (int)gg_bf16_wgrad_launch(p, 128, num_wg, s);
  if (v == MOE_GG_GG_PINGPONG_256 && !pingpong_ok) return MOE_GG_EUNSUPPORTED;
  if (v == MOE_GG_GG_PINGPONG_256 || (v < 0 && pingpong_ok && t256 * 4 >= (int64_t)num_wg * 3))
    return (int)gg_bf16_pingpong_wgrad_launch(p, num_wg, s);
  if (v < 0 && t256 >= num_wg) return (int)gg_bf16_wgrad_launch(p, 256, num_wg, s);
  return (int)gg_bf16_wgrad_launch(p, 128, num_wg, s);
}

int moe_gg_grouped_gemm_backward_bf16(const void* grad_out, int64_t ld_go, int grad_layout, const void* x, const void* w,
                                      const int32_t* m_sizes, int G, int64_t M, int N, int K, void* grad_x, void* grad_w,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  return backward_bf16_impl(grad_out, ld_go, grad_layout, x, w, m_sizes, G, M, N, K, grad_x, grad_w, workspace,
                            workspace_bytes, false, stream);
}

int moe_gg_grouped_gemm_backward_bf16_static(const void* grad_out, int64_t ld_go, int grad_layout, const void* x,
                                             const void* w, const int32_t* m_sizes, int G, int64_t M, int N, int K,
                                             void* grad_x, void* grad_w, void* stream) {
  return backward_bf16_impl(grad_out, ld_go, grad_layout, x, w, m_sizes, G, M, N, K, grad_x, grad_w, nullptr, 0, true,
                            stream);
}

static int silu_and_mul_any(const void* in, void* out, int64_t rows, int n, bool fp16, void* stream) {
  if (rows < 0 || n < 0) return MOE_GG_EINVAL;
  if (rows == 0 || n == 0) return MOE_GG_OK;
  if (!in || !out) return MOE_GG_EINVAL;
  if (n % 8 != 0) return MOE_GG_ESHAPE;
  if (!aligned(in, 16) || !aligned(out, 16)) return MOE_GG_EALIGN;
  return (int)silu_and_mul_launch(in, out, rows, n, fp16, (hipStream_t)stream);
}

int moe_gg_silu_and_mul(const void* in, void* out, int64_t rows, int n, void* stream) {
  return silu_and_mul_any(in, out, rows, n, false, stream);
}

int moe_gg_silu_and_mul_f16(const void* in, void* out, int64_t rows, int n, void* stream) {
  return silu_and_mul_any(in, out, rows, n, true, stream);
}

int moe_gg_invert_perm(const int32_t* perm, int32_t* inv, int64_t n, const int32_t* n_valid, void* stream) {
  if (n < 0) return MOE_GG_EINVAL;
  if (n == 0) return MOE_GG_OK;
  if (!perm || !inv) return MOE_GG_EINVAL;
  if (n > INT32_MAX) return MOE_GG_EUNSUPPORTED;
  return (int)invert_perm_launch(perm, inv, (int)n, n_valid, (hipStream_t)stream);
}

static int combine_topk_any(const void* y, const int32_t* inv, const void* weights, int weights_dtype, bool fp16,
                            void* out, int64_t T, int k, int d, int64_t n_rows, void* stream) {
  if (T < 0 || k <= 0 || d < 0 || n_rows < 0) return MOE_GG_EINVAL;
  if (weights_dtype != MOE_GG_DTYPE_FP32 && weights_dtype != (fp16 ? MOE_GG_DTYPE_FP16 : MOE_GG_DTYPE_BF16)) return MOE_GG_EINVAL;
  if (T == 0 || d == 0) return MOE_GG_OK;
  if (!y || !inv || !weights || !out) return MOE_GG_EINVAL;
  if (d % 8 != 0) return MOE_GG_ESHAPE;
  if (T > INT32_MAX || n_rows > INT32_MAX || T * k > INT32_MAX) return MOE_GG_EUNSUPPORTED;
  if (!aligned(y, 16) || !aligned(out, 16) || !aligned(weights, weights_dtype == MOE_GG_DTYPE_FP32 ? 4 : 2))
    return MOE_GG_EALIGN;
  return (int)combine_topk_launch(y, inv, weights, weights_dtype != MOE_GG_DTYPE_FP32, fp16, out, (int)T, k, d,
                                  (int)n_rows, (hipStream_t)stream);
}

int moe_gg_combine_topk(const void* y, const int32_t* inv, const void* weights, int weights_dtype, void* out,
                        int64_t T, int k, int d, int64_t n_rows, void* stream) {
  return combine_topk_any(y, inv, weights, weights_dtype, false, out, T, k, d, n_rows, stream);
}

int moe_gg_combine_topk_f16(const void* y, const int32_t* inv, const void* weights, int weights_dtype, void* out,
                            int64_t T, int k, int d, int64_t n_rows, void* stream) {
  return combine_topk_any(y, inv, weights, weights_dtype, true, out, T, k, d, n_rows, stream);
}

int moe_gg_fp8_groupwise_quant(const void* in, int dtype, void* out, float* scales, int64_t numel, void* stream) {
  if (numel < 0) return MOE_GG_EINVAL;
  if (dtype != MOE_GG_DTYPE_BF16 && dtype != MOE_GG_DTYPE_FP32) return MOE_GG_EINVAL;
  if (numel % 128 != 0) return MOE_GG_ESHAPE;
  if (numel == 0) return MOE_GG_OK;
  if (!in || !out || !scales) return MOE_GG_EINVAL;
  if (!aligned(in, 8) || !aligned(out, 2) || !aligned(scales, 4)) return MOE_GG_EALIGN;
  return (int)fp8_groupwise_quant_launch(in, dtype == MOE_GG_DTYPE_BF16, out, scales, numel / 128, (hipStream_t)stream);
}

int moe_gg_fp8_block128_quant(const void* in, int dtype, void* out, float* scales, int64_t rows, int K, void* stream) {
  if (rows < 0 || K < 0) return MOE_GG_EINVAL;
  if (dtype != MOE_GG_DTYPE_BF16 && dtype != MOE_GG_DTYPE_FP32) return MOE_GG_EINVAL;
  if (rows % 128 != 0 || K % 128 != 0) return MOE_GG_ESHAPE;
  if (rows == 0 || K == 0) return MOE_GG_OK;
  if (!in || !out || !scales) return MOE_GG_EINVAL;
  if (rows / 128 > 65535) return MOE_GG_EUNSUPPORTED;
  if (!aligned(in, 16) || !aligned(out, 16) || !aligned(scales, 4)) return MOE_GG_EALIGN;
  return (int)fp8_block128_quant_launch(in, dtype == MOE_GG_DTYPE_BF16, out, scales, rows, K, (hipStream_t)stream);
}

int moe_gg_host_enumerate_tiles(const int32_t* m_sizes_host, int G, int64_t M, int N, int block_m,
                                int block_n, int num_workgroups, int xcds, int32_t* out,
                                int max_tiles) {
  if (!m_sizes_host || !out || G <= 0 || G > MOE_GG_MAX_GROUPS_ABI || block_m <= 0 || block_n <= 0 ||
      num_workgroups <= 0 || xcds <= 0 || num_workgroups % xcds != 0 || M < 0 || N <= 0)
    return MOE_GG_EINVAL;
  static thread_local int32_t row_off[MOE_GG_MAX_GROUPS_ABI + 1], tile_off[MOE_GG_MAX_GROUPS_ABI + 1];
  const int ntn = moe_gg_cdiv(N, block_n);
  const int total = moe_gg_build_tables(m_sizes_host, G, M, block_m, ntn, row_off, tile_off);
  int written = 0;
  for (int wg = 0; wg < num_workgroups; ++wg) {
    for (int round = 0; round * num_workgroups < total; ++round) {
      const int L = moe_gg_tile_of(wg, num_workgroups, xcds, round);
      if (L >= total) continue;
      if (written >= max_tiles) return written;
      MoeGgTile t = moe_gg_decode_tile(row_off, tile_off, G, L, block_m);
      int32_t* o = out + (size_t)written * 5;
      o[0] = wg; o[1] = t.g; o[2] = t.tm; o[3] = t.tn; o[4] = t.row0;
      ++written;
    }
  }
  return written;
}

int moe_gg_host_tails_apart(const int32_t* m_sizes_host, int G, int64_t M, int N, int K, int num_workgroups) {
  if (!m_sizes_host || G <= 0 || G > MOE_GG_MAX_GROUPS_ABI || num_workgroups <= 0 || M < 0 || N <= 0 || K <= 0)
    return MOE_GG_EINVAL;
  const int ntn = moe_gg_cdiv(N, 256);
  int64_t r = 0, nl = 0, ns = 0, passes = 0;
  for (int g = 0; g < G; ++g) {
    const int m = moe_gg_clamp_rows(m_sizes_host[g], r, M);
    r += m;
    nl += moe_gg_long_row_tiles(m, 256) * ntn;
    ns += moe_gg_low_row_tiles(m, 256) * ntn;
    passes += (int64_t)moe_gg_low_passes(m, 256) * ntn;
  }
  if (nl > INT32_MAX || ns > INT32_MAX) return MOE_GG_EUNSUPPORTED;
  return G <= TAILS_APART_MAX_GROUPS && K >= TAILS_APART_MIN_K && K % 128 == 0 &&
                 moe_gg_tails_apart((int)nl, (int)ns, passes, num_workgroups)
             ? 1
             : 0;
}

int moe_gg_host_tail_pieces(int n_long, int n_low, int num_workgroups) {
  if (n_long < 0 || n_low < 0 || num_workgroups <= 0) return MOE_GG_EINVAL;
  return split_tails_on() ? moe_gg_tail_pieces_low(n_long, n_low, num_workgroups) : moe_gg_tail_pieces(n_long, num_workgroups);
}

int moe_gg_host_enumerate_tiles_two_lists(const int32_t* m_sizes_host, int G, int64_t M, int N, int block_m,
                                          int block_n, int num_workgroups, int xcds, int32_t* out,
                                          int max_tiles) {
  if (!m_sizes_host || !out || G <= 0 || G > MOE_GG_MAX_GROUPS_ABI || block_m != 256 || block_n <= 0 ||
      num_workgroups <= 0 || xcds <= 0 || num_workgroups % xcds != 0 || M < 0 || N <= 0)
    return MOE_GG_EINVAL;
  static thread_local int32_t row_off[MOE_GG_MAX_GROUPS_ABI + 1], long_off[MOE_GG_MAX_GROUPS_ABI + 1],
      low_off[MOE_GG_MAX_GROUPS_ABI + 1];
  // The lists of a launch that computes its low tiles itself, in the tile order that is in force
  // (MOE_GG_OP_TILE_ORDER); the decode below is the kernels' own.
  const bool tall = g_variant[MOE_GG_OP_TILE_ORDER].load() == MOE_GG_ORDER_TALL_TILES;
  const bool split = !tall && split_tails_on() != 0;
  const int ntn = moe_gg_cdiv(N, block_n);
  int64_t r = 0;
  int nl = 0, ns = 0;
  for (int g = 0; g < G; ++g) {
    row_off[g] = (int32_t)r; long_off[g] = nl; low_off[g] = ns;
    const int m = moe_gg_clamp_rows(m_sizes_host[g], r, M);
    r += m;
    nl += (tall ? moe_gg_long_row_tiles_tall(m, block_m) : moe_gg_long_row_tiles2(m, block_m, split)) * ntn;
    ns += (tall ? moe_gg_low_row_tiles_tall(m, block_m) : moe_gg_low_row_tiles2(m, block_m, split)) * ntn;
  }
  row_off[G] = (int32_t)r; long_off[G] = nl; low_off[G] = ns;
  const int tail_s = split ? moe_gg_tail_pieces_low(nl, ns, num_workgroups) : moe_gg_tail_pieces(nl, num_workgroups);
  const int tail_first = moe_gg_tail_first_s(nl, num_workgroups, tail_s);
  const int long_ids = moe_gg_long_ids_s(nl, num_workgroups, tail_s);
  const int total = long_ids + ns;
  int written = 0;
  for (int wg = 0; wg < num_workgroups; ++wg) {
    int n_long = 0, n_low = 0;
    while (n_long * num_workgroups < long_ids && moe_gg_tile_of(wg, num_workgroups, xcds, n_long) < long_ids) ++n_long;
    while ((n_long + n_low) * num_workgroups < total && moe_gg_tile_of(wg, num_workgroups, xcds, n_long + n_low) < total) ++n_low;
    const int n_my = n_long + n_low, phase = moe_gg_low_phase(wg, xcds);
    for (int seq = 0; seq < n_my; ++seq) {
      const int L = moe_gg_tile_of(wg, num_workgroups, xcds, moe_gg_seq_round(seq, n_my, n_low, phase));
      if (written >= max_tiles) return written;
      if (L >= total) return MOE_GG_EINVAL;  // cannot happen
      const MoeGgListTile t = tall ? moe_gg_two_list_decode_tall(row_off, long_off, low_off, G, L, long_ids, tail_first,
                                                                 tail_s, block_m, block_n)
                                   : moe_gg_two_list_decode(row_off, long_off, low_off, G, L, long_ids, tail_first, tail_s,
                                                            block_m, block_n, split);
      int32_t* o = out + (size_t)written * 6;
      o[0] = wg; o[1] = t.g; o[2] = t.m0; o[3] = t.h; o[4] = t.n0; o[5] = block_n;
      ++written;
    }
  }
  return written;
}

}  // extern "C"
