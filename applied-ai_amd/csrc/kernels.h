// Internal launch interface between the C-ABI layer (api.hip) and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// Arguments of the grouped GEMM kernels. x is [M, K] row-major, w is [G * N, K] row-major
// (expert g owns rows g*N .. (g+1)*N), y has leading dimension ldy; expert g writes its rows at
// column offset g * col_block (0 for the [M, N] layout, N for the [M, N*G] block layout).
struct GgParams {
  const void* x;
  const void* w;
  void* y;
  const int32_t* m_sizes;  // device, G entries
  const float* x_scale;    // fp8 only
  const float* w_scale;    // fp8 only
  int G, M, N, K;
  int ldy;
  int col_block;
  int vec_store;  // 1: 8-byte aligned row segments can be stored as one dwordx2; 2: also 16-byte ones as dwordx4
  int xcds;       // number of XCDs the persistent grid is spread over
  int skip_rows;  // tiled fp8 kernel: experts with at most this many rows are left to the streaming kernel
  int ldx;          // gg_bf16_pingpong_nt / _wgrad_direct: leading dimension of x (the output gradient)
  int x_col_block;  // gg_bf16_pingpong_nt / _wgrad_direct: expert g reads x at column offset g * x_col_block
  // gg_bf16_pingpong + gg_bf16_decode_tails pair: 0, or the ping-pong launch's workgroup count; the low tiles are
  // then computed by the small-M kernel whenever moe_gg_tails_apart() says so (both kernels evaluate it).
  int tails_apart;
  int fp16;  // forward kernels: x, w and y are IEEE half instead of bf16 (same layouts)
  // gg_bf16_pingpong_swiglu with a row gather: when gather_perm is set, x is the token matrix [gather_rows, K] and row
  // i of the expert-sorted order (M of them) is its row gather_perm[i] / gather_k.
  const int32_t* gather_perm;
  int gather_k;
  int gather_rows;
  // Forward ping-pong kernels: 1 = split-tail tile order (moe_gg_split_tail, row pieces chosen by
  // moe_gg_tail_pieces_low), 0 = the plain two-list order (row pieces by moe_gg_tail_pieces).
  int split_tails;
};

// block_m in {256, 128, 64}, or GG_TILED_256_FOUR_WAVES for the 256 x 256 tile on a four-wave workgroup; the matching
// tile width is gg_bf16_tiled_block_n(block_m).
constexpr int GG_TILED_256_FOUR_WAVES = 2564;
hipError_t gg_bf16_tiled_launch(const GgParams& p, int block_m, int num_wg, hipStream_t stream);
int gg_bf16_tiled_block_n(int block_m);
// 256 x 256 tiles, ping-pong schedule (gg_pingpong.hip); the fp8 form takes the scale modes of gg_fp8_launch
// and honours p.skip_rows.
hipError_t gg_bf16_pingpong_launch(const GgParams& p, int num_wg, hipStream_t stream);
// The same tiles, tile order and LDS stages on four waves of 128 x 128 outputs each (bf16 / fp16 forward only).
// tall: tiles of up to 256 + 32 rows (the lists of moe_gg_tall_tail)
hipError_t gg_bf16_fourwave_launch(const GgParams& p, bool tall, int num_wg, hipStream_t stream);
// ... and its form with SiLU-and-mul in the epilogue (the arguments of gg_bf16_pingpong_swiglu_launch, no row gather).
hipError_t gg_bf16_fourwave_swiglu_launch(const GgParams& p, bool tall, int num_wg, hipStream_t stream);
hipError_t gg_fp8_pingpong_launch(const GgParams& p, int scale_mode, int num_wg, hipStream_t stream);
hipError_t gg_bf16_generic_launch(const GgParams& p, hipStream_t stream);
// Small-M split-K kernel; nf = 16-row weight fragments per wave (2 or 4), mf = 16-row activation
// fragments per pass (1, 2 or 4). Needs K % 128 == 0 and 16-byte aligned x and w.
hipError_t gg_bf16_decode_launch(const GgParams& p, int nf, int mf, hipStream_t stream);
// The same kernel over the low tiles only (rows of an expert beyond its last full 256-row tile, when
// moe_gg_low_row_tiles counts them as a low tile), and only if moe_gg_tails_apart() holds for the launch;
// p.tails_apart = workgroup count of the ping-pong launch it completes.
hipError_t gg_bf16_decode_tails_launch(const GgParams& p, hipStream_t stream);

// W4A16 split-K dequant GEMM (w4a16.hip). a, scales, c share one 16-bit float type.
struct W4Params {
  const void* a;           // [M, K]
  const int32_t* qweight;  // [K/8, N]
  const void* scales;      // [K/group_size, N]
  const int32_t* qzeros;   // [K/group_size, N/8]
  void* c;                 // [M, N]
  int M, N, K;
  int group_size;
  int zero_offset;
  // Grouped (MoE) call: m_sizes != nullptr, G experts; a / c are [M, K] / [M, N] with rows sorted by expert,
  // qweight [G, K/8, N], scales [G, K/group_size, N], qzeros [G, K/group_size, N/8]; M is the total row count.
  const int32_t* m_sizes;
  int G;
  // fp8 output instead of c (c may be nullptr then): cq [M, N] e4m3fn and cscale [M, N/128] fp32, the 1 x 128
  // group-wise quantisation of the 16-bit result; needs N % 128 == 0.
  void* cq = nullptr;
  float* cscale = nullptr;
};
// variant: bits of MOE_GG_OP_W4A16's variant (0 = the kernels chosen by default), group size 128 and 16-bit output only:
// 1: more than 32 rows (per expert, on average): passes of four activation fragments on four waves;
// 2: up to 16 rows: two extra waves per workgroup that request every line of its weight strip ahead of the
//    consumer waves, and lanes of activation rows that do not exist issue no loads;
// 4: the activations of a quantisation group go through the wave's own LDS area (whole-line loads).
hipError_t w4a16_splitk_launch(const W4Params& p, bool fp16, int variant, hipStream_t stream);

// fp8 e4m3 grouped GEMM (gg_fp8.hip). scale_mode 0: x_scale [M], w_scale [G*N]; 1: x_scale [M, K/128],
// w_scale [G*N/128, K/128]. Needs K % 128 == 0 (and N % 128 == 0 in block mode), 16-byte aligned x, w.
hipError_t gg_fp8_launch(const GgParams& p, int scale_mode, int num_wg, hipStream_t stream);
// Streaming split-K kernel for experts with 1 .. gg_fp8_stream_max_rows() rows (gg_fp8_stream.hip); experts
// outside that range are not touched. Pair it with gg_fp8_launch and p.skip_rows = gg_fp8_stream_max_rows().
hipError_t gg_fp8_stream_launch(const GgParams& p, int scale_mode, hipStream_t stream);
int gg_fp8_stream_max_rows();

// Routing (routing.hip). E <= MOE_GG_MAX_ROUTE_EXPERTS; ids are int32.
hipError_t route_topk_launch(const float* logits, int T, int E, int k, int32_t* ids, hipStream_t stream);
hipError_t route_group_launch(const int32_t* flat, int n, int E, int32_t* perm, int32_t* m_sizes, int32_t* offsets,
                              hipStream_t stream);
// sorted_ids [n + E * (block_size - 1)], expert_ids [n + E], num_post_pad [1]; perm / m_sizes as route_group_launch wrote them.
hipError_t align_block_size_launch(const int32_t* perm, const int32_t* m_sizes, int E, int n, int block_size,
                                   int32_t* sorted_ids, int32_t* expert_ids, int32_t* num_post_pad,
                                   hipStream_t stream);
hipError_t gather_rows_launch(const void* x, const int32_t* perm, int k, void* out, int n, int64_t row_bytes,
                              int64_t src_rows, const int32_t* n_valid, hipStream_t stream);
// 1 x 128 fp8 quantiser (quant.hip); `groups` groups of 128 consecutive elements.
hipError_t fp8_groupwise_quant_launch(const void* in, bool bf16_in, void* out, float* scales, int64_t groups,
                                      hipStream_t stream);

// 128 x 128 block quantiser of a [rows, K] matrix (quant.hip); rows % 128 == 0, K % 128 == 0; scales [rows/128, K/128].
hipError_t fp8_block128_quant_launch(const void* in, bool bf16_in, void* out, float* scales, int64_t rows, int K,
                                     hipStream_t stream);

// MoE layer glue (moe_layer.hip). bf16 data; n and d multiples of 8; 16-byte aligned pointers.
hipError_t silu_and_mul_launch(const void* in, void* out, int64_t rows, int n, bool fp16, hipStream_t stream);
hipError_t invert_perm_launch(const int32_t* perm, int32_t* inv, int n, const int32_t* n_valid, hipStream_t stream);
hipError_t combine_topk_launch(const void* y, const int32_t* inv, const void* weights, bool weights_16bit, bool fp16,
                               void* out, int T, int k, int d, int n_rows, hipStream_t stream);

// Backward pass (gg_backward.hip, gg_bf16_prefill.hip). bf16.
// src [B, R, C] -> dst [B, C, R].
hipError_t transpose_batched_launch(const void* src, void* dst, int B, int R, int C, hipStream_t stream);
// dst[c][pad_off[g] + i] = src[row_off[g] + i][g * col_block + c], experts padded to multiples of 64 columns with zeros.
hipError_t transpose_padded_launch(const void* src, void* dst, const int32_t* m_sizes, int G, int M, int C,
                                   int64_t src_pitch, int col_block, int64_t ldm, hipStream_t stream);
// dst [M, C] <- the expert's own C columns (at g * col_block) of src [M, src_pitch]. C % 4 == 0, 8-byte aligned rows.
hipError_t compact_block_launch(const void* src, void* dst, const int32_t* m_sizes, int G, int M, int C, int64_t src_pitch,
                                int col_block, hipStream_t stream);
// y [M, n] = silu(x w_gate^T) * (x w_up^T) with w [G * 2n, K] (gate rows first); p.N = 2n, p.ldy >= n, p.col_block unused.
hipError_t gg_bf16_pingpong_swiglu_launch(const GgParams& p, int num_wg, hipStream_t stream);
// y [M, N] = x [M, K] times w[g] [K, N] (weights row-major along N, not along the reduction): p.w = [G * K, N];
// x has leading dimension p.ldx and expert g reads it at column offset g * p.x_col_block. K % 64 == 0, N % 8 == 0.
hipError_t gg_bf16_pingpong_nt_launch(const GgParams& p, int num_wg, hipStream_t stream);
// dW[g] [N, K] = dY_g^T X_g read from the operands as stored: p.x = dY [M, ldx] (expert g at column offset
// g * x_col_block), p.w = X [M, K], p.M = number of rows, p.y = dW [G * N, K], p.ldy = K. N % 8 == 0, K % 8 == 0,
// ldx % 8 == 0.
hipError_t gg_bf16_pingpong_wgrad_direct_launch(const GgParams& p, int num_wg, hipStream_t stream);
hipError_t gg_bf16_pingpong_wgrad_launch(const GgParams& p, int num_wg, hipStream_t stream);
// dW = dY^T X per expert on the transposed, padded operands; p.x = dY^T [N, ldm], p.w = X^T [K, ldm], p.M = ldm,
// p.skip_rows = number of gradient rows (bound for m_sizes), p.y = dW [G * N, K] with p.ldy = K. block in {256, 128}.
hipError_t gg_bf16_wgrad_launch(const GgParams& p, int block, int num_wg, hipStream_t stream);
