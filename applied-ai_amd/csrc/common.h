// Shared device-side types and helpers for the gfx950 (CDNA4) MoE grouped-GEMM kernels.
// Everything here assumes 64-wide wavefronts and the 16x16xK MFMA register layouts:
//   A operand: lane l holds row (l % 16), 8 (bf16) / 8 (fp8, x32) consecutive K elements of chunk (l / 16)
//   B operand: lane l holds column (l % 16), same K chunk
//   C/D:       lane l holds rows 4*(l/16)+{0,1,2,3} of column (l % 16)
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2_t;

#define MOE_GG_MAX_GROUPS 1024  // size of the in-LDS group offset table (== MOE_GG_MAX_GROUPS_ABI)

#define DEVINL __device__ __forceinline__

// Round-to-nearest-even fp32 -> bf16 pair packed in one dword (lo = a, hi = b).
DEVINL uint32_t pack_bf16x2(float a, float b) {
  bf16x2_t v;
  v[0] = (__bf16)a;
  v[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, v);
}

DEVINL int lane_id() { return threadIdx.x & 63; }
DEVINL int wave_id() { return threadIdx.x >> 6; }

// Byte offset of 16-byte chunk `c` (0..7) of row `r` in an LDS tile whose rows hold 64 bf16 (128 B).
// The XOR term spreads the 16 rows a 16x16 MFMA fragment touches over all 64 LDS banks
// for ds_read_b128, while a row's 8 chunks stay inside its own 128-byte line.
DEVINL int lds_swizzle_off(int r, int c) { return r * 128 + ((c ^ ((r >> 1) & 7)) << 4); }
