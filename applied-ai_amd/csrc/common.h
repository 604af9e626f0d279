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

// The same for IEEE half.
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
DEVINL uint32_t pack_f16x2(float a, float b) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)a) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)b) << 16);
}
// 16-bit float type of a kernel instantiation: F16 = IEEE half, else bf16. Both are 2 bytes, so the data movement of
// the kernels is the same; only the MFMA instruction and the conversions of the epilogue differ.
template <bool F16> DEVINL uint32_t pack_16x2(float a, float b) { return F16 ? pack_f16x2(a, b) : pack_bf16x2(a, b); }
template <bool F16> DEVINL uint16_t cvt_16(float a) {
  return F16 ? __builtin_bit_cast(uint16_t, (_Float16)a) : __builtin_bit_cast(uint16_t, (__bf16)a);
}
template <bool F16> DEVINL float f32_of_16(uint16_t h) {
  return F16 ? (float)__builtin_bit_cast(_Float16, h) : __builtin_bit_cast(float, (uint32_t)h << 16);
}
template <bool F16> DEVINL f32x4_t mfma_16x16x32(u32x4_t a, u32x4_t b, f32x4_t c) {
  if (F16) return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// A point where all lanes of a wave are known to be together again: the top of a loop whose body ends in lane-masked
// blocks. Nothing on the GPU (no instruction, no constraint on the compiler's scheduling). A host build of the kernels
// that runs the lanes of a wave as separate threads of control defines wave_whole() as the place where they meet.
#ifndef wave_whole
DEVINL void wave_whole() {}
#endif

DEVINL int lane_id() { return threadIdx.x & 63; }
DEVINL int wave_id() { return threadIdx.x >> 6; }

// Byte offset of 16-byte chunk `c` (0..7) of row `r` in an LDS tile whose rows hold 64 bf16 (128 B).
// The XOR term spreads the 16 rows a 16x16 MFMA fragment touches over all 64 LDS banks
// for ds_read_b128, while a row's 8 chunks stay inside its own 128-byte line.
DEVINL int lds_swizzle_off(int r, int c) { return r * 128 + ((c ^ ((r >> 1) & 7)) << 4); }
