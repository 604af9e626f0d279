// Host stand-in for <hip/hip_runtime.h>: lets the library's .hip sources compile as plain C++ (clang++, x86-64) and
// run on the CPU under a lockstep-wave emulation (emu_core.cpp). Test infrastructure only: nothing in the product
// includes or links it. A kernel launch runs its workgroups one after the other; the threads of a workgroup are
// fibers that switch at barriers and at wave-wide operations (shuffles, readfirstlane, MFMA, transposing LDS reads),
// so data exchanged between lanes takes the same routes as on the GPU. What is modelled: 64-lane waves, the register
// layouts of the 16x16 MFMAs, LDS as one address range with 32-bit addresses, global->LDS loads that land only when
// the issuing wave waits on its counter (or at issue, see EMU_DMA). What is not: timing, caches, bank conflicts.
#pragma once
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <functional>

using std::max;
using std::min;

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __shared__ static __attribute__((section("emu_lds")))
#define __align__(n) __attribute__((aligned(n)))

typedef int hipError_t;
enum : int { hipSuccess = 0, hipErrorInvalidValue = 1, hipErrorLaunchFailure = 719 };
typedef void* hipStream_t;
struct dim3 {
  unsigned x, y, z;
  dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct hipDeviceProp_t { int multiProcessorCount; };
struct float2 { float x, y; };

extern dim3 threadIdx, blockIdx, blockDim, gridDim;

namespace emu {
struct i32x8 { int32_t v[8]; };
typedef __attribute__((__vector_size__(16))) float f32x4;
typedef __attribute__((__vector_size__(16))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16))) _Float16 f16x8;
typedef __attribute__((__vector_size__(32))) int i32x8v;
typedef short i16x4 __attribute__((ext_vector_type(4)));

void launch(dim3 grid, dim3 block, size_t dyn_lds, const std::function<void()>& body);
void* dyn_lds();
void syncthreads();
// One wave-wide exchange: every lane deposits `bytes` (<= 64) bytes, then may read any lane's deposit until it
// calls exchange_done(). Lanes of a wave that are not at the same exchange (divergent control flow) do not take
// part; `site` identifies the place (default: the caller's address).
const unsigned char* exchange(const void* mine, int bytes, const void* site = nullptr);  // returns the table [64][64]
unsigned long long exchange_mask();                            // lanes that took part in the current exchange
void exchange_done(const void* site = nullptr);
int lane();
void dma(int bytes, const void* sbase, uint32_t voff, uint32_t lds_addr);
void wait_vm(int n);
void wait_lds();
char* lds_ptr(uint32_t addr, int bytes);
void fail(const char* what);

template <class T> inline T get_lane(T v, int src, const void* site = nullptr) {
  static_assert(sizeof(T) <= 8, "");
  const unsigned char* t = exchange(&v, sizeof(T), site);
  T r = v;
  if (src >= 0 && src < 64 && ((exchange_mask() >> src) & 1)) memcpy(&r, t + 64 * src, sizeof(T));
  exchange_done(site);
  return r;
}
int readfirstlane(int v);
void wave_join();
unsigned long long ballot(int pred);
f32x4 mfma_16x16x32_bf16(bf16x8 a, bf16x8 b, f32x4 c);
f32x4 mfma_16x16x32_f16(f16x8 a, f16x8 b, f32x4 c);
f32x4 mfma_16x16x128_fp8(i32x8v a, i32x8v b, f32x4 c);
i16x4 ds_read_tr16_b64(uint32_t lds_addr);
uint32_t perm(uint32_t s0, uint32_t s1, uint32_t sel);
int ds_swizzle(int v, int pattern);
int cvt_pk_fp8_f32(float a, float b, int old, bool hi);
}  // namespace emu

#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...) \
  emu::launch((grid), (block), (shmem), [=]() { kernel(__VA_ARGS__); })
#define HIP_SYMBOL(x) (&(x))
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
inline const char* hipGetErrorString(hipError_t) { return "emulated HIP error"; }
hipError_t hipGetDeviceProperties(hipDeviceProp_t* p, int dev);
enum hipDeviceAttribute_t { hipDeviceAttributeNumberOfXccs };
hipError_t hipDeviceGetAttribute(int* value, hipDeviceAttribute_t attr, int dev);
template <class T> inline hipError_t hipGetSymbolAddress(void** p, T* sym) { *p = (void*)sym; return hipSuccess; }

inline void __syncthreads() { emu::syncthreads(); }
template <class T> inline T __shfl_xor(T v, int d, int = 64) { return emu::get_lane(v, emu::lane() ^ d); }
template <class T> inline T __shfl_up(T v, int d, int = 64) { return emu::get_lane(v, emu::lane() - d); }
template <class T> inline T __shfl(T v, int src, int = 64) { return emu::get_lane(v, src & 63); }
inline unsigned long long __ballot(int pred) { return emu::ballot(pred); }
inline int __popcll(unsigned long long v) { return __builtin_popcountll(v); }
inline int __ffsll(long long v) { return __builtin_ffsll(v); }
template <class T> inline T atomicAdd(T* p, T v) { return __atomic_fetch_add(p, v, __ATOMIC_RELAXED); }

// Fast-math exponential of the device library: the host's expf (results differ in the last bits).
#define __expf(x) expf(x)
#define __builtin_amdgcn_readfirstlane(v) emu::readfirstlane((int)(v))
#define __builtin_amdgcn_wave_barrier() emu::wave_join()
#define wave_whole() emu::wave_join()   // common.h's marker of a point where a wave's lanes are together again
#define __builtin_amdgcn_sched_barrier(m) ((void)0)
#define __builtin_amdgcn_sched_group_barrier(a, b, c) ((void)0)
#define __builtin_amdgcn_s_setprio(p) ((void)0)
#define __builtin_amdgcn_perm(a, b, s) emu::perm((a), (b), (s))
#define __builtin_amdgcn_ds_swizzle(v, p) emu::ds_swizzle((v), (p))
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, x, y, z) emu::mfma_16x16x32_bf16((a), (b), (c))
#define __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, x, y, z) emu::mfma_16x16x32_f16((a), (b), (c))
// Scale operands that are all the constant 0 select the unscaled instruction on the GPU; nothing else is used.
#define __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, cbsz, blgp, oa, sa, ob, sb) \
  emu::mfma_16x16x128_fp8(__builtin_bit_cast(emu::i32x8v, (a)), __builtin_bit_cast(emu::i32x8v, (b)), (c))
#define __builtin_amdgcn_ds_read_tr16_b64_v4i16(p) emu::ds_read_tr16_b64((uint32_t)(uintptr_t)(p))
#define __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, hi) emu::cvt_pk_fp8_f32((a), (b), (old), (hi))
