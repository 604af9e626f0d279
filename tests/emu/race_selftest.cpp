// Positive and negative controls for the data-race check (tests/emu/race_check.cpp): two small kernels written against
// the stand-in HIP header, compiled under ThreadSanitizer like the library's kernels. In each, wave 0 fills a slab of
// LDS (once with ordinary stores, once with a global->LDS load retired by a counter wait) and wave 1 reads it; with
// `barrier` the two are separated by __syncthreads(), without it they race. The sanitizer must report the second
// form and stay silent on the first.
#include <hip/hip_runtime.h>

namespace {
__global__ void stores_then_reads(const int* in, int* out, int barrier) {
  __shared__ int slab[64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (wave == 0) slab[lane] = in[lane];
  if (barrier) __syncthreads();
  if (wave == 1) out[lane] = slab[63 - lane];
}
__global__ void dma_then_reads(const int* in, int* out, int barrier) {
  __shared__ __attribute__((aligned(256))) int slab[64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (wave == 0) {
    emu::dma(4, in, (uint32_t)lane * 4u, (uint32_t)(uintptr_t)slab);
    emu::wait_vm(0);
  }
  if (barrier) __syncthreads();
  if (wave == 1) out[lane] = slab[63 - lane];
}
}  // namespace

// Returns the sum of what wave 1 read (2016 when it saw all of wave 0's slab), so that the reads cannot be optimised away.
extern "C" int race_selftest(int kernel, int barrier) {
  static int in[64], out[64];
  for (int i = 0; i < 64; ++i) in[i] = i;
  if (kernel == 0) hipLaunchKernelGGL(stores_then_reads, dim3(1), dim3(128), 0, nullptr, in, out, barrier);
  else hipLaunchKernelGGL(dma_then_reads, dim3(1), dim3(128), 0, nullptr, in, out, barrier);
  int sum = 0;
  for (int i = 0; i < 64; ++i) sum += out[i];
  return sum;
}
