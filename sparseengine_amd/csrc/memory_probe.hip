// What this box's memory delivers: a kernel that only reads a buffer and one that copies it.
// Every weight-streaming kernel of the engine is priced against the first (the published 8 TB/s of
// HBM3E is what the interface could carry, not what a kernel sees); the benchmarks time both over
// buffers far larger than the chip's caches and report them beside the published figure.
#include "common.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kLoads = 8;      // 16-byte loads a thread has in flight at once

// Block b reads the 16-byte words b * kThreads * kLoads + ..., grid-stride.  The words are folded into
// one value per thread with exclusive-or (the cheapest use that keeps the loads) and the block's value
// is written only to its own slot of `sink`, so that the compiler keeps every load.
__global__ __launch_bounds__(kThreads) void stream_read_kernel(const u32x4* __restrict__ src, int64_t words,
                                                              uint32_t* __restrict__ sink) {
  u32x4 acc = {0u, 0u, 0u, 0u};
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads * kLoads;
  for (int64_t base = static_cast<int64_t>(blockIdx.x) * kThreads * kLoads + threadIdx.x; base < words;
       base += stride) {
    u32x4 v[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int64_t at = base + static_cast<int64_t>(i) * kThreads;
      v[i] = at < words ? __builtin_nontemporal_load(src + at) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int i = 0; i < kLoads; ++i) acc ^= v[i];
  }
  uint32_t folded = acc.x ^ acc.y ^ acc.z ^ acc.w;
  for (int offset = SE_WAVE / 2; offset > 0; offset >>= 1) folded ^= __shfl_xor(folded, offset);
  __shared__ uint32_t per_wave[kThreads / SE_WAVE];
  if (threadIdx.x % SE_WAVE == 0) per_wave[threadIdx.x / SE_WAVE] = folded;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t all = 0;
    for (int w = 0; w < kThreads / SE_WAVE; ++w) all ^= per_wave[w];
    sink[blockIdx.x] = all;
  }
}

__global__ __launch_bounds__(kThreads) void stream_copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                              int64_t words) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads * kLoads;
  for (int64_t base = static_cast<int64_t>(blockIdx.x) * kThreads * kLoads + threadIdx.x; base < words;
       base += stride) {
    u32x4 v[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int64_t at = base + static_cast<int64_t>(i) * kThreads;
      if (at < words) v[i] = __builtin_nontemporal_load(src + at);
    }
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int64_t at = base + static_cast<int64_t>(i) * kThreads;
      if (at < words) __builtin_nontemporal_store(v[i], dst + at);
    }
  }
}

}  // namespace

extern "C" {

// Reads `bytes` (a multiple of 16, 16-byte aligned) once; `sink` takes one 32-bit word per block
// (`blocks` of them, at most 65536): the exclusive-or of everything the block read.
int se_stream_read(const void* src, int64_t bytes, uint32_t* sink, int blocks, hipStream_t stream) {
  if (bytes <= 0 || bytes % 16 || reinterpret_cast<uintptr_t>(src) % 16 || blocks <= 0 || blocks > 65536)
    return SE_ERR_SHAPE;
  hipLaunchKernelGGL(stream_read_kernel, dim3(blocks), dim3(kThreads), 0, stream,
                     static_cast<const u32x4*>(src), bytes / 16, sink);
  SE_CHECK_LAUNCH();
  return SE_OK;
}

// Copies `bytes` (a multiple of 16, both 16-byte aligned, not overlapping) from `src` to `dst`.
int se_stream_copy(const void* src, void* dst, int64_t bytes, int blocks, hipStream_t stream) {
  if (bytes <= 0 || bytes % 16 || reinterpret_cast<uintptr_t>(src) % 16 || reinterpret_cast<uintptr_t>(dst) % 16 ||
      blocks <= 0 || blocks > 65536)
    return SE_ERR_SHAPE;
  hipLaunchKernelGGL(stream_copy_kernel, dim3(blocks), dim3(kThreads), 0, stream,
                     static_cast<const u32x4*>(src), static_cast<u32x4*>(dst), bytes / 16);
  SE_CHECK_LAUNCH();
  return SE_OK;
}

}  // extern "C"
