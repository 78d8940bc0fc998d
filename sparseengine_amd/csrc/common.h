// Shared device helpers for the gfx950 kernels: storage types, conversions, wave and
// block reductions.  Wavefronts are 64 lanes wide everywhere in this library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define SE_WAVE 64

// Every entry point returns 0 on success or a negative code the Python side turns into
// an exception; shapes are validated on the host before a launch.
#define SE_OK 0
#define SE_ERR_SHAPE -1
#define SE_ERR_LAUNCH -2

#define SE_CHECK_LAUNCH()                                  \
  do {                                                     \
    hipError_t e__ = hipGetLastError();                    \
    if (e__ != hipSuccess) return SE_ERR_LAUNCH;           \
  } while (0)

// bfloat16 is carried as its 16 raw bits; arithmetic is always done in float.
struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) {
  return __uint_as_float(static_cast<uint32_t>(b) << 16);
}

// round to nearest even, NaN kept quiet (same rule as the framework's tensor library)
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return bf16_bits_to_float(v.bits); }

template <typename T>
__device__ __forceinline__ T from_float(float v);
template <>
__device__ __forceinline__ float from_float<float>(float v) {
  return v;
}
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float v) {
  bf16_t r;
  r.bits = float_to_bf16_bits(v);
  return r;
}

// value after a round trip through the storage type T (identity for float)
template <typename T>
__device__ __forceinline__ float round_to(float v) {
  return to_float(from_float<T>(v));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = SE_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, SE_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = SE_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, SE_WAVE));
  return v;
}

// Sum over a whole block of up to 1024 threads; every thread gets the result.
// `scratch` holds at least 16 floats of shared memory and may be reused after the call.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int lane = threadIdx.x & (SE_WAVE - 1);
  const int wave = threadIdx.x / SE_WAVE;
  const int nwaves = (blockDim.x + SE_WAVE - 1) / SE_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}

enum SeDtype { SE_F32 = 0, SE_BF16 = 1 };

// 16-byte vectors of storage elements
template <typename T>
struct Vec16;
template <>
struct Vec16<float> {
  static constexpr int N = 4;
  float4 v;
  __device__ __forceinline__ float get(int i) const { return (&v.x)[i]; }
  __device__ __forceinline__ void set(int i, float f) { (&v.x)[i] = f; }
};
template <>
struct Vec16<bf16_t> {
  static constexpr int N = 8;
  uint4 v;
  __device__ __forceinline__ float get(int i) const {
    const uint32_t word = (&v.x)[i >> 1];
    return __uint_as_float((i & 1) ? (word & 0xffff0000u) : (word << 16));
  }
  __device__ __forceinline__ void set(int i, float f) {
    uint32_t& word = (&v.x)[i >> 1];
    const uint32_t bits = float_to_bf16_bits(f);
    word = (i & 1) ? ((word & 0x0000ffffu) | (bits << 16)) : ((word & 0xffff0000u) | bits);
  }
};

// Bring n elements (n % Vec16<T>::N == 0, 16-byte aligned) into shared memory as float with a block
// of 256 threads.  Every load is issued before the first one is used: a row is a handful of
// vectors per thread, and a loop that waits for each load in turn costs a memory latency apiece.
template <typename T, int MAXV>
__device__ __forceinline__ void stage_row(const T* src, float* dst, int n) {
  constexpr int VN = Vec16<T>::N;
  const int nvec = n / VN;
  Vec16<T> v[MAXV];
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int idx = threadIdx.x + i * 256;
    if (idx < nvec) v[i].v = *reinterpret_cast<const decltype(v[i].v)*>(src + static_cast<int64_t>(idx) * VN);
  }
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int idx = threadIdx.x + i * 256;
    if (idx < nvec) {
#pragma unroll
      for (int j = 0; j < VN; ++j) dst[idx * VN + j] = v[i].get(j);
    }
  }
}
