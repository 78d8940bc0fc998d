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

// A kernel that waits by hand for its loads into shared memory while it also has loads into registers under
// way marks each load with this: nothing on the GPU; a build of the sources for the host (a test aid) counts
// the loads with it, as the chip's counter does.
#ifndef SE_NOTE_VECTOR_LOAD
#define SE_NOTE_VECTOR_LOAD()
#endif

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

// Two floats to two bfloat16, round to nearest even (the rule of the framework's tensor library;
// NaN stays a quiet NaN): the chip's own conversion, one instruction, where doing the same with
// integer arithmetic takes eight and made the norm and rotation kernels arithmetic-bound.
typedef __bf16 se_bf16x2 __attribute__((ext_vector_type(2)));
typedef float se_floatx2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t floats_to_bf16x2_bits(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(se_floatx2{lo, hi}, se_bf16x2));
}
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  return static_cast<uint16_t>(floats_to_bf16x2_bits(f, 0.f));
}

// 16 bytes that this kernel reads once and nobody else reads soon (a weight streamed through a decode
// step, a request's keys and values): loaded with the "non-temporal" hint, so that the caches do not
// keep them in place of data that is read again.  Measured on MI355X: the streaming expert kernel reads
// at 6.5 / 7.0 TB/s with the hint against 6.1 / 6.4 without (8 / 64 tokens), a kernel that does nothing
// but read at 7.1.
typedef uint32_t se_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load16_once(const void* p) {
  return __builtin_bit_cast(uint4, __builtin_nontemporal_load(reinterpret_cast<const se_u32x4*>(p)));
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
template <>
__device__ __forceinline__ float round_to<bf16_t>(float v) {
  return __uint_as_float(floats_to_bf16x2_bits(0.f, v) & 0xffff0000u);   // the upper half is v's bfloat16
}

// Exchange steps of a reduction over the 64 lanes of a wavefront, all inside the vector unit:
// neighbours within four lanes, mirrors within 8 and 16 lanes (after the earlier steps all lanes
// of a group hold the same value, so a mirror is as good as an exchange), then swaps between
// rows of 16 and between halves.  Shuffles through the shared-memory crossbar cost a memory
// latency apiece, and a reduction is six of them in a row.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_move(uint32_t v) {
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xf, 0xf, false));
}
#define SE_DPP_XOR1 0xB1          // quad_perm [1, 0, 3, 2]
#define SE_DPP_XOR2 0x4E          // quad_perm [2, 3, 0, 1]
#define SE_DPP_HALF_MIRROR 0x141  // lane i <-> 7 - i within 8
#define SE_DPP_MIRROR 0x140       // lane i <-> 15 - i within 16

__device__ __forceinline__ uint32_t word_of(float v) { return __float_as_uint(v); }
__device__ __forceinline__ uint32_t word_of(int v) { return static_cast<uint32_t>(v); }
__device__ __forceinline__ void word_to(uint32_t w, float& v) { v = __uint_as_float(w); }
__device__ __forceinline__ void word_to(uint32_t w, int& v) { v = static_cast<int>(w); }

// `op(a, b)` must be commutative and associative up to rounding; every lane gets the result.
// T is float or int.
template <typename T, typename Op>
__device__ __forceinline__ T wave_reduce(T v, Op op) {
  T o;
  word_to(dpp_move<SE_DPP_XOR1>(word_of(v)), o);
  v = op(v, o);
  word_to(dpp_move<SE_DPP_XOR2>(word_of(v)), o);
  v = op(v, o);
  word_to(dpp_move<SE_DPP_HALF_MIRROR>(word_of(v)), o);
  v = op(v, o);
  word_to(dpp_move<SE_DPP_MIRROR>(word_of(v)), o);
  v = op(v, o);
  const auto rows = __builtin_amdgcn_permlane16_swap(word_of(v), word_of(v), false, false);
  word_to(rows[0], v);
  word_to(rows[1], o);
  v = op(v, o);
  const auto halves = __builtin_amdgcn_permlane32_swap(word_of(v), word_of(v), false, false);
  word_to(halves[0], v);
  word_to(halves[1], o);
  return op(v, o);
}

// The same for a (value, index) pair.  `take_other(v, i, ov, oi)` says whether the other pair
// wins; it must order distinct pairs strictly, so that both sides of an exchange agree.
template <typename Better>
__device__ __forceinline__ void wave_reduce_pair(float& v, int& i, Better take_other) {
  auto step = [&](float ov, int oi) {
    if (take_other(v, i, ov, oi)) {
      v = ov;
      i = oi;
    }
  };
#define SE_PAIR_DPP(CTRL) \
  step(__uint_as_float(dpp_move<CTRL>(__float_as_uint(v))), static_cast<int>(dpp_move<CTRL>(static_cast<uint32_t>(i))))
  SE_PAIR_DPP(SE_DPP_XOR1);
  SE_PAIR_DPP(SE_DPP_XOR2);
  SE_PAIR_DPP(SE_DPP_HALF_MIRROR);
  SE_PAIR_DPP(SE_DPP_MIRROR);
#undef SE_PAIR_DPP
  {
    const uint32_t a = __float_as_uint(v), b = static_cast<uint32_t>(i);
    const auto va = __builtin_amdgcn_permlane16_swap(a, a, false, false);
    const auto ia = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    v = __uint_as_float(va[0]);
    i = static_cast<int>(ia[0]);
    step(__uint_as_float(va[1]), static_cast<int>(ia[1]));
  }
  {
    const uint32_t a = __float_as_uint(v), b = static_cast<uint32_t>(i);
    const auto va = __builtin_amdgcn_permlane32_swap(a, a, false, false);
    const auto ia = __builtin_amdgcn_permlane32_swap(b, b, false, false);
    v = __uint_as_float(va[0]);
    i = static_cast<int>(ia[0]);
    step(__uint_as_float(va[1]), static_cast<int>(ia[1]));
  }
}

__device__ __forceinline__ float wave_sum(float v) {
  return wave_reduce(v, [](float a, float b) { return a + b; });
}

__device__ __forceinline__ float wave_max(float v) {
  return wave_reduce(v, [](float a, float b) { return fmaxf(a, b); });
}

__device__ __forceinline__ int wave_sum(int v) {
  return wave_reduce(v, [](int a, int b) { return a + b; });
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

// What a gated feed-forward applies to its gate before the product with the up projection.
enum SeActivation { SE_ACT_SILU = 0, SE_ACT_GELU_TANH = 1 };
template <bool FAST_EXP>
__device__ __forceinline__ float gate_activation(float g, int activation) {
  if (activation == SE_ACT_GELU_TANH)     // 0.5 g (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3)))
    return 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
  return g / (1.f + (FAST_EXP ? __expf(-g) : expf(-g)));
}

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

// Bring n elements (n % Vec16<T>::N == 0, 16-byte aligned, n <= MAXV * 256 vectors) into shared
// memory as float with a block of at least 256 threads.  Every load is issued before the first one
// is used: a row is a handful of vectors per thread, and a loop that waits for each load in turn
// costs a memory latency apiece.
template <typename T, int MAXV>
__device__ __forceinline__ void stage_row(const T* src, float* dst, int n) {
  constexpr int VN = Vec16<T>::N;
  const int nvec = n / VN;
  const int threads = blockDim.x;
  Vec16<T> v[MAXV];
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int idx = threadIdx.x + i * threads;
    if (idx < nvec) v[i].v = *reinterpret_cast<const decltype(v[i].v)*>(src + static_cast<int64_t>(idx) * VN);
  }
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int idx = threadIdx.x + i * threads;
    if (idx < nvec) {
#pragma unroll
      for (int j = 0; j < VN; ++j) dst[idx * VN + j] = v[i].get(j);
    }
  }
}

// Where an element of a kv head lies inside its page (page_size * head_dim elements), for keys
// and for values.  Loads of 16 bytes per lane reach the caches fastest when neighbouring lanes
// read neighbouring addresses; a matrix-core operand puts neighbouring *rows* into neighbouring
// lanes, eight elements each.  So the cache keeps eight-element groups of neighbouring rows side
// by side:
//   keys:   [head_dim / 8][page_size][8]   lanes = keys, a lane's eight elements = eight dims
//   values: [page_size / 8][head_dim][8]   lanes = dims, a lane's eight elements = eight keys
// (measured on MI355X: 16 lanes x 16 bytes from 16 different rows arrive at 16 bytes a clock and
// CU, from one contiguous stretch at three times that).  page_size % 8 == 0, head_dim % 8 == 0.
__host__ __device__ __forceinline__ int64_t key_place(int page_size, int off, int d) {
  return (static_cast<int64_t>(d >> 3) * page_size + off) * 8 + (d & 7);
}
__host__ __device__ __forceinline__ int64_t value_place(int head_dim, int off, int d) {
  return (static_cast<int64_t>(off >> 3) * head_dim + d) * 8 + (off & 7);
}

// 16 bytes per lane from global memory straight into shared memory, no register in between: lane l's
// bytes land at (wave-uniform) lds_addr + 16 l.  The compiler does not see the write: the caller
// waits for it by hand (s_waitcnt vmcnt) before a barrier, and reads the data only after that barrier.
// (m0, the destination's base, is set and used inside one statement; naming it as clobbered draws a
// warning about reserved registers that does not apply here)
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void load16_to_lds(const void* src, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(src)   // the base is the same in all lanes
               : "memory", "m0");
}
// The same with the address in two parts: a base that is the same in all lanes (it stays in scalar
// registers, and so does the arithmetic that made it) and a lane's own offset in bytes.
__device__ __forceinline__ const void* same_in_all_lanes(const void* p) {   // tells the compiler so
  const uint64_t bits = reinterpret_cast<uint64_t>(p);
  const uint64_t lo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(bits)));
  const uint64_t hi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(bits >> 32)));
  return reinterpret_cast<const void*>((hi << 32) | lo);
}
__device__ __forceinline__ void load16_to_lds_at(const void* base, uint32_t offset, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(offset), "s"(same_in_all_lanes(base))
               : "memory", "m0");
}


