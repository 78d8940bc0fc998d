// Token sampling over float logits [rows, vocab] for gfx950; one block per row.
//
//   temperature <= 1e-10 : arg-max (lowest index among equal values)
//   otherwise            : l = logit / temperature; keep the top_k largest (top_k <= 0: all;
//                          values equal to the k-th are all kept); among those keep token i while
//                          the probability mass of strictly more probable tokens is <= top_p;
//                          draw from the renormalised rest by arg-max of l_i + Gumbel noise.
// The noise of token i is a pure function of (seed of the row, i): a row's draw does not depend
// on which other rows share the launch.
#include "common.h"
#include "no_alloc.h"

#define SAMPLE_THREADS 1024

__device__ __forceinline__ uint32_t ordered_key(float v) {
  const uint32_t u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ float uniform_open(uint64_t seed, uint32_t index) {
  uint64_t x = seed + 0x9E3779B97F4A7C15ull * (static_cast<uint64_t>(index) + 1ull);
  x ^= x >> 30;
  x *= 0xBF58476D1CE4E5B9ull;
  x ^= x >> 27;
  x *= 0x94D049BB133111EBull;
  x ^= x >> 31;
  // 23 random bits: (n + 0.5) / 2^23 is exact in float and lies strictly inside (0, 1)
  return (static_cast<float>(static_cast<uint32_t>(x >> 41)) + 0.5f) * (1.0f / 8388608.0f);
}

struct ArgBest {
  float value;
  int index;
};

__device__ __forceinline__ ArgBest better(ArgBest a, ArgBest b) {
  if (b.index < 0) return a;
  if (a.index < 0) return b;
  if (b.value > a.value || (b.value == a.value && b.index < a.index)) return b;
  return a;
}

// larger value, lower index among equals, over the wavefront; every lane gets the result
__device__ __forceinline__ ArgBest wave_argbest(ArgBest v) {
  wave_reduce_pair(v.value, v.index, [](float av, int ai, float bv, int bi) {
    if (bi < 0) return false;
    if (ai < 0) return true;
    return bv > av || (bv == av && bi < ai);
  });
  return v;
}

__device__ ArgBest block_argbest(ArgBest v, ArgBest* scratch) {
  v = wave_argbest(v);
  const int lane = threadIdx.x & (SE_WAVE - 1), wave = threadIdx.x / SE_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  ArgBest r = scratch[0];
  for (int w = 1; w < SAMPLE_THREADS / SE_WAVE; ++w) r = better(r, scratch[w]);
  return r;
}

__device__ float block_sum_f(float v, float* scratch) { return block_sum(v, scratch); }

__device__ int block_sum_i(int v, int* scratch) {
  v = wave_sum(v);
  const int lane = threadIdx.x & (SE_WAVE - 1), wave = threadIdx.x / SE_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  int total = 0;
  for (int w = 0; w < SAMPLE_THREADS / SE_WAVE; ++w) total += scratch[w];
  return total;
}

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, int64_t stride, int vocab,
              const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
              const float* __restrict__ top_p, const uint64_t* __restrict__ seeds,
              int32_t* __restrict__ out) {
  __shared__ ArgBest arg_scratch[SAMPLE_THREADS / SE_WAVE];
  __shared__ float f_scratch[SAMPLE_THREADS / SE_WAVE];
  __shared__ int i_scratch[SAMPLE_THREADS / SE_WAVE];
  const int row = blockIdx.x;
  const float* l = logits + static_cast<int64_t>(row) * stride;
  const float temp = temperature ? temperature[row] : 0.f;

  if (!(temp > 1e-10f)) {
    ArgBest best = {-INFINITY, -1};
    for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) {
      ArgBest c = {l[i], i};
      if (c.value != c.value) c.value = INFINITY;  // NaN wins, as in a library arg-max
      best = better(best, c);
    }
    best = block_argbest(best, arg_scratch);
    if (threadIdx.x == 0) out[row] = best.index;
    return;
  }

  const float inv_temp = 1.f / temp;
  const int k = top_k ? top_k[row] : 0;
  const float p = top_p ? top_p[row] : 1.f;
  // smallest ordered key that is kept
  uint32_t keep_from = 0;
  if (k > 0 && k < vocab) {
    uint32_t ans = 0;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = ans | (1u << bit);
      int cnt = 0;
      for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS)
        cnt += ordered_key(l[i] * inv_temp) >= cand;
      if (block_sum_i(cnt, i_scratch) >= k) ans = cand;
    }
    keep_from = ans;
  }
  float vmax = -INFINITY;
  for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) vmax = fmaxf(vmax, l[i] * inv_temp);
  {
    ArgBest m = {vmax, 0};
    vmax = block_argbest(m, arg_scratch).value;
  }
  if (p < 1.f) {
    float z = 0.f;
    for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) {
      const float v = l[i] * inv_temp;
      if (ordered_key(v) >= keep_from) z += expf(v - vmax);
    }
    z = block_sum_f(z, f_scratch);
    const float budget = p * z;
    uint32_t ans = 0;  // largest key c with mass{kept key >= c} > budget, built bit by bit
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = ans | (1u << bit);
      float mass = 0.f;
      for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) {
        const float v = l[i] * inv_temp;
        const uint32_t key = ordered_key(v);
        if (key >= cand && key >= keep_from) mass += expf(v - vmax);
      }
      if (block_sum_f(mass, f_scratch) > budget) ans = cand;
    }
    if (ans > keep_from) keep_from = ans;
  }
  const uint64_t seed = seeds ? seeds[row] : 0ull;
  ArgBest best = {-INFINITY, -1};
  for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) {
    const float v = l[i] * inv_temp;
    if (ordered_key(v) < keep_from) continue;
    const float u = uniform_open(seed, static_cast<uint32_t>(i));
    ArgBest c = {v - logf(-logf(u)), i};
    best = better(best, c);
  }
  best = block_argbest(best, arg_scratch);
  if (threadIdx.x == 0) out[row] = best.index;
}

// Rows without top-k / top-p are one arg-max each (of the logits, or of scaled logits plus
// noise): many blocks per row find partial maxima over stretches of the vocabulary, one
// wavefront per row picks among them.
#define SAMPLE_CHUNK 4096
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_partial_kernel(const float* __restrict__ logits, int64_t stride, int vocab,
                      const float* __restrict__ temperature, const uint64_t* __restrict__ seeds,
                      float* __restrict__ part_value, int32_t* __restrict__ part_index, int chunks) {
  __shared__ ArgBest arg_scratch[SAMPLE_THREADS / SE_WAVE];
  const int row = blockIdx.x, chunk = blockIdx.y;
  const float* l = logits + static_cast<int64_t>(row) * stride;
  const float temp = temperature ? temperature[row] : 0.f;
  const bool greedy = !(temp > 1e-10f);
  const float inv_temp = greedy ? 1.f : 1.f / temp;
  const uint64_t seed = seeds ? seeds[row] : 0ull;
  const int begin = chunk * SAMPLE_CHUNK;
  const int end = begin + SAMPLE_CHUNK < vocab ? begin + SAMPLE_CHUNK : vocab;
  ArgBest best = {-INFINITY, -1};
#pragma unroll
  for (int j = 0; j < SAMPLE_CHUNK / SAMPLE_THREADS; ++j) {
    const int i = begin + threadIdx.x + j * SAMPLE_THREADS;
    if (i < end) {
      float v = l[i];
      if (greedy) {
        if (v != v) v = INFINITY;
      } else {
        v = v * inv_temp - logf(-logf(uniform_open(seed, static_cast<uint32_t>(i))));
      }
      ArgBest c = {v, i};
      best = better(best, c);
    }
  }
  best = block_argbest(best, arg_scratch);
  if (threadIdx.x == 0) {
    part_value[row * chunks + chunk] = best.value;
    part_index[row * chunks + chunk] = best.index;
  }
}

__global__ void sample_final_kernel(const float* __restrict__ part_value,
                                    const int32_t* __restrict__ part_index, int chunks,
                                    int32_t* __restrict__ out) {
  const int row = blockIdx.x;
  ArgBest best = {-INFINITY, -1};
  for (int c = threadIdx.x; c < chunks; c += SE_WAVE) {
    ArgBest cand = {part_value[row * chunks + c], part_index[row * chunks + c]};
    best = better(best, cand);
  }
  best = wave_argbest(best);
  if (threadIdx.x == 0) out[row] = best.index;
}

// scratch: rows * ceil(vocab / 4096) floats and as many int32
extern "C" int se_sample_unfiltered(const float* logits, int64_t stride, int rows, int vocab,
                                    const float* temperature, const uint64_t* seeds,
                                    float* part_value, int32_t* part_index, int32_t* out,
                                    hipStream_t stream) {
  if (rows <= 0) return SE_OK;
  if (vocab <= 0 || !part_value || !part_index) return SE_ERR_SHAPE;
  const int chunks = (vocab + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
  if (chunks > 65535) return SE_ERR_SHAPE;
  sample_partial_kernel<<<dim3(rows, chunks), SAMPLE_THREADS, 0, stream>>>(
      logits, stride, vocab, temperature, seeds, part_value, part_index, chunks);
  SE_CHECK_LAUNCH();
  sample_final_kernel<<<rows, SE_WAVE, 0, stream>>>(part_value, part_index, chunks, out);
  SE_CHECK_LAUNCH();
  return SE_OK;
}

extern "C" int se_sample(const float* logits, int64_t stride, int rows, int vocab,
                         const float* temperature, const int32_t* top_k, const float* top_p,
                         const uint64_t* seeds, int32_t* out, hipStream_t stream) {
  if (rows <= 0) return SE_OK;
  if (vocab <= 0) return SE_ERR_SHAPE;
  sample_kernel<<<rows, SAMPLE_THREADS, 0, stream>>>(logits, stride, vocab, temperature, top_k,
                                                     top_p, seeds, out);
  SE_CHECK_LAUNCH();
  return SE_OK;
}

// ---------------------------------------------------------------------------------------- //
// The same arg-max sampling for callers that cannot allocate (no_alloc.h): the partial maxima go
// to a fixed array in device memory instead of a workspace of the caller's.
// ---------------------------------------------------------------------------------------- //
static __device__ __align__(256) unsigned char scratch[SE_NO_ALLOC_SAMPLE_SLOTS * (sizeof(float) + sizeof(int32_t))];

#define SE_NO_ALLOC_MAX_DEVICES 64
static unsigned char* scratch_of_device[SE_NO_ALLOC_MAX_DEVICES];   // the array's address on each GPU, once asked for

extern "C" int se_sample_unfiltered_no_alloc(const float* logits, int64_t stride, int rows, int vocab,
                                             const float* temperature, const uint64_t* seeds,
                                             int32_t* out, hipStream_t stream) {
  if (rows <= 0) return SE_OK;
  if (vocab <= 0) return SE_ERR_SHAPE;
  const int chunks = (vocab + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
  if (chunks > 65535 || static_cast<int64_t>(rows) * chunks > SE_NO_ALLOC_SAMPLE_SLOTS) return SE_ERR_SHAPE;
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= SE_NO_ALLOC_MAX_DEVICES) return SE_ERR_LAUNCH;
  if (!scratch_of_device[device]) {
    // in host code the array's name is a stand-in, not a device address: every GPU holds its own
    // copy at its own address, which is asked for once with that GPU current
    void* address = nullptr;
    if (hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)) != hipSuccess || !address) return SE_ERR_LAUNCH;
    scratch_of_device[device] = static_cast<unsigned char*>(address);
  }
  // every slot a call reads has been written by the same call: nothing has to start at zero
  float* part_value = reinterpret_cast<float*>(scratch_of_device[device]);
  int32_t* part_index = reinterpret_cast<int32_t*>(scratch_of_device[device] + SE_NO_ALLOC_SAMPLE_SLOTS * sizeof(float));
  sample_partial_kernel<<<dim3(rows, chunks), SAMPLE_THREADS, 0, stream>>>(
      logits, stride, vocab, temperature, seeds, part_value, part_index, chunks);
  SE_CHECK_LAUNCH();
  sample_final_kernel<<<rows, SE_WAVE, 0, stream>>>(part_value, part_index, chunks, out);
  SE_CHECK_LAUNCH();
  return SE_OK;
}
