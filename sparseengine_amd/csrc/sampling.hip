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

// ---------------------------------------------------------------------------------------- //
// Rows with top-k or top-p.  Both filters keep a prefix of the row's tokens in descending order,
// that is all tokens whose ordered key is at least some threshold.  A threshold is found eight
// bits at a time: a pass over the row counts (top-k) or weighs (top-p) the tokens in the 256 bins
// of the next eight key bits, among those that agree with the bits found so far; many blocks per
// row share a pass and add their bins into the row's histogram, and every block of the next pass
// reads the histograms so far and works the bits out again (a few hundred additions) rather than
// wait for another launch to do it.  Sums are integers (a token's weight is exp(l - max) in units of
// 2^-40), so the order in which blocks and wavefronts add them does not matter: the same row gives
// the same token on every run and in every batch.
//   hist [rows][2 * FILTER_PASSES][FILTER_BINS] uint64: passes 0-3 counts, 4-7 weights; zero at the start
// ---------------------------------------------------------------------------------------- //
#define FILTER_BINS 256
#define FILTER_PASSES 4
typedef unsigned long long u64;

__device__ __forceinline__ u64 lane_value64(u64 v, int source) {
  const uint32_t lo = __shfl(static_cast<uint32_t>(v), source);
  const uint32_t hi = __shfl(static_cast<uint32_t>(v >> 32), source);
  return (static_cast<u64>(hi) << 32) | lo;
}

// One wavefront, lane l holding bins 4 l ... 4 l + 3 of a pass: the largest bin d for which
// `above` + (sum of the bins d ... 255) reaches `target` (strictly exceeds it if `strict`), and what
// lies above that bin (`above` + sum of the bins d + 1 ... 255).  Bin 0 if none does.
__device__ __forceinline__ int pick_bin(const u64 (&bin)[4], u64 above, u64 target, bool strict, u64& above_out) {
  const int lane = threadIdx.x & (SE_WAVE - 1);
  const u64 mine = bin[0] + bin[1] + bin[2] + bin[3];
  u64 from_here = mine;      // becomes the sum over this lane and all lanes after it
#pragma unroll
  for (int off = 1; off < SE_WAVE; off <<= 1) {
    const u64 other = lane_value64(from_here, (lane + off) & (SE_WAVE - 1));
    if (lane + off < SE_WAVE) from_here += other;
  }
  u64 tail = above + from_here - mine;      // everything above this lane's last bin
  int found = -1;
  u64 above_found = 0;
#pragma unroll
  for (int j = 3; j >= 0; --j) {
    const u64 with = tail + bin[j];
    if (found < 0 && (strict ? with > target : with >= target)) {
      found = j;
      above_found = tail;
    }
    tail = with;
  }
  const uint64_t who = __ballot(found >= 0);
  if (who == 0) {       // cannot happen with consistent histograms; bin 0 keeps every token
    above_out = above + lane_value64(from_here, 0);
    return 0;
  }
  const int top = 63 - __builtin_clzll(who);
  above_out = lane_value64(above_found, top);
  return 4 * top + __shfl(found, top);
}

// The bits found by the first `passes` passes of one kind (run by one whole wavefront).
__device__ __forceinline__ uint32_t bits_found(const u64* __restrict__ hist_kind, int passes, u64 target, bool strict) {
  const int lane = threadIdx.x & (SE_WAVE - 1);
  uint32_t prefix = 0;
  u64 above = 0;
  for (int pass = 0; pass < passes; ++pass) {
    const u64* h = hist_kind + pass * FILTER_BINS + 4 * lane;
    const u64 bin[4] = {h[0], h[1], h[2], h[3]};
    prefix = (prefix << 8) | static_cast<uint32_t>(pick_bin(bin, above, target, strict, above));
  }
  return prefix;
}

// the largest of the row's chunk maxima (one wavefront)
__device__ __forceinline__ float row_max(const float* __restrict__ part_max, int chunks) {
  const int lane = threadIdx.x & (SE_WAVE - 1);
  float m = -INFINITY;
  for (int c = lane; c < chunks; c += SE_WAVE) m = fmaxf(m, part_max[c]);
  return wave_max(m);
}

__device__ __forceinline__ u64 weight_of(float v, float vmax) {
  const float w = expf(v - vmax) * 1099511627776.f;      // 2^40: the largest token weighs exactly that
  return w == w ? static_cast<u64>(w) : 0;
}

// the weight that the tokens kept by top-p may have above them: top_p times the weight of all tokens that top-k kept
__device__ __forceinline__ u64 nucleus_budget(const u64* __restrict__ hist_weights, float p) {
  const int lane = threadIdx.x & (SE_WAVE - 1);
  u64 total = hist_weights[4 * lane] + hist_weights[4 * lane + 1] + hist_weights[4 * lane + 2] + hist_weights[4 * lane + 3];
#pragma unroll
  for (int off = 1; off < SE_WAVE; off <<= 1) total += lane_value64(total, lane ^ off);
  return static_cast<u64>(static_cast<double>(p) * static_cast<double>(total));
}

#define SAMPLE_CHUNK 4096
// the chunk maxima of logit / temperature, for the weights
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_chunk_max_kernel(const float* __restrict__ logits, int64_t stride, int vocab,
                        const float* __restrict__ temperature, const float* __restrict__ top_p,
                        float* __restrict__ part_max, int chunks) {
  __shared__ float scratch[SAMPLE_THREADS / SE_WAVE];
  const int row = blockIdx.x, chunk = blockIdx.y;
  const float temp = temperature[row];
  if (!(temp > 1e-10f) || !(top_p[row] < 1.f)) return;     // the whole block
  const float inv_temp = 1.f / temp;
  const float* l = logits + static_cast<int64_t>(row) * stride;
  const int begin = chunk * SAMPLE_CHUNK;
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < SAMPLE_CHUNK / SAMPLE_THREADS; ++j) {
    const int i = begin + threadIdx.x + j * SAMPLE_THREADS;
    if (i < vocab) m = fmaxf(m, l[i] * inv_temp);
  }
  m = wave_max(m);
  const int lane = threadIdx.x & (SE_WAVE - 1), wave = threadIdx.x / SE_WAVE;
  if (lane == 0) scratch[wave] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < SAMPLE_THREADS / SE_WAVE; ++w) m = fmaxf(m, scratch[w]);
    part_max[row * chunks + chunk] = m;
  }
}

template <bool WEIGHTS>    // false: a top-k pass (counts), true: a top-p pass (weights)
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_filter_pass_kernel(const float* __restrict__ logits, int64_t stride, int vocab,
                          const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
                          const float* __restrict__ top_p, const float* __restrict__ part_max,
                          u64* __restrict__ hist, int pass, int chunks) {
  __shared__ u64 bins[SAMPLE_THREADS / SE_WAVE][FILTER_BINS];     // one set per wavefront: fewer collisions
  __shared__ uint32_t found[2];
  __shared__ float shared_max;
  const int row = blockIdx.x, chunk = blockIdx.y;
  const float temp = temperature[row];
  const int k = top_k ? top_k[row] : 0;
  const float p = top_p ? top_p[row] : 1.f;
  const bool has_k = k > 0 && k < vocab, has_p = p < 1.f;
  if (!(temp > 1e-10f) || (WEIGHTS ? !has_p : !has_k)) return;     // the whole block
  const int lane = threadIdx.x & (SE_WAVE - 1), wave = threadIdx.x / SE_WAVE;
  for (int i = threadIdx.x; i < (SAMPLE_THREADS / SE_WAVE) * FILTER_BINS; i += SAMPLE_THREADS) (&bins[0][0])[i] = 0;
  u64* hist_row = hist + static_cast<int64_t>(row) * 2 * FILTER_PASSES * FILTER_BINS;
  if (wave == 0) {
    uint32_t k_bits = 0, p_bits = 0;
    if (has_k) k_bits = bits_found(hist_row, WEIGHTS ? FILTER_PASSES : pass, static_cast<u64>(k), false);
    if (WEIGHTS) {
      const u64* weights = hist_row + FILTER_PASSES * FILTER_BINS;
      if (pass > 0) p_bits = bits_found(weights, pass, nucleus_budget(weights, p), true);
      const float m = row_max(part_max + row * chunks, chunks);
      if (lane == 0) shared_max = m;
    }
    if (lane == 0) {
      found[0] = k_bits;
      found[1] = p_bits;
    }
  }
  __syncthreads();
  const uint32_t k_bits = found[0], p_bits = found[1];
  const float vmax = WEIGHTS ? shared_max : 0.f;
  const float inv_temp = 1.f / temp;
  const float* l = logits + static_cast<int64_t>(row) * stride;
  const int begin = chunk * SAMPLE_CHUNK;
  const int high = 32 - 8 * pass;       // bits above the pass's eight (32 in the first pass: no shift by that)
#pragma unroll
  for (int j = 0; j < SAMPLE_CHUNK / SAMPLE_THREADS; ++j) {
    const int i = begin + threadIdx.x + j * SAMPLE_THREADS;
    if (i >= vocab) continue;
    const float v = l[i] * inv_temp;
    const uint32_t key = ordered_key(v);
    const uint32_t bin = (key >> (high - 8)) & (FILTER_BINS - 1);
    if (WEIGHTS) {
      if (has_k && key < k_bits) continue;      // top-k has dropped it
      if (pass > 0 && (key >> high) != p_bits) continue;
      atomicAdd(&bins[wave][bin], weight_of(v, vmax));
    } else {
      if (pass > 0 && (key >> high) != k_bits) continue;
      atomicAdd(&bins[wave][bin], static_cast<u64>(1));
    }
  }
  __syncthreads();
  if (threadIdx.x < FILTER_BINS) {
    u64 total = 0;
    for (int w = 0; w < SAMPLE_THREADS / SE_WAVE; ++w) total += bins[w][threadIdx.x];
    if (total) atomicAdd(hist_row + ((WEIGHTS ? FILTER_PASSES : 0) + pass) * FILTER_BINS + threadIdx.x, total);
  }
}

__global__ void zero_words_kernel(u64* __restrict__ words, int64_t count) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < count) words[i] = 0;
}

// Rows without top-k / top-p are one arg-max each (of the logits, or of scaled logits plus
// noise): many blocks per row find partial maxima over stretches of the vocabulary, one
// wavefront per row picks among them.
// With `hist` (filled by the passes above) a row's tokens below its thresholds are left out.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_partial_kernel(const float* __restrict__ logits, int64_t stride, int vocab,
                      const float* __restrict__ temperature, const uint64_t* __restrict__ seeds,
                      float* __restrict__ part_value, int32_t* __restrict__ part_index, int chunks,
                      const int32_t* __restrict__ top_k, const float* __restrict__ top_p,
                      const u64* __restrict__ hist) {
  __shared__ ArgBest arg_scratch[SAMPLE_THREADS / SE_WAVE];
  __shared__ uint32_t shared_keep_from;
  const int row = blockIdx.x, chunk = blockIdx.y;
  const float* l = logits + static_cast<int64_t>(row) * stride;
  const float temp = temperature ? temperature[row] : 0.f;
  const bool greedy = !(temp > 1e-10f);
  const float inv_temp = greedy ? 1.f : 1.f / temp;
  const uint64_t seed = seeds ? seeds[row] : 0ull;
  uint32_t keep_from = 0;      // the smallest ordered key that is kept
  if (hist && !greedy) {       // the same for the whole block
    if (threadIdx.x < SE_WAVE) {
      const int k = top_k ? top_k[row] : 0;
      const float p = top_p ? top_p[row] : 1.f;
      const u64* hist_row = hist + static_cast<int64_t>(row) * 2 * FILTER_PASSES * FILTER_BINS;
      uint32_t from = 0;
      if (k > 0 && k < vocab) from = bits_found(hist_row, FILTER_PASSES, static_cast<u64>(k), false);
      if (p < 1.f) {
        const u64* weights = hist_row + FILTER_PASSES * FILTER_BINS;
        const uint32_t nucleus = bits_found(weights, FILTER_PASSES, nucleus_budget(weights, p), true);
        if (nucleus > from) from = nucleus;
      }
      if (threadIdx.x == 0) shared_keep_from = from;
    }
    __syncthreads();
    keep_from = shared_keep_from;
  }
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
        v = v * inv_temp;
        if (ordered_key(v) < keep_from) continue;
        v -= logf(-logf(uniform_open(seed, static_cast<uint32_t>(i))));
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
      logits, stride, vocab, temperature, seeds, part_value, part_index, chunks, nullptr, nullptr, nullptr);
  SE_CHECK_LAUNCH();
  sample_final_kernel<<<rows, SE_WAVE, 0, stream>>>(part_value, part_index, chunks, out);
  SE_CHECK_LAUNCH();
  return SE_OK;
}

// Rows with top_k and / or top_p (either may be null: off for every row); `temperature` is needed.
// Workspace: part_value, part_index as above, part_max [rows * ceil(vocab / 4096)] floats,
// hist [rows * 2048] 64-bit words (cleared here).
extern "C" int se_sample(const float* logits, int64_t stride, int rows, int vocab,
                         const float* temperature, const int32_t* top_k, const float* top_p,
                         const uint64_t* seeds, float* part_value, int32_t* part_index, float* part_max,
                         unsigned long long* hist, int32_t* out, hipStream_t stream) {
  if (rows <= 0) return SE_OK;
  if (vocab <= 0 || !temperature || !part_value || !part_index || !part_max || !hist) return SE_ERR_SHAPE;
  const int chunks = (vocab + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
  if (chunks > 65535) return SE_ERR_SHAPE;
  const dim3 grid(rows, chunks);
  const int64_t words = static_cast<int64_t>(rows) * 2 * FILTER_PASSES * FILTER_BINS;
  zero_words_kernel<<<static_cast<unsigned>((words + 255) / 256), 256, 0, stream>>>(hist, words);
  if (top_k)
    for (int pass = 0; pass < FILTER_PASSES; ++pass)
      sample_filter_pass_kernel<false><<<grid, SAMPLE_THREADS, 0, stream>>>(
          logits, stride, vocab, temperature, top_k, top_p, part_max, hist, pass, chunks);
  if (top_p) {
    sample_chunk_max_kernel<<<grid, SAMPLE_THREADS, 0, stream>>>(logits, stride, vocab, temperature, top_p,
                                                                 part_max, chunks);
    for (int pass = 0; pass < FILTER_PASSES; ++pass)
      sample_filter_pass_kernel<true><<<grid, SAMPLE_THREADS, 0, stream>>>(
          logits, stride, vocab, temperature, top_k, top_p, part_max, hist, pass, chunks);
  }
  SE_CHECK_LAUNCH();
  sample_partial_kernel<<<grid, SAMPLE_THREADS, 0, stream>>>(
      logits, stride, vocab, temperature, seeds, part_value, part_index, chunks, top_k, top_p, hist);
  SE_CHECK_LAUNCH();
  sample_final_kernel<<<rows, SE_WAVE, 0, stream>>>(part_value, part_index, chunks, out);
  SE_CHECK_LAUNCH();
  return SE_OK;
}

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
      logits, stride, vocab, temperature, seeds, part_value, part_index, chunks, nullptr, nullptr, nullptr);
  SE_CHECK_LAUNCH();
  sample_final_kernel<<<rows, SE_WAVE, 0, stream>>>(part_value, part_index, chunks, out);
  SE_CHECK_LAUNCH();
  return SE_OK;
}
