// Paged causal GQA attention, general form, for gfx950: one wavefront per (token, query head).
//
// Works for every head size that is a multiple of 8 up to 512, any number of heads and groups,
// page sizes in steps of 8, float and bfloat16 storage, with an optional sliding window.  It is the
// float path of the engine and the fallback for shapes the matrix-core kernels refuse.
//
// Cache layer layout: [pages, 2, kv_heads, page_size * head_dim]; inside a page a head's keys and
// values lie in groups of eight elements (key_place / value_place in common.h); page_size % 8 == 0.
//
// For the query at position p of a request the keys n in [max(0, p - window + 1), p] are read
// from the request's pages through its block-table row: this step's own keys were written
// before the call.  Scores, running maximum, running sum and the output accumulator are float;
// the probabilities are rounded to the storage type before they weight the values.
#include "common.h"

#define ATT_MAX_D_PER_LANE 8  // head_dim <= 64 * 8

template <typename T>
__global__ void paged_attention_generic_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ cache,
    const int32_t* __restrict__ block_table, int bt_stride, const int32_t* __restrict__ token_row,
    const int32_t* __restrict__ positions, T* __restrict__ out, int64_t out_stride, int tokens,
    int heads, int kv_heads, int head_dim, int page_size, float scale, int window) {
  extern __shared__ float q_shared[];  // [waves per block][head_dim]
  const int lane = threadIdx.x & (SE_WAVE - 1);
  const int wave = threadIdx.x / SE_WAVE;
  const int waves_per_block = blockDim.x / SE_WAVE;
  const int64_t work = static_cast<int64_t>(blockIdx.x) * waves_per_block + wave;
  const bool active = work < static_cast<int64_t>(tokens) * heads;
  const int token = active ? static_cast<int>(work / heads) : 0;
  const int head = active ? static_cast<int>(work % heads) : 0;
  const int kv_head = head / (heads / kv_heads);
  float* qs = q_shared + wave * head_dim;
  if (active) {
    const T* qr = q + static_cast<int64_t>(token) * q_stride + static_cast<int64_t>(head) * head_dim;
    for (int d = lane; d < head_dim; d += SE_WAVE) qs[d] = to_float(qr[d]);
  }
  __syncthreads();
  if (!active) return;

  const int pos = positions[token];
  const int32_t* table = block_table + static_cast<int64_t>(token_row[token]) * bt_stride;
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int64_t plane = static_cast<int64_t>(kv_heads) * page_size * head_dim;
  const int64_t head_off = static_cast<int64_t>(kv_head) * page_size * head_dim;
  constexpr int VN = Vec16<T>::N;

  float acc[ATT_MAX_D_PER_LANE];
#pragma unroll
  for (int i = 0; i < ATT_MAX_D_PER_LANE; ++i) acc[i] = 0.f;
  float run_max = -INFINITY, run_sum = 0.f;

  for (int base = first; base <= pos; base += SE_WAVE) {
    const int n = base + lane;
    const bool valid = n <= pos;
    int slot = -1;
    float score = -INFINITY;
    if (valid) {
      const int page = table[n / page_size];
      slot = page * page_size + (n % page_size);
      const T* kr = cache + (static_cast<int64_t>(page) * 2) * plane + head_off;
      float dot = 0.f;
      for (int d = 0; d < head_dim; d += VN) {
        Vec16<T> kv;
        kv.v = *reinterpret_cast<const decltype(kv.v)*>(kr + key_place(page_size, n % page_size, d));
#pragma unroll
        for (int i = 0; i < VN; ++i) dot += qs[d + i] * kv.get(i);
      }
      score = dot * scale;
    }
    const float new_max = fmaxf(run_max, wave_max(score));
    const float p = valid ? expf(score - new_max) : 0.f;
    const float alpha = expf(run_max - new_max);  // 0 on the first chunk (run_max = -inf)
    run_sum = run_sum * alpha + wave_sum(p);
    run_max = new_max;
#pragma unroll
    for (int i = 0; i < ATT_MAX_D_PER_LANE; ++i) acc[i] *= alpha;
    const float p_store = round_to<T>(p);
    const int count = (pos - base + 1 < SE_WAVE) ? pos - base + 1 : SE_WAVE;
    for (int j = 0; j < count; ++j) {
      const float pj = __shfl(p_store, j, SE_WAVE);
      const int sj = __shfl(slot, j, SE_WAVE);
      const T* vr = cache + (static_cast<int64_t>(sj / page_size) * 2 + 1) * plane + head_off;
      const int off_j = sj % page_size;
#pragma unroll
      for (int i = 0; i < ATT_MAX_D_PER_LANE; ++i) {
        const int d = lane + i * SE_WAVE;
        if (d < head_dim) acc[i] += pj * to_float(vr[value_place(head_dim, off_j, d)]);
      }
    }
  }
  T* o = out + static_cast<int64_t>(token) * out_stride + static_cast<int64_t>(head) * head_dim;
  const float inv = 1.f / run_sum;
#pragma unroll
  for (int i = 0; i < ATT_MAX_D_PER_LANE; ++i) {
    const int d = lane + i * SE_WAVE;
    if (d < head_dim) o[d] = from_float<T>(acc[i] * inv);
  }
}

extern "C" int se_paged_attention_generic(const void* q, int64_t q_stride, const void* cache,
                                          const int32_t* block_table, int bt_stride,
                                          const int32_t* token_row, const int32_t* positions,
                                          void* out, int64_t out_stride, int tokens, int heads,
                                          int kv_heads, int head_dim, int page_size, float scale,
                                          int window, int dtype, hipStream_t stream) {
  if (tokens <= 0) return SE_OK;
  if (head_dim <= 0 || head_dim % 8 || head_dim > SE_WAVE * ATT_MAX_D_PER_LANE) return SE_ERR_SHAPE;
  if (kv_heads <= 0 || heads % kv_heads || page_size <= 0 || page_size % 8) return SE_ERR_SHAPE;
  if (q_stride % 8 || (dtype != SE_F32 && dtype != SE_BF16)) return SE_ERR_SHAPE;
  const int waves = 4;
  const int64_t work = static_cast<int64_t>(tokens) * heads;
  const int blocks = static_cast<int>((work + waves - 1) / waves);
  const size_t shmem = static_cast<size_t>(waves) * head_dim * sizeof(float);
  if (dtype == SE_F32)
    paged_attention_generic_kernel<float><<<blocks, waves * SE_WAVE, shmem, stream>>>(
        static_cast<const float*>(q), q_stride, static_cast<const float*>(cache), block_table,
        bt_stride, token_row, positions, static_cast<float*>(out), out_stride, tokens, heads,
        kv_heads, head_dim, page_size, scale, window);
  else
    paged_attention_generic_kernel<bf16_t><<<blocks, waves * SE_WAVE, shmem, stream>>>(
        static_cast<const bf16_t*>(q), q_stride, static_cast<const bf16_t*>(cache), block_table,
        bt_stride, token_row, positions, static_cast<bf16_t*>(out), out_stride, tokens, heads,
        kv_heads, head_dim, page_size, scale, window);
  SE_CHECK_LAUNCH();
  return SE_OK;
}
