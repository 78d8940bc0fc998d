// Fused per-token attention input preparation for gfx950:
//   flat QK RMSNorm (one statistic per token over all heads, optional)
//   -> partial NeoX rotation of dims [0, R) of every q and k head (pairs (d, d + R/2))
//   -> q written back in place, k (normed, rotated) and v (raw) written to their cache page.
//
// Statistics, rsqrt and the rotation are float.  The flat norm rounds (x * inv_rms) to the
// storage type and multiplies by the weight in the storage type before the rotation, as a
// two-step tensor expression would; in float storage both roundings are the identity.
//
// Cache layer layout: [num_pages, 2 (k, v), kv_heads, page_size * head_dim]; inside a page a kv
// head's keys lie [page_size][head_dim] and its values transposed, [head_dim][page_size] (the
// matrix-core attention reads eight consecutive keys of one value dim as one operand).  A
// token's slot is page * page_size + offset; negative slots are skipped.
#include "common.h"

template <typename T, typename W>
__device__ __forceinline__ float normed(const T* row, const W* weight, int idx, float inv,
                                        bool use_norm) {
  const float x = to_float(row[idx]);
  if (!use_norm) return x;
  const float scaled = round_to<T>(x * inv);
  return round_to<T>(scaled * round_to<T>(to_float(weight[idx])));
}

template <typename T, typename W>
__global__ void qk_norm_rope_store_kernel(T* qkv, int64_t row_stride,
                                          const int32_t* __restrict__ positions,
                                          const float* __restrict__ cos_sin,
                                          const W* __restrict__ q_weight,
                                          const W* __restrict__ k_weight, float eps, int heads,
                                          int kv_heads, int head_dim, int rotary_dim, T* cache,
                                          const int32_t* __restrict__ slots, int page_size,
                                          int write_kv) {
  __shared__ float scratch[16];
  const int token = blockIdx.x;
  T* q = qkv + static_cast<int64_t>(token) * row_stride;
  T* k = q + heads * head_dim;
  T* v = k + kv_heads * head_dim;
  const int q_width = heads * head_dim;
  const int k_width = kv_heads * head_dim;
  const bool use_norm = q_weight != nullptr;

  float q_inv = 1.f, k_inv = 1.f;
  if (use_norm) {
    float sq = 0.f;
    for (int c = threadIdx.x; c < q_width; c += blockDim.x) {
      const float x = to_float(q[c]);
      sq += x * x;
    }
    q_inv = rsqrtf(block_sum(sq, scratch) / static_cast<float>(q_width) + eps);
    sq = 0.f;
    for (int c = threadIdx.x; c < k_width; c += blockDim.x) {
      const float x = to_float(k[c]);
      sq += x * x;
    }
    k_inv = rsqrtf(block_sum(sq, scratch) / static_cast<float>(k_width) + eps);
  }

  const int half = rotary_dim / 2;
  const float* cs = cos_sin + static_cast<int64_t>(positions[token]) * rotary_dim;

  int64_t k_dst = -1, v_dst = -1;
  const int slot = write_kv ? slots[token] : -1;
  if (slot >= 0) {
    const int64_t page = slot / page_size;
    const int64_t off = slot % page_size;
    const int64_t plane = static_cast<int64_t>(kv_heads) * page_size * head_dim;
    k_dst = (page * 2) * plane + off * head_dim;   // + head * page_size * head_dim + d
    v_dst = (page * 2 + 1) * plane + off;          // + head * page_size * head_dim + d * page_size
  }

  // q: one thread per element; the thread of dim d < R/2 also produces its partner d + R/2.
  for (int c = threadIdx.x; c < q_width; c += blockDim.x) {
    const int d = c % head_dim;
    if (d < half) {
      const float x1 = normed(q, q_weight, c, q_inv, use_norm);
      const float x2 = normed(q, q_weight, c + half, q_inv, use_norm);
      const float cosv = cs[d], sinv = cs[half + d];
      q[c] = from_float<T>(x1 * cosv - x2 * sinv);
      q[c + half] = from_float<T>(x2 * cosv + x1 * sinv);
    } else if (d >= rotary_dim) {
      q[c] = from_float<T>(normed(q, q_weight, c, q_inv, use_norm));
    }
  }
  for (int c = threadIdx.x; c < k_width; c += blockDim.x) {
    const int head = c / head_dim;
    const int d = c % head_dim;
    const int64_t head_off = static_cast<int64_t>(head) * page_size * head_dim;
    if (d < half) {
      const float x1 = normed(k, k_weight, c, k_inv, use_norm);
      const float x2 = normed(k, k_weight, c + half, k_inv, use_norm);
      const float cosv = cs[d], sinv = cs[half + d];
      const T y1 = from_float<T>(x1 * cosv - x2 * sinv);
      const T y2 = from_float<T>(x2 * cosv + x1 * sinv);
      k[c] = y1;
      k[c + half] = y2;
      if (k_dst >= 0) {
        cache[k_dst + head_off + d] = y1;
        cache[k_dst + head_off + d + half] = y2;
      }
    } else if (d >= rotary_dim) {
      const T y = from_float<T>(normed(k, k_weight, c, k_inv, use_norm));
      k[c] = y;
      if (k_dst >= 0) cache[k_dst + head_off + d] = y;
    }
    if (v_dst >= 0) cache[v_dst + head_off + static_cast<int64_t>(d) * page_size] = v[c];
  }
}

template <typename T, typename W>
static int launch(void* qkv, int64_t row_stride, const int32_t* positions, const float* cos_sin,
                  const void* qw, const void* kw, float eps, int tokens, int heads, int kv_heads,
                  int head_dim, int rotary_dim, void* cache, const int32_t* slots, int page_size,
                  int write_kv, hipStream_t stream) {
  qk_norm_rope_store_kernel<T, W><<<tokens, 256, 0, stream>>>(
      static_cast<T*>(qkv), row_stride, positions, cos_sin, static_cast<const W*>(qw),
      static_cast<const W*>(kw), eps, heads, kv_heads, head_dim, rotary_dim, static_cast<T*>(cache),
      slots, page_size, write_kv);
  SE_CHECK_LAUNCH();
  return SE_OK;
}

extern "C" int se_qk_norm_rope_store(void* qkv, int64_t row_stride, const int32_t* positions,
                                     const float* cos_sin, const void* q_weight,
                                     const void* k_weight, float eps, int tokens, int heads,
                                     int kv_heads, int head_dim, int rotary_dim, void* cache,
                                     const int32_t* slots, int page_size, int write_kv, int dtype,
                                     int weight_dtype, hipStream_t stream) {
  if (tokens <= 0) return SE_OK;
  if (rotary_dim < 0 || rotary_dim % 2 || rotary_dim > head_dim) return SE_ERR_SHAPE;
  if ((q_weight == nullptr) != (k_weight == nullptr)) return SE_ERR_SHAPE;
  if (write_kv && (!cache || !slots || page_size <= 0)) return SE_ERR_SHAPE;
  if (dtype == SE_F32) {
    if (q_weight && weight_dtype != SE_F32) return SE_ERR_SHAPE;
    return launch<float, float>(qkv, row_stride, positions, cos_sin, q_weight, k_weight, eps, tokens,
                                heads, kv_heads, head_dim, rotary_dim, cache, slots, page_size,
                                write_kv, stream);
  }
  if (q_weight && weight_dtype == SE_F32)
    return launch<bf16_t, float>(qkv, row_stride, positions, cos_sin, q_weight, k_weight, eps,
                                 tokens, heads, kv_heads, head_dim, rotary_dim, cache, slots,
                                 page_size, write_kv, stream);
  return launch<bf16_t, bf16_t>(qkv, row_stride, positions, cos_sin, q_weight, k_weight, eps, tokens,
                                heads, kv_heads, head_dim, rotary_dim, cache, slots, page_size,
                                write_kv, stream);
}
