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

// the storage value whose widening to float is `v`, bit for bit (NaN payloads included)
template <typename T>
__device__ __forceinline__ T narrow_exact(float v);
template <>
__device__ __forceinline__ float narrow_exact<float>(float v) {
  return v;
}
template <>
__device__ __forceinline__ bf16_t narrow_exact<bf16_t>(float v) {
  bf16_t r;
  r.bits = static_cast<uint16_t>(__float_as_uint(v) >> 16);
  return r;
}

template <typename T, typename W>
__global__ void qk_norm_rope_store_kernel(T* qkv, int64_t row_stride,
                                          const int32_t* __restrict__ positions,
                                          const float* __restrict__ cos_sin,
                                          const W* __restrict__ q_weight,
                                          const W* __restrict__ k_weight, float eps, int heads,
                                          int kv_heads, int head_dim, int rotary_dim, T* cache,
                                          const int32_t* __restrict__ slots, int page_size,
                                          int write_kv, int vector_path) {
  // The token's whole q|k|v row is first brought into shared memory (as float); everything after
  // the barrier reads from there, so no global load waits behind a store to the same row.
  extern __shared__ float row[];
  __shared__ float scratch[16];
  const int token = blockIdx.x;
  // With few tokens the block is 1024 threads wide: a thread then has one vector, and every load
  // it needs is in flight at once.
  const int first = threadIdx.x;
  const int stride = blockDim.x;
  // what the later phases need from small tables is asked for before the row itself
  const int position = positions[token];
  const int slot = write_kv ? slots[token] : -1;
  T* src = qkv + static_cast<int64_t>(token) * row_stride;
  const int q_width = heads * head_dim;
  const int k_width = kv_heads * head_dim;
  const int width = q_width + 2 * k_width;
  const bool use_norm = q_weight != nullptr;

  constexpr int VN = Vec16<T>::N;
  float q_sq = 0.f, k_sq = 0.f;
  if (vector_path) {
    stage_row<T, 8>(src, row, width);      // width <= 15360 elements = 8 vectors of 8 per thread
    __syncthreads();
    for (int c = threadIdx.x; c < q_width + k_width; c += blockDim.x) {
      const float x = row[c];
      if (c < q_width) q_sq += x * x;
      else k_sq += x * x;
    }
  } else {
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
      const float x = to_float(src[c]);
      row[c] = x;
      if (c < q_width) q_sq += x * x;
      else if (c < q_width + k_width) k_sq += x * x;
    }
  }
  float q_inv = 1.f, k_inv = 1.f;
  if (use_norm) {
    q_inv = rsqrtf(block_sum(q_sq, scratch) / static_cast<float>(q_width) + eps);
    k_inv = rsqrtf(block_sum(k_sq, scratch) / static_cast<float>(k_width) + eps);
  } else {
    __syncthreads();
  }

  const int half = rotary_dim / 2;
  const float* cs = cos_sin + static_cast<int64_t>(position) * rotary_dim;
  int64_t k_dst = -1, v_dst = -1;
  if (slot >= 0) {
    const int64_t page = slot / page_size;
    const int64_t off = slot % page_size;
    const int64_t plane = static_cast<int64_t>(kv_heads) * page_size * head_dim;
    k_dst = (page * 2) * plane + off * head_dim;   // + head * page_size * head_dim + d
    v_dst = (page * 2 + 1) * plane + off;          // + head * page_size * head_dim + d * page_size
  }

  if (vector_path) {
    // one thread per 16-byte vector of q and k; a vector lies inside one head and on one side of
    // the rotary boundaries (head_dim, rotary_dim / 2 are multiples of the vector length)
    constexpr int WN = Vec16<W>::N;
    constexpr int WV = VN / WN;
    for (int vi = first; vi < (q_width + k_width) / VN; vi += stride) {
      const int c0 = vi * VN;
      const bool is_q = c0 < q_width;
      const int base = is_q ? 0 : q_width;
      const int local0 = c0 - base;
      const int d0 = local0 % head_dim;
      const float inv = is_q ? q_inv : k_inv;
      const W* weight = is_q ? q_weight : k_weight;
      const bool rotated = d0 < rotary_dim;
      const bool lower = d0 < half;
      const int partner0 = lower ? local0 + half : local0 - half;
      Vec16<W> w_own[WV], w_partner[WV];
      float4 cos_v[VN / 4], sin_v[VN / 4];
      if (use_norm) {
#pragma unroll
        for (int k = 0; k < WV; ++k) {
          w_own[k].v = *reinterpret_cast<const decltype(w_own[k].v)*>(weight + local0 + k * WN);
          if (rotated) w_partner[k].v = *reinterpret_cast<const decltype(w_own[k].v)*>(weight + partner0 + k * WN);
        }
      }
      if (rotated) {
        const int pair0 = lower ? d0 : d0 - half;
#pragma unroll
        for (int k = 0; k < VN / 4; ++k) {
          cos_v[k] = *reinterpret_cast<const float4*>(cs + pair0 + 4 * k);
          sin_v[k] = *reinterpret_cast<const float4*>(cs + half + pair0 + 4 * k);
        }
      }
      Vec16<T> outv;
#pragma unroll
      for (int j = 0; j < VN; ++j) {
        float own = row[base + local0 + j];
        if (use_norm) own = round_to<T>(round_to<T>(own * inv) * round_to<T>(w_own[j / WN].get(j % WN)));
        float y = own;
        if (rotated) {
          float other = row[base + partner0 + j];
          if (use_norm)
            other = round_to<T>(round_to<T>(other * inv) * round_to<T>(w_partner[j / WN].get(j % WN)));
          const float cosv = (&cos_v[j / 4].x)[j % 4], sinv = (&sin_v[j / 4].x)[j % 4];
          y = lower ? own * cosv - other * sinv : own * cosv + other * sinv;
        }
        outv.set(j, y);
      }
      *reinterpret_cast<decltype(outv.v)*>(src + c0) = outv.v;
      if (!is_q && k_dst >= 0) {
        const int head = local0 / head_dim;
        *reinterpret_cast<decltype(outv.v)*>(cache + k_dst + static_cast<int64_t>(head) * page_size * head_dim + d0) = outv.v;
      }
    }
  } else {
  // one thread per element of q and k: normed value, then the rotation with its partner
  for (int c = first; c < q_width + k_width; c += stride) {
    const bool is_q = c < q_width;
    const int local = is_q ? c : c - q_width;
    const int d = local % head_dim;
    const float inv = is_q ? q_inv : k_inv;
    const W* weight = is_q ? q_weight : k_weight;
    auto normed = [&](int idx) {        // idx: element of q or of k
      const float x = row[(is_q ? 0 : q_width) + idx];
      if (!use_norm) return x;
      const float scaled = round_to<T>(x * inv);
      return round_to<T>(scaled * round_to<T>(to_float(weight[idx])));
    };
    float y;
    if (d < half) {
      y = normed(local) * cs[d] - normed(local + half) * cs[half + d];
    } else if (d < rotary_dim) {
      y = normed(local) * cs[d - half] + normed(local - half) * cs[d];
    } else {
      y = normed(local);
    }
    const T stored = from_float<T>(y);
    src[c] = stored;
    if (!is_q && k_dst >= 0) {
      const int head = local / head_dim;
      cache[k_dst + static_cast<int64_t>(head) * page_size * head_dim + d] = stored;
    }
  }
  }
  if (v_dst >= 0) {
    // the staged floats are the stored values widened; narrowing them again gives back the same bits
    const float* v = row + q_width + k_width;
    for (int c = first; c < k_width; c += stride) {
      const int head = c / head_dim, d = c % head_dim;
      cache[v_dst + static_cast<int64_t>(head) * page_size * head_dim + static_cast<int64_t>(d) * page_size] =
          narrow_exact<T>(v[c]);
    }
  }
}

template <typename T, typename W>
static int launch(void* qkv, int64_t row_stride, const int32_t* positions, const float* cos_sin,
                  const void* qw, const void* kw, float eps, int tokens, int heads, int kv_heads,
                  int head_dim, int rotary_dim, void* cache, const int32_t* slots, int page_size,
                  int write_kv, int vector_ok, hipStream_t stream) {
  // wide path: 16-byte aligned rows, vectors that never straddle a head or a rotary boundary
  constexpr int VN = Vec16<T>::N;
  const int vector_path = vector_ok && head_dim % VN == 0 && (rotary_dim / 2) % VN == 0 && row_stride % VN == 0 &&
                          (rotary_dim / 2) % 4 == 0 && (Vec16<W>::N <= VN);
  const size_t shmem = static_cast<size_t>(heads + 2 * kv_heads) * head_dim * sizeof(float);
  // few tokens: wide blocks, so that the step is not a handful of long-running narrow ones
  const int threads = tokens < 128 ? 1024 : 256;
  qk_norm_rope_store_kernel<T, W><<<tokens, threads, shmem, stream>>>(
      static_cast<T*>(qkv), row_stride, positions, cos_sin, static_cast<const W*>(qw),
      static_cast<const W*>(kw), eps, heads, kv_heads, head_dim, rotary_dim, static_cast<T*>(cache),
      slots, page_size, write_kv, vector_path);
  SE_CHECK_LAUNCH();
  return SE_OK;
}

extern "C" int se_qk_norm_rope_store(void* qkv, int64_t row_stride, const int32_t* positions,
                                     const float* cos_sin, const void* q_weight,
                                     const void* k_weight, float eps, int tokens, int heads,
                                     int kv_heads, int head_dim, int rotary_dim, void* cache,
                                     const int32_t* slots, int page_size, int write_kv, int dtype,
                                     int weight_dtype, int vector_ok, hipStream_t stream) {
  if (tokens <= 0) return SE_OK;
  if (rotary_dim < 0 || rotary_dim % 2 || rotary_dim > head_dim) return SE_ERR_SHAPE;
  if ((q_weight == nullptr) != (k_weight == nullptr)) return SE_ERR_SHAPE;
  if (write_kv && (!cache || !slots || page_size <= 0)) return SE_ERR_SHAPE;
  if (static_cast<int64_t>(heads + 2 * kv_heads) * head_dim > 15360) return SE_ERR_SHAPE;  // row kept in LDS
  if (dtype == SE_F32) {
    if (q_weight && weight_dtype != SE_F32) return SE_ERR_SHAPE;
    return launch<float, float>(qkv, row_stride, positions, cos_sin, q_weight, k_weight, eps, tokens,
                                heads, kv_heads, head_dim, rotary_dim, cache, slots, page_size,
                                write_kv, vector_ok, stream);
  }
  if (q_weight && weight_dtype == SE_F32)
    return launch<bf16_t, float>(qkv, row_stride, positions, cos_sin, q_weight, k_weight, eps,
                                 tokens, heads, kv_heads, head_dim, rotary_dim, cache, slots,
                                 page_size, write_kv, vector_ok, stream);
  return launch<bf16_t, bf16_t>(qkv, row_stride, positions, cos_sin, q_weight, k_weight, eps, tokens,
                                heads, kv_heads, head_dim, rotary_dim, cache, slots, page_size,
                                write_kv, vector_ok, stream);
}
