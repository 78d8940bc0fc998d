// Fused per-token attention input preparation for gfx950:
//   QK RMSNorm, optional: flat (one statistic per token over all heads of q, one over all of k; weights
//      [heads * head_dim]) or per head (one statistic per token and head; weights [head_dim], the general
//      kernel only)
//   -> partial rotation of dims [0, R) of every q and k head: pairs (d, d + R/2) ("NeoX", pairing 0)
//      or pairs (2 j, 2 j + 1) ("interleaved", pairing 1; the general kernel only); pair j turns by
//      the angle whose cosine and sine are the table's entries j and R/2 + j
//   -> q written back in place, k (normed, rotated) and v (raw) written to their cache page.
//
// Statistics, rsqrt and the rotation are float.  The flat norm rounds (x * inv_rms) to the
// storage type and multiplies by the weight in the storage type before the rotation, as a
// two-step tensor expression would; the norm per head multiplies in float and rounds once, as a norm
// kernel does.  In float storage the roundings are the identity.
//
// Cache layer layout: [num_pages, 2 (k, v), kv_heads, page_size * head_dim]; inside a page a kv
// head's keys and values lie in groups of eight elements (key_place / value_place in common.h),
// so that what one matrix-core operand load of sixteen lanes takes is one contiguous stretch.  A
// token's slot is page * page_size + offset; negative slots are skipped.  page_size % 8 == 0 and
// head_dim % 8 == 0.
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
                                          int write_kv, int pairing, int per_head) {
  // General sizes, one element at a time.  The token's whole q|k|v row is first brought into shared
  // memory (as float); everything after the barrier reads from there, so no global load waits
  // behind a store to the same row.
  extern __shared__ float row[];      // the row; then (norm per head) heads + kv_heads reciprocal roots
  __shared__ float scratch[16];
  const int token = blockIdx.x;
  const int position = positions[token];
  const int slot = write_kv ? slots[token] : -1;
  T* src = qkv + static_cast<int64_t>(token) * row_stride;
  const int q_width = heads * head_dim;
  const int k_width = kv_heads * head_dim;
  const int width = q_width + 2 * k_width;
  const bool use_norm = q_weight != nullptr;

  float q_sq = 0.f, k_sq = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float x = to_float(src[c]);
    row[c] = x;
    if (c < q_width) q_sq += x * x;
    else if (c < q_width + k_width) k_sq += x * x;
  }
  float q_inv = 1.f, k_inv = 1.f;
  float* head_inv = row + width;      // [heads + kv_heads], q heads first
  if (use_norm && per_head) {
    __syncthreads();
    for (int h = threadIdx.x; h < heads + kv_heads; h += blockDim.x) {   // a thread adds up a head's squares, in order
      float sq = 0.f;
      for (int d = 0; d < head_dim; ++d) sq += row[h * head_dim + d] * row[h * head_dim + d];
      head_inv[h] = rsqrtf(sq / static_cast<float>(head_dim) + eps);
    }
    __syncthreads();
  } else if (use_norm) {
    q_inv = rsqrtf(block_sum(q_sq, scratch) / static_cast<float>(q_width) + eps);
    k_inv = rsqrtf(block_sum(k_sq, scratch) / static_cast<float>(k_width) + eps);
  } else {
    __syncthreads();
  }

  const int half = rotary_dim / 2;
  const float* cs = cos_sin + static_cast<int64_t>(position) * rotary_dim;
  int64_t k_dst = -1, v_dst = -1;
  int page_off = 0;
  if (slot >= 0) {
    const int64_t page = slot / page_size;
    const int64_t off = slot % page_size;
    const int64_t plane = static_cast<int64_t>(kv_heads) * page_size * head_dim;
    k_dst = (page * 2) * plane;       // + head * page_size * head_dim + key_place(page_size, off, d)
    v_dst = (page * 2 + 1) * plane;   // + head * page_size * head_dim + value_place(head_dim, off, d)
    page_off = static_cast<int>(off);
  }

  // one thread per element of q and k: normed value, then the rotation with its partner
  for (int c = threadIdx.x; c < q_width + k_width; c += blockDim.x) {
    const bool is_q = c < q_width;
    const int local = is_q ? c : c - q_width;
    const int d = local % head_dim;
    const float inv = is_q ? q_inv : k_inv;
    const W* weight = is_q ? q_weight : k_weight;
    auto normed = [&](int idx) {        // idx: element of q or of k
      const float x = row[(is_q ? 0 : q_width) + idx];
      if (!use_norm) return x;
      if (per_head)                     // q heads, then k heads: head (is_q ? 0 : heads) + idx / head_dim of the row
        return round_to<T>(x * head_inv[(is_q ? 0 : heads) + idx / head_dim] * to_float(weight[idx % head_dim]));
      const float scaled = round_to<T>(x * inv);
      return round_to<T>(scaled * round_to<T>(to_float(weight[idx])));
    };
    float y;
    if (d >= rotary_dim) {
      y = normed(local);
    } else if (pairing == 1) {   // neighbours: (2 j, 2 j + 1) turn by angle j
      const int j = d >> 1;
      y = (d & 1) ? normed(local) * cs[j] + normed(local - 1) * cs[half + j]
                  : normed(local) * cs[j] - normed(local + 1) * cs[half + j];
    } else if (d < half) {
      y = normed(local) * cs[d] - normed(local + half) * cs[half + d];
    } else {
      y = normed(local) * cs[d - half] + normed(local - half) * cs[d];
    }
    const T stored = from_float<T>(y);
    src[c] = stored;
    if (!is_q && k_dst >= 0) {
      const int head = local / head_dim;
      cache[k_dst + static_cast<int64_t>(head) * page_size * head_dim + key_place(page_size, page_off, d)] = stored;
    }
  }
  if (v_dst >= 0) {
    // the staged floats are the stored values widened; narrowing them again gives back the same bits
    const float* v = row + q_width + k_width;
    for (int c = threadIdx.x; c < k_width; c += blockDim.x) {
      const int head = c / head_dim, d = c % head_dim;
      cache[v_dst + static_cast<int64_t>(head) * page_size * head_dim + value_place(head_dim, page_off, d)] =
          narrow_exact<T>(v[c]);
    }
  }
}

// The same for sizes whose 16-byte vectors never straddle a head or a rotary boundary (head_dim and
// rotary_dim / 2 multiples of the vector length, 16-byte aligned rows).  A thread owns up to MAXV
// vectors of the row: it loads them all at once, adds up their squares from registers, leaves them
// in shared memory in the storage type (only rotation partners and the value copy read them
// there), and after the two reductions normalises and rotates its own vectors.  With few tokens
// the block is 1024 threads wide and a thread has one or two vectors.
template <typename T, typename W, int MAXV>
__global__ void __launch_bounds__(1024)
qk_norm_rope_store_vec_kernel(T* qkv, int64_t row_stride, const int32_t* __restrict__ positions,
                              const float* __restrict__ cos_sin, const W* __restrict__ q_weight,
                              const W* __restrict__ k_weight, float eps, int heads, int kv_heads,
                              int head_dim, int rotary_dim, T* cache,
                              const int32_t* __restrict__ slots, int page_size, int write_kv) {
  constexpr int VN = Vec16<T>::N;
  constexpr int WN = Vec16<W>::N;
  constexpr int WV = VN / WN;
  typedef decltype(Vec16<T>().v) raw_t;
  typedef decltype(Vec16<W>().v) wraw_t;
  extern __shared__ __align__(16) unsigned char row_bytes[];
  raw_t* row = reinterpret_cast<raw_t*>(row_bytes);      // the row's vectors, storage type
  __shared__ float scratch[16];
  const int token = blockIdx.x;
  const int threads = blockDim.x;
  // what the later phases need from small tables is asked for before the row itself
  const int position = positions[token];
  const int slot = write_kv ? slots[token] : -1;
  T* src = qkv + static_cast<int64_t>(token) * row_stride;
  const int q_width = heads * head_dim;
  const int k_width = kv_heads * head_dim;
  const int nvec = (q_width + 2 * k_width) / VN;
  const int qvec = q_width / VN, qkvec = (q_width + k_width) / VN;
  const bool use_norm = q_weight != nullptr;

  const int half = rotary_dim / 2;
  Vec16<T> own[MAXV];
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int idx = threadIdx.x + i * threads;
    if (idx < nvec) own[i].v = *reinterpret_cast<const raw_t*>(src + static_cast<int64_t>(idx) * VN);
  }

  // Norm weights and rotation angles of a thread's vectors.  With one or two vectors per thread (few
  // tokens, where the kernel's time is a chain of memory latencies) they are asked for now, before
  // the reductions; with more they would take too many registers and are fetched vector by vector.
  constexpr bool EARLY = MAXV <= 2;
  constexpr int SLOTS = EARLY ? MAXV : 1;
  Vec16<W> w_own[SLOTS][WV], w_partner[SLOTS][WV];
  float4 cos_v[SLOTS][VN / 4], sin_v[SLOTS][VN / 4];
  const float* cs = cos_sin + static_cast<int64_t>(position) * rotary_dim;
  // (a macro, not a lambda: register arrays reached through a reference end up in scratch memory)
#define QK_FETCH_TABLES(VI, SLOT)                                                                  \
  {                                                                                                \
    const int fc0 = (VI) * VN;                                                                     \
    const bool f_is_q = fc0 < q_width;                                                             \
    const int f_local0 = fc0 - (f_is_q ? 0 : q_width);                                             \
    const int f_d0 = f_local0 % head_dim;                                                          \
    const W* f_weight = f_is_q ? q_weight : k_weight;                                              \
    const bool f_rotated = f_d0 < rotary_dim;                                                      \
    const bool f_lower = f_d0 < half;                                                              \
    if (use_norm) {                                                                                \
      const int f_partner0 = f_lower ? f_local0 + half : f_local0 - half;                          \
      _Pragma("unroll") for (int k = 0; k < WV; ++k) {                                             \
        w_own[SLOT][k].v = *reinterpret_cast<const wraw_t*>(f_weight + f_local0 + k * WN);         \
        if (f_rotated)                                                                             \
          w_partner[SLOT][k].v = *reinterpret_cast<const wraw_t*>(f_weight + f_partner0 + k * WN); \
      }                                                                                            \
    }                                                                                              \
    if (f_rotated) {                                                                               \
      const int f_pair0 = f_lower ? f_d0 : f_d0 - half;                                            \
      _Pragma("unroll") for (int k = 0; k < VN / 4; ++k) {                                         \
        cos_v[SLOT][k] = *reinterpret_cast<const float4*>(cs + f_pair0 + 4 * k);                   \
        sin_v[SLOT][k] = *reinterpret_cast<const float4*>(cs + half + f_pair0 + 4 * k);            \
      }                                                                                            \
    }                                                                                              \
  }
  if constexpr (EARLY) {
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
      const int vi = threadIdx.x + i * threads;
      if (vi < qkvec) QK_FETCH_TABLES(vi, i)
    }
  }

  float q_sq = 0.f, k_sq = 0.f;
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int idx = threadIdx.x + i * threads;
    if (idx < nvec) {
      row[idx] = own[i].v;
      float sq = 0.f;
#pragma unroll
      for (int j = 0; j < VN; ++j) sq += own[i].get(j) * own[i].get(j);
      if (idx < qvec) q_sq += sq;
      else if (idx < qkvec) k_sq += sq;
    }
  }
  float q_inv = 1.f, k_inv = 1.f;
  if (use_norm) {
    q_inv = rsqrtf(block_sum(q_sq, scratch) / static_cast<float>(q_width) + eps);
    k_inv = rsqrtf(block_sum(k_sq, scratch) / static_cast<float>(k_width) + eps);
  } else {
    __syncthreads();
  }

  int64_t k_dst = -1, v_dst = -1;
  int page_off = 0;
  if (slot >= 0) {
    const int64_t page = slot / page_size;
    const int64_t off = slot % page_size;
    const int64_t plane = static_cast<int64_t>(kv_heads) * page_size * head_dim;
    k_dst = (page * 2) * plane;       // + head * page_size * head_dim + key_place(page_size, off, d)
    v_dst = (page * 2 + 1) * plane;   // + head * page_size * head_dim + value_place(head_dim, off, d)
    page_off = static_cast<int>(off);
  }

#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int vi = threadIdx.x + i * threads;
    if (vi >= qkvec) continue;
    const int ti = EARLY ? i : 0;
    if constexpr (!EARLY) QK_FETCH_TABLES(vi, 0)
    const int c0 = vi * VN;
    const bool is_q = c0 < q_width;
    const int base = is_q ? 0 : q_width;
    const int local0 = c0 - base;
    const int d0 = local0 % head_dim;
    const float inv = is_q ? q_inv : k_inv;
    const bool rotated = d0 < rotary_dim;
    const bool lower = d0 < half;
    const int partner0 = lower ? local0 + half : local0 - half;
    Vec16<T> partner;
    if (rotated) partner.v = row[(base + partner0) / VN];
    Vec16<T> outv;
#pragma unroll
    for (int j = 0; j < VN; ++j) {
      float mine = own[i].get(j);
      if (use_norm) mine = round_to<T>(round_to<T>(mine * inv) * round_to<T>(w_own[ti][j / WN].get(j % WN)));
      float y = mine;
      if (rotated) {
        float other = partner.get(j);
        if (use_norm)
          other = round_to<T>(round_to<T>(other * inv) * round_to<T>(w_partner[ti][j / WN].get(j % WN)));
        const float cosv = (&cos_v[ti][j / 4].x)[j % 4], sinv = (&sin_v[ti][j / 4].x)[j % 4];
        y = lower ? mine * cosv - other * sinv : mine * cosv + other * sinv;
      }
      outv.set(j, y);
    }
    *reinterpret_cast<raw_t*>(src + c0) = outv.v;
    if (!is_q && k_dst >= 0) {
      const int head = local0 / head_dim;
      *reinterpret_cast<raw_t*>(cache + k_dst + static_cast<int64_t>(head) * page_size * head_dim +
                                key_place(page_size, page_off, d0)) = outv.v;
    }
  }
#undef QK_FETCH_TABLES
  if (v_dst >= 0) {   // values: a copy, bit for bit, to their place among the page's groups of eight keys
    const T* v = reinterpret_cast<const T*>(row_bytes) + q_width + k_width;
    for (int c = threadIdx.x; c < k_width; c += threads) {
      const int head = c / head_dim, d = c % head_dim;
      cache[v_dst + static_cast<int64_t>(head) * page_size * head_dim + value_place(head_dim, page_off, d)] = v[c];
    }
  }
}

template <typename T, typename W, int MAXV>
static void launch_vec(int threads, size_t shmem, void* qkv, int64_t row_stride, const int32_t* positions,
                       const float* cos_sin, const void* qw, const void* kw, float eps, int tokens,
                       int heads, int kv_heads, int head_dim, int rotary_dim, void* cache,
                       const int32_t* slots, int page_size, int write_kv, hipStream_t stream) {
  qk_norm_rope_store_vec_kernel<T, W, MAXV><<<tokens, threads, shmem, stream>>>(
      static_cast<T*>(qkv), row_stride, positions, cos_sin, static_cast<const W*>(qw),
      static_cast<const W*>(kw), eps, heads, kv_heads, head_dim, rotary_dim, static_cast<T*>(cache),
      slots, page_size, write_kv);
}

template <typename T, typename W>
static int launch(void* qkv, int64_t row_stride, const int32_t* positions, const float* cos_sin,
                  const void* qw, const void* kw, float eps, int tokens, int heads, int kv_heads,
                  int head_dim, int rotary_dim, void* cache, const int32_t* slots, int page_size,
                  int write_kv, int vector_ok, int pairing, int per_head, hipStream_t stream) {
  // wide path: 16-byte aligned rows, vectors that never straddle a head or a rotary boundary
  constexpr int VN = Vec16<T>::N;
  const bool vector_path = vector_ok && pairing == 0 && !(per_head && qw) && head_dim % VN == 0 && (rotary_dim / 2) % VN == 0 && row_stride % VN == 0 &&
                           (rotary_dim / 2) % 4 == 0 && (Vec16<W>::N <= VN);
  const int width = (heads + 2 * kv_heads) * head_dim;
  if (vector_path) {
    // few tokens: wide blocks, so that the step is not a handful of long-running narrow ones
    const int threads = tokens < 128 ? 1024 : 256;
    const int per_thread = (width / VN + threads - 1) / threads;
    const size_t shmem = static_cast<size_t>(width) * sizeof(T);
#define SE_QK_VEC(MAXV)                                                                              \
  launch_vec<T, W, MAXV>(threads, shmem, qkv, row_stride, positions, cos_sin, qw, kw, eps, tokens, heads, \
                         kv_heads, head_dim, rotary_dim, cache, slots, page_size, write_kv, stream)
    if (per_thread <= 1) SE_QK_VEC(1);
    else if (per_thread <= 2) SE_QK_VEC(2);
    else if (per_thread <= 4) SE_QK_VEC(4);
    else if (per_thread <= 8) SE_QK_VEC(8);
    else if (VN == 4 && per_thread <= 16) {
      if constexpr (VN == 4) SE_QK_VEC(16);   // only float rows are that many vectors long
    } else return SE_ERR_SHAPE;
#undef SE_QK_VEC
  } else {
    const size_t shmem = static_cast<size_t>(width + heads + kv_heads) * sizeof(float);
    qk_norm_rope_store_kernel<T, W><<<tokens, 256, shmem, stream>>>(
        static_cast<T*>(qkv), row_stride, positions, cos_sin, static_cast<const W*>(qw),
        static_cast<const W*>(kw), eps, heads, kv_heads, head_dim, rotary_dim, static_cast<T*>(cache),
        slots, page_size, write_kv, pairing, per_head);
  }
  SE_CHECK_LAUNCH();
  return SE_OK;
}

extern "C" int se_qk_norm_rope_store(void* qkv, int64_t row_stride, const int32_t* positions,
                                     const float* cos_sin, const void* q_weight,
                                     const void* k_weight, float eps, int tokens, int heads,
                                     int kv_heads, int head_dim, int rotary_dim, void* cache,
                                     const int32_t* slots, int page_size, int write_kv, int dtype,
                                     int weight_dtype, int vector_ok, int pairing, int per_head,
                                     hipStream_t stream) {
  // per_head: the norm's statistic is one per token and head, its weights are [head_dim] (else flat, see above)
  if (tokens <= 0) return SE_OK;
  if (per_head != 0 && per_head != 1) return SE_ERR_SHAPE;
  if (rotary_dim < 0 || rotary_dim % 2 || rotary_dim > head_dim) return SE_ERR_SHAPE;
  if (pairing != 0 && pairing != 1) return SE_ERR_SHAPE;
  if ((q_weight == nullptr) != (k_weight == nullptr)) return SE_ERR_SHAPE;
  if (write_kv && (!cache || !slots || page_size <= 0)) return SE_ERR_SHAPE;
  if (static_cast<int64_t>(heads + 2 * kv_heads) * head_dim > 15360) return SE_ERR_SHAPE;  // row kept in LDS
  if (dtype == SE_F32) {
    if (q_weight && weight_dtype != SE_F32) return SE_ERR_SHAPE;
    return launch<float, float>(qkv, row_stride, positions, cos_sin, q_weight, k_weight, eps, tokens,
                                heads, kv_heads, head_dim, rotary_dim, cache, slots, page_size,
                                write_kv, vector_ok, pairing, per_head, stream);
  }
  if (q_weight && weight_dtype == SE_F32)
    return launch<bf16_t, float>(qkv, row_stride, positions, cos_sin, q_weight, k_weight, eps,
                                 tokens, heads, kv_heads, head_dim, rotary_dim, cache, slots,
                                 page_size, write_kv, vector_ok, pairing, per_head, stream);
  return launch<bf16_t, bf16_t>(qkv, row_stride, positions, cos_sin, q_weight, k_weight, eps, tokens,
                                heads, kv_heads, head_dim, rotary_dim, cache, slots, page_size,
                                write_kv, vector_ok, pairing, per_head, stream);
}
