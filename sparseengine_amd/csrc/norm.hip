// Embedding gather and RMSNorm (plain, fused residual add, row-selected) for gfx950.
//
// RMSNorm: y = z * rsqrt(mean(z^2) + eps) * w with z = x (+ residual).  The sum, the mean,
// rsqrt and the weight product are float; when a residual is given the rounded sum is
// written back as the new residual while the norm uses the unrounded sum.
#include "common.h"

// TT: storage of the table, T: storage of the activations (a table kept in float under a
// bfloat16 engine is rounded on the way out)
template <typename TT, typename T>
__global__ void embedding_kernel(const int32_t* __restrict__ ids, const TT* __restrict__ table,
                                 T* __restrict__ out, int hidden) {
  const int64_t row = ids[blockIdx.x];
  const TT* src = table + row * hidden;
  T* dst = out + static_cast<int64_t>(blockIdx.x) * hidden;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) dst[c] = from_float<T>(to_float(src[c]));
}

// One block per output row.  rows == nullptr: input row = output row = blockIdx.x.
// rows != nullptr: input row rows[blockIdx.x], output row blockIdx.x (residual is read only).
template <typename T, typename W>
__global__ void rms_norm_kernel(const T* x, T* residual, const W* __restrict__ weight, T* out,
                                const int32_t* __restrict__ rows, int hidden, float eps,
                                int64_t x_stride, int64_t res_stride, int64_t out_stride,
                                int write_residual) {
  extern __shared__ float row_cache[];  // hidden floats, then 16 floats for the reduction
  float* scratch = row_cache + hidden;
  const int64_t in_row = rows ? rows[blockIdx.x] : blockIdx.x;
  const T* xr = x + in_row * x_stride;
  T* rr = residual ? residual + in_row * res_stride : nullptr;
  // all loads come before any store: x, residual and out may be the same memory, and a store in
  // the loading loop would keep the loads from overlapping each other
  float sq = 0.f;
#pragma unroll 4
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    float v = to_float(xr[c]);
    if (rr) v += to_float(rr[c]);
    row_cache[c] = v;
    sq += v * v;
  }
  const float total = block_sum(sq, scratch);
  const float inv = rsqrtf(total / static_cast<float>(hidden) + eps);
  T* o = out + static_cast<int64_t>(blockIdx.x) * out_stride;
#pragma unroll 4
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    const float v = row_cache[c];
    if (rr && write_residual) rr[c] = from_float<T>(v);
    o[c] = from_float<T>(v * inv * to_float(weight[c]));
  }
}

// The same with 16-byte loads and stores, all loads of a phase issued before their first use;
// needs hidden and the row strides to be multiples of the vector length and 16-byte alignment.
template <typename T, typename W, int MAXV>
__global__ void __launch_bounds__(256)
rms_norm_vec_kernel(const T* x, T* residual, const W* __restrict__ weight, T* out,
                    const int32_t* __restrict__ rows, int hidden, float eps, int64_t x_stride,
                    int64_t res_stride, int64_t out_stride, int write_residual, int slots) {
  extern __shared__ float row_cache[];  // hidden floats, then 16 floats for the reduction
  float* scratch = row_cache + hidden;
  constexpr int VN = Vec16<T>::N;
  constexpr int WN = Vec16<W>::N;
  constexpr int WV = VN / WN;           // weight vectors per activation vector (1, or 2 for float weights)
  const int nvec = hidden / VN;
  const int64_t in_row = rows ? rows[blockIdx.x] : blockIdx.x;
  const T* xr = x + in_row * slots * x_stride;
  T* rr = residual ? residual + in_row * res_stride : nullptr;

  // x as float: the row itself, or (slots > 1) the sum of the row's `slots` consecutive rows of x,
  // added up in float in slot order and rounded to the storage type, as a separate sum would leave it
  float val[MAXV][VN];
  Vec16<T> rv[MAXV];
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int idx = threadIdx.x + i * 256;
    if (idx < nvec && rr) rv[i].v = *reinterpret_cast<const decltype(rv[i].v)*>(rr + idx * VN);
  }
  if (slots == 1) {
    Vec16<T> xv[MAXV];
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
      const int idx = threadIdx.x + i * 256;
      if (idx < nvec) xv[i].v = *reinterpret_cast<const decltype(xv[i].v)*>(xr + idx * VN);
    }
#pragma unroll
    for (int i = 0; i < MAXV; ++i)
#pragma unroll
      for (int j = 0; j < VN; ++j) val[i][j] = xv[i].get(j);
  } else if constexpr (MAXV <= 4) {
#pragma unroll
    for (int i = 0; i < MAXV; ++i)
#pragma unroll
      for (int j = 0; j < VN; ++j) val[i][j] = 0.f;
    for (int k0 = 0; k0 < slots; k0 += 8) {
      Vec16<T> sv[8][MAXV];
#pragma unroll
      for (int k = 0; k < 8; ++k)
#pragma unroll
        for (int i = 0; i < MAXV; ++i) {
          const int idx = threadIdx.x + i * 256;
          if (k0 + k < slots && idx < nvec)
            sv[k][i].v = *reinterpret_cast<const decltype(sv[k][i].v)*>(xr + (k0 + k) * x_stride + idx * VN);
        }
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (k0 + k < slots) {
#pragma unroll
          for (int i = 0; i < MAXV; ++i)
#pragma unroll
            for (int j = 0; j < VN; ++j) val[i][j] += sv[k][i].get(j);
        }
    }
#pragma unroll
    for (int i = 0; i < MAXV; ++i)
#pragma unroll
      for (int j = 0; j < VN; ++j) val[i][j] = round_to<T>(val[i][j]);
  }
  // the sums stay in registers (a thread's own vectors are all it needs after the reduction)
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int idx = threadIdx.x + i * 256;
    if (idx < nvec) {
#pragma unroll
      for (int j = 0; j < VN; ++j) {
        float v = val[i][j];
        if (rr) v += rv[i].get(j);
        val[i][j] = v;
        sq += v * v;
      }
    }
  }
  Vec16<W> wv[MAXV][WV];
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int idx = threadIdx.x + i * 256;
    if (idx < nvec) {
#pragma unroll
      for (int k = 0; k < WV; ++k)
        wv[i][k].v = *reinterpret_cast<const decltype(wv[i][k].v)*>(weight + idx * VN + k * WN);
    }
  }
  const float total = block_sum(sq, scratch);
  const float inv = rsqrtf(total / static_cast<float>(hidden) + eps);
  T* o = out + static_cast<int64_t>(blockIdx.x) * out_stride;
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int idx = threadIdx.x + i * 256;
    if (idx < nvec) {
      Vec16<T> ov, sv;
#pragma unroll
      for (int j = 0; j < VN; ++j) {
        const float v = val[i][j];
        sv.set(j, v);
        ov.set(j, v * inv * wv[i][j / WN].get(j % WN));
      }
      if (rr && write_residual) *reinterpret_cast<decltype(sv.v)*>(rr + idx * VN) = sv.v;
      *reinterpret_cast<decltype(ov.v)*>(o + idx * VN) = ov.v;
    }
  }
}

template <typename T, typename W>
static int launch_rms(const void* x, void* residual, const void* weight, void* out,
                      const int32_t* rows, int n_out, int hidden, float eps, int64_t xs, int64_t rs,
                      int64_t os, int write_residual, int vector_ok, hipStream_t stream, int slots = 1) {
  const size_t shmem = (static_cast<size_t>(hidden) + 16) * sizeof(float);
  constexpr int VN = Vec16<T>::N;
  const T* xp = static_cast<const T*>(x);
  T* rp = static_cast<T*>(residual);
  const W* wp = static_cast<const W*>(weight);
  T* op = static_cast<T*>(out);
  if (vector_ok && hidden % VN == 0 && xs % VN == 0 && rs % VN == 0 && os % VN == 0) {
    const int per_thread = (hidden / VN + 255) / 256;
    if (slots > 1 && per_thread > 4) return SE_ERR_SHAPE;   // rows summed on the fly: up to four vectors a thread
#define SE_RMS(MAXV)                                                                             \
  rms_norm_vec_kernel<T, W, MAXV><<<n_out, 256, shmem, stream>>>(xp, rp, wp, op, rows, hidden, eps, \
                                                                 xs, rs, os, write_residual, slots)
    if (per_thread <= 1) SE_RMS(1);
    else if (per_thread <= 2) SE_RMS(2);
    else if (per_thread <= 4) SE_RMS(4);
    else if (per_thread <= 8) SE_RMS(8);
    else SE_RMS(16);
#undef SE_RMS
  } else {
    if (slots > 1) return SE_ERR_SHAPE;
    rms_norm_kernel<T, W><<<n_out, 256, shmem, stream>>>(xp, rp, wp, op, rows, hidden, eps, xs, rs, os,
                                                         write_residual);
  }
  SE_CHECK_LAUNCH();
  return SE_OK;
}

extern "C" {

int se_embedding(const int32_t* ids, const void* table, void* out, int tokens, int hidden,
                 int dtype, int table_dtype, hipStream_t stream) {
  if (tokens <= 0) return SE_OK;
  if (dtype == SE_F32 && table_dtype == SE_F32)
    embedding_kernel<float, float><<<tokens, 256, 0, stream>>>(ids, static_cast<const float*>(table),
                                                               static_cast<float*>(out), hidden);
  else if (dtype == SE_BF16 && table_dtype == SE_F32)
    embedding_kernel<float, bf16_t><<<tokens, 256, 0, stream>>>(ids, static_cast<const float*>(table),
                                                                static_cast<bf16_t*>(out), hidden);
  else if (dtype == SE_BF16 && table_dtype == SE_BF16)
    embedding_kernel<bf16_t, bf16_t><<<tokens, 256, 0, stream>>>(ids, static_cast<const bf16_t*>(table),
                                                                 static_cast<bf16_t*>(out), hidden);
  else
    return SE_ERR_SHAPE;
  SE_CHECK_LAUNCH();
  return SE_OK;
}

// x, residual (optional), out: [*, hidden] with the given row strides (in elements).
// vector_ok: every pointer is 16-byte aligned (the wide kernel is then used where strides allow).
// hidden is limited by the row cache kept in shared memory.
int se_rms_norm(const void* x, void* residual, const void* weight, void* out, const int32_t* rows,
                int n_out, int hidden, float eps, int64_t x_stride, int64_t res_stride,
                int64_t out_stride, int write_residual, int dtype, int weight_dtype, int vector_ok,
                hipStream_t stream) {
  if (n_out <= 0) return SE_OK;
  if (hidden <= 0 || hidden > 15360) return SE_ERR_SHAPE;
  if (dtype == SE_F32) {
    if (weight_dtype != SE_F32) return SE_ERR_SHAPE;
    return launch_rms<float, float>(x, residual, weight, out, rows, n_out, hidden, eps, x_stride,
                                    res_stride, out_stride, write_residual, vector_ok, stream);
  }
  if (weight_dtype == SE_F32)
    return launch_rms<bf16_t, float>(x, residual, weight, out, rows, n_out, hidden, eps, x_stride,
                                     res_stride, out_stride, write_residual, vector_ok, stream);
  return launch_rms<bf16_t, bf16_t>(x, residual, weight, out, rows, n_out, hidden, eps, x_stride,
                                    res_stride, out_stride, write_residual, vector_ok, stream);
}

// The same with every input row the sum of `slots` consecutive rows of x (row r: rows r * slots ... of
// x), added up in float in slot order and rounded to the storage type first: the sum over a token's
// expert slots, done while the norm reads.  Sizes the wide kernel takes, up to four vectors a thread;
// out must not be x.
int se_rms_norm_slots(const void* x, void* residual, const void* weight, void* out, const int32_t* rows,
                      int n_out, int hidden, float eps, int64_t x_stride, int64_t res_stride,
                      int64_t out_stride, int write_residual, int dtype, int weight_dtype, int vector_ok,
                      int slots, hipStream_t stream) {
  if (n_out <= 0) return SE_OK;
  if (hidden <= 0 || hidden > 15360 || slots < 1 || !vector_ok || x == out) return SE_ERR_SHAPE;
  if (dtype == SE_F32) {
    if (weight_dtype != SE_F32) return SE_ERR_SHAPE;
    return launch_rms<float, float>(x, residual, weight, out, rows, n_out, hidden, eps, x_stride,
                                    res_stride, out_stride, write_residual, vector_ok, stream, slots);
  }
  if (weight_dtype == SE_F32)
    return launch_rms<bf16_t, float>(x, residual, weight, out, rows, n_out, hidden, eps, x_stride,
                                     res_stride, out_stride, write_residual, vector_ok, stream, slots);
  return launch_rms<bf16_t, bf16_t>(x, residual, weight, out, rows, n_out, hidden, eps, x_stride,
                                    res_stride, out_stride, write_residual, vector_ok, stream, slots);
}

}  // extern "C"
