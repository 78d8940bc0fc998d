// Embedding gather and RMSNorm (plain, fused residual add, row-selected) for gfx950.
//
// RMSNorm: y = z * rsqrt(mean(z^2) + eps) * w with z = x (+ residual).  The sum, the mean,
// rsqrt and the weight product are float; when a residual is given the rounded sum is
// written back as the new residual while the norm uses the unrounded sum.
#include "common.h"

template <typename T>
__global__ void embedding_kernel(const int32_t* __restrict__ ids, const T* __restrict__ table,
                                 T* __restrict__ out, int hidden) {
  const int64_t row = ids[blockIdx.x];
  const T* src = table + row * hidden;
  T* dst = out + static_cast<int64_t>(blockIdx.x) * hidden;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) dst[c] = src[c];
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
  float sq = 0.f;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    float v = to_float(xr[c]);
    if (rr) {
      v += to_float(rr[c]);
      if (write_residual) rr[c] = from_float<T>(v);
    }
    row_cache[c] = v;
    sq += v * v;
  }
  const float total = block_sum(sq, scratch);
  const float inv = rsqrtf(total / static_cast<float>(hidden) + eps);
  T* o = out + static_cast<int64_t>(blockIdx.x) * out_stride;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x)
    o[c] = from_float<T>(row_cache[c] * inv * to_float(weight[c]));
}

template <typename T, typename W>
static int launch_rms(const void* x, void* residual, const void* weight, void* out,
                      const int32_t* rows, int n_out, int hidden, float eps, int64_t xs, int64_t rs,
                      int64_t os, int write_residual, hipStream_t stream) {
  const size_t shmem = (static_cast<size_t>(hidden) + 16) * sizeof(float);
  rms_norm_kernel<T, W><<<n_out, 256, shmem, stream>>>(
      static_cast<const T*>(x), static_cast<T*>(residual), static_cast<const W*>(weight),
      static_cast<T*>(out), rows, hidden, eps, xs, rs, os, write_residual);
  SE_CHECK_LAUNCH();
  return SE_OK;
}

extern "C" {

int se_embedding(const int32_t* ids, const void* table, void* out, int tokens, int hidden,
                 int dtype, hipStream_t stream) {
  if (tokens <= 0) return SE_OK;
  if (dtype == SE_F32)
    embedding_kernel<float><<<tokens, 256, 0, stream>>>(ids, static_cast<const float*>(table),
                                                        static_cast<float*>(out), hidden);
  else
    embedding_kernel<bf16_t><<<tokens, 256, 0, stream>>>(ids, static_cast<const bf16_t*>(table),
                                                         static_cast<bf16_t*>(out), hidden);
  SE_CHECK_LAUNCH();
  return SE_OK;
}

// x, residual (optional), out: [*, hidden] with the given row strides (in elements).
// hidden is limited by the row cache kept in shared memory.
int se_rms_norm(const void* x, void* residual, const void* weight, void* out, const int32_t* rows,
                int n_out, int hidden, float eps, int64_t x_stride, int64_t res_stride,
                int64_t out_stride, int write_residual, int dtype, int weight_dtype,
                hipStream_t stream) {
  if (n_out <= 0) return SE_OK;
  if (hidden <= 0 || hidden > 15360) return SE_ERR_SHAPE;
  if (dtype == SE_F32) {
    if (weight_dtype != SE_F32) return SE_ERR_SHAPE;
    return launch_rms<float, float>(x, residual, weight, out, rows, n_out, hidden, eps, x_stride,
                                    res_stride, out_stride, write_residual, stream);
  }
  if (weight_dtype == SE_F32)
    return launch_rms<bf16_t, float>(x, residual, weight, out, rows, n_out, hidden, eps, x_stride,
                                     res_stride, out_stride, write_residual, stream);
  return launch_rms<bf16_t, bf16_t>(x, residual, weight, out, rows, n_out, hidden, eps, x_stride,
                                    res_stride, out_stride, write_residual, stream);
}

}  // extern "C"
