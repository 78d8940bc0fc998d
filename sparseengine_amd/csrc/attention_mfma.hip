// Paged causal GQA attention on the matrix cores (bfloat16) for gfx950: one kernel for portions
// of prompts and for single decoded tokens, with split keys where a step has too few rows to
// fill the chip, and a merge kernel for the splits.
//
// A *row* is one (query token, query head) pair.  For one request and one kv head the rows
// (q_len * group of them, ordered token-major) are cut into tiles of 16; a work unit is one tile
// and one range of keys, and one wavefront runs it:
//
//   S^T = K Q^T   v_mfma_f32_16x16x32_bf16, A = 16 keys x 32 dims, B = 32 dims x 16 rows.  The key of
//                 A-row m in block b is k0 + 8 * (m / 4) + m % 4 + 4 * b, so that a lane ends up with
//                 the scores of eight consecutive keys for its row: exactly the B operand of
//   O^T += V^T P^T  A = 16 value dims x 32 keys (values lie transposed in a page, eight consecutive
//                 keys of one dim are one 16-byte load), B = 32 keys x 16 rows.
//
// Softmax is online, in float, in base 2 (scale * log2(e) folded into the scores); probabilities
// are rounded to bfloat16 for the value product, the running sum uses them unrounded.
// Masked: keys after the row's position, keys more than `window` before it.  A split unit
// writes its unnormalised O, running maximum and sum; the merge kernel combines a tile's splits
// in the order of the key ranges.
//
// Cache layer: [pages, 2, kv_heads, page_size * head_dim]; keys [page_size][head_dim], values
// [head_dim][page_size].  Requires head_dim % 32 == 0, head_dim <= 256, page_size % 8 == 0.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

#define UNIT_FIELDS 6  // item, row_tile, key_begin, key_end, partial_slot (-1: writes out), unused

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return static_cast<uint32_t>(float_to_bf16_bits(lo)) |
         (static_cast<uint32_t>(float_to_bf16_bits(hi)) << 16);
}

template <int DSTEPS>  // head_dim = 32 * DSTEPS
__global__ void __launch_bounds__(256)
paged_attention_mfma_kernel(const bf16_t* __restrict__ q, int64_t q_stride,
                            const bf16_t* __restrict__ cache,
                            const int32_t* __restrict__ block_table, int bt_stride,
                            const int32_t* __restrict__ item_meta, int num_items,
                            const int32_t* __restrict__ units, int num_units,
                            bf16_t* __restrict__ out, int64_t out_stride,
                            float* __restrict__ part_o, float* __restrict__ part_ml, int heads,
                            int kv_heads, int page_size, float scale_log2e, int window) {
  constexpr int D = 32 * DSTEPS;
  constexpr int DBLOCKS = 2 * DSTEPS;  // blocks of 16 value dims
  const int lane = threadIdx.x & (SE_WAVE - 1);
  const int unit = blockIdx.x * (blockDim.x / SE_WAVE) + threadIdx.x / SE_WAVE;
  if (unit >= num_units) return;  // whole waves leave together; there is no block barrier below
  const int n = lane & 15;        // row of the tile (B operand column) / A operand row
  const int g = lane >> 4;        // which 8 of a step's 32 reduction indices this lane holds
  const int kvh = blockIdx.y;
  const int group = heads / kv_heads;

  const int32_t* u = units + static_cast<int64_t>(unit) * UNIT_FIELDS;
  const int item = u[0], row_tile = u[1], key_begin = u[2], slot = u[4];
  int key_end = u[3];
  const int q_start = item_meta[item], q_len = item_meta[num_items + item],
            ctx_len = item_meta[2 * num_items + item];
  const int rows_total = q_len * group;

  const int rho = row_tile * 16 + n;
  const bool row_valid = rho < rows_total;
  const int rho_c = row_valid ? rho : rows_total - 1;   // padding rows repeat the last row
  const int q_idx = rho_c / group;
  const int head = kvh * group + rho_c % group;
  const int token = q_start + q_idx;
  const int pos = ctx_len - q_len + q_idx;

  // this tile's largest and smallest position bound the keys that matter
  const int last_row = (row_tile * 16 + 15 < rows_total) ? row_tile * 16 + 15 : rows_total - 1;
  const int pos_max = ctx_len - q_len + last_row / group;
  if (key_end > pos_max + 1) key_end = pos_max + 1;
  int k_first = key_begin;
  if (window > 0) {
    const int pos_min = ctx_len - q_len + (row_tile * 16) / group;
    const int lowest = pos_min - window + 1;
    if (lowest > k_first) k_first = lowest & ~31;
  }

  const bf16_t* q_row = q + static_cast<int64_t>(token) * q_stride + static_cast<int64_t>(head) * D + g * 8;
  uint4 qf[DSTEPS];
#pragma unroll
  for (int ds = 0; ds < DSTEPS; ++ds) qf[ds] = *reinterpret_cast<const uint4*>(q_row + ds * 32);

  const int32_t* table = block_table + static_cast<int64_t>(item) * bt_stride;
  const int64_t head_span = static_cast<int64_t>(page_size) * D;
  const int64_t plane = static_cast<int64_t>(kv_heads) * head_span;
  const int last_key = ctx_len - 1;

  floatx4 o[DBLOCKS];
#pragma unroll
  for (int db = 0; db < DBLOCKS; ++db) o[db] = floatx4{0.f, 0.f, 0.f, 0.f};
  float run_max = -INFINITY, run_sum = 0.f;

  for (int k0 = k_first; k0 < key_end; k0 += 32) {
    // ---- scores of 32 keys x 16 rows
    floatx4 s[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      s[b] = floatx4{0.f, 0.f, 0.f, 0.f};
      int key = k0 + 8 * (n >> 2) + (n & 3) + 4 * b;
      if (key > last_key) key = last_key;           // reads stay inside the request's pages
      const int page = table[key / page_size];
      const bf16_t* k_row = cache + (static_cast<int64_t>(page) * 2) * plane + kvh * head_span +
                            static_cast<int64_t>(key % page_size) * D + g * 8;
#pragma unroll
      for (int ds = 0; ds < DSTEPS; ++ds) {
        const uint4 kf = *reinterpret_cast<const uint4*>(k_row + ds * 32);
        s[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf),
                                                       __builtin_bit_cast(bf16x8, qf[ds]), s[b], 0, 0, 0);
      }
    }
    // lane (g, n): s[b][i] is the score of key k0 + 8 g + 4 b + i for row n
    float p[8];
    float tile_max = -INFINITY;
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = k0 + 8 * g + 4 * b + i;
        const bool masked = key > pos || (window > 0 && key <= pos - window);
        const float v = masked ? -INFINITY : s[b][i] * scale_log2e;
        p[b * 4 + i] = v;
        tile_max = fmaxf(tile_max, v);
      }
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, SE_WAVE));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, SE_WAVE));
    const float new_max = fmaxf(run_max, tile_max);
    const float ref = (new_max == -INFINITY) ? 0.f : new_max;   // a row with no key yet
    const float alpha = exp2f(run_max - ref);
    float tile_sum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      p[j] = exp2f(p[j] - ref);
      tile_sum += p[j];
    }
    tile_sum += __shfl_xor(tile_sum, 16, SE_WAVE);
    tile_sum += __shfl_xor(tile_sum, 32, SE_WAVE);
    run_sum = run_sum * alpha + tile_sum;
    run_max = new_max;
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) o[db] *= alpha;

    uint4 pf;
    pf.x = pack_bf16x2(p[0], p[1]);
    pf.y = pack_bf16x2(p[2], p[3]);
    pf.z = pack_bf16x2(p[4], p[5]);
    pf.w = pack_bf16x2(p[6], p[7]);

    // ---- values: lane (g, n) reads value dim db * 16 + n at keys k0 + 8 g .. + 7
    int vkey = k0 + 8 * g;
    const bool beyond = vkey + 7 > last_key;        // only in the request's last step
    if (vkey > last_key) vkey = last_key & ~7;
    const int vpage = table[vkey / page_size];
    const bf16_t* v_col = cache + (static_cast<int64_t>(vpage) * 2 + 1) * plane + kvh * head_span +
                          static_cast<int64_t>(n) * page_size + (vkey % page_size);
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) {
      uint4 vf = *reinterpret_cast<const uint4*>(v_col + static_cast<int64_t>(db) * 16 * page_size);
      if (beyond) {
        // slots past the request's last key hold whatever an earlier owner left: make them zero
        uint32_t* w32 = &vf.x;
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (vkey + j > last_key) w32[j >> 1] &= (j & 1) ? 0x0000ffffu : 0xffff0000u;
      }
      o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vf),
                                                     __builtin_bit_cast(bf16x8, pf), o[db], 0, 0, 0);
    }
  }

  // lane (g, n): o[db][i] is value dim db * 16 + 4 g + i of row n
  if (slot < 0) {
    if (!row_valid) return;
    const float inv = 1.f / run_sum;
    bf16_t* o_row = out + static_cast<int64_t>(token) * out_stride + static_cast<int64_t>(head) * D + 4 * g;
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) {
      uint2 packed;
      packed.x = pack_bf16x2(o[db][0] * inv, o[db][1] * inv);
      packed.y = pack_bf16x2(o[db][2] * inv, o[db][3] * inv);
      *reinterpret_cast<uint2*>(o_row + db * 16) = packed;
    }
  } else {
    const int64_t base = (static_cast<int64_t>(slot) * kv_heads + kvh) * 16 + n;
    float* po = part_o + base * D + 4 * g;
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) *reinterpret_cast<floatx4*>(po + db * 16) = o[db];
    if (g == 0) {
      part_ml[base * 2] = run_max;
      part_ml[base * 2 + 1] = run_sum;
    }
  }
}

// One block per (merge task, kv head): task = {item, row_tile, first_slot, num_splits}.
// Thread (n, j) of the 16 x 16 block first turns the splits' maxima and sums of row n into
// weights in shared memory, then adds the weighted partial outputs for its value dims.
#define MERGE_MAX_SPLITS 256
__global__ void __launch_bounds__(256)
attention_merge_kernel(const int32_t* __restrict__ tasks, const int32_t* __restrict__ item_meta,
                       int num_items, const float* __restrict__ part_o,
                       const float* __restrict__ part_ml, bf16_t* __restrict__ out,
                       int64_t out_stride, int heads, int kv_heads, int head_dim) {
  __shared__ float weight[16][MERGE_MAX_SPLITS];
  __shared__ float inv_denom[16];
  const int32_t* t = tasks + static_cast<int64_t>(blockIdx.x) * 4;
  const int item = t[0], row_tile = t[1], first_slot = t[2], splits = t[3];
  const int kvh = blockIdx.y;
  const int group = heads / kv_heads;
  const int q_start = item_meta[item], q_len = item_meta[num_items + item];
  const int n = threadIdx.x >> 4;        // row of the tile
  const int j = threadIdx.x & 15;
  const int rho = row_tile * 16 + n;
  const bool valid = rho < q_len * group;
  const int64_t stride = static_cast<int64_t>(kv_heads) * 16;     // partial rows between two splits
  const int64_t base0 = (static_cast<int64_t>(first_slot) * kv_heads + kvh) * 16 + n;
  // maxima: 16 threads per row share the splits
  float m = -INFINITY;
  for (int s = j; s < splits; s += 16) {
    const float ms = part_ml[(base0 + s * stride) * 2];
    weight[n][s] = ms;
    m = fmaxf(m, ms);
  }
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, SE_WAVE));
  float denom = 0.f;
  for (int s = j; s < splits; s += 16) {
    const float w = exp2f(weight[n][s] - m);
    weight[n][s] = w;
    denom += part_ml[(base0 + s * stride) * 2 + 1] * w;
  }
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) denom += __shfl_xor(denom, off, SE_WAVE);
  if (j == 0) inv_denom[n] = 1.f / denom;
  __syncthreads();
  if (!valid) return;
  const int token = q_start + rho / group;
  const int head = kvh * group + rho % group;
  const float inv = inv_denom[n];
  bf16_t* o_row = out + static_cast<int64_t>(token) * out_stride + static_cast<int64_t>(head) * head_dim;
  for (int d = j; d < head_dim; d += 16) {
    float acc = 0.f;
#pragma unroll 4
    for (int s = 0; s < splits; ++s) acc += part_o[(base0 + s * stride) * head_dim + d] * weight[n][s];
    o_row[d] = from_float<bf16_t>(acc * inv);
  }
}

extern "C" int se_paged_attention_mfma(const void* q, int64_t q_stride, const void* cache,
                                       const int32_t* block_table, int bt_stride,
                                       const int32_t* item_meta, int num_items,
                                       const int32_t* units, int num_units, const int32_t* tasks,
                                       int num_tasks, void* out, int64_t out_stride, float* part_o,
                                       float* part_ml, int heads, int kv_heads, int head_dim,
                                       int page_size, float scale, int window, hipStream_t stream) {
  if (num_units <= 0) return SE_OK;
  if (head_dim % 32 || head_dim <= 0 || head_dim > 256) return SE_ERR_SHAPE;
  if (kv_heads <= 0 || heads % kv_heads || page_size <= 0 || page_size % 8) return SE_ERR_SHAPE;
  if (q_stride % 8 || out_stride % 4) return SE_ERR_SHAPE;
  if (num_tasks > 0 && (!part_o || !part_ml || !tasks)) return SE_ERR_SHAPE;  // splits per task <= 256 (host)
  const float scale_log2e = scale * 1.4426950408889634f;
  dim3 grid((num_units + 3) / 4, kv_heads);
#define SE_ATT(DS)                                                                                 \
  case DS:                                                                                         \
    paged_attention_mfma_kernel<DS><<<grid, 256, 0, stream>>>(                                     \
        static_cast<const bf16_t*>(q), q_stride, static_cast<const bf16_t*>(cache), block_table,  \
        bt_stride, item_meta, num_items, units, num_units, static_cast<bf16_t*>(out), out_stride, \
        part_o, part_ml, heads, kv_heads, page_size, scale_log2e, window);                        \
    break;
  switch (head_dim / 32) {
    SE_ATT(1) SE_ATT(2) SE_ATT(3) SE_ATT(4) SE_ATT(5) SE_ATT(6) SE_ATT(7) SE_ATT(8)
    default: return SE_ERR_SHAPE;
  }
#undef SE_ATT
  SE_CHECK_LAUNCH();
  if (num_tasks > 0) {
    attention_merge_kernel<<<dim3(num_tasks, kv_heads), 256, 0, stream>>>(
        tasks, item_meta, num_items, part_o, part_ml, static_cast<bf16_t*>(out), out_stride, heads,
        kv_heads, head_dim);
    SE_CHECK_LAUNCH();
  }
  return SE_OK;
}
