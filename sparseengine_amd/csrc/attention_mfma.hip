// Paged causal GQA attention on the matrix cores (bfloat16) for gfx950.  Two kernels share one
// formulation: one wavefront per unit, with split keys and a merge kernel, for steps with few rows
// (decoding, short portions); blocks that share keys and values through shared memory for steps
// with many rows (prompt portions).  The host's work list decides which one a step takes.
//
// A *row* is one (query token, query head) pair.  For one request and one kv head the rows
// (q_len * group of them, ordered token-major) are cut into tiles of 16; a work unit is one tile
// and one range of keys, and one wavefront runs it:
//
//   S^T = K Q^T   v_mfma_f32_16x16x32_bf16, A = 16 keys x 32 dims, B = 32 dims x 16 rows.  The key of
//                 A-row m in block b is k0 + 8 * (m / 4) + m % 4 + 4 * b, so that a lane ends up with
//                 the scores of eight consecutive keys for its row: exactly the B operand of
//   O^T += V^T P^T  A = 16 value dims x 32 keys (eight consecutive keys of one dim lie side by side
//                 in a page and are one 16-byte load), B = 32 keys x 16 rows.
//
// Softmax is online, in float, in base 2 (scale * log2(e) folded into the scores); probabilities
// are rounded to bfloat16 for the value product, the running sum uses them unrounded.
// Masked: keys after the row's position, keys more than `window` before it.  A split unit
// writes its unnormalised O, running maximum and sum; the merge kernel combines a tile's splits
// in the order of the key ranges.
//
// Cache layer: [pages, 2, kv_heads, page_size * head_dim]; inside a page a head's keys lie
// [head_dim / 8][page_size][8] and its values [page_size / 8][head_dim][8] (common.h: key_place,
// value_place): the sixteen lanes that hold neighbouring rows of an operand read one contiguous
// stretch.  Requires head_dim % 32 == 0, head_dim <= 256, page_size % 8 == 0.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// A unit carries what its wavefront needs to start (one 32-byte record, no second look-up):
#define UNIT_FIELDS 8  // item, row_tile, key_begin, key_end, partial_slot (-1: writes out), q_start, q_len, ctx_len
#define TASK_FIELDS 6  // item, row_tile, first_slot, num_splits, q_start, q_len
// a block's record: item, first_tile, key_begin, key_end, partial_slot of its first tile (-1: writes
// out), q_start, q_len, ctx_len, slots between two of its tiles (= key ranges per tile), 3 unused
#define BLOCK_UNIT_FIELDS 12

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return static_cast<uint32_t>(float_to_bf16_bits(lo)) |
         (static_cast<uint32_t>(float_to_bf16_bits(hi)) << 16);
}

// Eight consecutive keys of one value dim; those after `last_key` are made zero: slots past a
// request's last key hold whatever an earlier owner of the page left (possibly not finite).
__device__ __forceinline__ uint4 zero_keys_beyond(uint4 v, int first_key, int last_key) {
  const int keep = last_key - first_key + 1;   // keys 0 .. keep - 1 of the eight stay
  auto word = [&](uint32_t w, int k) {
    const uint32_t m = (2 * k < keep ? 0x0000ffffu : 0u) | (2 * k + 1 < keep ? 0xffff0000u : 0u);
    return w & m;
  };
  v.x = word(v.x, 0);
  v.y = word(v.y, 1);
  v.z = word(v.z, 2);
  v.w = word(v.w, 3);
  return v;
}

template <int DSTEPS>  // head_dim = 32 * DSTEPS
__global__ void __launch_bounds__(256)
paged_attention_mfma_kernel(const bf16_t* __restrict__ q, int64_t q_stride,
                            const bf16_t* __restrict__ cache,
                            const int32_t* __restrict__ block_table, int bt_stride,
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

  const int4* u = reinterpret_cast<const int4*>(units + static_cast<int64_t>(unit) * UNIT_FIELDS);
  const int4 u0 = u[0], u1 = u[1];
  const int item = u0.x, row_tile = u0.y, key_begin = u0.z, slot = u1.x;
  int key_end = u0.w;
  const int q_start = u1.y, q_len = u1.z, ctx_len = u1.w;
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
  // With a window the first step of 32 keys may begin before the tile's lowest key, in a page that
  // the request has given back (its table entry is -1).  No page is looked up and nothing is loaded
  // for a key below `low_key`: such a key takes the place of `low_key` (its score is masked, so
  // whatever finite values stand in for it count for nothing).
  int k_first = key_begin;
  int low_key = 0;
  if (window > 0) {
    const int pos_min = ctx_len - q_len + (row_tile * 16) / group;
    const int lowest = pos_min - window + 1;
    if (lowest > k_first) k_first = lowest & ~31;
    if (lowest > 0) low_key = lowest;
    if (key_end <= low_key) key_end = k_first;   // the whole range lies before every row's window
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

  // One step = 32 keys.  Two register sets (A, B) take turns: while the matrix cores and the
  // softmax work on one step, the key and value operands of the next are already being loaded,
  // and the page ids of the step after that are looked up.  Without this every step costs two
  // memory round trips (keys, then values) and the kernel is bound by latency, not by bandwidth.
  auto page_of_keys = [&](int k0) {     // page of the lane's two key rows (both lie in one group of 8)
    int key = k0 + 8 * (n >> 2);
    if (key > last_key) key = last_key;
    if (key < low_key) key = low_key;
    return table[key / page_size];
  };
  auto page_of_values = [&](int k0) {   // page of the lane's eight consecutive keys
    int key = k0 + 8 * g;
    if (key > last_key) key = last_key & ~7;
    if (key + 7 < low_key) key = low_key & ~7;
    return table[key / page_size];
  };

#define ATT_LOAD(KF, VF, K0, PK, PV)                                                              \
  {                                                                                               \
    _Pragma("unroll") for (int b = 0; b < 2; ++b) {                                               \
      int key = (K0) + 8 * (n >> 2) + (n & 3) + 4 * b;                                            \
      if (key > last_key) key = last_key; /* reads stay inside the request's pages */            \
      if (key < low_key) key = low_key;                                                           \
      /* dims 32 ds + 8 g ... of the key: group 4 ds + g of the page's [head_dim / 8][page_size][8] */ \
      const bf16_t* k_row = cache + (static_cast<int64_t>(PK) * 2) * plane + kvh * head_span +    \
                            (static_cast<int64_t>(g) * page_size + key % page_size) * 8;          \
      _Pragma("unroll") for (int ds = 0; ds < DSTEPS; ++ds)                                       \
          KF[b][ds] = load16_once(k_row + static_cast<int64_t>(ds) * 32 * page_size);             \
    }                                                                                             \
    int vkey = (K0) + 8 * g;                                                                      \
    if (vkey > last_key) vkey = last_key & ~7;                                                    \
    if (vkey + 7 < low_key) vkey = low_key & ~7;                                                  \
    /* eight keys of dim 16 db + n: the page's [page_size / 8][head_dim][8] */                     \
    const bf16_t* v_col = cache + (static_cast<int64_t>(PV) * 2 + 1) * plane + kvh * head_span +  \
                          static_cast<int64_t>(vkey % page_size) * D + n * 8;                     \
    _Pragma("unroll") for (int db = 0; db < DBLOCKS; ++db)                                        \
        VF[db] = load16_once(v_col + db * 128);                                                   \
  }

#define ATT_COMPUTE(KF, VF, K0)                                                                   \
  {                                                                                               \
    floatx4 s[2];                                                                                 \
    _Pragma("unroll") for (int b = 0; b < 2; ++b) {                                               \
      s[b] = floatx4{0.f, 0.f, 0.f, 0.f};                                                         \
      _Pragma("unroll") for (int ds = 0; ds < DSTEPS; ++ds)                                       \
          s[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, KF[b][ds]),   \
                                                         __builtin_bit_cast(bf16x8, qf[ds]), s[b], 0, 0, 0); \
    }                                                                                             \
    /* lane (g, n): s[b][i] is the score of key K0 + 8 g + 4 b + i for row n */                   \
    float p[8];                                                                                   \
    float tile_max = -INFINITY;                                                                   \
    _Pragma("unroll") for (int b = 0; b < 2; ++b)                                                 \
      _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                             \
        const int key = (K0) + 8 * g + 4 * b + i;                                                 \
        const bool masked = key > pos || (window > 0 && key <= pos - window);                     \
        const float v = masked ? -INFINITY : s[b][i] * scale_log2e;                               \
        p[b * 4 + i] = v;                                                                         \
        tile_max = fmaxf(tile_max, v);                                                            \
      }                                                                                           \
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, SE_WAVE));                                \
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, SE_WAVE));                                \
    const float new_max = fmaxf(run_max, tile_max);                                               \
    const float ref = (new_max == -INFINITY) ? 0.f : new_max; /* a row with no key yet */         \
    const float alpha = exp2f(run_max - ref);                                                     \
    float tile_sum = 0.f;                                                                         \
    _Pragma("unroll") for (int j = 0; j < 8; ++j) {                                               \
      p[j] = exp2f(p[j] - ref);                                                                   \
      tile_sum += p[j];                                                                           \
    }                                                                                             \
    tile_sum += __shfl_xor(tile_sum, 16, SE_WAVE);                                                \
    tile_sum += __shfl_xor(tile_sum, 32, SE_WAVE);                                                \
    run_sum = run_sum * alpha + tile_sum;                                                         \
    run_max = new_max;                                                                            \
    _Pragma("unroll") for (int db = 0; db < DBLOCKS; ++db) o[db] *= alpha;                        \
    uint4 pf;                                                                                     \
    pf.x = pack_bf16x2(p[0], p[1]);                                                               \
    pf.y = pack_bf16x2(p[2], p[3]);                                                               \
    pf.z = pack_bf16x2(p[4], p[5]);                                                               \
    pf.w = pack_bf16x2(p[6], p[7]);                                                               \
    /* values: lane (g, n) holds value dim db * 16 + n at keys K0 + 8 g .. + 7 */                 \
    int vkey = (K0) + 8 * g; /* clamped as in the load */                                         \
    if (vkey > last_key) vkey = last_key & ~7;                                                    \
    if (vkey + 7 < low_key) vkey = low_key & ~7;                                                  \
    const bool beyond = vkey + 7 > last_key; /* the request's last group of eight */              \
    _Pragma("unroll") for (int db = 0; db < DBLOCKS; ++db) {                                      \
      uint4 vf = VF[db];                                                                          \
      if (beyond) vf = zero_keys_beyond(vf, vkey, last_key);                                      \
      o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vf),             \
                                                     __builtin_bit_cast(bf16x8, pf), o[db], 0, 0, 0); \
    }                                                                                             \
  }

  if (k_first < key_end) {
    uint4 kfA[2][DSTEPS], vfA[DBLOCKS];
    if constexpr (DSTEPS <= 4) {
      uint4 kfB[2][DSTEPS], vfB[DBLOCKS];
      int pk = page_of_keys(k_first), pv = page_of_values(k_first);
      ATT_LOAD(kfA, vfA, k_first, pk, pv)
      pk = page_of_keys(k_first + 32);
      pv = page_of_values(k_first + 32);
      for (int k0 = k_first; k0 < key_end; k0 += 64) {
        const bool second = k0 + 32 < key_end;
        if (second) {
          ATT_LOAD(kfB, vfB, k0 + 32, pk, pv)
          pk = page_of_keys(k0 + 64);
          pv = page_of_values(k0 + 64);
        }
        ATT_COMPUTE(kfA, vfA, k0)
        if (!second) break;
        if (k0 + 64 < key_end) {
          ATT_LOAD(kfA, vfA, k0 + 64, pk, pv)
          pk = page_of_keys(k0 + 96);
          pv = page_of_values(k0 + 96);
        }
        ATT_COMPUTE(kfB, vfB, k0 + 32)
      }
    } else {   // large heads: one register set; keys and values of a step are still loaded together
      for (int k0 = k_first; k0 < key_end; k0 += 32) {
        const int pk = page_of_keys(k0), pv = page_of_values(k0);
        ATT_LOAD(kfA, vfA, k0, pk, pv)
        ATT_COMPUTE(kfA, vfA, k0)
      }
    }
  }
#undef ATT_LOAD
#undef ATT_COMPUTE

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

// Prompt portions: the same product with the keys and values of a step shared by a whole block.
// A block of four wavefronts takes 4 * RT consecutive row tiles of one request and one kv head
// (wave w the tiles first + w * RT ...).  Each step of 32 keys is brought into shared memory once,
// by loads that go from the cache straight into shared memory (no register in between), NS - 1
// steps ahead of the step that is being computed; every wave reads its operands from there and
// each operand feeds RT products.  The one-wavefront kernel above reads every key once per 16
// rows, which binds a long prompt to the L2's bandwidth and to the latency of each step's loads.
//
// Such a load writes lane l's 16 bytes at (wave-uniform base) + 16 l, so shared memory holds
// chunks of 1024 bytes in the order the loading lanes chose: per 16 value dims db one chunk in
// which lane l's piece is exactly what lane l feeds the matrix core, and per (sixteen consecutive
// keys, 32 dims ds) one chunk from which the lanes pick their operand's key when they read (the
// places are chosen so that these reads are conflict-free too; see where `key_at` is set).
// The compiler does not see these writes; the waits for them (vmcnt) are placed by hand, and the
// barrier is a bare s_barrier: the usual fence would wait for every load in flight.
// The request's page ids for the block's keys are copied to shared memory first (at most
// TILED_MAX_PAGES), so that no load in the loop depends on another.
// A unit covers a run of tiles and a range of keys; with the whole range of its rows it writes the
// output itself, else partial results for the merge kernel, like the units of the kernel above.
#define TILED_MAX_PAGES 2048
#define TILED_ROW_TILES 2   // row tiles per wavefront: 8 per block
#define TILED_STAGES 4      // steps of keys in shared memory at a time

// Maximum / sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 that share a row: two register swaps
// between halves and between rows of 16 lanes instead of trips through the shared-memory crossbar.
// The library's fmaxf quiets signalling NaNs first, one more instruction per operand; scores are
// products of finite numbers or -inf, so the bare instructions do.
__device__ __forceinline__ float max_bare(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ float max3_bare(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ __forceinline__ float quad_max(float v) {
  const uint32_t u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  v = max_bare(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const uint32_t w = __float_as_uint(v);
  const auto b = __builtin_amdgcn_permlane16_swap(w, w, false, false);
  return max_bare(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float quad_sum(float v) {
  const uint32_t u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const uint32_t w = __float_as_uint(v);
  const auto b = __builtin_amdgcn_permlane16_swap(w, w, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2_rne(float lo, float hi) {   // one v_cvt_pk_bf16_f32
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{lo, hi}, bf16x2));
}

// Online softmax of one step for the wave's RT tiles (float, base 2).  The reference maximum of a
// row is only raised when the step's maximum exceeds it by more than SOFTMAX_SLACK (probabilities
// may then reach 2^SLACK, which float sums and bfloat16 operands hold as well as values below 1):
// the rescaling of the accumulators, the costly part, becomes rare.  A row's sum is kept per
// lane and added up over its four lanes at the end.
#define SOFTMAX_SLACK 8.f
#define TILED_SOFTMAX(MASKED)                                                                      \
  _Pragma("unroll") for (int rt = 0; rt < RT; ++rt) {                                              \
    float v[8];                                                                                    \
    _Pragma("unroll") for (int b = 0; b < 2; ++b)                                                  \
      _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                              \
        float x = s[rt][b][i];                                                                     \
        if (MASKED) {                                                                              \
          const int key = k0 + 8 * g + 4 * b + i;                                                  \
          if (key > pos[rt] || (window > 0 && key <= pos[rt] - window)) x = -INFINITY;             \
        }                                                                                          \
        v[b * 4 + i] = x;                                                                          \
      }                                                                                            \
    float m = max_bare(max3_bare(v[0], v[1], v[2]), max3_bare(max3_bare(v[3], v[4], v[5]), v[6], v[7])); \
    m = quad_max(m) * scale_log2e; /* scale > 0: the maximum commutes with it */                   \
    const bool grow = m > run_max[rt] + SOFTMAX_SLACK || (run_max[rt] == -INFINITY && m > -INFINITY); \
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(grow) != 0, 0)) {                             \
      const float alpha = grow ? __builtin_amdgcn_exp2f(run_max[rt] - m) : 1.f;                    \
      if (grow) run_max[rt] = m;                                                                   \
      run_sum[rt] *= alpha;                                                                        \
      _Pragma("unroll") for (int db = 0; db < DBLOCKS; ++db) o[rt][db] *= alpha;                   \
    }                                                                                              \
    /* a row whose keys are all masked so far has no reference yet; its probabilities are 0 */     \
    const float ref = (MASKED && run_max[rt] == -INFINITY) ? 0.f : run_max[rt];                    \
    float sum = 0.f;                                                                               \
    _Pragma("unroll") for (int j = 0; j < 8; ++j) {                                                \
      v[j] = __builtin_amdgcn_exp2f(fmaf(v[j], scale_log2e, -ref));                                \
      sum += v[j];                                                                                 \
    }                                                                                              \
    run_sum[rt] += sum;                                                                            \
    pf[rt].x = pack_bf16x2_rne(v[0], v[1]);                                                        \
    pf[rt].y = pack_bf16x2_rne(v[2], v[3]);                                                        \
    pf[rt].z = pack_bf16x2_rne(v[4], v[5]);                                                        \
    pf[rt].w = pack_bf16x2_rne(v[6], v[7]);                                                        \
  }

template <int DSTEPS, int RT, int NS, bool STEP_IN_PAGE>   // STEP_IN_PAGE: pages hold a multiple of 32 keys
__global__ void __launch_bounds__(256, 2)
paged_attention_tiled_kernel(const bf16_t* __restrict__ q, int64_t q_stride,
                             const bf16_t* __restrict__ cache,
                             const int32_t* __restrict__ block_table, int bt_stride,
                             const int32_t* __restrict__ units, bf16_t* __restrict__ out,
                             int64_t out_stride, float* __restrict__ part_o,
                             float* __restrict__ part_ml, int heads, int kv_heads, int page_size,
                             float scale_log2e, int window) {
  constexpr int D = 32 * DSTEPS;
  constexpr int DBLOCKS = 2 * DSTEPS;
  constexpr int CHUNKS = 4 * DSTEPS;              // per step: 2 * DSTEPS of keys, then 2 * DSTEPS of values
  // the destination of a load into shared memory is a 16-bit offset: the stages lie in the first 64 KB
  static_assert(NS * CHUNKS * 1024 <= 65536, "stages must lie within the first 64 KB of shared memory");
  // dynamic: NS stages of CHUNKS x 64 vectors, then TILED_MAX_PAGES page ids (more than a block's
  // static allowance when NS = 4 and head_dim = 128)
  extern __shared__ __align__(16) uint4 tiled_shared[];
  uint4(*stage)[CHUNKS][64] = reinterpret_cast<uint4(*)[CHUNKS][64]>(tiled_shared);
  int32_t* page_ids = reinterpret_cast<int32_t*>(tiled_shared + NS * CHUNKS * 64);

  const int tid = threadIdx.x;
  const int lane = tid & (SE_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / SE_WAVE);   // known to be the same in all lanes
  const int n = lane & 15;
  const int g = lane >> 4;
  const int kvh = blockIdx.x % kv_heads;   // units come longest first: all kv heads of one, then the next
  const int group = heads / kv_heads;

  const int32_t* u = units + static_cast<int64_t>(blockIdx.x / kv_heads) * BLOCK_UNIT_FIELDS;
  const int item = u[0], first_tile = u[1], key_begin = u[2], slot = u[4], slot_stride = u[8];
  int key_end = u[3];
  const int q_start = u[5], q_len = u[6], ctx_len = u[7];
  const int rows_total = q_len * group;
  const int pos0 = ctx_len - q_len;
  const int last_key = ctx_len - 1;

  // the block's rows bound the keys that are loaded; the wave's rows bound what it computes
  const int block_last_row = min((first_tile + 4 * RT) * 16, rows_total) - 1;
  key_end = min(key_end, pos0 + block_last_row / group + 1);
  // as in the kernel above: nothing is looked up or loaded for a key below `low_key`, whose page the
  // request may have given back; `low_key` stands in for it
  int k_first = key_begin;
  int low_key = 0;
  if (window > 0) {
    const int lowest = pos0 + (first_tile * 16) / group - window + 1;
    if (lowest > k_first) k_first = lowest & ~31;
    if (lowest > 0) low_key = lowest;
    if (key_end <= low_key) key_end = k_first;   // the whole range lies before every row's window
  }
  const int tile0 = first_tile + wave * RT;
  const bool wave_active = tile0 * 16 < rows_total;
  const int wave_last_row = min((tile0 + RT) * 16, rows_total) - 1;
  const int wave_hi = wave_active ? pos0 + wave_last_row / group : -1;          // largest position
  const int wave_lo = wave_active ? pos0 + (tile0 * 16) / group : 0;            // smallest position

  const int32_t* table = block_table + static_cast<int64_t>(item) * bt_stride;
  const int kmax = key_end - 1;                    // loads are clamped to the block's last key
  // The page ids of the block's keys, as many as fit; a longer range is brought in window by
  // window as the steps reach it (a very long context on small pages).
  int window_base = k_first / page_size;          // first page held in page_ids
  int window_end = (window_base + TILED_MAX_PAGES) * page_size;   // first key whose page is not held
  const int last_page = kmax / page_size;
  if (k_first < key_end) {
    const int pages = min(last_page - window_base + 1, TILED_MAX_PAGES);
    for (int i = tid; i < pages; i += 256) page_ids[i] = table[window_base + i];
  }
  // a lane's row of tile rt: whether the item has it, its token, head and position.  Worked out again
  // where it is needed (the masked steps, the end): kept, it would cost eight registers all through
  // a loop that has none to spare.
  auto row_of = [&](int rt, bool& valid, int& token, int& head, int& position) {
    const int rho = (tile0 + rt) * 16 + n;
    valid = rho < rows_total;
    const int rho_c = valid ? rho : rows_total - 1;   // padding rows repeat the last row
    const int q_idx = rho_c / group;
    head = kvh * group + rho_c % group;
    token = q_start + q_idx;
    position = pos0 + q_idx;
  };
  uint4 qf[RT][DSTEPS];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    bool valid;
    int token, head, position;
    row_of(rt, valid, token, head, position);
    const bf16_t* q_row = q + static_cast<int64_t>(token) * q_stride +
                          static_cast<int64_t>(head) * D + g * 8;
#pragma unroll
    for (int ds = 0; ds < DSTEPS; ++ds) qf[rt][ds] = *reinterpret_cast<const uint4*>(q_row + ds * 32);
  }

  const int64_t head_span = static_cast<int64_t>(page_size) * D;
  const int64_t plane = static_cast<int64_t>(kv_heads) * head_span;
  const bf16_t* cache_head = cache + kvh * head_span;

  floatx4 o[RT][DBLOCKS];
  float run_max[RT], run_sum[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    run_max[rt] = -INFINITY;
    run_sum[rt] = 0.f;
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) o[rt][db] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  __syncthreads();   // page ids are in place
  // The query operands must have arrived before the loop: a wait for them inside it would also
  // wait for the loads into shared memory that were issued just before.
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int ds = 0; ds < DSTEPS; ++ds)
      asm volatile("" : "+v"(qf[rt][ds].x), "+v"(qf[rt][ds].y), "+v"(qf[rt][ds].z), "+v"(qf[rt][ds].w));

  // Waves 0 and 1 bring sixteen keys of a step each, waves 2 and 3 one half of the value dims each:
  // wave w fills chunks w * DSTEPS ... of a stage.  Steps are issued in order, so a lane follows its
  // key's page and place in the page by adding 32 (no division in the loop); a key past the block's
  // last one is replaced by that one (values: by its group of eight).
  // The sixteen keys of a key chunk are consecutive ones, 256 contiguous bytes per group of eight
  // dims (whole cache lines; the score layout wants keys 0-3, 8-11, 16-19, 24-27 in one operand and
  // the others in the second, and chunks loaded in that order would take every line in two halves,
  // by two waves).  The operands are gathered when they are read: row n of key block b is key
  // 8 (n / 4) + n % 4 + 4 b.  Wave 1 brings its keys with bit 2 of their place flipped, so that the
  // sixteen lanes of a read, half of which look into each chunk, fall on sixteen different bank groups.
  const uint32_t stage_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(&stage[0][0][0]));
  const bool loads_keys = wave < 2;
  const int lane_key = loads_keys ? 16 * wave + (n ^ (4 * wave)) : 8 * g;
  const int clamp_key = loads_keys ? kmax : (kmax & ~7);
  const int clamp_page = clamp_key / page_size, clamp_off = clamp_key % page_size;
  // a lane's key (values: its group of eight) wholly below `low_key` is replaced by that one's
  const int low_clamp = loads_keys ? low_key : (low_key & ~7);
  const int low_page = low_clamp / page_size, low_off = low_clamp % page_size;
  int key_at[2];     // where the lane's vector of key block b lies among a stage's vectors, for the first 32 dims
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const int key = 8 * (n >> 2) + (n & 3) + 4 * b, half = key >> 4;
    key_at[b] = half * DSTEPS * 64 + 16 * g + ((key & 15) ^ (4 * half));
  }
  int next_key = k_first + lane_key;                     // the lane's key of the next step to be issued
  int next_page = next_key / page_size, next_off = next_key % page_size;
  // keys lie [head_dim / 8][page_size][8], values [page_size / 8][head_dim][8]: sixteen lanes of a
  // chunk (keys: runs of four; values: all sixteen) read one contiguous stretch
  const int64_t lane_base = loads_keys ? static_cast<int64_t>(g) * page_size * 8
                                       : plane + static_cast<int64_t>((wave - 2) * DSTEPS * 16 + n) * 8;
  const int off_scale = loads_keys ? 8 : D;
  const int64_t load_stride = loads_keys ? static_cast<int64_t>(32) * page_size : 128;
  // a page's keys and values of all heads: fewer than 2^32 elements (the host checks it), so that a
  // page's place is one multiplication of unsigned words
  const uint32_t page_span = static_cast<uint32_t>(2 * plane);
  const bf16_t* lane_src = cache_head + lane_base;
  // Pages of a multiple of 32 keys hold all keys of a step, so the step's page and the address of its
  // first key are the same in all lanes: that arithmetic stays in scalar registers, beside the vector
  // instructions that the loop is short of, and a lane adds only its own constant offset.  The steps at
  // a unit's ends, where lanes are clamped to the first or the last key, take the lane-by-lane form.
  constexpr bool page_per_step = STEP_IN_PAGE;
  const uint32_t lane_bytes = static_cast<uint32_t>((lane_base + static_cast<int64_t>(lane_key) * off_scale) * 2);
  int step_page = k_first / page_size, step_off = k_first % page_size;   // of the next step to be issued
  auto issue = [&](int step) {
    const uint32_t dst = stage_base + static_cast<uint32_t>((step % NS) * CHUNKS + wave * DSTEPS) * 1024u;
    if constexpr (page_per_step) {
      const int k = k_first + 32 * step;
      if (k + 31 <= kmax && k >= low_key) {
        const uint32_t page = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(page_ids[step_page - window_base]));
        const bf16_t* base = cache_head + static_cast<uint64_t>(page) * page_span +
                             static_cast<uint32_t>(step_off * off_scale);
#pragma unroll
        for (int j = 0; j < DSTEPS; ++j)
          load16_to_lds_at(base + j * load_stride, lane_bytes, dst + static_cast<uint32_t>(j) * 1024u);
      } else {
        int key = k + lane_key;
        if (key > kmax) key = clamp_key;
        if (key < low_clamp) key = low_clamp;
        const uint32_t page = static_cast<uint32_t>(page_ids[key / page_size - window_base]);
        const bf16_t* src = lane_src + static_cast<uint64_t>(page) * page_span +
                            static_cast<uint32_t>((key % page_size) * off_scale);
#pragma unroll
        for (int j = 0; j < DSTEPS; ++j) load16_to_lds(src + j * load_stride, dst + static_cast<uint32_t>(j) * 1024u);
      }
      step_off += 32;
      if (step_off >= page_size) {
        step_off -= page_size;
        ++step_page;
      }
    } else {
    const bool over = next_key > kmax;
    const uint32_t page = static_cast<uint32_t>(page_ids[(over ? clamp_page : next_page) - window_base]);
    const bf16_t* src = lane_src + static_cast<uint64_t>(page) * page_span +
                        static_cast<uint32_t>((over ? clamp_off : next_off) * off_scale);
#pragma unroll
    for (int j = 0; j < DSTEPS; ++j) load16_to_lds(src + j * load_stride, dst + static_cast<uint32_t>(j) * 1024u);
    next_key += 32;
    next_off += 32;
#pragma unroll
    for (int i = 0; i < 4; ++i)          // pages hold at least 8 keys
      if (next_off >= page_size) {
        next_off -= page_size;
        ++next_page;
      }
    }
  };

  const int nsteps = (key_end - k_first + 31) / 32;
  if (nsteps > 0) {
    // The loop below works on two steps at a time: while the vector unit turns the scores of step t
    // into probabilities, the matrix unit already makes the scores of step t + 1 (both from one wave's
    // instruction stream, which is the only way the two units of a SIMD overlap reliably).  So keys
    // are needed one step before values: the waves that bring keys run one step ahead of those that
    // bring values, in the same ring of stages.
    const int lead = loads_keys ? 1 : 0;
    // Only a unit's first step can begin before `low_key` (it begins less than 32 keys before it): a
    // lane whose key lies there takes `low_key`'s place for that one load and then goes on from its
    // own key.  (Done here and not inside `issue`, which is the loop's hot path.)
    const bool under = next_key < low_clamp;
    if (under) {
      next_page = low_page;
      next_off = low_off;
    }
    issue(0);
    if (under) {       // next_key has moved on by 32
      next_page = next_key / page_size;
      next_off = next_key % page_size;
    }
#pragma unroll
    for (int j = 1; j < NS; ++j)
      if (j < NS - 1 + lead && j < nsteps) issue(j);
    // What every wave does at the start of step t, whatever it computes then: wait for its part of the
    // data that the step needs (the values of step t, the keys of step t + 1), meet the others, issue
    // the loads of the step NS - 1 after that.
    auto begin_step = [&](int t) {
      const int mine = t + lead;
      // all but the loads of the NS - 2 steps after `mine` must have come back
      if (mine + NS - 2 < nsteps) {
        __builtin_amdgcn_s_waitcnt(0x0F70 | ((NS - 2) * DSTEPS));     // vmcnt((NS - 2) * DSTEPS)
      } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);                           // vmcnt(0)
      }
      __builtin_amdgcn_s_barrier();   // everyone's part is in; everyone has left step t - 1
      asm volatile("" ::: "memory");
      if (t + NS - 1 < nsteps) {      // values of step t + NS - 1, keys of step t + NS if there is one
        const int k_near = k_first + 32 * (t + NS - 1);
        const int k_far = k_first + 32 * min(t + NS, nsteps - 1);
        if (min(k_far + 31, kmax) >= window_end) {
          // nobody reads page_ids between the barrier above and its own issue below
          window_base = k_near / page_size;
          window_end = (window_base + TILED_MAX_PAGES) * page_size;
          const int pages = min(last_page - window_base + 1, TILED_MAX_PAGES);
          for (int i = tid; i < pages; i += 256) page_ids[i] = table[window_base + i];
          __syncthreads();
        }
        if (mine + NS - 1 < nsteps) issue(mine + NS - 1);   // into the buffer whose last readers have met the barrier
      }
    };
    auto active = [&](int step) {      // has the wave a row that sees a key of this step?
      const int k0 = k_first + 32 * step;
      return k0 <= wave_hi && (window <= 0 || k0 + 31 > wave_lo - window);
    };
    // lane (g, n): s[rt][b][i] becomes the score of key k0 + 8 g + 4 b + i for row n of tile rt
    auto scores = [&](int step, floatx4 (&s)[RT][2]) {
      const uint4* keys = &stage[step % NS][0][0];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) s[rt][0] = s[rt][1] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ds = 0; ds < DSTEPS; ++ds)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          const uint4 kf = keys[key_at[b] + 64 * ds];
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
            s[rt][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf),
                                                               __builtin_bit_cast(bf16x8, qf[rt][ds]),
                                                               s[rt][b], 0, 0, 0);
        }
    };
    // A step in full, from its scores: the rows' ranges of keys, the reference maxima and the end of the
    // cache all looked at.
    auto whole_step = [&](int step, floatx4 (&s)[RT][2]) {
      const int k0 = k_first + 32 * step;
      if (active(step)) {
        const uint4(*buf)[64] = stage[step % NS];
        // Most steps lie wholly inside every row's range of keys and need no mask.
        uint4 pf[RT];
        if (k0 + 31 > wave_lo || (window > 0 && k0 <= wave_hi - window)) {
          int pos[RT];
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
            bool valid;
            int token, head;
            row_of(rt, valid, token, head, pos[rt]);
          }
          TILED_SOFTMAX(1)
        } else {
          const int* pos = nullptr;      // not looked at without masks
          (void)pos;
          TILED_SOFTMAX(0)
        }
        // the block's last step may hold slots past the request's last key: whatever an earlier owner
        // of the page left there, possibly not finite.  The loader's clamping is repeated here.
        // Two copies of the loop: folded into one, the masking would be paid in every step.
        if (__builtin_expect(k0 + 31 > kmax, 0)) {
          int vkey = k0 + 8 * g;      // clamped as the loader clamps it
          if (vkey > kmax) vkey = kmax & ~7;
          if (vkey < (low_key & ~7)) vkey = low_key & ~7;
#pragma unroll
          for (int db = 0; db < DBLOCKS; ++db) {
            const uint4 vf = zero_keys_beyond(buf[2 * DSTEPS + db][lane], vkey, last_key);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
              o[rt][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vf),
                                                                 __builtin_bit_cast(bf16x8, pf[rt]),
                                                                 o[rt][db], 0, 0, 0);
          }
        } else {
#pragma unroll
          for (int db = 0; db < DBLOCKS; ++db) {
            const uint4 vf = buf[2 * DSTEPS + db][lane];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
              o[rt][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vf),
                                                                 __builtin_bit_cast(bf16x8, pf[rt]),
                                                                 o[rt][db], 0, 0, 0);
          }
        }
      }
    };
    // Most steps of a long context lie before every row's own position, inside every row's window and
    // before the block's last key, and raise no row's maximum beyond the slack: steps [plain_begin,
    // plain_end) are tried without masks, without the exchange of maxima between lanes and, above all,
    // without a path that rescales the accumulators.  (With that path inside the loop the compiler keeps
    // the accumulators in two sets of registers and copies all 64 of them between the sets in every
    // step; vector instructions, not matrix instructions, are what this kernel waits for.)  A step that
    // would raise a maximum is done in full instead.
    // a lane looks at its own eight keys only: any lane of a row that sees the maximum raised says so
    auto raised = [&](const floatx4 (&s)[RT][2]) {
      bool over = false;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const float m = max_bare(max3_bare(s[rt][0][0], s[rt][0][1], s[rt][0][2]),
                                 max3_bare(max3_bare(s[rt][0][3], s[rt][1][0], s[rt][1][1]), s[rt][1][2], s[rt][1][3]));
        over = over || !(m * scale_log2e <= run_max[rt] + SOFTMAX_SLACK);   // also with no maximum yet
      }
      return __builtin_amdgcn_ballot_w64(over) != 0;
    };
    auto plain_step = [&](int step, const floatx4 (&s)[RT][2]) {
      const uint4(*buf)[64] = stage[step % NS];
      uint4 pf[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        float v[8];
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          v[j] = __builtin_amdgcn_exp2f(fmaf(s[rt][j >> 2][j & 3], scale_log2e, -run_max[rt]));
          sum += v[j];
        }
        run_sum[rt] += sum;
        pf[rt].x = pack_bf16x2_rne(v[0], v[1]);
        pf[rt].y = pack_bf16x2_rne(v[2], v[3]);
        pf[rt].z = pack_bf16x2_rne(v[4], v[5]);
        pf[rt].w = pack_bf16x2_rne(v[6], v[7]);
      }
      // The wavefront asks for the instruction arbiter's favour while it feeds the matrix unit: the SIMD's
      // other wavefront is then mostly in its exponentials, which would otherwise take turns with these
      // instructions and leave the matrix unit waiting (a portion of 8192 tokens at context 65536: +6 %).
      // (Reading the value operands ahead of the exponentials instead of just before their use changes nothing.)
      __builtin_amdgcn_s_setprio(1);
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db) {
        const uint4 vf = buf[2 * DSTEPS + db][lane];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          o[rt][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vf),
                                                             __builtin_bit_cast(bf16x8, pf[rt]),
                                                             o[rt][db], 0, 0, 0);
      }
      __builtin_amdgcn_s_setprio(0);
    };
    const int plain_limit = min(wave_lo, kmax) - 31;              // last first-key of a plain step
    // (a plain step also makes the scores of the step after it, without asking whether there is one: the
    // unit's last step is never among them)
    const int plain_end = plain_limit >= k_first ? min(nsteps - 1, (plain_limit - k_first) / 32 + 1) : 0;
    const int plain_begin =
        window > 0 && wave_hi - window >= k_first ? (wave_hi - window - k_first) / 32 + 1 : 0;

    // the keys of step 0 have to be in before the loop: of the steps issued so far (a wave that brings
    // values has issued one fewer, and waits for nothing here) all but the first may still be under way
    {
      const int issued = min(NS, nsteps);
      if (issued >= 4) {
        __builtin_amdgcn_s_waitcnt(0x0F70 | (3 * DSTEPS));
      } else if (issued == 3) {
        __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * DSTEPS));
      } else if (issued == 2) {
        __builtin_amdgcn_s_waitcnt(0x0F70 | (1 * DSTEPS));
      } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);
      }
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
    }
    floatx4 sa[RT][2], sb[RT][2];     // the scores of the step at hand and of the one after it
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) sa[rt][0] = sa[rt][1] = sb[rt][0] = sb[rt][1] = floatx4{0.f, 0.f, 0.f, 0.f};
    if (active(0)) scores(0, sa);
    // The row maxima are taken with bare instructions (inline assembly), which the compiler does not
    // guard against reading a matrix instruction's result too early.  Inside the loop the scores that
    // are looked at were issued a whole step before (sixteen more matrix instructions lie between);
    // here the distance is made by hand.
    asm volatile("s_nop 15\n\ts_nop 15" : "+v"(sa[0][0]), "+v"(sa[0][1]), "+v"(sa[RT - 1][0]), "+v"(sa[RT - 1][1]));
    asm volatile("" ::: "memory");
    int t = 0;
    while (t < nsteps) {
      bool begun = false;     // the step's data is in and its barrier met
      if (t >= plain_begin && t < plain_end) {
        bool in_b = false;    // the scores of step t are in `sb`
        while (t < plain_end) {        // two steps a round, the two sets of scores taking turns
          begin_step(t);
          if (__builtin_expect(raised(sa), 0)) {
            begun = true;
            break;
          }
          scores(t + 1, sb);
          plain_step(t, sa);
          asm volatile("" ::: "memory");
          ++t;
          in_b = true;
          if (t >= plain_end) break;
          begin_step(t);
          if (__builtin_expect(raised(sb), 0)) {
            begun = true;
            break;
          }
          scores(t + 1, sa);
          plain_step(t, sb);
          asm volatile("" ::: "memory");
          ++t;
          in_b = false;
        }
        if (in_b) {
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
            sa[rt][0] = sb[rt][0];
            sa[rt][1] = sb[rt][1];
          }
        }
        if (!begun) continue;     // the plain steps are done
      }
      if (!begun) begin_step(t);
      if (t + 1 < nsteps && active(t + 1)) scores(t + 1, sb);
      whole_step(t, sa);
      asm volatile("" ::: "memory");
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        sa[rt][0] = sb[rt][0];
        sa[rt][1] = sb[rt][1];
      }
      ++t;
    }
  }

#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const float total = quad_sum(run_sum[rt]);   // every lane takes part
    if (slot >= 0) {
      // one key range of several: the unnormalised sums, their reference and the sum of weights, for
      // the merge kernel (padding rows included, tiles past the item's rows not: they have no slot)
      if ((tile0 + rt) * 16 >= rows_total) continue;
      const int64_t base =
          (static_cast<int64_t>(slot + (tile0 + rt - first_tile) * slot_stride) * kv_heads + kvh) * 16 + n;
      float* po = part_o + base * D + 4 * g;
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db) *reinterpret_cast<floatx4*>(po + db * 16) = o[rt][db];
      if (g == 0) {
        part_ml[base * 2] = run_max[rt];
        part_ml[base * 2 + 1] = total;
      }
      continue;
    }
    bool valid;
    int token, head, position;
    row_of(rt, valid, token, head, position);
    if (!valid || !wave_active) continue;
    const float inv = 1.f / total;
    bf16_t* o_row = out + static_cast<int64_t>(token) * out_stride +
                    static_cast<int64_t>(head) * D + 4 * g;
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) {
      uint2 packed;
      packed.x = pack_bf16x2(o[rt][db][0] * inv, o[rt][db][1] * inv);
      packed.y = pack_bf16x2(o[rt][db][2] * inv, o[rt][db][3] * inv);
      *reinterpret_cast<uint2*>(o_row + db * 16) = packed;
    }
  }
}

// One block per (merge task, kv head): task = {item, row_tile, first_slot, num_splits, q_start, q_len}.
// Thread (n, j) of the 16 x 16 block first turns the splits' maxima and sums of row n into weights
// in shared memory; then every thread owns float4 pieces of the tile's 16 x head_dim output and
// adds the weighted partial outputs, eight splits' loads in flight at a time.
#define MERGE_MAX_SPLITS 256
__global__ void __launch_bounds__(256)
attention_merge_kernel(const int32_t* __restrict__ tasks, const float* __restrict__ part_o,
                       const float* __restrict__ part_ml, bf16_t* __restrict__ out,
                       int64_t out_stride, int heads, int kv_heads, int head_dim) {
  __shared__ float weight[16][MERGE_MAX_SPLITS];
  __shared__ float inv_denom[16];
  const int32_t* t = tasks + static_cast<int64_t>(blockIdx.x) * TASK_FIELDS;
  const int row_tile = t[1], first_slot = t[2], splits = t[3], q_start = t[4], q_len = t[5];
  const int kvh = blockIdx.y;
  const int group = heads / kv_heads;
  const int64_t stride = static_cast<int64_t>(kv_heads) * 16;     // partial rows between two splits
  const int64_t tile_base = (static_cast<int64_t>(first_slot) * kv_heads + kvh) * 16;
  {
    const int n = threadIdx.x >> 4;        // row of the tile
    const int j = threadIdx.x & 15;        // 16 threads per row share the splits
    const int64_t base0 = tile_base + n;
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
  }
  __syncthreads();
  const int vecs_per_row = head_dim / 4;
  for (int piece = threadIdx.x; piece < 16 * vecs_per_row; piece += 256) {
    const int n = piece / vecs_per_row, d4 = (piece % vecs_per_row) * 4;
    const int rho = row_tile * 16 + n;
    if (rho >= q_len * group) continue;
    const float* src = part_o + (tile_base + n) * head_dim + d4;
    float4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < splits; s0 += 8) {
      float4 v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (s0 + i < splits) v[i] = *reinterpret_cast<const float4*>(src + (s0 + i) * stride * head_dim);
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (s0 + i < splits) {   // the splits are always added in the order of their key ranges
          const float w = weight[n][s0 + i];
          acc.x += v[i].x * w;
          acc.y += v[i].y * w;
          acc.z += v[i].z * w;
          acc.w += v[i].w * w;
        }
    }
    const float inv = inv_denom[n];
    const int token = q_start + rho / group;
    const int head = kvh * group + rho % group;
    uint2 packed;
    packed.x = pack_bf16x2(acc.x * inv, acc.y * inv);
    packed.y = pack_bf16x2(acc.z * inv, acc.w * inv);
    *reinterpret_cast<uint2*>(out + static_cast<int64_t>(token) * out_stride +
                              static_cast<int64_t>(head) * head_dim + d4) = packed;
  }
}

extern "C" int se_paged_attention_mfma(const void* q, int64_t q_stride, const void* cache,
                                       const int32_t* block_table, int bt_stride,
                                       const int32_t* units, int num_units, const int32_t* tasks,
                                       int num_tasks, void* out, int64_t out_stride, float* part_o,
                                       float* part_ml, int heads, int kv_heads, int head_dim,
                                       int page_size, float scale, int window, hipStream_t stream) {
  if (num_units <= 0 && num_tasks <= 0) return SE_OK;
  if (head_dim % 32 || head_dim <= 0 || head_dim > 256) return SE_ERR_SHAPE;
  if (kv_heads <= 0 || heads % kv_heads || page_size <= 0 || page_size % 8) return SE_ERR_SHAPE;
  if (q_stride % 8 || out_stride % 4) return SE_ERR_SHAPE;
  if (num_tasks > 0 && (!part_o || !part_ml || !tasks)) return SE_ERR_SHAPE;  // splits per task <= 256 (host)
  const float scale_log2e = scale * 1.4426950408889634f;
  dim3 grid((num_units + 3) / 4, kv_heads);
  if (num_units > 0) {
#define SE_ATT(DS)                                                                                 \
  case DS:                                                                                         \
    paged_attention_mfma_kernel<DS><<<grid, 256, 0, stream>>>(                                     \
        static_cast<const bf16_t*>(q), q_stride, static_cast<const bf16_t*>(cache), block_table,  \
        bt_stride, units, num_units, static_cast<bf16_t*>(out), out_stride,                       \
        part_o, part_ml, heads, kv_heads, page_size, scale_log2e, window);                        \
    break;
  switch (head_dim / 32) {
    SE_ATT(1) SE_ATT(2) SE_ATT(3) SE_ATT(4) SE_ATT(5) SE_ATT(6) SE_ATT(7) SE_ATT(8)
    default: return SE_ERR_SHAPE;
  }
#undef SE_ATT
  SE_CHECK_LAUNCH();
  }
  if (num_tasks > 0) {   // also merges what the block kernel has left in the same buffers
    attention_merge_kernel<<<dim3(num_tasks, kv_heads), 256, 0, stream>>>(
        tasks, part_o, part_ml, static_cast<bf16_t*>(out), out_stride, heads,
        kv_heads, head_dim);
    SE_CHECK_LAUNCH();
  }
  return SE_OK;
}

// Prompt portions through shared memory: units of BLOCK_UNIT_FIELDS ints, each covering
// `tiles_per_block` (8) row tiles; head_dim % 32 == 0, head_dim <= 128.  Units with a partial slot
// need part_o / part_ml and a merge afterwards (se_paged_attention_mfma with the tiles' tasks).
extern "C" int se_paged_attention_tiled(const void* q, int64_t q_stride, const void* cache,
                                        const int32_t* block_table, int bt_stride,
                                        const int32_t* units, int num_units, void* out,
                                        int64_t out_stride, float* part_o, float* part_ml, int heads,
                                        int kv_heads, int head_dim, int page_size, float scale,
                                        int window, int tiles_per_block, hipStream_t stream) {
  if (num_units <= 0) return SE_OK;
  if (head_dim % 32 || head_dim <= 0 || head_dim > 128) return SE_ERR_SHAPE;
  if (kv_heads <= 0 || heads % kv_heads || page_size <= 0 || page_size % 8) return SE_ERR_SHAPE;
  if (q_stride % 8 || out_stride % 4 || tiles_per_block != 4 * TILED_ROW_TILES) return SE_ERR_SHAPE;
  const float scale_log2e = scale * 1.4426950408889634f;
  if (static_cast<int64_t>(num_units) * kv_heads > 0x7fffffff) return SE_ERR_SHAPE;
  if (2 * static_cast<int64_t>(kv_heads) * page_size * head_dim > 0xffffffffLL) return SE_ERR_SHAPE;   // a page's span is a 32-bit word in the kernel
  dim3 grid(num_units * kv_heads);
#define SE_ATT_LAUNCH(DS, IN_PAGE)                                                                  \
  {                                                                                                \
    constexpr size_t shared = TILED_STAGES * 4 * DS * 1024 + TILED_MAX_PAGES * sizeof(int32_t);    \
    static bool allowed = false; /* more than 64 KB of shared memory has to be asked for, once */  \
    if (!allowed) {                                                                                \
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(                                       \
                                  &paged_attention_tiled_kernel<DS, TILED_ROW_TILES, TILED_STAGES, IN_PAGE>), \
                              hipFuncAttributeMaxDynamicSharedMemorySize,                          \
                              static_cast<int>(shared)) != hipSuccess)                             \
        return SE_ERR_LAUNCH;                                                                      \
      allowed = true;                                                                              \
    }                                                                                              \
    paged_attention_tiled_kernel<DS, TILED_ROW_TILES, TILED_STAGES, IN_PAGE><<<grid, 256, shared, stream>>>( \
        static_cast<const bf16_t*>(q), q_stride, static_cast<const bf16_t*>(cache), block_table,  \
        bt_stride, units, static_cast<bf16_t*>(out), out_stride, part_o, part_ml, heads,          \
        kv_heads, page_size, scale_log2e, window);                                                 \
  }
#define SE_ATT(DS)                                                                                 \
  case DS:                                                                                         \
    if (page_size % 32 == 0) SE_ATT_LAUNCH(DS, true) else SE_ATT_LAUNCH(DS, false)                 \
    break;
  switch (head_dim / 32) {
    SE_ATT(1) SE_ATT(2) SE_ATT(3) SE_ATT(4)
    default: return SE_ERR_SHAPE;
  }
#undef SE_ATT
#undef SE_ATT_LAUNCH
  SE_CHECK_LAUNCH();
  return SE_OK;
}
