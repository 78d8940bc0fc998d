// Mixture-of-experts support kernels for gfx950: router top-k, grouping of (token, slot)
// assignments by expert, a general tiled grouped GEMM (float and bfloat16, any sizes), the
// sum over a token's slots, and the SwiGLU product of a dense feed-forward.
//
// Router: score = sigmoid(logit) (or softmax over the experts); experts are chosen by
// score + bias, NaN counting as +inf, lowest index first among equal values; the output
// holds the chosen experts with a value strictly above the k-th one in index order, then the
// ties at the k-th value in index order.  Weights are the unbiased scores of the chosen
// experts, optionally divided by their sum, times a scaling factor.  All float.
#include "common.h"

#define ROUTER_MAX_PER_LANE 16  // experts <= 64 * 16

// One wavefront routes one token.
template <int PER_LANE>  // experts <= 64 * PER_LANE
__device__ __forceinline__ void route_token(const float* __restrict__ logits, int64_t stride,
                                            const float* __restrict__ bias, int32_t* __restrict__ ids,
                                            float* __restrict__ weights, int token, int experts,
                                            int top_k, int softmax_scoring, int normalize,
                                            float scaling, int32_t* ids_copy = nullptr) {
  const int lane = threadIdx.x & (SE_WAVE - 1);
  const float* row = logits + static_cast<int64_t>(token) * stride;

  float score[PER_LANE], sel[PER_LANE];
  float row_max = -INFINITY;
#pragma unroll
  for (int i = 0; i < PER_LANE; ++i) {
    const int e = i * SE_WAVE + lane;
    score[i] = e < experts ? row[e] : -INFINITY;
    row_max = fmaxf(row_max, score[i]);
  }
  if (softmax_scoring) {
    row_max = wave_max(row_max);
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) {
      const int e = i * SE_WAVE + lane;
      score[i] = e < experts ? expf(score[i] - row_max) : 0.f;
      part += score[i];
    }
    const float denom = wave_sum(part);
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) score[i] /= denom;
  } else {
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) score[i] = 1.f / (1.f + expf(-score[i]));
  }
  uint32_t taken = 0;     // bit i: element i of this lane is chosen
  uint32_t excluded = 0;  // bit i: element i does not exist
#pragma unroll
  for (int i = 0; i < PER_LANE; ++i) {
    const int e = i * SE_WAVE + lane;
    if (e < experts) {
      float s = score[i] + (bias ? bias[e] : 0.f);
      sel[i] = (s == s) ? s : INFINITY;
    } else {
      sel[i] = -INFINITY;
      excluded |= 1u << i;
    }
  }
  // k rounds of arg-max (largest value, lowest index among equals); the last value is the threshold.
  // A round is one reduction over the wave, the maximum of the values, and a few ballots for the lowest index
  // among the elements that hold it (a reduction over (value, index) pairs costs twice the instructions, a
  // second reduction for the index half as many again, and with few tokens this kernel is a lone
  // wavefront's chain of dependent instructions).
  float threshold = 0.f;
  for (int round = 0; round < top_k; ++round) {
    float best = -INFINITY;
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i)
      if (!((taken | excluded) & (1u << i)) && sel[i] > best) best = sel[i];
    const float top = wave_max(best);
    // the lowest index among the elements that hold it: the lowest element slot i that any lane holds it in
    // (index = 64 i + lane), then the lowest such lane; the lanes' answers are masks in scalar registers
    int winner = -1;
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) {
      const uint64_t holders = __ballot(!((taken | excluded) & (1u << i)) && sel[i] == top);
      if (winner < 0 && holders) winner = i * SE_WAVE + __builtin_ctzll(holders);
    }
    if ((winner & (SE_WAVE - 1)) == lane) taken |= 1u << (winner / SE_WAVE);
    threshold = top;
  }
  // output order: strictly greater than the threshold by index, then the chosen ties by index
  int greater_before = 0, ties_before = 0;
  int my_slot[PER_LANE];
  const uint64_t lower_lanes = (lane == 0) ? 0ull : (~0ull >> (SE_WAVE - lane));
#pragma unroll
  for (int i = 0; i < PER_LANE; ++i) {
    const bool chosen = taken & (1u << i);
    const bool greater = chosen && sel[i] > threshold;
    const bool tie = chosen && !greater;
    const uint64_t gmask = __ballot(greater);
    const uint64_t tmask = __ballot(tie);
    my_slot[i] = greater ? greater_before + __popcll(gmask & lower_lanes)
                         : -(1 + ties_before + __popcll(tmask & lower_lanes));
    greater_before += __popcll(gmask);
    ties_before += __popcll(tmask);
  }
  float part = 0.f;
#pragma unroll
  for (int i = 0; i < PER_LANE; ++i)
    if (taken & (1u << i)) part += score[i];
  const float total = wave_sum(part);
#pragma unroll
  for (int i = 0; i < PER_LANE; ++i) {
    if (!(taken & (1u << i))) continue;
    const int slot = my_slot[i] >= 0 ? my_slot[i] : greater_before + (-my_slot[i] - 1);
    ids[static_cast<int64_t>(token) * top_k + slot] = i * SE_WAVE + lane;
    if (ids_copy) ids_copy[token * top_k + slot] = i * SE_WAVE + lane;
    weights[static_cast<int64_t>(token) * top_k + slot] =
        (normalize ? score[i] / total : score[i]) * scaling;
  }
}

template <int PER_LANE>
__global__ void router_topk_kernel(const float* __restrict__ logits, int64_t stride,
                                   const float* __restrict__ bias, int32_t* __restrict__ ids,
                                   float* __restrict__ weights, int tokens, int experts, int top_k,
                                   int softmax_scoring, int normalize, float scaling) {
  const int token = blockIdx.x * (blockDim.x / SE_WAVE) + threadIdx.x / SE_WAVE;
  if (token >= tokens) return;  // whole waves leave together; there is no block barrier
  route_token<PER_LANE>(logits, stride, bias, ids, weights, token, experts, top_k, softmax_scoring,
                        normalize, scaling);
}

// ---------------------------------------------------------------------------------------- //
// Router logits of a step with few tokens: logits[t, e] = x[t] . w[e], float accumulate from
// float weights; the activations are widened as they are read (no float copy of x, no library
// call whose launch and set-up cost more than the product).  One wavefront per expert; a lane
// takes 8 consecutive k out of every 512 and keeps the sums of up to TG (1, 2, 4, 8) tokens.
// Requires K % 8 == 0 and 16-byte aligned rows.
// ---------------------------------------------------------------------------------------- //
template <typename T, int TG>   // TG tokens at a time share the weight loads
__global__ void __launch_bounds__(256)
router_logits_kernel(const T* __restrict__ x, int64_t x_stride, const float* __restrict__ w,
                     float* __restrict__ logits, int64_t out_stride, int tokens, int experts, int K) {
  const int lane = threadIdx.x & (SE_WAVE - 1);
  const int expert = blockIdx.x * 4 + threadIdx.x / SE_WAVE;
  if (expert >= experts) return;   // whole waves leave together; there is no block barrier below
  constexpr int XV = 8 / Vec16<T>::N;            // 16-byte vectors of 8 activations
  // steps of 512 along K whose loads go out together: with one token the product is a chain of
  // memory round trips otherwise (measured at 256 x 3072: 5.8 -> 4.7 us)
  constexpr int UNROLL = TG <= 2 ? 8 : (TG == 4 ? 6 : 3);
  const float* w_row = w + static_cast<int64_t>(expert) * K;
  for (int t0 = 0; t0 < tokens; t0 += TG) {
    float acc[TG];
#pragma unroll
    for (int g = 0; g < TG; ++g) acc[g] = 0.f;
#pragma unroll UNROLL
    for (int k = lane * 8; k < K; k += SE_WAVE * 8) {
      const float4 w0 = *reinterpret_cast<const float4*>(w_row + k);
      const float4 w1 = *reinterpret_cast<const float4*>(w_row + k + 4);
      Vec16<T> xv[TG][XV];
#pragma unroll
      for (int g = 0; g < TG; ++g) {
        const int t = min(t0 + g, tokens - 1);     // rows past the end repeat the last one
        const T* xr = x + static_cast<int64_t>(t) * x_stride + k;
#pragma unroll
        for (int v = 0; v < XV; ++v)
          xv[g][v].v = *reinterpret_cast<const decltype(xv[g][v].v)*>(xr + v * Vec16<T>::N);
      }
      const float wk[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
      for (int g = 0; g < TG; ++g)
#pragma unroll
        for (int j = 0; j < 8; ++j)
          acc[g] = fmaf(xv[g][j / Vec16<T>::N].get(j % Vec16<T>::N), wk[j], acc[g]);
    }
#pragma unroll
    for (int g = 0; g < TG; ++g) {
      const float total = wave_sum(acc[g]);
      if (lane == 0 && t0 + g < tokens) logits[static_cast<int64_t>(t0 + g) * out_stride + expert] = total;
    }
  }
}

// ---------------------------------------------------------------------------------------- //
// Group the A = tokens * top_k assignments by expert.  Every expert's run is padded to a
// multiple of `tile_rows`; padding entries hold A.  One block does the whole job.
//   sorted[capacity]      assignment ids in expert order (capacity >= A + experts*(tile_rows-1))
//   tile_expert[max_tiles] expert of each tile of `tile_rows` sorted entries
//   counters[0] = number of tiles, counters[1] = number of sorted entries
// The order of assignments inside one expert's run is not fixed; every row of a tile is
// computed independently of its neighbours, so results do not depend on it.
// ---------------------------------------------------------------------------------------- //
// The work of one block of 64 ... 1024 threads (a multiple of 64); sh holds 3 * experts + 1 ints.
// `other_rows` > 0: the tile height is chosen here, where the counts are known, between `tile_rows` (the kernel
// that streams an expert's table once per tile) and `other_rows` (the kernel that shares a table among many rows):
// with t tiles of `tile_rows` the former reads t tables; the latter reads one table per expert that got rows,
// or, when the rows are many, is bound by its arithmetic, which takes as long as reading a table per
// `heavy_rows` rows.  The former is chosen if t * percent / 100 is at most the larger of the two (percent: how
// much faster it reads).  counters[2] says which (0 / 1); the launch that follows holds both kernels' code.
__device__ __forceinline__ void align_assignments(const int32_t* __restrict__ ids, int assignments,
                                                  int experts, int tile_rows, int32_t* __restrict__ sorted,
                                                  int32_t* __restrict__ tile_expert,
                                                  int32_t* __restrict__ counters, int32_t* sh,
                                                  int other_rows = 0, int percent = 0, int heavy_rows = 1) {
  int32_t* counts = sh;                 // [experts]
  int32_t* offsets = sh + experts;      // [experts + 1] start of each run in `sorted`
  int32_t* cursor = offsets + experts + 1;  // [experts]
  for (int e = threadIdx.x; e < experts; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  // eight loads of a thread are asked for before the first is used: one by one, each costs a
  // round trip to memory (16384 assignments: 18.6 -> 12 us)
  for (int a0 = threadIdx.x; a0 < assignments; a0 += 8 * blockDim.x) {
    int32_t e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int a = a0 + j * blockDim.x;
      e[j] = a < assignments ? ids[a] : -1;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (e[j] >= 0) atomicAdd(&counts[e[j]], 1);
  }
  __syncthreads();
  if (other_rows > 0) {
    __shared__ int32_t touched, tiles;
    if (threadIdx.x == 0) touched = tiles = 0;
    __syncthreads();
    int32_t mine = 0, my_tiles = 0;
    for (int e = threadIdx.x; e < experts; e += blockDim.x) {
      mine += counts[e] > 0;
      my_tiles += (counts[e] + tile_rows - 1) / tile_rows;
    }
    if (mine) {
      atomicAdd(&touched, mine);
      atomicAdd(&tiles, my_tiles);
    }
    __syncthreads();
    const int64_t tables = max(touched, assignments / heavy_rows);
    const bool few = static_cast<int64_t>(tiles) * percent <= 100 * tables;
    if (!few) tile_rows = other_rows;
    if (threadIdx.x == 0) counters[2] = few ? 0 : 1;
  }
  // exclusive prefix sum of the padded counts: every thread scans its own stretch of experts,
  // wave 0 scans the stretch totals
  {
    const int per_thread = (experts + blockDim.x - 1) / blockDim.x;
    const int first = threadIdx.x * per_thread;
    int32_t mine = 0;
    for (int e = first; e < first + per_thread && e < experts; ++e)
      mine += (counts[e] + tile_rows - 1) / tile_rows * tile_rows;
    __shared__ int32_t stretch[1024];
    stretch[threadIdx.x] = mine;
    __syncthreads();
    if (threadIdx.x < SE_WAVE) {
      // blockDim / 64 consecutive stretch totals per lane
      const int per_lane = blockDim.x / SE_WAVE;
      int32_t lane_total = 0;
      for (int i = 0; i < per_lane; ++i) lane_total += stretch[threadIdx.x * per_lane + i];
      int32_t inclusive = lane_total;
#pragma unroll
      for (int off = 1; off < SE_WAVE; off <<= 1) {
        const int32_t up = __shfl_up(inclusive, off, SE_WAVE);
        if (static_cast<int>(threadIdx.x) >= off) inclusive += up;
      }
      int32_t run = inclusive - lane_total;
      for (int i = 0; i < per_lane; ++i) {
        const int32_t v = stretch[threadIdx.x * per_lane + i];
        stretch[threadIdx.x * per_lane + i] = run;
        run += v;
      }
      if (threadIdx.x == SE_WAVE - 1) {
        offsets[experts] = run;
        counters[0] = run / tile_rows;
        counters[1] = run;
      }
    }
    __syncthreads();
    int32_t run = stretch[threadIdx.x];
    for (int e = first; e < first + per_thread && e < experts; ++e) {
      offsets[e] = run;
      run += (counts[e] + tile_rows - 1) / tile_rows * tile_rows;
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < experts; e += blockDim.x) cursor[e] = offsets[e];
  // Padding entries and the tiles' experts.  Large tiles, many wavefronts: a wavefront per run, its
  // lanes side by side (a thread per run would write up to tile_rows - 1 padding entries in a row:
  // 18 us for 64 tokens on tiles of 128).  Small tiles or a narrow block (the router's own launch
  // for a few tokens): a thread per run, since most runs are empty and a run has few entries.
  if (tile_rows > 32 && blockDim.x >= 4 * SE_WAVE) {
    const int lane = threadIdx.x & (SE_WAVE - 1);
    const int waves = blockDim.x / SE_WAVE;
    for (int e = threadIdx.x / SE_WAVE; e < experts; e += waves) {
      const int begin = offsets[e], end = offsets[e + 1];
      for (int p = begin + counts[e] + lane; p < end; p += SE_WAVE) sorted[p] = assignments;
      for (int t = begin / tile_rows + lane; t < end / tile_rows; t += SE_WAVE) tile_expert[t] = e;
    }
  } else {
    for (int e = threadIdx.x; e < experts; e += blockDim.x) {
      for (int p = offsets[e] + counts[e]; p < offsets[e + 1]; ++p) sorted[p] = assignments;
      for (int t = offsets[e] / tile_rows; t < offsets[e + 1] / tile_rows; ++t) tile_expert[t] = e;
    }
  }
  __syncthreads();
  for (int a0 = threadIdx.x; a0 < assignments; a0 += 8 * blockDim.x) {
    int32_t e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int a = a0 + j * blockDim.x;
      e[j] = a < assignments ? ids[a] : -1;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (e[j] >= 0) sorted[atomicAdd(&cursor[e[j]], 1)] = a0 + j * blockDim.x;
  }
}

__global__ void moe_align_kernel(const int32_t* __restrict__ ids, int assignments, int experts,
                                 int tile_rows, int32_t* __restrict__ sorted,
                                 int32_t* __restrict__ tile_expert, int32_t* __restrict__ counters,
                                 int other_rows, int percent, int heavy_rows) {
  extern __shared__ int32_t sh[];
  align_assignments(ids, assignments, experts, tile_rows, sorted, tile_expert, counters, sh, other_rows, percent,
                    heavy_rows);
}

// A step with few tokens (at most 16): one block routes them, a wavefront each, and then groups
// the assignments, which saves a launch where launches are most of the time.
template <int PER_LANE>
__global__ void router_topk_align_kernel(const float* __restrict__ logits, int64_t stride,
                                         const float* __restrict__ bias, int32_t* __restrict__ ids,
                                         float* __restrict__ weights, int tokens, int experts,
                                         int top_k, int softmax_scoring, int normalize, float scaling,
                                         int tile_rows, int32_t* __restrict__ sorted,
                                         int32_t* __restrict__ tile_expert,
                                         int32_t* __restrict__ counters) {
  extern __shared__ int32_t sh[];
  // the chosen experts also stay in shared memory: grouping them from there saves the round trip
  // of writing them to memory and reading them back (about 1.5 us of a 9 us launch)
  int32_t* chosen = sh + 3 * experts + 1;   // [tokens * top_k]
  route_token<PER_LANE>(logits, stride, bias, ids, weights, threadIdx.x / SE_WAVE, experts, top_k,
                        softmax_scoring, normalize, scaling, chosen);
  __syncthreads();
  if (tokens == 1 && top_k <= SE_WAVE) {
    // One token: its experts are all different, every run is one row.  Tile t belongs to the t-th smallest of
    // them (the order the general grouping gives); nothing has to be counted or scanned.
    const int lane = threadIdx.x;
    if (lane < top_k) {
      const int mine = chosen[lane];
      int tile = 0;
      for (int j = 0; j < top_k; ++j) tile += chosen[j] < mine;
      tile_expert[tile] = mine;
      sorted[tile * tile_rows] = lane;
      for (int r = 1; r < tile_rows; ++r) sorted[tile * tile_rows + r] = top_k;     // padding
    }
    if (lane == 0) {
      counters[0] = top_k;
      counters[1] = top_k * tile_rows;
    }
    return;
  }
  align_assignments(chosen, tokens * top_k, experts, tile_rows, sorted, tile_expert, counters, sh);
}

// ---------------------------------------------------------------------------------------- //
// General grouped GEMM over the sorted assignments, float accumulation, any sizes.
// A tile is GM = 16 sorted rows; a block computes GN = 64 output columns of it.
//   MODE 0 (gate-up + SwiGLU): in row = x[a / top_k, :K]; w = w13[e] of shape [2N, K];
//       out[a, n] = silu(g) * u with g = in . w[n], u = in . w[N + n]; g and u are rounded to
//       the storage type, silu is taken in float and rounded, the product is rounded.
//   MODE 1 (down): in row = act[a, :K]; w = w2[e] of shape [N, K];
//       out[a, n] = (in . w[n]) * route_weight[a]   (weight applied to the float accumulator)
// ---------------------------------------------------------------------------------------- //
#define GG_M 16
#define GG_N 64
#define GG_K 32

template <typename T, int MODE>
__global__ void grouped_gemm_generic_kernel(const T* __restrict__ in, const T* __restrict__ w,
                                            T* __restrict__ out,
                                            const int32_t* __restrict__ sorted,
                                            const int32_t* __restrict__ tile_expert,
                                            const int32_t* __restrict__ counters,
                                            const float* __restrict__ route_weight, int assignments,
                                            int top_k, int N, int K, int activation) {
  const int tile = blockIdx.y;
  if (tile >= counters[0]) return;  // uniform over the block
  __shared__ float xs[GG_M][GG_K + 1];
  __shared__ float wg[GG_N][GG_K + 1];
  __shared__ float wu[MODE == 0 ? GG_N : 1][GG_K + 1];
  __shared__ int32_t rows[GG_M];
  const int expert = tile_expert[tile];
  const int n0 = blockIdx.x * GG_N;
  if (threadIdx.x < GG_M) rows[threadIdx.x] = sorted[tile * GG_M + threadIdx.x];
  __syncthreads();
  const int64_t w_rows = MODE == 0 ? 2 * static_cast<int64_t>(N) : N;
  const T* we = w + static_cast<int64_t>(expert) * w_rows * K;
  const int r = threadIdx.x / 16;          // row of the tile
  const int cg = threadIdx.x % 16;         // column group: columns cg, cg+16, cg+32, cg+48
  float g[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += GG_K) {
    for (int idx = threadIdx.x; idx < GG_M * GG_K; idx += blockDim.x) {
      const int rr = idx / GG_K, kk = idx % GG_K;
      const int a = rows[rr];
      float v = 0.f;
      if (a < assignments && k0 + kk < K) {
        const int64_t src = MODE == 0 ? a / top_k : a;
        v = to_float(in[src * K + k0 + kk]);
      }
      xs[rr][kk] = v;
    }
    for (int idx = threadIdx.x; idx < GG_N * GG_K; idx += blockDim.x) {
      const int nn = idx / GG_K, kk = idx % GG_K;
      const bool ok = n0 + nn < N && k0 + kk < K;
      wg[nn][kk] = ok ? to_float(we[static_cast<int64_t>(n0 + nn) * K + k0 + kk]) : 0.f;
      if (MODE == 0)
        wu[nn][kk] = ok ? to_float(we[static_cast<int64_t>(N + n0 + nn) * K + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < GG_K; ++kk) {
      const float xv = xs[r][kk];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        g[j] += xv * wg[cg + 16 * j][kk];
        if (MODE == 0) u[j] += xv * wu[cg + 16 * j][kk];
      }
    }
    __syncthreads();
  }
  const int a = rows[r];
  if (a >= assignments) return;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + cg + 16 * j;
    if (n >= N) continue;
    float y;
    if (MODE == 0) {
      const float gate = round_to<T>(g[j]);
      const float up = round_to<T>(u[j]);
      const float act = round_to<T>(gate_activation<false>(gate, activation));
      y = act * up;
    } else {
      y = g[j] * route_weight[a];
    }
    out[static_cast<int64_t>(a) * N + n] = from_float<T>(y);
  }
}

// out[t, c] = sum over the token's top_k slots of y[t * top_k + k, c], float accumulation in slot
// order; one thread per output element (grid: tokens x column blocks)
template <typename T>
__global__ void moe_sum_kernel(const T* __restrict__ y, T* __restrict__ out, int top_k,
                               int hidden) {
  const int64_t t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= hidden) return;
  float acc = 0.f;
#pragma unroll 8
  for (int k = 0; k < top_k; ++k) acc += to_float(y[(t * top_k + k) * hidden + c]);
  out[t * hidden + c] = from_float<T>(acc);
}

// The same with 16-byte vectors (hidden a multiple of the vector length, 16-byte aligned rows): a
// thread owns one vector of the output row and asks for up to eight slots' vectors at once.
template <typename T>
__global__ void __launch_bounds__(256)
moe_sum_vec_kernel(const T* __restrict__ y, T* __restrict__ out, int top_k, int hidden) {
  constexpr int VN = Vec16<T>::N;
  typedef decltype(Vec16<T>().v) raw_t;
  const int64_t t = blockIdx.x;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * VN;
  if (c >= hidden) return;
  float acc[VN];
#pragma unroll
  for (int j = 0; j < VN; ++j) acc[j] = 0.f;
  for (int k0 = 0; k0 < top_k; k0 += 8) {
    Vec16<T> v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (k0 + i < top_k) v[i].v = *reinterpret_cast<const raw_t*>(y + (t * top_k + k0 + i) * hidden + c);
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (k0 + i < top_k) {   // slot order, as in the scalar kernel
#pragma unroll
        for (int j = 0; j < VN; ++j) acc[j] += v[i].get(j);
      }
  }
  Vec16<T> o;
#pragma unroll
  for (int j = 0; j < VN; ++j) o.set(j, acc[j]);
  *reinterpret_cast<raw_t*>(out + t * hidden + c) = o.v;
}

// out[t, c] = act(x[t, c]) * x[t, width + c] (act: silu or gelu) with the roundings of the fused expert path
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ x, T* __restrict__ out, int width, int activation) {
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float gate = to_float(x[t * 2 * width + c]);
    const float up = to_float(x[t * 2 * width + width + c]);
    const float act = round_to<T>(gate_activation<false>(gate, activation));
    out[t * width + c] = from_float<T>(act * up);
  }
}

extern "C" {

int se_router_topk(const float* logits, int64_t stride, const float* bias, int32_t* ids,
                   float* weights, int tokens, int experts, int top_k, int softmax_scoring,
                   int normalize, float scaling, hipStream_t stream) {
  if (tokens <= 0) return SE_OK;
  if (experts <= 0 || experts > SE_WAVE * ROUTER_MAX_PER_LANE) return SE_ERR_SHAPE;
  if (top_k <= 0 || top_k > experts) return SE_ERR_SHAPE;
  const int waves = 4;
  const dim3 grid((tokens + waves - 1) / waves);
  if (experts <= SE_WAVE * 4) {
    router_topk_kernel<4><<<grid, waves * SE_WAVE, 0, stream>>>(
        logits, stride, bias, ids, weights, tokens, experts, top_k, softmax_scoring, normalize, scaling);
  } else {
    router_topk_kernel<ROUTER_MAX_PER_LANE><<<grid, waves * SE_WAVE, 0, stream>>>(
        logits, stride, bias, ids, weights, tokens, experts, top_k, softmax_scoring, normalize, scaling);
  }
  SE_CHECK_LAUNCH();
  return SE_OK;
}

// logits[tokens, experts] (float) = x[tokens, K] (dtype) . w[experts, K]^T (float), for few tokens
int se_router_logits(const void* x, int64_t x_stride, const float* w, float* logits,
                     int64_t out_stride, int tokens, int experts, int K, int dtype,
                     hipStream_t stream) {
  if (tokens <= 0) return SE_OK;
  if (experts <= 0 || K <= 0 || K % 8 || x_stride % 8) return SE_ERR_SHAPE;
  const dim3 grid((experts + 3) / 4);
#define SE_RL(T, TG)                                                                              \
  router_logits_kernel<T, TG><<<grid, 256, 0, stream>>>(static_cast<const T*>(x), x_stride, w, logits, \
                                                        out_stride, tokens, experts, K)
#define SE_RL_TG(T)                                                                               \
  if (tokens <= 1) SE_RL(T, 1);                                                                   \
  else if (tokens <= 2) SE_RL(T, 2);                                                              \
  else if (tokens <= 4) SE_RL(T, 4);                                                              \
  else SE_RL(T, 8)
  if (dtype == SE_F32) { SE_RL_TG(float); } else { SE_RL_TG(bf16_t); }
#undef SE_RL_TG
#undef SE_RL
  SE_CHECK_LAUNCH();
  return SE_OK;
}

// router_topk for at most 16 tokens followed by moe_align, in one launch
int se_router_topk_align(const float* logits, int64_t stride, const float* bias, int32_t* ids,
                         float* weights, int tokens, int experts, int top_k, int softmax_scoring,
                         int normalize, float scaling, int tile_rows, int32_t* sorted,
                         int32_t* tile_expert, int32_t* counters, hipStream_t stream) {
  if (tokens <= 0) return SE_OK;
  if (tokens > 16 || experts <= 0 || experts > SE_WAVE * ROUTER_MAX_PER_LANE) return SE_ERR_SHAPE;
  if (top_k <= 0 || top_k > experts || tile_rows <= 0) return SE_ERR_SHAPE;
  const size_t shmem = (3 * static_cast<size_t>(experts) + 1 + static_cast<size_t>(tokens) * top_k) * sizeof(int32_t);
  if (shmem > 64 * 1024) return SE_ERR_SHAPE;
  if (experts <= SE_WAVE * 4) {
    router_topk_align_kernel<4><<<1, tokens * SE_WAVE, shmem, stream>>>(
        logits, stride, bias, ids, weights, tokens, experts, top_k, softmax_scoring, normalize, scaling,
        tile_rows, sorted, tile_expert, counters);
  } else {
    router_topk_align_kernel<ROUTER_MAX_PER_LANE><<<1, tokens * SE_WAVE, shmem, stream>>>(
        logits, stride, bias, ids, weights, tokens, experts, top_k, softmax_scoring, normalize, scaling,
        tile_rows, sorted, tile_expert, counters);
  }
  SE_CHECK_LAUNCH();
  return SE_OK;
}

int se_moe_align(const int32_t* ids, int assignments, int experts, int tile_rows, int32_t* sorted,
                 int32_t* tile_expert, int32_t* counters, hipStream_t stream) {
  if (assignments <= 0) return SE_OK;
  if (experts <= 0 || experts > 4096 || tile_rows <= 0) return SE_ERR_SHAPE;
  const size_t shmem = (3 * static_cast<size_t>(experts) + 1) * sizeof(int32_t);
  moe_align_kernel<<<1, 1024, shmem, stream>>>(ids, assignments, experts, tile_rows, sorted,
                                               tile_expert, counters, 0, 0, 1);
  SE_CHECK_LAUNCH();
  return SE_OK;
}

// The same with the tile height chosen on the device, where the counts are (see align_assignments): tiles of
// `few_tile_rows` or of `many_tile_rows`; counters[2] = 0 / 1.  (The host knows how many tokens a step has, not
// how they spread over the experts: a prompt whose tokens agree on a few dozen experts and one that uses them all
// want different kernels.)
int se_moe_align_choice(const int32_t* ids, int assignments, int experts, int few_tile_rows, int many_tile_rows,
                        int percent, int heavy_rows, int32_t* sorted, int32_t* tile_expert, int32_t* counters,
                        hipStream_t stream) {
  if (assignments <= 0) return SE_OK;
  if (experts <= 0 || experts > 4096 || few_tile_rows <= 0 || many_tile_rows <= 0 || percent <= 0 || heavy_rows <= 0)
    return SE_ERR_SHAPE;
  const size_t shmem = (3 * static_cast<size_t>(experts) + 1) * sizeof(int32_t);
  moe_align_kernel<<<1, 1024, shmem, stream>>>(ids, assignments, experts, few_tile_rows, sorted,
                                               tile_expert, counters, many_tile_rows, percent, heavy_rows);
  SE_CHECK_LAUNCH();
  return SE_OK;
}

// mode 0: gate-up + SwiGLU (w = [experts, 2N, K]); mode 1: down (w = [experts, N, K]).
// max_tiles bounds the grid; tiles beyond counters[0] leave at once.
int se_grouped_gemm_generic(const void* in, const void* w, void* out, const int32_t* sorted,
                            const int32_t* tile_expert, const int32_t* counters,
                            const float* route_weight, int assignments, int top_k, int N, int K,
                            int max_tiles, int mode, int dtype, int activation, hipStream_t stream) {
  if (assignments <= 0) return SE_OK;
  if (N <= 0 || K <= 0 || max_tiles <= 0 || max_tiles > 65535) return SE_ERR_SHAPE;
  if (activation != SE_ACT_SILU && activation != SE_ACT_GELU_TANH) return SE_ERR_SHAPE;
  dim3 grid((N + GG_N - 1) / GG_N, max_tiles);
#define SE_GG(T, MODE)                                                                          \
  grouped_gemm_generic_kernel<T, MODE><<<grid, 256, 0, stream>>>(                               \
      static_cast<const T*>(in), static_cast<const T*>(w), static_cast<T*>(out), sorted,        \
      tile_expert, counters, route_weight, assignments, top_k, N, K, activation)
  if (dtype == SE_F32) {
    if (mode == 0) SE_GG(float, 0); else SE_GG(float, 1);
  } else {
    if (mode == 0) SE_GG(bf16_t, 0); else SE_GG(bf16_t, 1);
  }
#undef SE_GG
  SE_CHECK_LAUNCH();
  return SE_OK;
}

int se_moe_sum(const void* y, void* out, int tokens, int top_k, int hidden, int dtype,
               hipStream_t stream) {
  if (tokens <= 0) return SE_OK;
  if (hidden <= 0) return SE_ERR_SHAPE;
  const int vn = dtype == SE_F32 ? 4 : 8;
  const bool aligned = (reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(out)) % 16 == 0;
  if (hidden % vn == 0 && aligned) {
    dim3 vgrid(tokens, (hidden / vn + 255) / 256);
    if (dtype == SE_F32)
      moe_sum_vec_kernel<float><<<vgrid, 256, 0, stream>>>(static_cast<const float*>(y),
                                                           static_cast<float*>(out), top_k, hidden);
    else
      moe_sum_vec_kernel<bf16_t><<<vgrid, 256, 0, stream>>>(static_cast<const bf16_t*>(y),
                                                            static_cast<bf16_t*>(out), top_k, hidden);
    SE_CHECK_LAUNCH();
    return SE_OK;
  }
  dim3 grid(tokens, (hidden + 255) / 256);
  if (dtype == SE_F32)
    moe_sum_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(y),
                                                    static_cast<float*>(out), top_k, hidden);
  else
    moe_sum_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<const bf16_t*>(y),
                                                     static_cast<bf16_t*>(out), top_k, hidden);
  SE_CHECK_LAUNCH();
  return SE_OK;
}

int se_silu_mul(const void* x, void* out, int tokens, int width, int dtype, int activation, hipStream_t stream) {
  if (tokens <= 0) return SE_OK;
  if (activation != SE_ACT_SILU && activation != SE_ACT_GELU_TANH) return SE_ERR_SHAPE;
  if (dtype == SE_F32)
    silu_mul_kernel<float><<<tokens, 256, 0, stream>>>(static_cast<const float*>(x),
                                                       static_cast<float*>(out), width, activation);
  else
    silu_mul_kernel<bf16_t><<<tokens, 256, 0, stream>>>(static_cast<const bf16_t*>(x),
                                                        static_cast<bf16_t*>(out), width, activation);
  SE_CHECK_LAUNCH();
  return SE_OK;
}

}  // extern "C"
