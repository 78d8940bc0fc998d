// Grouped expert GEMMs on the matrix cores (bfloat16 in, float accumulate) for gfx950.
//
// Work is a list of tiles of BM = 16 * MB sorted assignments that share one expert (see
// moe_align in moe.hip).  A workgroup of four wavefronts computes BN = 16 * NB output columns of
// one tile; the wavefronts split the reduction dimension K into equal parts (quarters, or more
// for the dense products of a step with few rows, which have few blocks), each streaming
// its part of the expert's weight rows straight from memory into MFMA operands
// (v_mfma_f32_16x16x32_bf16: weights are the A operand, the tile's activation rows the B
// operand), and the partial tiles are summed through LDS before the epilogue.
//
//   MODE 0 (gate-up + SwiGLU): in row = x[a / top_k]; w = w13[e] = [gate rows; up rows], [2N, K];
//       out[a, n] = silu(g) * u; g and u are rounded to bfloat16, silu is taken in float and
//       rounded, the product is rounded.
//   MODE 1 (down): in row = act[a]; w = w2[e], [N, K]; out[a, n] = (in . w[n]) * route_weight[a].
//   MODE 2 (dense, few rows): out[t, n] = x[t] . w[n] for one weight matrix [N, K]; tile t holds rows
//       16 * MB * t ...; the same streaming loop serves the skinny projections of decode steps.
//   MODE 3: MODE 2 with the weight matrix in tiles, as the expert tables are (below).
//
// Expert tables (MODE 0 and 1, in all three kernels of this file) lie in tiles: tile
// (n / 16, k / 32) of an expert is 512 consecutive elements in the order [(k % 32) / 8][n % 16][k % 8],
// which is the order of the lanes that hold the tile as an A operand, so a wavefront's load of a
// tile is one contiguous kilobyte (kernels/hip_ops.py: tile_expert_weights puts a table into this
// order).  Dense tables lie in rows (MODE 2), as the BLAS library reads them, or in a tiled copy made
// for steps of few rows (MODE 3): a wavefront's load of 16 rows x 32 k of a table in rows is 64 bytes
// from each of 16 rows, which arrive at a third of the rate of one contiguous kilobyte, and a block of
// an output projection (16 rows x 6144) then takes 6 us for its loads alone; tiled loads also take the
// read-once hint, which on half cache lines fetches every line twice.
//
// Every output element is one dot product in a fixed order of K, so a row's result does not
// depend on its place in the tile or on what else is in the batch.
// Requires K % 128 == 0 and N % BN == 0; other sizes take the general kernel in moe.hip.
#include "common.h"
#include <type_traits>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Work item (tile, column block) of a block in a 1-D grid.  Consecutive block ids go to
// different XCDs (id % 8), and every XCD has an L2 of its own: so each XCD gets one contiguous
// stretch of the work, and the column blocks of a tile - which all read the tile's activation
// rows - and the tiles of one expert - which read the same weights - meet in one L2.
__device__ __forceinline__ bool xcd_work_item(int column_blocks, int num_tiles, int& tile, int& column_block) {
  const int total = num_tiles * column_blocks;
  const int per_xcd = (total + 7) >> 3;
  const int xcd = blockIdx.x & 7, index = blockIdx.x >> 3;
  if (index >= per_xcd) return false;
  const int item = xcd * per_xcd + index;
  if (item >= total) return false;
  tile = item / column_blocks;
  column_block = item % column_blocks;
  return true;
}

// A lane's 16 bytes of a weight tile: tiled tables are read once, in whole cache lines (load16_once);
// a table in rows gives a lane half a cache line, whose other half the next step reads.
template <bool TILED>
__device__ __forceinline__ uint4 load_weights(const bf16_t* p) {
  if constexpr (TILED) return load16_once(p);
  return *reinterpret_cast<const uint4*>(p);
}

template <int MODE, int MB, int NB, int U, int KW = 4>   // KW wavefronts split K
__global__ void __launch_bounds__(64 * KW)
grouped_gemm_mfma_kernel(const bf16_t* __restrict__ in, const bf16_t* __restrict__ w,
                         bf16_t* __restrict__ out, const int32_t* __restrict__ sorted,
                         const int32_t* __restrict__ tile_expert,
                         const int32_t* __restrict__ counters,
                         const float* __restrict__ route_weight, int assignments, int top_k, int N,
                         int K, int max_tiles, int activation) {
  constexpr int BM = 16 * MB;
  constexpr int BN = 16 * NB;
  constexpr int NBT = MODE == 0 ? 2 * NB : NB;  // weight blocks per wave: gate blocks, then up blocks
  int tile, column_block;
  constexpr bool DENSE = MODE >= 2;
  if (!xcd_work_item(N / BN, DENSE ? max_tiles : counters[0], tile, column_block)) return;  // uniform

  constexpr bool TILED = MODE != 2;
  constexpr int KSCALE = TILED ? 16 : 1;       // a step of 32 along k is 512 elements further in a tiled table
  constexpr int P = NB * MB;                   // output blocks of 16 x 16 (gate/up pairs in MODE 0)
  constexpr int PARTS = MODE == 0 ? 2 : 1;
  // block p is finished by wave p % KW; the other waves leave their partial sums here
  __shared__ floatx4 partial[P][KW - 1][PARTS][SE_WAVE];
  __shared__ int32_t rows[BM];

  const int lane = threadIdx.x & (SE_WAVE - 1);
  const int wave = threadIdx.x / SE_WAVE;
  const int expert = DENSE ? 0 : tile_expert[tile];
  const int n0 = column_block * BN;
  if (threadIdx.x < BM)
    rows[threadIdx.x] = DENSE ? tile * BM + static_cast<int>(threadIdx.x) : sorted[tile * BM + threadIdx.x];
  __syncthreads();

  const int col = lane & 15;   // row of the weight block (A) / row of the activation block (B)
  const int kgroup = lane >> 4;  // which 8 of the 32 k of a step this lane holds
  const int64_t w_rows = MODE == 0 ? 2 * static_cast<int64_t>(N) : N;
  const bf16_t* we = w + static_cast<int64_t>(expert) * w_rows * K;

  const bf16_t* a_ptr[NBT];
#pragma unroll
  for (int nb = 0; nb < NBT; ++nb) {
    const int block_row = (MODE == 0 && nb >= NB) ? N + n0 + (nb - NB) * 16 : n0 + nb * 16;
    // expert tables lie in tiles of 16 rows x 32 k, each 1 KB in the order of the lanes that hold it
    // as an operand (tile_expert_weights in kernels/hip_ops.py); dense tables lie in rows
    a_ptr[nb] = TILED ? we + static_cast<int64_t>(block_row / 16) * (K / 32) * 512 + lane * 8
                      : we + static_cast<int64_t>(block_row + col) * K + kgroup * 8;
  }
  const bf16_t* b_ptr[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int a = rows[mb * 16 + col];
    const int64_t src = a < assignments ? (MODE == 0 ? a / top_k : a) : 0;  // padding reads row 0
    b_ptr[mb] = in + src * K + kgroup * 8;
  }

  floatx4 acc[NBT][MB];
#pragma unroll
  for (int nb = 0; nb < NBT; ++nb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[nb][mb] = floatx4{0.f, 0.f, 0.f, 0.f};

  // A stage is U steps of 32 along K.  Two register sets take turns: while the matrix cores work
  // on one stage the loads of the next are already under way (the loop is memory-latency bound
  // otherwise: one round trip per stage and wave).
  const int k_begin = wave * (K / KW);
  const int k_end = k_begin + K / KW;
  if constexpr (U == 0) {
    // tall tiles: registers go to accumulators; one step at a time, the compiler overlaps what it can
#pragma unroll 2
    for (int k = k_begin; k < k_end; k += 32) {
      uint4 af[NBT], bf[MB];
#pragma unroll
      for (int nb = 0; nb < NBT; ++nb) af[nb] = load_weights<TILED>(a_ptr[nb] + static_cast<int64_t>(k) * KSCALE);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) bf[mb] = *reinterpret_cast<const uint4*>(b_ptr[mb] + k);
#pragma unroll
      for (int nb = 0; nb < NBT; ++nb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          acc[nb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              __builtin_bit_cast(bf16x8, af[nb]), __builtin_bit_cast(bf16x8, bf[mb]), acc[nb][mb], 0, 0, 0);
    }
  } else {
  constexpr int STAGE = 32 * (U == 0 ? 1 : U);
  constexpr int UU = U == 0 ? 1 : U;
  uint4 a0[UU][NBT], b0[UU][MB], a1[UU][NBT], b1[UU][MB];
  auto load_stage = [&](uint4 (&af)[UU][NBT], uint4 (&bf)[UU][MB], int k) {
#pragma unroll
    for (int u = 0; u < UU; ++u) {
#pragma unroll
      for (int nb = 0; nb < NBT; ++nb)
        af[u][nb] = load_weights<TILED>(a_ptr[nb] + static_cast<int64_t>(k + 32 * u) * KSCALE);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) bf[u][mb] = *reinterpret_cast<const uint4*>(b_ptr[mb] + k + 32 * u);
    }
  };
  auto run_stage = [&](const uint4 (&af)[UU][NBT], const uint4 (&bf)[UU][MB]) {
#pragma unroll
    for (int u = 0; u < UU; ++u)
#pragma unroll
      for (int nb = 0; nb < NBT; ++nb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          acc[nb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              __builtin_bit_cast(bf16x8, af[u][nb]), __builtin_bit_cast(bf16x8, bf[u][mb]), acc[nb][mb], 0, 0, 0);
  };
  load_stage(a0, b0, k_begin);
  for (int k = k_begin; k < k_end; k += 2 * STAGE) {
    const bool more1 = k + STAGE < k_end;
    if (more1) load_stage(a1, b1, k + STAGE);
    run_stage(a0, b0);
    if (!more1) break;
    if (k + 2 * STAGE < k_end) load_stage(a0, b0, k + 2 * STAGE);
    run_stage(a1, b1);
  }
  }

  // lane (kgroup, col) holds, for i < 4, the sum for weight row 4 * kgroup + i and activation row col
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int p = nb * MB + mb;
      const int owner = p % KW;
      if (wave != owner) {
        const int slot = ((wave - owner + KW) % KW) - 1;
#pragma unroll
        for (int part = 0; part < PARTS; ++part) partial[p][slot][part][lane] = acc[part * NB + nb][mb];
      }
    }
  __syncthreads();

#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int p = nb * MB + mb;
      if ((p % KW) != wave) continue;
      floatx4 total[PARTS];
#pragma unroll
      for (int part = 0; part < PARTS; ++part) {
        total[part] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KW; ++s) {  // the parts of K are always added in the same order
          if (s == wave)
            total[part] += acc[part * NB + nb][mb];
          else
            total[part] += partial[p][((s - wave + KW) % KW) - 1][part][lane];
        }
      }
      const int a = rows[mb * 16 + col];
      if (a >= assignments) continue;
      uint16_t y[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v;
        if (MODE == 0) {
          const float gate = round_to<bf16_t>(total[0][i]);
          const float up = round_to<bf16_t>(total[PARTS - 1][i]);
          const float act = round_to<bf16_t>(gate_activation<true>(gate, activation));
          v = act * up;
        } else if (MODE == 1) {
          v = total[0][i] * route_weight[a];
        } else {
          v = total[0][i];
        }
        y[i] = float_to_bf16_bits(v);
      }
      uint2 packed;
      packed.x = static_cast<uint32_t>(y[0]) | (static_cast<uint32_t>(y[1]) << 16);
      packed.y = static_cast<uint32_t>(y[2]) | (static_cast<uint32_t>(y[3]) << 16);
      *reinterpret_cast<uint2*>(out + static_cast<int64_t>(a) * N + n0 + nb * 16 + 4 * kgroup) = packed;
    }
}

template <int MODE, int MB, int NB, int U>
static void launch_u(const void* in, const void* w, void* out, const int32_t* sorted,
                   const int32_t* tile_expert, const int32_t* counters, const float* route_weight,
                   int assignments, int top_k, int N, int K, int max_tiles, int activation, hipStream_t stream) {
  const int64_t items = static_cast<int64_t>(N / (16 * NB)) * max_tiles;
  const int grid = static_cast<int>((items + 7) / 8 * 8);
  grouped_gemm_mfma_kernel<MODE, MB, NB, U><<<grid, 256, 0, stream>>>(
      static_cast<const bf16_t*>(in), static_cast<const bf16_t*>(w), static_cast<bf16_t*>(out), sorted,
      tile_expert, counters, route_weight, assignments, top_k, N, K, max_tiles, activation);
}

// steps of 32 per stage: as many as divide a wave's quarter of K, fewer for taller tiles (registers)
template <int MODE, int MB, int NB>
static void launch(const void* in, const void* w, void* out, const int32_t* sorted,
                   const int32_t* tile_expert, const int32_t* counters, const float* route_weight,
                   int assignments, int top_k, int N, int K, int max_tiles, int activation, hipStream_t stream) {
  constexpr int UMAX = MB == 1 ? 4 : (MB == 2 ? 2 : 0);
  const int quarter = K / 4;
  if (UMAX == 0) {
    launch_u<MODE, MB, NB, 0>(in, w, out, sorted, tile_expert, counters, route_weight, assignments, top_k,
                              N, K, max_tiles, activation, stream);
    return;
  }
  if (UMAX >= 4 && quarter % 128 == 0)
    launch_u<MODE, MB, NB, UMAX >= 4 ? 4 : 1>(in, w, out, sorted, tile_expert, counters, route_weight,
                                              assignments, top_k, N, K, max_tiles, activation, stream);
  else if (UMAX >= 2 && quarter % 64 == 0)
    launch_u<MODE, MB, NB, UMAX >= 2 ? 2 : 1>(in, w, out, sorted, tile_expert, counters, route_weight,
                                              assignments, top_k, N, K, max_tiles, activation, stream);
  else
    launch_u<MODE, MB, NB, 1>(in, w, out, sorted, tile_expert, counters, route_weight, assignments,
                              top_k, N, K, max_tiles, activation, stream);
}

// ---------------------------------------------------------------------------------------- //
// Tall tiles (an expert has dozens of rows, as in the prefill of a long prompt): the weights of a
// tile are used by many rows, so they are staged through LDS and shared by the block's four
// waves.  A block computes BM = 16 * MB rows x 128 weight rows (MODE 0: 64 gate + 64 up rows ->
// 64 outputs; MODE 1: 128 outputs) in steps of 64 along K, double-buffered: the loads of the next
// step are in flight while the matrix cores work on the current one.  The weights stay in the
// order of their tiles in LDS, the activation rows lie in padded rows.  Wave w owns 32 of the
// weight rows (MODE 0: gate rows 16 w .. and the matching up rows) and all rows of the tile.
// Each output is one dot product in the order of K, as in the streaming kernel.
// ---------------------------------------------------------------------------------------- //
#define TALL_BK 64
#define TALL_LD 72          // stride of an activation row in LDS (elements): 64 + 8 keeps 16-byte reads off the same banks

template <int MODE, int MB>
__global__ void __launch_bounds__(256)
grouped_gemm_tall_kernel(const bf16_t* __restrict__ in, const bf16_t* __restrict__ w,
                         bf16_t* __restrict__ out, const int32_t* __restrict__ sorted,
                         const int32_t* __restrict__ tile_expert,
                         const int32_t* __restrict__ counters,
                         const float* __restrict__ route_weight, int assignments, int top_k, int N,
                         int K, int activation) {
  constexpr int BM = 16 * MB;
  constexpr int WROWS = 128;
  int tile, column_block;
  if (!xcd_work_item(N / (MODE == 0 ? 64 : 128), counters[0], tile, column_block)) return;  // uniform
  // the weights of a step: 8 row blocks x 2 halves of k, each a tile of 64 16-byte vectors in the
  // order of the lanes that hold it as an operand, as it lies in memory
  __shared__ __attribute__((aligned(16))) uint4 ws[2][WROWS / 16 * 2][SE_WAVE];
  __shared__ __attribute__((aligned(16))) uint16_t xs[2][BM][TALL_LD];
  __shared__ int32_t rows[BM];

  const int tid = threadIdx.x;
  const int lane = tid & (SE_WAVE - 1);
  const int wave = tid / SE_WAVE;
  const int col = lane & 15, kgroup = lane >> 4;
  const int expert = tile_expert[tile];
  const int out_cols = MODE == 0 ? 64 : 128;
  const int n0 = column_block * out_cols;
  if (tid < BM) rows[tid] = sorted[tile * BM + tid];
  __syncthreads();

  const int64_t w_rows = MODE == 0 ? 2 * static_cast<int64_t>(N) : N;
  const bf16_t* we = w + static_cast<int64_t>(expert) * w_rows * K;

  // global -> LDS assignment: a chunk is 8 elements (16 bytes), a 64-wide row has 8 chunks; thread
  // t moves chunk t & 7 of rows (t >> 3) + 32 j.  Everything is kept in named scalars so that the
  // loads stay in registers while they are in flight.
  static_assert(MB == 4, "the staging below moves exactly two activation chunks per thread");
  const int r0 = tid >> 3, kc = (tid & 7) * 8;
  // weights: wave w brings row blocks 2 w and 2 w + 1 of the step's 8 (MODE 0: blocks 0-3 are gate
  // rows n0 + 16 b, blocks 4-7 the matching up rows; MODE 1: rows n0 + 16 b), both halves of k;
  // a lane brings its own 16 bytes of each tile
  auto block_row = [&](int rb) -> int64_t {
    return MODE == 0 ? (rb < 4 ? 0 : static_cast<int64_t>(N)) + n0 + 16 * (rb & 3) : n0 + 16 * rb;
  };
  const int64_t tiles_per_row_block = K / 32;
  const bf16_t* wp0 = we + (block_row(2 * wave) / 16) * tiles_per_row_block * 512 + lane * 8;   // + 512 for the second half
  const bf16_t* wp2 = we + (block_row(2 * wave + 1) / 16) * tiles_per_row_block * 512 + lane * 8;
  const bf16_t* wp1 = wp0 + 512;
  const bf16_t* wp3 = wp2 + 512;
  const int a0 = rows[r0], a1 = rows[r0 + 32];
  const bf16_t* xp0 = in + (a0 < assignments ? static_cast<int64_t>(MODE == 0 ? a0 / top_k : a0) : 0) * K + kc;
  const bf16_t* xp1 = in + (a1 < assignments ? static_cast<int64_t>(MODE == 0 ? a1 / top_k : a1) : 0) * K + kc;
  const int lds0 = r0 * TALL_LD + kc;               // element offset of the thread's first activation chunk
  constexpr int LDS32 = 32 * TALL_LD;

  floatx4 acc[2][MB];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[nb][mb] = floatx4{0.f, 0.f, 0.f, 0.f};

  // row blocks of the step's weights this wave multiplies
  const int a_block0 = MODE == 0 ? wave : 2 * wave;
  const int a_block1 = MODE == 0 ? 4 + wave : 2 * wave + 1;

#define TALL_FETCH(S, K0)                                        \
  S##w0 = *reinterpret_cast<const uint4*>(wp0 + static_cast<int64_t>(K0) * 16); /* 32 k = one tile = 512 elements */ \
  S##w1 = *reinterpret_cast<const uint4*>(wp1 + static_cast<int64_t>(K0) * 16); \
  S##w2 = *reinterpret_cast<const uint4*>(wp2 + static_cast<int64_t>(K0) * 16); \
  S##w3 = *reinterpret_cast<const uint4*>(wp3 + static_cast<int64_t>(K0) * 16); \
  S##x0 = *reinterpret_cast<const uint4*>(xp0 + (K0));           \
  S##x1 = *reinterpret_cast<const uint4*>(xp1 + (K0));
#define TALL_STASH(S, BUF)                                                          \
  ws[BUF][4 * wave][lane] = S##w0;                                                  \
  ws[BUF][4 * wave + 1][lane] = S##w1;                                              \
  ws[BUF][4 * wave + 2][lane] = S##w2;                                              \
  ws[BUF][4 * wave + 3][lane] = S##w3;                                              \
  *reinterpret_cast<uint4*>(&xs[BUF][0][0] + lds0) = S##x0;                         \
  *reinterpret_cast<uint4*>(&xs[BUF][0][0] + lds0 + LDS32) = S##x1;
#define TALL_COMPUTE(BUF)                                                                              \
  _Pragma("unroll") for (int sub = 0; sub < TALL_BK / 32; ++sub) {                                     \
    const int ko = sub * 32 + kgroup * 8;                                                              \
    const uint4 af0 = ws[BUF][2 * a_block0 + sub][lane];                                               \
    const uint4 af1 = ws[BUF][2 * a_block1 + sub][lane];                                               \
    _Pragma("unroll") for (int mb = 0; mb < MB; ++mb) {                                                \
      const uint4 bf = *reinterpret_cast<const uint4*>(&xs[BUF][mb * 16 + col][ko]);                   \
      acc[0][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af0),            \
                                                           __builtin_bit_cast(bf16x8, bf), acc[0][mb], 0, 0, 0); \
      acc[1][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af1),            \
                                                           __builtin_bit_cast(bf16x8, bf), acc[1][mb], 0, 0, 0); \
    }                                                                                                  \
  }

  // Two register sets (p, q) hold the loads of the next two steps: a load has a whole step of
  // matrix work, and the other block of the CU, to arrive before it is written to LDS.
  uint4 pw0, pw1, pw2, pw3, px0, px1, qw0, qw1, qw2, qw3, qx0, qx1;
  const int steps = K / TALL_BK;     // even: K % 128 == 0
  TALL_FETCH(p, 0)
  TALL_FETCH(q, TALL_BK)
  TALL_STASH(p, 0)
  __syncthreads();
  for (int kt = 0; kt < steps; kt += 2) {
    // step kt: LDS buffer 0 is current, set q holds step kt + 1, set p is free
    if (kt + 2 < steps) { TALL_FETCH(p, (kt + 2) * TALL_BK) }
    TALL_COMPUTE(0)
    TALL_STASH(q, 1)
    __syncthreads();
    // step kt + 1: buffer 1 is current, set p holds step kt + 2, set q is free
    if (kt + 3 < steps) { TALL_FETCH(q, (kt + 3) * TALL_BK) }
    TALL_COMPUTE(1)
    if (kt + 2 < steps) { TALL_STASH(p, 0) }
    __syncthreads();
  }
#undef TALL_FETCH
#undef TALL_STASH
#undef TALL_COMPUTE

  // lane (kgroup, col): acc[nb][mb][i] belongs to weight row 4 * kgroup + i of block nb, tile row mb * 16 + col
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int a = rows[mb * 16 + col];
    if (a >= assignments) continue;
    if (MODE == 0) {
      uint16_t y[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float gate = round_to<bf16_t>(acc[0][mb][i]);
        const float up = round_to<bf16_t>(acc[1][mb][i]);
        const float act = round_to<bf16_t>(gate_activation<true>(gate, activation));
        y[i] = float_to_bf16_bits(act * up);
      }
      uint2 packed;
      packed.x = static_cast<uint32_t>(y[0]) | (static_cast<uint32_t>(y[1]) << 16);
      packed.y = static_cast<uint32_t>(y[2]) | (static_cast<uint32_t>(y[3]) << 16);
      *reinterpret_cast<uint2*>(out + static_cast<int64_t>(a) * N + n0 + 16 * wave + 4 * kgroup) = packed;
    } else {
      const float rw = route_weight[a];
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        uint2 packed;
        packed.x = static_cast<uint32_t>(float_to_bf16_bits(acc[nb][mb][0] * rw)) |
                   (static_cast<uint32_t>(float_to_bf16_bits(acc[nb][mb][1] * rw)) << 16);
        packed.y = static_cast<uint32_t>(float_to_bf16_bits(acc[nb][mb][2] * rw)) |
                   (static_cast<uint32_t>(float_to_bf16_bits(acc[nb][mb][3] * rw)) << 16);
        *reinterpret_cast<uint2*>(out + static_cast<int64_t>(a) * N + n0 + 32 * wave + 16 * nb + 4 * kgroup) = packed;
      }
    }
  }
}

// tile_rows: 64.  MODE 0 needs N % 64 == 0, MODE 1 N % 128 == 0; K % 64 == 0.
extern "C" int se_grouped_gemm_tall(const void* in, const void* w, void* out, const int32_t* sorted,
                                    const int32_t* tile_expert, const int32_t* counters,
                                    const float* route_weight, int assignments, int top_k, int N,
                                    int K, int max_tiles, int mode, int tile_rows, int activation, hipStream_t stream) {
  if (assignments <= 0) return SE_OK;
  if (K <= 0 || K % (2 * TALL_BK) || N <= 0 || N % (mode == 0 ? 64 : 128)) return SE_ERR_SHAPE;
  if (activation != SE_ACT_SILU && activation != SE_ACT_GELU_TANH) return SE_ERR_SHAPE;
  if (max_tiles <= 0 || max_tiles > (1 << 22) || (mode != 0 && mode != 1)) return SE_ERR_SHAPE;
  const int64_t items = static_cast<int64_t>(N / (mode == 0 ? 64 : 128)) * max_tiles;
  const int grid = static_cast<int>((items + 7) / 8 * 8);
#define SE_TALL(MODE, MB)                                                                          \
  grouped_gemm_tall_kernel<MODE, MB><<<grid, 256, 0, stream>>>(                                    \
      static_cast<const bf16_t*>(in), static_cast<const bf16_t*>(w), static_cast<bf16_t*>(out), sorted, \
      tile_expert, counters, route_weight, assignments, top_k, N, K, activation)
  if (tile_rows == 64) { if (mode == 0) SE_TALL(0, 4); else SE_TALL(1, 4); }
  else return SE_ERR_SHAPE;
#undef SE_TALL
  SE_CHECK_LAUNCH();
  return SE_OK;
}

// ---------------------------------------------------------------------------------------- //
// Wide tiles (an expert has sixteen rows or more: prompt portions from 512 tokens on).  The 64 x 128
// kernel above brings its operands through registers, and registers are fed at about 16 bytes a
// clock and CU whatever the addresses; loads that go straight into LDS are fed at three times that
// when the lanes of a load read one contiguous stretch, which the tiled expert tables provide.
// Here a block computes 128 rows x 256 weight rows (87 flop per byte) with eight wavefronts, each
// 64 rows x 64 weight rows (MODE 0: 32 gate rows and the matching 32 up rows, so that the SwiGLU
// product stays inside a lane).  A step of 32 along K is 24 chunks of 1 KB that go from memory
// straight into shared memory in operand order (lane l's 16 bytes of a chunk are what lane l feeds
// the matrix core), three stages deep, three chunks per wavefront and step; 72 KB of LDS, so that
// two blocks share a CU and one computes while the other waits at its barrier.  Measured at 16384
// tokens (gate-up + down): four wavefronts of 64 x 128 and steps of 64, one block per CU: 6.2 ms;
// eight wavefronts: 5.9 (LDS reads issue at 220 instead of 120 bytes a clock); steps of 32 and two
// blocks per CU: 5.1.
//   MODE 0: columns n0 + 32 wc + 16 cb + ... from gate rows n0 + 32 wc ..., up rows N + n0 + 32 wc ...; the result
//           lies in operand tiles by sorted position (see the epilogue), which MODE 1 reads as its activations
//   MODE 1: out[a, n0 + 64 wc + 16 cb + ...] * route_weight[a]
// Requires K % 64 == 0, N % 128 == 0 (MODE 0) / N % 256 == 0 (MODE 1); tiles of 128 sorted rows (BM = 64:
// four wavefronts on 64 rows, measured equal to the tall kernel where that one is used).
// ---------------------------------------------------------------------------------------- //
#define WIDE_STAGES 3
#ifndef WIDE_KSTEP
#define WIDE_KSTEP 32    // k per stage
#endif

template <int MODE, int BM, int KSTEP>   // BM: 64 or 128 rows per tile; KSTEP: 32 or 64 along K per stage
__device__ __forceinline__ void wide_tile(const bf16_t* __restrict__ in, const bf16_t* __restrict__ w,
                                          bf16_t* __restrict__ out, const int32_t* __restrict__ sorted,
                                          const int32_t* __restrict__ tile_expert,
                                          const int32_t* __restrict__ counters,
                                          const float* __restrict__ route_weight, int assignments, int top_k, int N,
                                          int K, int activation) {
  constexpr int OUT_COLS = MODE == 0 ? 128 : 256;
  constexpr int WAVES = BM / 16;                 // 4 or 8: each wavefront 64 rows x 64 weight rows
  constexpr int WCOLS = 4;                       // wave columns: the tile's 256 weight rows in 4 parts
  constexpr int CB = 16 / WCOLS;                 // weight row blocks of a wave
  constexpr int ROW_BLOCKS = 16 + BM / 16;       // weight and activation row blocks of a step
  constexpr int PAIRS = ROW_BLOCKS / WAVES;      // row blocks a wave brings per step: 5 or 3
  constexpr int HALVES = KSTEP / 32;             // chunks of 32 k per row block and step
  constexpr int CHUNKS = ROW_BLOCKS * HALVES;    // per stage
  static_assert(ROW_BLOCKS % WAVES == 0, "the step's row blocks are shared out evenly");
  int tile, column_block;
  if (!xcd_work_item(N / OUT_COLS, counters[0], tile, column_block)) return;  // uniform
  extern __shared__ __align__(16) uint4 wide_shared[];     // WIDE_STAGES x CHUNKS x 64 vectors, then the rows
  int32_t* rows = reinterpret_cast<int32_t*>(wide_shared + WIDE_STAGES * CHUNKS * 64);
  static_assert(WIDE_STAGES * CHUNKS * 1024 <= 160 * 1024 - 1024, "stages must fit shared memory");

  const int tid = threadIdx.x;
  const int lane = tid & (SE_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / SE_WAVE);
  const int col = lane & 15, kgroup = lane >> 4;
  // wave (wr, wc): row blocks wr, RW + wr, 2 RW + wr, 3 RW + wr of the tile (16 rows each) and part wc of the weight rows
  constexpr int RW = BM / 64;
  const int wr = wave / WCOLS, wc = wave % WCOLS;
  const int expert = tile_expert[tile];
  const int n0 = column_block * OUT_COLS;
  if (tid < BM) rows[tid] = sorted[tile * BM + tid];
  __syncthreads();
  // An expert's last tile is partly padding, which lies at its end.  Row blocks that are all padding are
  // left out of the matrix work (with the tokens of a prompt agreeing on a few dozen experts every third
  // tile is such a last tile); the row blocks alternate between the wave rows so that what is left is
  // shared evenly.
  int valid = 0;
#pragma unroll
  for (int r = 0; r < BM; r += SE_WAVE)
    valid += __popcll(__ballot(rows[r + lane] < assignments));
  const int live_blocks = __builtin_amdgcn_readfirstlane((valid + 15) / 16);
  const int my_blocks = (live_blocks - wr + RW - 1) / RW;     // 0 .. 4, the same for the whole wave

  const int64_t w_rows = MODE == 0 ? 2 * static_cast<int64_t>(N) : N;
  const bf16_t* we = w + static_cast<int64_t>(expert) * w_rows * K;

  // Row block rb (16 rows) of the tile's 256 weight rows: blocks CB wc' ... CB wc' + CB - 1 belong to
  // the wave column wc'; in MODE 0 the first half of them are gate rows, the second half the matching
  // up rows.
  auto weight_row = [&](int rb) -> int64_t {
    const int wcol = rb / CB, cb = rb % CB;
    if (MODE == 0)
      return (cb < CB / 2 ? 0 : static_cast<int64_t>(N)) + n0 + (8 * CB) * wcol + 16 * (cb % (CB / 2));
    return n0 + (16 * CB) * wcol + 16 * cb;
  };
  // The wave brings PAIRS "row block pairs" of a step: pair p < 16 is weight row block p, pair p >= 16
  // is activation row block p - 16; both halves of the step (chunks 2 p and 2 p + 1).
  const bf16_t* src[PAIRS];
#pragma unroll
  for (int j = 0; j < PAIRS; ++j) {
    const int p = wave * PAIRS + j;
    if (p < 16) {     // a tile of 16 rows x 32 k is 512 elements in the order of the lanes; the next 32 k follow it
      src[j] = we + (weight_row(p) / 16) * (K / 32) * 512 + lane * 8;
    } else if (MODE == 0) {
      const int a = rows[(p - 16) * 16 + col];
      const int64_t token = a < assignments ? static_cast<int64_t>(a / top_k) : 0;  // padding reads row 0
      src[j] = in + token * K + kgroup * 8;
    } else {
      // the gate-up launch has left its output in tiles by sorted position (below): row block p - 16
      // of this tile, like a weight row block.  (Gathering the gate-up launch's rows into such tiles
      // first was measured too: the extra pass costs more than it saves below 8192 tokens, and
      // saves 2 % from there on.)
      src[j] = in + (static_cast<int64_t>(tile) * (BM / 16) + (p - 16)) * (K / 32) * 512 + lane * 8;
    }
  }
  const uint32_t stage_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(wide_shared));
  auto issue = [&](int step) {
    const uint32_t dst =
        stage_base + static_cast<uint32_t>((step % WIDE_STAGES) * CHUNKS + wave * HALVES * PAIRS) * 1024u;
    const int k0 = step * KSTEP;
#pragma unroll
    for (int j = 0; j < PAIRS; ++j) {
      const bool tiles = MODE == 1 || wave * PAIRS + j < 16;      // the same for all lanes
      const bf16_t* first = tiles ? src[j] + static_cast<int64_t>(k0) * 16 : src[j] + k0;
      load16_to_lds(first, dst + static_cast<uint32_t>(HALVES * j) * 1024u);
      if (HALVES == 2) load16_to_lds(first + (tiles ? 512 : 32), dst + static_cast<uint32_t>(2 * j + 1) * 1024u);
    }
  };

  floatx4 acc[CB][4];      // [weight row block of the wave][row block of the wave]
#pragma unroll
  for (int cb = 0; cb < CB; ++cb)
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) acc[cb][mb] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int steps = K / KSTEP;
#pragma unroll
  for (int j = 0; j < WIDE_STAGES - 1; ++j)
    if (j < steps) issue(j);
  // the loop over K for a wave with MBS live row blocks: every wave brings its chunks and meets the
  // barriers, whatever it has to compute
  auto run = [&](auto mbs_tag) {
    constexpr int MBS = decltype(mbs_tag)::value;
    for (int step = 0; step < steps; ++step) {
      // this step's data: all but the loads of the steps after it must have come back
      if (step + WIDE_STAGES - 2 < steps) {
        __builtin_amdgcn_s_waitcnt(0x0F70 | ((WIDE_STAGES - 2) * HALVES * PAIRS));    // vmcnt((stages - 2) * loads per step)
      } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);                               // vmcnt(0)
      }
      __builtin_amdgcn_s_barrier();   // everyone's part of the step is in; everyone has left step - 1
      asm volatile("" ::: "memory");
      if (step + WIDE_STAGES - 1 < steps) issue(step + WIDE_STAGES - 1);   // into the buffer step - 1 used
      const uint4(*chunk)[64] = reinterpret_cast<const uint4(*)[64]>(wide_shared) + (step % WIDE_STAGES) * CHUNKS;
      if constexpr (MBS > 0) {
#pragma unroll
        for (int sub = 0; sub < HALVES; ++sub) {
          uint4 bfrag[MBS];
#pragma unroll
          for (int mb = 0; mb < MBS; ++mb) bfrag[mb] = chunk[HALVES * (16 + RW * mb + wr) + sub][lane];
#pragma unroll
          for (int cb = 0; cb < CB; ++cb) {
            const uint4 afrag = chunk[HALVES * (CB * wc + cb) + sub][lane];
#pragma unroll
            for (int mb = 0; mb < MBS; ++mb)
              acc[cb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, afrag),
                                                                   __builtin_bit_cast(bf16x8, bfrag[mb]),
                                                                   acc[cb][mb], 0, 0, 0);
          }
        }
      }
      asm volatile("" ::: "memory");
    }
  };
  if (my_blocks >= 4) run(std::integral_constant<int, 4>{});
  else if (my_blocks == 3) run(std::integral_constant<int, 3>{});
  else if (my_blocks == 2) run(std::integral_constant<int, 2>{});
  else if (my_blocks == 1) run(std::integral_constant<int, 1>{});
  else run(std::integral_constant<int, 0>{});
  // lane (kgroup, col): acc[cb][mb][i] belongs to weight row 4 * kgroup + i of block cb, tile row 16 (RW mb + wr) + col
#pragma unroll
  for (int mb = 0; mb < 4; ++mb) {
    const int a = rows[16 * (RW * mb + wr) + col];
    if (a >= assignments) continue;
    bf16_t* o_row = out + static_cast<int64_t>(a) * N + n0 + 4 * kgroup;
    if (MODE == 0) {
      // The result is the down launch's activation operand.  It is written in tiles of 16 sorted
      // rows x 32 columns, each 1 KB in the order of the lanes that will hold it ([column / 8][row]
      // [column % 8], like the expert tables), tile (sorted row block, column / 32): the down launch
      // then loads it as contiguous kilobytes instead of 64 bytes from each of 16 rows.  Rows of
      // padding are not written; what the down launch computes from them is not stored.
      bf16_t* t_row = out + (static_cast<int64_t>(tile) * (BM / 16) + RW * mb + wr) * (N / 32) * 512 + col * 8;
#pragma unroll
      for (int cb = 0; cb < CB / 2; ++cb) {
        uint16_t y[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float gate = round_to<bf16_t>(acc[cb][mb][i]);
          const float up = round_to<bf16_t>(acc[cb + CB / 2][mb][i]);
          const float act = round_to<bf16_t>(gate_activation<true>(gate, activation));
          y[i] = float_to_bf16_bits(act * up);
        }
        uint2 packed;
        packed.x = static_cast<uint32_t>(y[0]) | (static_cast<uint32_t>(y[1]) << 16);
        packed.y = static_cast<uint32_t>(y[2]) | (static_cast<uint32_t>(y[3]) << 16);
        const int n = n0 + (8 * CB) * wc + 16 * cb + 4 * kgroup;    // first of the lane's four columns
        *reinterpret_cast<uint2*>(t_row + static_cast<int64_t>(n / 32) * 512 + ((n % 32) / 8) * 128 + n % 8) = packed;
      }
    } else {
      const float rw = route_weight[a];
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) {
        uint2 packed;
        packed.x = static_cast<uint32_t>(float_to_bf16_bits(acc[cb][mb][0] * rw)) |
                   (static_cast<uint32_t>(float_to_bf16_bits(acc[cb][mb][1] * rw)) << 16);
        packed.y = static_cast<uint32_t>(float_to_bf16_bits(acc[cb][mb][2] * rw)) |
                   (static_cast<uint32_t>(float_to_bf16_bits(acc[cb][mb][3] * rw)) << 16);
        *reinterpret_cast<uint2*>(o_row + (16 * CB) * wc + 16 * cb) = packed;
      }
    }
  }
}

template <int MODE, int BM, int KSTEP>
__global__ void __launch_bounds__(4 * BM, KSTEP == 32 ? 2 : 1)
grouped_gemm_wide_kernel(const bf16_t* __restrict__ in, const bf16_t* __restrict__ w,
                         bf16_t* __restrict__ out, const int32_t* __restrict__ sorted,
                         const int32_t* __restrict__ tile_expert,
                         const int32_t* __restrict__ counters,
                         const float* __restrict__ route_weight, int assignments, int top_k, int N,
                         int K, int activation) {
  wide_tile<MODE, BM, KSTEP>(in, w, out, sorted, tile_expert, counters, route_weight, assignments, top_k, N, K, activation);
}

// tile_rows: 64 or 128.  MODE 0 needs N % 128 == 0, MODE 1 N % 256 == 0; K % 64 == 0.
template <int MODE, int BM>
static int launch_wide(const void* in, const void* w, void* out, const int32_t* sorted,
                       const int32_t* tile_expert, const int32_t* counters, const float* route_weight,
                       int assignments, int top_k, int N, int K, int max_tiles, int activation, hipStream_t stream) {
  const int64_t items = static_cast<int64_t>(N / (MODE == 0 ? 128 : 256)) * max_tiles;
  const int grid = static_cast<int>((items + 7) / 8 * 8);
  constexpr size_t shared = WIDE_STAGES * (16 + BM / 16) * (WIDE_KSTEP / 32) * 1024 + BM * sizeof(int32_t);
  static bool allowed = false;   // more than 64 KB of shared memory has to be asked for, once
  if (!allowed) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&grouped_gemm_wide_kernel<MODE, BM, WIDE_KSTEP>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(shared)) != hipSuccess)
      return SE_ERR_LAUNCH;
    allowed = true;
  }
  grouped_gemm_wide_kernel<MODE, BM, WIDE_KSTEP><<<grid, 4 * BM, shared, stream>>>(
      static_cast<const bf16_t*>(in), static_cast<const bf16_t*>(w), static_cast<bf16_t*>(out), sorted,
      tile_expert, counters, route_weight, assignments, top_k, N, K, activation);
  return SE_OK;
}

extern "C" int se_grouped_gemm_wide(const void* in, const void* w, void* out, const int32_t* sorted,
                                    const int32_t* tile_expert, const int32_t* counters,
                                    const float* route_weight, int assignments, int top_k, int N,
                                    int K, int max_tiles, int mode, int tile_rows, int activation, hipStream_t stream) {
  if (assignments <= 0) return SE_OK;
  if (K <= 0 || K % 64 || N <= 0 || N % (mode == 0 ? 128 : 256)) return SE_ERR_SHAPE;
  if (activation != SE_ACT_SILU && activation != SE_ACT_GELU_TANH) return SE_ERR_SHAPE;
  if (tile_rows != 64 && tile_rows != 128) return SE_ERR_SHAPE;
  if (max_tiles <= 0 || max_tiles > (1 << 22) || (mode != 0 && mode != 1)) return SE_ERR_SHAPE;
  int status;
  if (mode == 0)
    status = tile_rows == 128 ? launch_wide<0, 128>(in, w, out, sorted, tile_expert, counters, route_weight, assignments,
                                                    top_k, N, K, max_tiles, activation, stream)
                              : launch_wide<0, 64>(in, w, out, sorted, tile_expert, counters, route_weight, assignments,
                                                   top_k, N, K, max_tiles, activation, stream);
  else
    status = tile_rows == 128 ? launch_wide<1, 128>(in, w, out, sorted, tile_expert, counters, route_weight, assignments,
                                                    top_k, N, K, max_tiles, activation, stream)
                              : launch_wide<1, 64>(in, w, out, sorted, tile_expert, counters, route_weight, assignments,
                                                   top_k, N, K, max_tiles, activation, stream);
  if (status != SE_OK) return status;
  SE_CHECK_LAUNCH();
  return SE_OK;
}

// Dense product of a few rows: out[rows, N] = x[rows, K] . w[N, K]^T (bfloat16, float accumulate).
// A projection has only N / 16 blocks, far fewer than an expert layer: K is split over as many
// wavefronts per block (up to 16) as it takes to put a few thousand of them in flight.
template <int MB, int KW, int U>
static void launch_dense(const void* x, const void* w, void* out, int rows, int N, int K, int tiles,
                         bool tiled, hipStream_t stream) {
  const int64_t items = static_cast<int64_t>(N / 16) * tiles;
  const int grid = static_cast<int>((items + 7) / 8 * 8);
  if (tiled)
    grouped_gemm_mfma_kernel<3, MB, 1, U, KW><<<grid, 64 * KW, 0, stream>>>(
        static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<bf16_t*>(out), nullptr,
        nullptr, nullptr, nullptr, rows, 1, N, K, tiles, 0);
  else
    grouped_gemm_mfma_kernel<2, MB, 1, U, KW><<<grid, 64 * KW, 0, stream>>>(
        static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<bf16_t*>(out), nullptr,
        nullptr, nullptr, nullptr, rows, 1, N, K, tiles, 0);
}

// One choice of the stage depth U: K is split over 4, 8 or 16 wavefronts (until a few thousand are
// in flight) if a wavefront's share of K is whole stages; false if it is not.
template <int MB, int U>
static bool dense_with_stage(const void* x, const void* w, void* out, int rows, int N, int K, int tiles,
                             bool tiled, hipStream_t stream) {
  constexpr int STAGE = 32 * U;
  const int64_t blocks = static_cast<int64_t>(N / 16) * tiles;
  int kw = 4;
  while (kw < 16 && blocks * kw < 3072 && K % (2 * kw * STAGE) == 0) kw *= 2;
  if (K % (kw * STAGE)) return false;
  if (kw == 4) launch_dense<MB, 4, U>(x, w, out, rows, N, K, tiles, tiled, stream);
  else if (kw == 8) launch_dense<MB, 8, U>(x, w, out, rows, N, K, tiles, tiled, stream);
  else launch_dense<MB, 16, U>(x, w, out, rows, N, K, tiles, tiled, stream);
  return true;
}

template <int MB>
static void dense_by_split(const void* x, const void* w, void* out, int rows, int N, int K, int tiles,
                           bool tiled, hipStream_t stream) {
  // Two stages of a wavefront are in flight at a time, so the deeper the stage the more bytes it
  // has under way: with up to 16 rows a stage of six steps (96 registers for both sets) brings a
  // share of 384 along K (MiniMax-M2's qkv and output projections) in one round trip instead of
  // three.  With one weight block per wavefront even 64 rows leave registers for stages of two.
  if constexpr (MB == 1) {
    if (dense_with_stage<MB, 6>(x, w, out, rows, N, K, tiles, tiled, stream)) return;
    if (dense_with_stage<MB, 4>(x, w, out, rows, N, K, tiles, tiled, stream)) return;
  }
  if (dense_with_stage<MB, 2>(x, w, out, rows, N, K, tiles, tiled, stream)) return;
  dense_with_stage<MB, 1>(x, w, out, rows, N, K, tiles, tiled, stream);   // K % 128 == 0 always holds here
}

// `tiled`: w is a copy of the matrix in tiles of 16 rows x 32 k (tile_expert_weights), not in rows.
extern "C" int se_skinny_gemm_mfma(const void* x, const void* w, void* out, int rows, int N, int K,
                                   int tiled, hipStream_t stream) {
  if (rows <= 0) return SE_OK;
  if (K <= 0 || K % 128 || N <= 0 || N % 16 || rows > 65535 * 16) return SE_ERR_SHAPE;
  if (rows <= 16)
    dense_by_split<1>(x, w, out, rows, N, K, 1, tiled != 0, stream);
  else if (rows <= 32)
    dense_by_split<2>(x, w, out, rows, N, K, 1, tiled != 0, stream);
  else
    dense_by_split<4>(x, w, out, rows, N, K, (rows + 63) / 64, tiled != 0, stream);
  SE_CHECK_LAUNCH();
  return SE_OK;
}

// ---------------------------------------------------------------------------------------- //
// Mid tiles (an expert has a few dozen rows: a prompt of a thousand or two thousand tokens spread
// evenly over the experts, prompt portions beside decoded tokens).  The step is bound by the expert
// tables it has to read, like a decode step, but the streaming kernel above reads a table once per 16
// (32) rows, and the wide kernel, which stages everything through shared memory, has too few bytes
// under way to fill the memory system when its tiles are half empty (5.2 of 7.1 TB/s at 64 rows per
// expert).  Here a block of eight wavefronts takes a tile of 64 or 96 sorted rows x 128 (MODE 1: 256)
// output columns; the output columns are split over the wavefronts, so that
//   * every wavefront streams its own weight rows (MODE 0: 16 gate rows and the matching 16 up rows;
//     MODE 1: 32 rows) from the tiled tables straight into matrix-core operands, read-once hint and
//     all, three stages of 64 along K deep in registers (8 KB under way per wavefront, 128 KB per CU);
//   * the tile's activation rows, which all eight need, go once per block from memory straight into
//     shared memory in operand order (one or two kilobytes per wavefront and stage) and are read from
//     there, three stages deep;
//   * no partial sums cross wavefronts: a lane's accumulators are whole dot products in the order of K.
// The loads into shared memory are counted by the same counter as the loads into registers, which the
// compiler waits for by itself but does not know of the former: before each barrier the wavefront waits
// by hand until only the loads of the stages after this one are outstanding (an exact count; the
// compiler's own waits, which come later, then find their data there or wait a little too long, never
// too short).
//   MODE 0: act[a, n0 + 16 wave + ...] from gate rows n0 + 16 wave ..., up rows N + n0 + 16 wave ...
//   MODE 1: out[a, n0 + 32 wave + ...] * route_weight[a]
// Requires K % 64 == 0, N % 128 == 0 (MODE 0) / N % 256 == 0 (MODE 1).
// ---------------------------------------------------------------------------------------- //
#define MID_WAVES 8
#define MID_STAGES 3
#define MID_KSTEP 64

// bytes of shared memory before the tile's row list: the stages of activation rows or the tile of results
__host__ __device__ constexpr int mid_shared_bytes(int mode, int mb) {
  const int stages = MID_STAGES * mb * (MID_KSTEP / 32) * 1024;
  const int results = 16 * mb * ((mode == 0 ? 16 : 32) * MID_WAVES * 2 + 16);
  return stages > results ? stages : results;
}

template <int MODE, int MB>   // MB row blocks of 16: tiles of 64 or 96 sorted rows
__device__ __forceinline__ void mid_tile(const bf16_t* __restrict__ in, const bf16_t* __restrict__ w,
                                         bf16_t* __restrict__ out, const int32_t* __restrict__ sorted,
                                         const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ counters,
                                         const float* __restrict__ route_weight, int assignments, int top_k, int N,
                                         int K, int activation) {
  constexpr int BM = 16 * MB;
  constexpr int U = MID_KSTEP / 32;              // steps of 32 per stage
  constexpr int TILES = MB * U;                  // activation tiles (1 KB) of a stage
  constexpr int OUT_COLS = (MODE == 0 ? 16 : 32) * MID_WAVES;
  static_assert(TILES >= MID_WAVES && TILES <= 2 * MID_WAVES, "a wavefront brings one or two activation tiles per stage");
  int tile, column_block;
  if (!xcd_work_item(N / OUT_COLS, counters[0], tile, column_block)) return;  // uniform
  // MID_STAGES x TILES x 64 vectors, which the tile of results takes over in the end; then the rows
  extern __shared__ __align__(16) uint4 mid_shared[];
  uint4(*stage)[TILES][SE_WAVE] = reinterpret_cast<uint4(*)[TILES][SE_WAVE]>(mid_shared);
  int32_t* rows = reinterpret_cast<int32_t*>(reinterpret_cast<char*>(mid_shared) + mid_shared_bytes(MODE, MB));

  const int tid = threadIdx.x;
  const int lane = tid & (SE_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / SE_WAVE);
  const int col = lane & 15, kgroup = lane >> 4;
  const int expert = tile_expert[tile];
  const int n0 = column_block * OUT_COLS;
  if (tid < BM) rows[tid] = sorted[tile * BM + tid];
  __syncthreads();

  // the wavefront's two weight row blocks, as tiles of 16 rows x 32 k (1 KB each, 512 elements apart along k)
  const int64_t w_rows = MODE == 0 ? 2 * static_cast<int64_t>(N) : N;
  const bf16_t* we = w + static_cast<int64_t>(expert) * w_rows * K;
  const int64_t row_block0 = MODE == 0 ? (n0 + 16 * wave) / 16 : (n0 + 32 * wave) / 16;
  const int64_t row_block1 = MODE == 0 ? (static_cast<int64_t>(N) + n0 + 16 * wave) / 16 : row_block0 + 1;
  const bf16_t* a_ptr0 = we + row_block0 * (K / 32) * 512 + lane * 8;
  const bf16_t* a_ptr1 = we + row_block1 * (K / 32) * 512 + lane * 8;

  // the activation tiles this wavefront brings per stage: tile j = (step u = j / MB, row block j % MB);
  // lane (kgroup, col) brings 8 k of row 16 (j % MB) + col: its 16 bytes are what it feeds the matrix core
  const bool two_tiles = wave + MID_WAVES < TILES;      // the same for the whole wavefront
  const bf16_t* x_ptr[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int j = min(wave + t * MID_WAVES, TILES - 1);
    const int a = rows[(j % MB) * 16 + col];
    const int64_t src = a < assignments ? (MODE == 0 ? a / top_k : a) : 0;  // padding reads row 0
    x_ptr[t] = in + src * K + kgroup * 8 + 32 * (j / MB);
  }
  const uint32_t stage_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(mid_shared));
  auto bring_rows = [&](int s) {      // the loads of stage s into shared memory
    const uint32_t dst = stage_base + static_cast<uint32_t>((s % MID_STAGES) * TILES + wave) * 1024u;
    load16_to_lds(x_ptr[0] + static_cast<int64_t>(s) * MID_KSTEP, dst);
    if (two_tiles) load16_to_lds(x_ptr[1] + static_cast<int64_t>(s) * MID_KSTEP, dst + MID_WAVES * 1024u);
  };

  floatx4 acc[2][MB];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[nb][mb] = floatx4{0.f, 0.f, 0.f, 0.f};

  // three register sets take turns: while the matrix cores work on one stage the weights of the next two
  // are under way
  uint4 w0[U][2], w1[U][2], w2[U][2];
  auto bring_weights = [&](uint4 (&wf)[U][2], int s) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      wf[u][0] = load16_once(a_ptr0 + (static_cast<int64_t>(s) * MID_KSTEP + 32 * u) * 16);
      SE_NOTE_VECTOR_LOAD();
      wf[u][1] = load16_once(a_ptr1 + (static_cast<int64_t>(s) * MID_KSTEP + 32 * u) * 16);
      SE_NOTE_VECTOR_LOAD();
    }
  };
  const int steps = K / MID_KSTEP;
  auto run_stage = [&](const uint4 (&wf)[U][2], uint4 (&next)[U][2], int s) {
    // stage s of everyone's rows is in shared memory once every wavefront has seen its own loads of it
    // land: all but the loads of the stages after s (the weights of stage s + 1, issued before its rows)
    if (s + 1 < steps) {
      if (two_tiles) __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * U + 2));
      else __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * U + 1));
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    __builtin_amdgcn_s_barrier();   // and everyone has left stage s - 1, whose buffer stage s + 2 takes
    asm volatile("" ::: "memory");
    if (s + 2 < steps) {
      bring_weights(next, s + 2);
      bring_rows(s + 2);
    }
    const uint4(*rows_of)[SE_WAVE] = stage[s % MID_STAGES];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const uint4 bfrag = rows_of[u * MB + mb][lane];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
          acc[nb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wf[u][nb]),
                                                               __builtin_bit_cast(bf16x8, bfrag), acc[nb][mb], 0, 0, 0);
      }
    asm volatile("" ::: "memory");
  };
  bring_weights(w0, 0);
  bring_rows(0);
  if (steps > 1) {
    bring_weights(w1, 1);
    bring_rows(1);
  }
  for (int s = 0; s < steps; s += 3) {
    run_stage(w0, w2, s);
    if (s + 1 < steps) run_stage(w1, w0, s + 1);
    if (s + 2 < steps) run_stage(w2, w1, s + 2);
  }

  // The results leave through shared memory, a row's columns as whole cache lines: written from the lanes
  // that hold them (8 bytes each, 32 bytes of a row per wavefront) they take several times as long as their
  // bytes need, measured 230 us of a 1350 us layer at 64 rows per expert.
  // lane (kgroup, col): acc[nb][mb][i] belongs to weight row 4 * kgroup + i of the wavefront's block nb, tile row 16 mb + col
  constexpr int ROW_BYTES = OUT_COLS * 2;
  constexpr int ROW_STRIDE = ROW_BYTES + 16;      // rows 132 (260) words apart: the lanes of a store hit different banks
  __syncthreads();                                // everyone has left the last stage
  char* out_tile = reinterpret_cast<char*>(mid_shared);
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    char* t_row = out_tile + (16 * mb + col) * ROW_STRIDE + 8 * kgroup;
    if (MODE == 0) {
      uint16_t y[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float gate = round_to<bf16_t>(acc[0][mb][i]);
        const float up = round_to<bf16_t>(acc[1][mb][i]);
        const float act = round_to<bf16_t>(gate_activation<true>(gate, activation));
        y[i] = float_to_bf16_bits(act * up);
      }
      uint2 packed;
      packed.x = static_cast<uint32_t>(y[0]) | (static_cast<uint32_t>(y[1]) << 16);
      packed.y = static_cast<uint32_t>(y[2]) | (static_cast<uint32_t>(y[3]) << 16);
      *reinterpret_cast<uint2*>(t_row + 32 * wave) = packed;
    } else {
      const int a = rows[16 * mb + col];
      const float rw = a < assignments ? route_weight[a] : 0.f;
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        uint2 packed;
        packed.x = static_cast<uint32_t>(float_to_bf16_bits(acc[nb][mb][0] * rw)) |
                   (static_cast<uint32_t>(float_to_bf16_bits(acc[nb][mb][1] * rw)) << 16);
        packed.y = static_cast<uint32_t>(float_to_bf16_bits(acc[nb][mb][2] * rw)) |
                   (static_cast<uint32_t>(float_to_bf16_bits(acc[nb][mb][3] * rw)) << 16);
        *reinterpret_cast<uint2*>(t_row + 64 * wave + 32 * nb) = packed;
      }
    }
  }
  __syncthreads();
  constexpr int LANES_PER_ROW = ROW_BYTES / 16;   // 16 bytes a thread
  for (int r = tid / LANES_PER_ROW; r < BM; r += 64 * MID_WAVES / LANES_PER_ROW) {
    const int a = rows[r];
    if (a >= assignments) continue;               // padding
    const int piece = tid % LANES_PER_ROW;
    // written once and read by a later kernel: past the caches (measured: 1245 against 1335 us for a layer at 64 rows per expert)
    __builtin_nontemporal_store(*reinterpret_cast<const se_u32x4*>(out_tile + r * ROW_STRIDE + 16 * piece),
                                reinterpret_cast<se_u32x4*>(out + static_cast<int64_t>(a) * N + n0 + 8 * piece));
  }
}

template <int MODE, int MB>
__global__ void __launch_bounds__(64 * MID_WAVES, 2)
grouped_gemm_mid_kernel(const bf16_t* __restrict__ in, const bf16_t* __restrict__ w,
                        bf16_t* __restrict__ out, const int32_t* __restrict__ sorted,
                        const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ counters,
                        const float* __restrict__ route_weight, int assignments, int top_k, int N,
                        int K, int activation) {
  mid_tile<MODE, MB>(in, w, out, sorted, tile_expert, counters, route_weight, assignments, top_k, N, K, activation);
}

// The device's choice between the two (se_moe_align_choice leaves it in counters[2], with the sorted list in
// tiles of the height that goes with it): tiles of 96 rows through the mid kernel's code, tiles of 128 through
// the wide kernel's.  One launch serves both, since the host cannot know which it will be; both have blocks of
// eight wavefronts, two to a CU, and the same output columns per block.
#define CHOICE_MID_MB 6
#define CHOICE_WIDE_BM 128
template <int MODE>
__global__ void __launch_bounds__(512, 2)
grouped_gemm_choice_kernel(const bf16_t* __restrict__ in, const bf16_t* __restrict__ w,
                           bf16_t* __restrict__ out, const int32_t* __restrict__ sorted,
                           const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ counters,
                           const float* __restrict__ route_weight, int assignments, int top_k, int N,
                           int K, int activation) {
  if (counters[2] == 0)    // the same in the whole grid
    mid_tile<MODE, CHOICE_MID_MB>(in, w, out, sorted, tile_expert, counters, route_weight, assignments, top_k, N, K, activation);
  else
    wide_tile<MODE, CHOICE_WIDE_BM, WIDE_KSTEP>(in, w, out, sorted, tile_expert, counters, route_weight, assignments, top_k, N,
                                                K, activation);
}

template <int MODE>
static int launch_choice(const void* in, const void* w, void* out, const int32_t* sorted, const int32_t* tile_expert,
                         const int32_t* counters, const float* route_weight, int assignments, int top_k, int N, int K,
                         int max_tiles, int activation, hipStream_t stream) {
  const int64_t items = static_cast<int64_t>(N / (MODE == 0 ? 128 : 256)) * max_tiles;
  const int grid = static_cast<int>((items + 7) / 8 * 8);
  constexpr size_t wide = WIDE_STAGES * (16 + CHOICE_WIDE_BM / 16) * (WIDE_KSTEP / 32) * 1024 + CHOICE_WIDE_BM * sizeof(int32_t);
  constexpr size_t mid = mid_shared_bytes(MODE, CHOICE_MID_MB) + 16 * CHOICE_MID_MB * sizeof(int32_t);
  constexpr size_t shared = wide > mid ? wide : mid;
  static bool allowed = false;   // more than 64 KB of shared memory has to be asked for, once
  if (!allowed) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&grouped_gemm_choice_kernel<MODE>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(shared)) != hipSuccess)
      return SE_ERR_LAUNCH;
    allowed = true;
  }
  grouped_gemm_choice_kernel<MODE><<<grid, 512, shared, stream>>>(
      static_cast<const bf16_t*>(in), static_cast<const bf16_t*>(w), static_cast<bf16_t*>(out), sorted,
      tile_expert, counters, route_weight, assignments, top_k, N, K, activation);
  return SE_OK;
}

// max_tiles: a bound for either tile height.  MODE 0 needs N % 128 == 0, MODE 1 N % 256 == 0; K % 64 == 0.
extern "C" int se_grouped_gemm_choice(const void* in, const void* w, void* out, const int32_t* sorted,
                                      const int32_t* tile_expert, const int32_t* counters,
                                      const float* route_weight, int assignments, int top_k, int N,
                                      int K, int max_tiles, int mode, int activation, hipStream_t stream) {
  if (assignments <= 0) return SE_OK;
  if (K <= 0 || K % 64 || N <= 0 || N % (mode == 0 ? 128 : 256)) return SE_ERR_SHAPE;
  if (activation != SE_ACT_SILU && activation != SE_ACT_GELU_TANH) return SE_ERR_SHAPE;
  if (max_tiles <= 0 || max_tiles > (1 << 22) || (mode != 0 && mode != 1)) return SE_ERR_SHAPE;
  const int status = mode == 0 ? launch_choice<0>(in, w, out, sorted, tile_expert, counters, route_weight, assignments,
                                                  top_k, N, K, max_tiles, activation, stream)
                               : launch_choice<1>(in, w, out, sorted, tile_expert, counters, route_weight, assignments,
                                                  top_k, N, K, max_tiles, activation, stream);
  if (status != SE_OK) return status;
  SE_CHECK_LAUNCH();
  return SE_OK;
}

// tile_rows: 64 or 96.  MODE 0 needs N % 128 == 0, MODE 1 N % 256 == 0; K % 64 == 0.
extern "C" int se_grouped_gemm_mid(const void* in, const void* w, void* out, const int32_t* sorted,
                                   const int32_t* tile_expert, const int32_t* counters,
                                   const float* route_weight, int assignments, int top_k, int N,
                                   int K, int max_tiles, int mode, int tile_rows, int activation, hipStream_t stream) {
  if (assignments <= 0) return SE_OK;
  if (K <= 0 || K % MID_KSTEP || N <= 0 || N % (mode == 0 ? 128 : 256)) return SE_ERR_SHAPE;
  if (activation != SE_ACT_SILU && activation != SE_ACT_GELU_TANH) return SE_ERR_SHAPE;
  if (tile_rows != 64 && tile_rows != 96) return SE_ERR_SHAPE;
  if (max_tiles <= 0 || max_tiles > (1 << 22) || (mode != 0 && mode != 1)) return SE_ERR_SHAPE;
  const int64_t items = static_cast<int64_t>(N / (mode == 0 ? 128 : 256)) * max_tiles;
  const int grid = static_cast<int>((items + 7) / 8 * 8);
#define SE_MID(MODE, MB)                                                                           \
  grouped_gemm_mid_kernel<MODE, MB><<<grid, 64 * MID_WAVES,                                        \
                                      mid_shared_bytes(MODE, MB) + 16 * MB * sizeof(int32_t), stream>>>( \
      static_cast<const bf16_t*>(in), static_cast<const bf16_t*>(w), static_cast<bf16_t*>(out), sorted, \
      tile_expert, counters, route_weight, assignments, top_k, N, K, activation)
  if (tile_rows == 64) { if (mode == 0) SE_MID(0, 4); else SE_MID(1, 4); }
  else { if (mode == 0) SE_MID(0, 6); else SE_MID(1, 6); }
#undef SE_MID
  SE_CHECK_LAUNCH();
  return SE_OK;
}

// tile_rows: 16, 32 or 64 (the alignment the sorted list was built with); col_blocks: 1 or 2.
extern "C" int se_grouped_gemm_mfma(const void* in, const void* w, void* out, const int32_t* sorted,
                                    const int32_t* tile_expert, const int32_t* counters,
                                    const float* route_weight, int assignments, int top_k, int N,
                                    int K, int max_tiles, int mode, int tile_rows, int col_blocks,
                                    int activation, hipStream_t stream) {
  if (assignments <= 0) return SE_OK;
  if (activation != SE_ACT_SILU && activation != SE_ACT_GELU_TANH) return SE_ERR_SHAPE;
  if (K <= 0 || K % 128 || N <= 0 || N % (16 * col_blocks)) return SE_ERR_SHAPE;
  if (max_tiles <= 0 || max_tiles > (1 << 22)) return SE_ERR_SHAPE;
  if (mode != 0 && mode != 1) return SE_ERR_SHAPE;
#define SE_CASE(MB, NB)                                                                             \
  if (tile_rows == 16 * MB && col_blocks == NB) {                                                   \
    if (mode == 0)                                                                                  \
      launch<0, MB, NB>(in, w, out, sorted, tile_expert, counters, route_weight, assignments,      \
                        top_k, N, K, max_tiles, activation, stream);                                \
    else                                                                                            \
      launch<1, MB, NB>(in, w, out, sorted, tile_expert, counters, route_weight, assignments,      \
                        top_k, N, K, max_tiles, activation, stream);                                \
    SE_CHECK_LAUNCH();                                                                              \
    return SE_OK;                                                                                   \
  }
  SE_CASE(1, 1)
  SE_CASE(1, 2)
  SE_CASE(2, 1)
  SE_CASE(2, 2)
  SE_CASE(4, 1)
  SE_CASE(4, 2)
#undef SE_CASE
  return SE_ERR_SHAPE;
}
