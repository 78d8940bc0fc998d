// A small HIP-on-the-CPU runtime for tests: it runs the kernel sources of sparseengine_amd/csrc,
// unchanged but for their launches and inline assembly (tests/emu/build.py rewrites those), on the
// host, one block after the other, every thread of a block as a fibre.
//
// What it models
//   * blocks, threads, wavefronts of 64, static and dynamic shared memory, __syncthreads / s_barrier
//     (threads that have returned do not take part);
//   * the cross-lane operations the kernels use (shuffles, ballots, DPP moves, row and half swaps)
//     and v_mfma_f32_16x16x32_bf16, as wave-wide exchanges: every live lane of the wavefront has to
//     arrive at the same operation, otherwise the run stops with a message;
//   * loads that go from memory straight into shared memory (load16_to_lds): they are queued per lane
//     and carried out only when an s_waitcnt lets them complete (or at once, see emu_rt_lds_mode),
//     so a wait that is too weak shows as stale data;
//   * the order in which the threads of a block run between two synchronisation points can be
//     ascending, descending or shuffled (emu_rt_schedule): results must not depend on it.
// What it does not model: timing, caches, register limits, the accuracy of hardware
// transcendental instructions, memory that is not 16-byte aligned being slower rather than wrong
// (a misaligned 16-byte vector access traps here).
//
// Out-of-bounds accesses are caught by the memory the caller hands in: tests/emu/kernels.py puts every
// tensor argument right before (or right after) an inaccessible page; dynamic shared memory is
// placed the same way here.  A fault prints the kernel, block and thread and ends the process.
#pragma once
#include <signal.h>
#include <sys/mman.h>
#include <ucontext.h>
#include <unistd.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __shared__ static
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))

// ---------------------------------------------------------------------------------------------
// runtime shared by all emulated libraries (tests/emu/emu_rt.cpp, loaded first and globally)
extern "C" {
void emu_rt_enter(const char* kernel);                     // a launch begins
void emu_rt_leave();
void emu_rt_where(unsigned bx, unsigned by, unsigned bz, unsigned tx);   // the fibre that runs now
int emu_rt_schedule_mode();                                // 0 ascending, 1 descending, 2 shuffled
unsigned emu_rt_schedule_seed();
int emu_rt_lds_mode();                                     // 0 at the wait (latest), 1 at issue (earliest)
void* emu_rt_guarded(size_t bytes, int guard_before, size_t keep_alignment_of);   // see emu_rt.cpp
void emu_rt_release(void* p);
void emu_rt_fail(const char* message);                     // prints where, aborts
}

// ---------------------------------------------------------------------------------------------
// types
struct dim3 {
  unsigned x, y, z;
  dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct emu_index {
  unsigned x, y, z;
};
struct alignas(8) float2 { float x, y; };
struct alignas(16) float4 { float x, y, z, w; };
struct alignas(8) uint2 { uint32_t x, y; };
struct alignas(16) uint4 { uint32_t x, y, z, w; };
struct alignas(8) int2 { int32_t x, y; };
struct alignas(16) int4 { int32_t x, y, z, w; };

typedef void* hipStream_t;
enum hipError_t { hipSuccess = 0, hipErrorUnknown = 999 };
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize = 8 };
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipFuncSetAttribute(const void*, hipFuncAttribute, int) { return hipSuccess; }
inline hipError_t hipGetDevice(int* device) {
  *device = 0;
  return hipSuccess;
}
// a __device__ variable is an ordinary one here: its name is its address
#define HIP_SYMBOL(x) x
inline hipError_t hipGetSymbolAddress(void** address, const void* symbol) {
  *address = const_cast<void*>(symbol);
  return hipSuccess;
}

namespace {

emu_index threadIdx, blockIdx;
dim3 blockDim, gridDim;

constexpr int EMU_WAVE = 64;
constexpr int EMU_MAX_THREADS = 1024;
constexpr size_t EMU_STACK_BYTES = 256 * 1024;
constexpr int EMU_XCHG_WORDS = 8;

struct EmuPendingLoad {
  const void* src;
  void* dst;
};

struct EmuThread {
  ucontext_t context;
  bool done = true;
  int wait_kind = 0;          // 0 none, 1 block barrier, 2 wave exchange
  uint64_t wait_generation = 0;
  unsigned tx = 0;
  int lane = 0, wave = 0;
  unsigned collectives = 0;   // parity picks the exchange buffer
  std::vector<EmuPendingLoad> lds_loads;
};

struct EmuWave {
  int live = 0, arrived = 0;
  uint64_t generation = 0;
  bool lane_live[EMU_WAVE];
  uint32_t words[2][EMU_WAVE][EMU_XCHG_WORDS];
  int kind[2][EMU_WAVE];
  unsigned stamp[2][EMU_WAVE];    // which operation of its thread a lane's words belong to
};

struct EmuState {
  ucontext_t scheduler;
  EmuThread threads[EMU_MAX_THREADS];
  EmuWave waves[EMU_MAX_THREADS / EMU_WAVE];
  char* stacks = nullptr;
  int num_threads = 0, live = 0, block_arrived = 0;
  uint64_t block_generation = 0;
  EmuThread* current = nullptr;
  const std::function<void()>* body = nullptr;
  char* dynamic_shared = nullptr;
  size_t dynamic_bytes = 0;
  const char* kernel = "";
} emu;

inline void emu_yield() { swapcontext(&emu.current->context, &emu.scheduler); }

inline void emu_complete_lds(EmuThread* t, size_t leave) {
  const size_t n = t->lds_loads.size();
  if (n <= leave) return;
  for (size_t i = 0; i < n - leave; ++i)
    if (t->lds_loads[i].dst) memcpy(t->lds_loads[i].dst, t->lds_loads[i].src, 16);      // a load into registers: counted only
  t->lds_loads.erase(t->lds_loads.begin(), t->lds_loads.begin() + (n - leave));
}

inline void emu_block_barrier(bool completes_loads) {
  EmuThread* t = emu.current;
  if (completes_loads) emu_complete_lds(t, 0);
  const uint64_t generation = emu.block_generation;
  if (++emu.block_arrived == emu.live) {
    emu.block_arrived = 0;
    ++emu.block_generation;
    return;
  }
  t->wait_kind = 1;
  t->wait_generation = generation;
  while (emu.block_generation == generation) emu_yield();
  t->wait_kind = 0;
}

inline void emu_wave_sync() {
  EmuThread* t = emu.current;
  EmuWave& w = emu.waves[t->wave];
  const uint64_t generation = w.generation;
  if (++w.arrived == w.live) {
    w.arrived = 0;
    ++w.generation;
    return;
  }
  t->wait_kind = 2;
  t->wait_generation = generation;
  while (w.generation == generation) emu_yield();
  t->wait_kind = 0;
}

// Every live lane of the wavefront leaves `n` words and gets the table of all lanes' words.  Two
// buffers take turns, so one synchronisation per operation is enough: nobody can reach the operation
// after the next before everybody has read this one.
inline const uint32_t (*emu_exchange(int kind, const uint32_t* mine, int n))[EMU_XCHG_WORDS] {
  EmuThread* t = emu.current;
  EmuWave& w = emu.waves[t->wave];
  const unsigned count = ++t->collectives;
  const int buffer = count & 1;
  memcpy(w.words[buffer][t->lane], mine, sizeof(uint32_t) * n);
  w.kind[buffer][t->lane] = kind;
  w.stamp[buffer][t->lane] = count;
  emu_wave_sync();
  for (int l = 0; l < EMU_WAVE; ++l)
    if (w.stamp[buffer][l] == count && w.kind[buffer][l] != kind)
      emu_rt_fail("the lanes of a wavefront arrived at different cross-lane operations");
  return w.words[buffer];
}

// Whether `lane` took part in the operation this thread has just been through.  (A lane that has
// returned since - the threads of a wavefront do not run in lockstep here - still counts.)
inline bool emu_lane_live(int lane) {
  if (lane < 0 || lane >= EMU_WAVE) return false;
  const EmuThread* t = emu.current;
  return emu.waves[t->wave].stamp[t->collectives & 1][lane] == t->collectives;
}

inline void emu_thread_exit(EmuThread* t) {
  emu_complete_lds(t, 0);
  t->done = true;
  --emu.live;
  EmuWave& w = emu.waves[t->wave];
  w.lane_live[t->lane] = false;
  --w.live;
  // the rest may have been waiting for this thread only
  if (w.live > 0 && w.arrived == w.live) {
    w.arrived = 0;
    ++w.generation;
  }
  if (emu.live > 0 && emu.block_arrived == emu.live) {
    emu.block_arrived = 0;
    ++emu.block_generation;
  }
}

inline void emu_trampoline() {
  EmuThread* t = emu.current;
  (*emu.body)();
  emu_thread_exit(t);
}

inline bool emu_runnable(const EmuThread& t) {
  if (t.done) return false;
  if (t.wait_kind == 1) return emu.block_generation != t.wait_generation;
  if (t.wait_kind == 2) return emu.waves[t.wave].generation != t.wait_generation;
  return true;
}

inline void emu_run_block(unsigned threads) {
  if (!emu.stacks) {
    emu.stacks = static_cast<char*>(mmap(nullptr, EMU_STACK_BYTES * EMU_MAX_THREADS, PROT_READ | PROT_WRITE,
                                         MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0));
    if (emu.stacks == MAP_FAILED) emu_rt_fail("no memory for the fibres' stacks");
  }
  emu.num_threads = static_cast<int>(threads);
  emu.live = emu.num_threads;
  emu.block_arrived = 0;
  const int waves = (emu.num_threads + EMU_WAVE - 1) / EMU_WAVE;
  for (int w = 0; w < waves; ++w) {
    EmuWave& wave = emu.waves[w];
    wave.live = 0;
    wave.arrived = 0;
    for (int l = 0; l < EMU_WAVE; ++l) {
      wave.lane_live[l] = false;
      wave.stamp[0][l] = wave.stamp[1][l] = 0;
    }
  }
  if (emu.dynamic_bytes) memset(emu.dynamic_shared, 0xff, emu.dynamic_bytes);   // not-a-number / -1: no stale zeros
  for (int i = 0; i < emu.num_threads; ++i) {
    EmuThread& t = emu.threads[i];
    t.done = false;
    t.wait_kind = 0;
    t.tx = static_cast<unsigned>(i);
    t.lane = i % EMU_WAVE;
    t.wave = i / EMU_WAVE;
    t.collectives = 0;
    t.lds_loads.clear();
    emu.waves[t.wave].lane_live[t.lane] = true;
    ++emu.waves[t.wave].live;
    getcontext(&t.context);
    t.context.uc_stack.ss_sp = emu.stacks + EMU_STACK_BYTES * i;
    t.context.uc_stack.ss_size = EMU_STACK_BYTES;
    t.context.uc_link = &emu.scheduler;
    makecontext(&t.context, emu_trampoline, 0);
  }
  std::vector<int> order(emu.num_threads);
  for (int i = 0; i < emu.num_threads; ++i) order[i] = i;
  const int mode = emu_rt_schedule_mode();
  if (mode == 1) {
    for (int i = 0; i < emu.num_threads; ++i) order[i] = emu.num_threads - 1 - i;
  } else if (mode == 2) {
    uint64_t s = emu_rt_schedule_seed() * 6364136223846793005ull + blockIdx.x * 1442695040888963407ull + 1;
    for (int i = emu.num_threads - 1; i > 0; --i) {
      s = s * 6364136223846793005ull + 1442695040888963407ull;
      const int j = static_cast<int>((s >> 33) % static_cast<uint64_t>(i + 1));
      const int tmp = order[i];
      order[i] = order[j];
      order[j] = tmp;
    }
  }
  while (emu.live > 0) {
    bool progress = false;
    for (int k = 0; k < emu.num_threads; ++k) {
      EmuThread& t = emu.threads[order[k]];
      if (!emu_runnable(t)) continue;
      progress = true;
      emu.current = &t;
      threadIdx.x = t.tx;
      threadIdx.y = threadIdx.z = 0;
      emu_rt_where(blockIdx.x, blockIdx.y, blockIdx.z, t.tx);
      swapcontext(&emu.scheduler, &t.context);
    }
    if (!progress)
      emu_rt_fail("deadlock: some threads of a block wait at a barrier or a cross-lane operation that the "
                  "others never reach");
  }
  emu.current = nullptr;
}

// kernel<<<grid, block, shared, stream>>>(args...) becomes emu_launch("kernel", grid, block, shared, [&] { kernel(args...); })
template <typename Body>
inline void emu_launch(const char* kernel, dim3 grid, dim3 block, size_t shared_bytes, Body&& body) {
  if (block.y != 1 || block.z != 1) emu_rt_fail("only one-dimensional blocks are emulated");
  if (block.x == 0 || block.x > EMU_MAX_THREADS) emu_rt_fail("a block has 1 to 1024 threads");
  if (grid.x == 0 || grid.y == 0 || grid.z == 0) emu_rt_fail("an empty grid was launched");
  if (shared_bytes > 160 * 1024) emu_rt_fail("more dynamic shared memory than a CU has");
  emu_rt_enter(kernel);
  emu.kernel = kernel;
  const std::function<void()> fn = body;
  emu.body = &fn;
  emu.dynamic_bytes = shared_bytes;
  // dynamic shared memory ends right before an inaccessible page, and its addresses keep their
  // meaning when cut to 32 bits (the runtime hands out such memory)
  emu.dynamic_shared = shared_bytes ? static_cast<char*>(emu_rt_guarded(shared_bytes, 0, 16)) : nullptr;
  blockDim = block;
  gridDim = grid;
  for (unsigned z = 0; z < grid.z; ++z)
    for (unsigned y = 0; y < grid.y; ++y)
      for (unsigned x = 0; x < grid.x; ++x) {
        blockIdx.x = x;
        blockIdx.y = y;
        blockIdx.z = z;
        emu_run_block(block.x);
      }
  if (emu.dynamic_shared) emu_rt_release(emu.dynamic_shared);
  emu.dynamic_shared = nullptr;
  emu.body = nullptr;
  emu_rt_leave();
}
template <typename Body>
inline void emu_launch(const char* kernel, dim3 grid, dim3 block, size_t shared_bytes, hipStream_t, Body&& body) {
  emu_launch(kernel, grid, block, shared_bytes, static_cast<Body&&>(body));
}
template <typename Body>
inline void emu_launch(const char* kernel, dim3 grid, dim3 block, Body&& body) {
  emu_launch(kernel, grid, block, 0, static_cast<Body&&>(body));
}

inline void* emu_dynamic_shared() { return emu.dynamic_shared; }

}  // namespace

// ---------------------------------------------------------------------------------------------
// device functions of the HIP headers that the kernels use
inline void __syncthreads() { emu_block_barrier(true); }      // the real one waits for all memory operations first
inline void emu_s_barrier() { emu_block_barrier(false); }     // the bare instruction does not

inline uint32_t __float_as_uint(float f) { return __builtin_bit_cast(uint32_t, f); }
inline float __uint_as_float(uint32_t u) { return __builtin_bit_cast(float, u); }
inline int __popcll(uint64_t v) { return __builtin_popcountll(v); }
inline float __expf(float x) { return expf(x); }
inline float rsqrtf(float x) { return 1.0f / sqrtf(x); }
inline int min(int a, int b) { return a < b ? a : b; }
inline int max(int a, int b) { return a > b ? a : b; }
inline unsigned min(unsigned a, unsigned b) { return a < b ? a : b; }
inline unsigned max(unsigned a, unsigned b) { return a > b ? a : b; }
inline long long min(long long a, long long b) { return a < b ? a : b; }
inline long long max(long long a, long long b) { return a > b ? a : b; }
inline long min(long a, long b) { return a < b ? a : b; }
inline long max(long a, long b) { return a > b ? a : b; }
inline float min(float a, float b) { return fminf(a, b); }
inline float max(float a, float b) { return fmaxf(a, b); }

inline int atomicAdd(int* p, int v) {
  const int old = *p;
  *p = old + v;
  return old;
}
inline unsigned long long atomicAdd(unsigned long long* p, unsigned long long v) {
  const unsigned long long old = *p;
  *p = old + v;
  return old;
}

enum { EMU_OP_SHFL = 1, EMU_OP_BALLOT, EMU_OP_DPP, EMU_OP_SWAP16, EMU_OP_SWAP32, EMU_OP_MFMA };

inline uint32_t emu_read_lane(int kind, uint32_t mine, int source) {
  const auto table = emu_exchange(kind, &mine, 1);
  return emu_lane_live(source) ? table[source][0] : mine;
}
inline uint32_t emu_word(float v) { return __float_as_uint(v); }
inline uint32_t emu_word(int v) { return static_cast<uint32_t>(v); }
inline uint32_t emu_word(unsigned v) { return v; }
inline void emu_unword(uint32_t w, float& v) { v = __uint_as_float(w); }
inline void emu_unword(uint32_t w, int& v) { v = static_cast<int>(w); }
inline void emu_unword(uint32_t w, unsigned& v) { v = w; }

template <typename T>
inline T __shfl(T v, int source, int width = EMU_WAVE) {
  const int lane = emu.current->lane;
  const int from = (lane & ~(width - 1)) + (source & (width - 1));
  T out;
  emu_unword(emu_read_lane(EMU_OP_SHFL, emu_word(v), from), out);
  return out;
}
template <typename T>
inline T __shfl_xor(T v, int mask, int width = EMU_WAVE) {
  const int lane = emu.current->lane;
  int from = lane ^ mask;
  if ((from & ~(width - 1)) != (lane & ~(width - 1))) from = lane;
  T out;
  emu_unword(emu_read_lane(EMU_OP_SHFL, emu_word(v), from), out);
  return out;
}
template <typename T>
inline T __shfl_up(T v, unsigned delta, int width = EMU_WAVE) {
  const int lane = emu.current->lane;
  int from = lane - static_cast<int>(delta);
  if (from < (lane & ~(width - 1))) from = lane;
  T out;
  emu_unword(emu_read_lane(EMU_OP_SHFL, emu_word(v), from), out);
  return out;
}
inline uint64_t __ballot(int predicate) {
  const uint32_t mine = predicate ? 1u : 0u;
  const auto table = emu_exchange(EMU_OP_BALLOT, &mine, 1);
  uint64_t mask = 0;
  for (int l = 0; l < EMU_WAVE; ++l)
    if (emu_lane_live(l) && table[l][0]) mask |= 1ull << l;
  return mask;
}
inline uint64_t emu_ballot_w64(bool predicate) { return __ballot(predicate); }

// v_mov_b32 with a DPP control: the patterns the kernels use (bound_ctrl off, all rows and banks)
inline int emu_update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
  if (row_mask != 0xf || bank_mask != 0xf || bound_ctrl) emu_rt_fail("DPP masks other than 0xf are not emulated");
  const int lane = emu.current->lane;
  int from;
  if (ctrl >= 0 && ctrl <= 0xff) from = (lane & ~3) + ((ctrl >> (2 * (lane & 3))) & 3);      // quad_perm
  else if (ctrl == 0x140) from = (lane & ~15) + 15 - (lane & 15);                              // row_mirror
  else if (ctrl == 0x141) from = (lane & ~7) + 7 - (lane & 7);                                 // row_half_mirror
  else {
    emu_rt_fail("this DPP control is not emulated");
    from = lane;
  }
  const uint32_t mine = static_cast<uint32_t>(src);
  const auto table = emu_exchange(EMU_OP_DPP, &mine, 1);
  return emu_lane_live(from) ? static_cast<int>(table[from][0]) : old;
}

typedef unsigned emu_pair __attribute__((ext_vector_type(2)));
// v_permlane16_swap: odd rows of 16 lanes of the first operand change places with even rows of the
// second; element 0 of the result is the first operand afterwards, element 1 the second
inline emu_pair emu_permlane16_swap(unsigned first, unsigned second, bool, bool) {
  const int lane = emu.current->lane;
  const uint32_t mine[2] = {first, second};
  const auto table = emu_exchange(EMU_OP_SWAP16, mine, 2);
  emu_pair out = {first, second};
  const bool odd_row = (lane >> 4) & 1;
  if (odd_row && emu_lane_live(lane - 16)) out[0] = table[lane - 16][1];
  if (!odd_row && emu_lane_live(lane + 16)) out[1] = table[lane + 16][0];
  return out;
}
// v_permlane32_swap: the upper half of the first operand changes places with the lower half of the second
inline emu_pair emu_permlane32_swap(unsigned first, unsigned second, bool, bool) {
  const int lane = emu.current->lane;
  const uint32_t mine[2] = {first, second};
  const auto table = emu_exchange(EMU_OP_SWAP32, mine, 2);
  emu_pair out = {first, second};
  if (lane >= 32 && emu_lane_live(lane - 32)) out[0] = table[lane - 32][1];
  if (lane < 32 && emu_lane_live(lane + 32)) out[1] = table[lane + 32][0];
  return out;
}

inline float emu_bf16_to_float(uint16_t bits) { return __uint_as_float(static_cast<uint32_t>(bits) << 16); }

// D = A x B + C with A 16 x 32 and B 32 x 16 in bfloat16, C and D 16 x 16 in float.  Lane l holds
// A[l % 16][8 (l / 16) .. + 7], B[8 (l / 16) .. + 7][l % 16] and D[4 (l / 16) .. + 3][l % 16].
template <typename AB, typename CD>
inline CD emu_mfma_f32_16x16x32_bf16(AB a, AB b, CD c, int, int, int) {
  static_assert(sizeof(AB) == 16 && sizeof(CD) == 16, "operands are eight bfloat16, results four floats");
  uint32_t mine[8];
  memcpy(mine, &a, 16);
  memcpy(mine + 4, &b, 16);
  const auto table = emu_exchange(EMU_OP_MFMA, mine, 8);
  const int lane = emu.current->lane;
  const int n = lane & 15, g = lane >> 4;
  float cd[4];
  memcpy(cd, &c, 16);
  for (int i = 0; i < 4; ++i) {
    const int m = 4 * g + i;
    float sum = cd[i];
    for (int kg = 0; kg < 4; ++kg) {
      const uint16_t* arow = reinterpret_cast<const uint16_t*>(table[16 * kg + m]);        // A[m][8 kg ..]
      const uint16_t* bcol = reinterpret_cast<const uint16_t*>(table[16 * kg + n] + 4);    // B[8 kg ..][n]
      for (int j = 0; j < 8; ++j) sum = fmaf(emu_bf16_to_float(arow[j]), emu_bf16_to_float(bcol[j]), sum);
    }
    cd[i] = sum;
  }
  CD out;
  memcpy(&out, cd, 16);
  return out;
}

// global_load_lds_dwordx4: lane l's 16 bytes go to (wave-uniform) lds_address + 16 l
inline void emu_load16_to_lds(const void* src, uint32_t lds_address) {
  EmuThread* t = emu.current;
  const uintptr_t high = reinterpret_cast<uintptr_t>(emu.dynamic_shared) & ~static_cast<uintptr_t>(0xffffffffu);
  char* dst = reinterpret_cast<char*>(high | lds_address) + 16 * t->lane;
  if (dst < emu.dynamic_shared || dst + 16 > emu.dynamic_shared + emu.dynamic_bytes)
    emu_rt_fail("a load into shared memory lands outside the block's dynamic shared memory");
  volatile char probe = *static_cast<const volatile char*>(src);   // an address that cannot be read faults at issue
  (void)probe;
  probe = static_cast<const volatile char*>(src)[15];
  if (emu_rt_lds_mode() == 1) {
    memcpy(dst, src, 16);
    return;
  }
  t->lds_loads.push_back({src, dst});
}
// A load into registers of a kernel that waits by hand (SE_NOTE_VECTOR_LOAD): it takes its place in the queue
// that s_waitcnt counts, as on the chip, and has nothing to do when it completes.
inline void emu_note_vector_load() {
  if (emu_rt_lds_mode() != 1) emu.current->lds_loads.push_back({nullptr, nullptr});
}
#define SE_NOTE_VECTOR_LOAD() emu_note_vector_load()
// s_waitcnt: only the count of vector memory operations matters here (bits 3:0 and 15:14)
inline void emu_s_waitcnt(int imm) {
  const size_t vmcnt = static_cast<size_t>((imm & 0xf) | (((imm >> 14) & 0x3) << 4));
  emu_complete_lds(emu.current, vmcnt);
}

inline float emu_max_bare(float a, float b) { return fmaxf(a, b); }
inline float emu_max3_bare(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }

#define __builtin_amdgcn_mfma_f32_16x16x32_bf16 emu_mfma_f32_16x16x32_bf16
#define __builtin_amdgcn_update_dpp emu_update_dpp
#define __builtin_amdgcn_permlane16_swap emu_permlane16_swap
#define __builtin_amdgcn_permlane32_swap emu_permlane32_swap
#define __builtin_amdgcn_readfirstlane(x) (x)      /* the kernels use it on wave-uniform values only */
#define __builtin_amdgcn_ballot_w64 emu_ballot_w64
#define __builtin_amdgcn_exp2f exp2f
#define __builtin_amdgcn_s_waitcnt emu_s_waitcnt
#define __builtin_amdgcn_s_barrier emu_s_barrier
#define __builtin_amdgcn_s_setprio(level) ((void)(level))     // a hint to the instruction arbiter, nothing to emulate
