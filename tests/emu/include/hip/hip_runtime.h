// CPU stand-in for <hip/hip_runtime.h>, for TESTS ONLY.
//
// Putting this directory ahead of /opt/rocm/include lets the library's own
// .hip sources be compiled, unchanged, as ordinary C++ for the host, so that
// their indexing, bounds and arithmetic can be exercised (and run under
// AddressSanitizer) on a machine without a GPU.  It is a SIMT emulator, not a
// port: every lane of a workgroup is a fibre (ucontext) with its own stack;
// lanes run until they reach a cross-lane operation (__shfl_xor, DPP, readlane,
// ballot, MFMA) or __syncthreads(), where they wait for the other lanes of
// their 64-wide wavefront / their workgroup, exactly like the hardware's
// lock-step semantics for convergent code.  Workgroups are independent and run
// on a few OS threads.
//
// Only what the kernels of this repository use is provided.  The product
// never includes this file: libexact_hip.so is built by hipcc against the real
// HIP headers, and nothing under exact_amd/ refers to the emulator.
#pragma once

#include <ucontext.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <thread>
#include <vector>

#if defined(__has_feature)
#if __has_feature(address_sanitizer)
#define HIPEMU_ASAN 1
#include <sanitizer/common_interface_defs.h>
#endif
#endif

// ---- qualifiers --------------------------------------------------------------
#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __shared__ static thread_local
#define HIP_DYNAMIC_SHARED(type, var) type* var = reinterpret_cast<type*>(hipemu::dyn_shared());
// the kernels pin an fp32 value in a register before converting it to fp16; here that is an SSE register
#define EXACT_VALUE_BARRIER(r) asm("" : "+x"(r))

// ---- vector types ------------------------------------------------------------
struct float2 { float x, y; };
struct float4 { float x, y, z, w; };
struct uint2 { uint32_t x, y; };
struct uint3 { uint32_t x, y, z; };
static inline float2 make_float2(float x, float y) { return {x, y}; }
static inline float4 make_float4(float x, float y, float z, float w) { return {x, y, z, w}; }
static inline uint2 make_uint2(uint32_t x, uint32_t y) { return {x, y}; }
struct dim3 {
  uint32_t x, y, z;
  dim3(uint32_t x_ = 1, uint32_t y_ = 1, uint32_t z_ = 1) : x(x_), y(y_), z(z_) {}
};

typedef int hipError_t;
typedef void* hipStream_t;
constexpr hipError_t hipSuccess = 0;
static inline hipError_t hipGetLastError() { return hipSuccess; }
// one emulated device; a small CU count keeps the persistent kernels' grids small here
enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount = 63 };
static inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
static inline hipError_t hipDeviceGetAttribute(int* v, hipDeviceAttribute_t, int) { *v = 2; return hipSuccess; }
static inline const char* hipGetErrorString(hipError_t) { return "hip emulator: no error"; }

using std::max;
using std::min;

namespace hipemu {

constexpr int kWaveSize = 64;
constexpr size_t kStackBytes = 64 * 1024;
constexpr size_t kDynSharedBytes = 64 * 1024;

struct WaveState {
  uint64_t gen = 0;
  int arrived = 0;
  int active = 0;
  uint64_t mask[2] = {0, 0};
  uint64_t slot[2][kWaveSize];
};

struct LaneState {
  ucontext_t ctx;
  char* stack = nullptr;
  bool done = false;
  uint3 tid;
#ifdef HIPEMU_ASAN
  void* fake_stack = nullptr;
#endif
};

struct BlockState {
  int nthreads = 0;
  int remaining = 0;
  uint3 bid, bdim, gdim;
  std::vector<LaneState> lanes;
  std::vector<WaveState> waves;
  uint64_t block_gen = 0;
  int block_arrived = 0;
  ucontext_t sched;
  const std::function<void()>* body = nullptr;
  int cur = 0;
  uint64_t progress = 0;
#ifdef HIPEMU_ASAN
  const void* sched_stack_bottom = nullptr;
  size_t sched_stack_size = 0;
  void* sched_fake_stack = nullptr;
#endif
};

inline thread_local BlockState* g_block = nullptr;
inline thread_local char* g_dyn_shared = nullptr;

inline char* dyn_shared() { return g_dyn_shared; }
inline const uint3& cur_tid() { return g_block->lanes[g_block->cur].tid; }
inline const uint3& cur_bid() { return g_block->bid; }
inline const uint3& cur_bdim() { return g_block->bdim; }
inline const uint3& cur_gdim() { return g_block->gdim; }

inline void switch_to_sched(LaneState& me, bool dying) {
  BlockState* b = g_block;
#ifdef HIPEMU_ASAN
  __sanitizer_start_switch_fiber(dying ? nullptr : &me.fake_stack, b->sched_stack_bottom, b->sched_stack_size);
#endif
  swapcontext(&me.ctx, &b->sched);
#ifdef HIPEMU_ASAN
  __sanitizer_finish_switch_fiber(me.fake_stack, &b->sched_stack_bottom, &b->sched_stack_size);
#endif
  (void)dying;
}

inline void yield() { switch_to_sched(g_block->lanes[g_block->cur], false); }

// Every not-yet-finished lane of the calling lane's wavefront deposits `mine`;
// returns the buffer index holding all deposits once the last lane has arrived.
inline int wave_collect(uint64_t mine, WaveState*& w_out, int& lane_out) {
  BlockState* b = g_block;
  const int t = b->cur;
  WaveState& w = b->waves[t / kWaveSize];
  const int lane = t % kWaveSize;
  const int buf = static_cast<int>(w.gen & 1);
  w.slot[buf][lane] = mine;
  w.mask[buf] |= (uint64_t{1} << lane);
  const uint64_t my_gen = w.gen;
  ++w.arrived;
  ++b->progress;
  if (w.arrived >= w.active) {
    w.arrived = 0;
    w.mask[buf ^ 1] = 0;
    ++w.gen;
  } else {
    while (w.gen == my_gen) yield();
  }
  w_out = &w;
  lane_out = lane;
  return buf;
}

inline void lane_exit() {
  BlockState* b = g_block;
  const int t = b->cur;
  LaneState& me = b->lanes[t];
  WaveState& w = b->waves[t / kWaveSize];
  me.done = true;
  --w.active;
  --b->remaining;
  ++b->progress;
  if (w.arrived > 0 && w.arrived >= w.active) {  // the lanes still waiting are now complete
    const int buf = static_cast<int>(w.gen & 1);
    w.arrived = 0;
    w.mask[buf ^ 1] = 0;
    ++w.gen;
  }
  if (b->block_arrived > 0 && b->block_arrived >= b->remaining) {
    b->block_arrived = 0;
    ++b->block_gen;
  }
  switch_to_sched(me, true);
}

inline void trampoline() {
  BlockState* b = g_block;
#ifdef HIPEMU_ASAN
  __sanitizer_finish_switch_fiber(nullptr, &b->sched_stack_bottom, &b->sched_stack_size);
#endif
  (*b->body)();
  lane_exit();
}

inline void run_block(BlockState& b, std::vector<char>& stacks) {
  g_block = &b;
  b.remaining = b.nthreads;
  b.block_gen = 0;
  b.block_arrived = 0;
  const int nwaves = (b.nthreads + kWaveSize - 1) / kWaveSize;
  b.waves.assign(nwaves, WaveState());
  for (int t = 0; t < b.nthreads; ++t) {
    LaneState& l = b.lanes[t];
    l.done = false;
    l.tid = {static_cast<uint32_t>(t % b.bdim.x), static_cast<uint32_t>((t / b.bdim.x) % b.bdim.y),
             static_cast<uint32_t>(t / (b.bdim.x * b.bdim.y))};
    l.stack = stacks.data() + static_cast<size_t>(t) * kStackBytes;
    getcontext(&l.ctx);
    l.ctx.uc_stack.ss_sp = l.stack;
    l.ctx.uc_stack.ss_size = kStackBytes;
    l.ctx.uc_link = nullptr;
    makecontext(&l.ctx, reinterpret_cast<void (*)()>(trampoline), 0);
    b.waves[t / kWaveSize].active++;
  }
  while (b.remaining > 0) {
    const uint64_t before = b.progress;
    for (int t = 0; t < b.nthreads; ++t) {
      if (b.lanes[t].done) continue;
      b.cur = t;
#ifdef HIPEMU_ASAN
      __sanitizer_start_switch_fiber(&b.sched_fake_stack, b.lanes[t].stack, kStackBytes);
#endif
      swapcontext(&b.sched, &b.lanes[t].ctx);
#ifdef HIPEMU_ASAN
      __sanitizer_finish_switch_fiber(b.sched_fake_stack, nullptr, nullptr);
#endif
    }
    if (b.progress == before) {
      std::fprintf(stderr, "hip emulator: deadlock in block (%u,%u): lanes wait at a barrier or cross-lane "
                           "operation that other live lanes of the wavefront/workgroup never reach\n",
                   b.bid.x, b.bid.y);
      std::abort();
    }
  }
  g_block = nullptr;
}

inline int g_threads_override = 0;

inline void launch(dim3 grid, dim3 block, size_t shmem, const std::function<void()>& body) {
  const int64_t nblocks = static_cast<int64_t>(grid.x) * grid.y * grid.z;
  const int nthreads = static_cast<int>(block.x * block.y * block.z);
  if (nblocks == 0 || nthreads == 0) return;
  if (shmem > kDynSharedBytes) {
    std::fprintf(stderr, "hip emulator: %zu bytes of dynamic shared memory requested\n", shmem);
    std::abort();
  }
  int workers = g_threads_override > 0 ? g_threads_override : static_cast<int>(std::thread::hardware_concurrency());
  if (const char* e = std::getenv("HIPEMU_THREADS")) workers = std::atoi(e);
  workers = static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(workers, nblocks)));
  std::atomic<int64_t> next{0};
  auto worker = [&]() {
    std::vector<char> stacks(static_cast<size_t>(nthreads) * kStackBytes);
    std::vector<char> dyn(std::max<size_t>(shmem, 16));  // exactly what the launch asked for: the sanitizer sees an overrun
    g_dyn_shared = dyn.data();
    BlockState b;
    b.nthreads = nthreads;
    b.lanes.resize(nthreads);
    b.body = &body;
    b.bdim = {block.x, block.y, block.z};
    b.gdim = {grid.x, grid.y, grid.z};
    for (;;) {
      const int64_t i = next.fetch_add(1);
      if (i >= nblocks) break;
      b.bid = {static_cast<uint32_t>(i % grid.x), static_cast<uint32_t>((i / grid.x) % grid.y),
               static_cast<uint32_t>(i / (static_cast<int64_t>(grid.x) * grid.y))};
      run_block(b, stacks);
    }
    g_dyn_shared = nullptr;
  };
  if (workers == 1) {
    worker();
  } else {
    std::vector<std::thread> pool;
    for (int i = 0; i < workers; ++i) pool.emplace_back(worker);
    for (auto& th : pool) th.join();
  }
}

// ---- cross-lane operations ---------------------------------------------------
inline uint32_t shfl_xor_u32(uint32_t v, int m) {
  WaveState* w;
  int lane;
  const int buf = wave_collect(v, w, lane);
  const int src = lane ^ m;
  if (src < 0 || src >= kWaveSize || !((w->mask[buf] >> src) & 1)) return v;
  return static_cast<uint32_t>(w->slot[buf][src]);
}

// __shfl with the default width: every lane names the lane it reads (ds_bpermute)
inline uint32_t shfl_u32(uint32_t v, int src) {
  WaveState* w;
  int lane;
  const int buf = wave_collect(v, w, lane);
  src &= kWaveSize - 1;
  if (!((w->mask[buf] >> src) & 1)) return v;
  return static_cast<uint32_t>(w->slot[buf][src]);
}

inline uint32_t readlane_u32(uint32_t v, int src) {
  WaveState* w;
  int lane;
  const int buf = wave_collect(v, w, lane);
  if (src < 0 || src >= kWaveSize || !((w->mask[buf] >> src) & 1)) {
    std::fprintf(stderr, "hip emulator: readlane from inactive lane %d\n", src);
    std::abort();
  }
  return static_cast<uint32_t>(w->slot[buf][src]);
}

inline uint32_t readfirstlane_u32(uint32_t v) {
  WaveState* w;
  int lane;
  const int buf = wave_collect(v, w, lane);
  return static_cast<uint32_t>(w->slot[buf][__builtin_ctzll(w->mask[buf])]);
}

inline uint64_t ballot(bool pred) {
  WaveState* w;
  int lane;
  const int buf = wave_collect(pred ? 1 : 0, w, lane);
  uint64_t out = 0;
  for (int l = 0; l < kWaveSize; ++l)
    if (((w->mask[buf] >> l) & 1) && w->slot[buf][l]) out |= uint64_t{1} << l;
  return out;
}

// DPP controls the kernels use: quad_perm (0x00..0xFF), row_ror:8 (0x128, the
// only rotation whose direction does not matter), row_mirror (0x140),
// row_half_mirror (0x141).  bound_ctrl = true: an inactive source reads as 0.
inline int mov_dpp(int v, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
  WaveState* w;
  int lane;
  const int buf = wave_collect(static_cast<uint32_t>(v), w, lane);
  if (row_mask != 0xF || bank_mask != 0xF || !bound_ctrl) {
    std::fprintf(stderr, "hip emulator: unsupported DPP masks\n");
    std::abort();
  }
  int src;
  if (ctrl >= 0 && ctrl <= 0xFF) src = (lane & ~3) | ((ctrl >> (2 * (lane & 3))) & 3);
  else if (ctrl == 0x128) src = (lane & ~15) | ((lane + 8) & 15);
  else if (ctrl == 0x140) src = (lane & ~15) | (15 - (lane & 15));
  else if (ctrl == 0x141) src = (lane & ~7) | (7 - (lane & 7));
  else {
    std::fprintf(stderr, "hip emulator: unsupported DPP control 0x%x\n", ctrl);
    std::abort();
  }
  if (!((w->mask[buf] >> src) & 1)) return 0;
  return static_cast<int>(static_cast<uint32_t>(w->slot[buf][src]));
}

inline float update_dpp_f32(float v, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
  int bits;
  std::memcpy(&bits, &v, 4);
  bits = mov_dpp(bits, ctrl, row_mask, bank_mask, bound_ctrl);
  std::memcpy(&v, &bits, 4);
  return v;
}

inline int update_dpp_i32(int v, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
  return mov_dpp(v, ctrl, row_mask, bank_mask, bound_ctrl);
}
inline float update_dpp_any(float v, int c, int rm, int bm, bool bc) { return update_dpp_f32(v, c, rm, bm, bc); }
inline int update_dpp_any(int v, int c, int rm, int bm, bool bc) { return update_dpp_i32(v, c, rm, bm, bc); }

// v_med3_f32: the median; with a NaN among the operands, v_min3_f32 of them
// (each v_min_f32 step returns the operand that is not a NaN)
inline float fmed3(float a, float b, float c) {
  if (std::isnan(a) || std::isnan(b) || std::isnan(c)) return std::fmin(std::fmin(a, b), c);
  const float hi = std::fmax(std::fmax(a, b), c);
  if (hi == a) return std::fmax(b, c);
  if (hi == b) return std::fmax(a, c);
  return std::fmax(a, b);
}

// v_perm_b32: byte i of the result is byte sel[i] of the eight bytes {hi, lo}
// (0..3 = lo, 4..7 = hi); 8..11 replicate a sign bit, 12 gives 0x00, above 0xFF
inline uint32_t byte_perm(uint32_t hi, uint32_t lo, uint32_t sel) {
  const uint64_t pool = (static_cast<uint64_t>(hi) << 32) | lo;
  uint32_t out = 0;
  for (int i = 0; i < 4; ++i) {
    const uint32_t s = (sel >> (8 * i)) & 0xFFu;
    uint32_t byte;
    if (s < 8) byte = static_cast<uint32_t>(pool >> (8 * s)) & 0xFFu;
    else if (s < 12) byte = ((pool >> (16 * (s - 8) + 15)) & 1u) ? 0xFFu : 0u;
    else byte = s == 12 ? 0u : 0xFFu;
    out |= byte << (8 * i);
  }
  return out;
}

// v_bitop3_b32: bit i of the result = truth table bit ((a_i << 2) | (b_i << 1) | c_i)
inline uint32_t bitop3(uint32_t a, uint32_t b, uint32_t c, int table) {
  uint32_t out = 0;
  for (int i = 0; i < 32; ++i) {
    const int idx = (((a >> i) & 1) << 2) | (((b >> i) & 1) << 1) | ((c >> i) & 1);
    out |= static_cast<uint32_t>((table >> idx) & 1) << i;
  }
  return out;
}

typedef float floatx16_t __attribute__((ext_vector_type(16)));

// v_mfma_f32_32x32x2_f32: A-operand lane l = A[l % 32][l / 32], B-operand lane l
// = B[l / 32][l % 32]; accumulator register v of lane l is
// C[8 * (v / 4) + 4 * (l / 32) + v % 4][l % 32].
inline floatx16_t mfma_f32_32x32x2f32(float a, float b, floatx16_t c, int, int, int) {
  uint32_t ab[2];
  std::memcpy(&ab[0], &a, 4);
  std::memcpy(&ab[1], &b, 4);
  WaveState* w;
  int lane;
  const int buf = wave_collect(static_cast<uint64_t>(ab[0]) | (static_cast<uint64_t>(ab[1]) << 32), w, lane);
  if (w->mask[buf] != ~uint64_t{0}) {
    std::fprintf(stderr, "hip emulator: MFMA with inactive lanes\n");
    std::abort();
  }
  auto a_of = [&](int l) { float f; uint32_t u = static_cast<uint32_t>(w->slot[buf][l]); std::memcpy(&f, &u, 4); return f; };
  auto b_of = [&](int l) { float f; uint32_t u = static_cast<uint32_t>(w->slot[buf][l] >> 32); std::memcpy(&f, &u, 4); return f; };
  const int j = lane % 32;
  for (int v = 0; v < 16; ++v) {
    const int i = 8 * (v / 4) + 4 * (lane / 32) + (v % 4);
    float acc = c[v];
    acc = std::fmaf(a_of(i), b_of(j), acc);
    acc = std::fmaf(a_of(i + 32), b_of(j + 32), acc);
    c[v] = acc;
  }
  return c;
}

// v_mfma_f32_32x32x16_bf16: lane l holds row (A) / column (B) l % 32 and the eight
// k-slots 8 * (l / 32) .. + 7 as bf16; accumulator layout as for 32x32x2.  The
// products of two bf16 numbers are exact in fp32; they are added one after the
// other in fp32 (the hardware's own order is not specified, so tests compare
// against float64 with a tolerance, and launches that must agree bit for bit
// with each other go through this same routine).
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
inline floatx16_t mfma_f32_32x32x16_bf16(bf16x8_t a, bf16x8_t b, floatx16_t c, int, int, int) {
  uint64_t words[4];
  std::memcpy(&words[0], &a, 16);
  std::memcpy(&words[2], &b, 16);
  uint64_t all[4][64];
  WaveState* w = nullptr;
  int lane = 0;
  for (int q = 0; q < 4; ++q) {
    const int buf = wave_collect(words[q], w, lane);
    if (w->mask[buf] != ~uint64_t{0}) {
      std::fprintf(stderr, "hip emulator: MFMA with inactive lanes\n");
      std::abort();
    }
    for (int l = 0; l < 64; ++l) all[q][l] = w->slot[buf][l];
  }
  auto element = [&](int base, int l, int e) {      // bf16 element e (0..7) of lane l's operand -> float
    const uint64_t word = all[base + e / 4][l];
    const uint32_t bits = static_cast<uint32_t>((word >> (16 * (e % 4))) & 0xFFFFu) << 16;
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
  };
  const int j = lane % 32;
  for (int v = 0; v < 16; ++v) {
    const int i = 8 * (v / 4) + 4 * (lane / 32) + (v % 4);
    float acc = c[v];
    for (int kk = 0; kk < 16; ++kk) acc = std::fmaf(element(0, i + 32 * (kk / 8), kk % 8), element(2, j + 32 * (kk / 8), kk % 8), acc);
    c[v] = acc;
  }
  return c;
}

inline void syncthreads() {
  BlockState* b = g_block;
  const uint64_t my_gen = b->block_gen;
  ++b->block_arrived;
  ++b->progress;
  if (b->block_arrived >= b->remaining) {
    b->block_arrived = 0;
    ++b->block_gen;
  } else {
    while (b->block_gen == my_gen) yield();
  }
}

inline void atomic_add_f32(float* p, float v) {
  uint32_t* u = reinterpret_cast<uint32_t*>(p);
  uint32_t old = __atomic_load_n(u, __ATOMIC_RELAXED);
  for (;;) {
    float f;
    std::memcpy(&f, &old, 4);
    f += v;
    uint32_t nu;
    std::memcpy(&nu, &f, 4);
    if (__atomic_compare_exchange_n(u, &old, nu, false, __ATOMIC_RELAXED, __ATOMIC_RELAXED)) return;
  }
}

template <typename F>
inline void launch_fn(dim3 grid, dim3 block, size_t shmem, F&& f) {
  const std::function<void()> body = std::forward<F>(f);
  launch(grid, block, shmem, body);
}

}  // namespace hipemu

#define threadIdx (hipemu::cur_tid())
#define blockIdx (hipemu::cur_bid())
#define blockDim (hipemu::cur_bdim())
#define gridDim (hipemu::cur_gdim())

#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...) \
  hipemu::launch_fn((grid), (block), (shmem), [&]() { kernel(__VA_ARGS__); })

static inline void __syncthreads() { hipemu::syncthreads(); }
static inline float __shfl_xor(float v, int m) {
  uint32_t u;
  std::memcpy(&u, &v, 4);
  u = hipemu::shfl_xor_u32(u, m);
  std::memcpy(&v, &u, 4);
  return v;
}
static inline uint32_t __shfl_xor(uint32_t v, int m) { return hipemu::shfl_xor_u32(v, m); }
static inline int __shfl_xor(int v, int m) { return static_cast<int>(hipemu::shfl_xor_u32(static_cast<uint32_t>(v), m)); }
static inline uint32_t __shfl(uint32_t v, int src) { return hipemu::shfl_u32(v, src); }
static inline uint64_t __ballot(bool p) { return hipemu::ballot(p); }
#define __builtin_amdgcn_readlane(v, l) static_cast<int>(hipemu::readlane_u32(static_cast<uint32_t>(v), (l)))
#define __builtin_amdgcn_readfirstlane(v) static_cast<int>(hipemu::readfirstlane_u32(static_cast<uint32_t>(v)))
#define __builtin_amdgcn_mov_dpp(v, ctrl, rm, bm, bc) hipemu::mov_dpp((v), (ctrl), (rm), (bm), (bc))
#define __builtin_amdgcn_update_dpp(old, v, ctrl, rm, bm, bc) hipemu::update_dpp_any((v), (ctrl), (rm), (bm), (bc))
#define __builtin_amdgcn_bitop3_b32(a, b, c, table) hipemu::bitop3((a), (b), (c), (table))
#define __builtin_amdgcn_perm(hi, lo, sel) hipemu::byte_perm((hi), (lo), (sel))
#define __builtin_amdgcn_fmed3f(a, b, c) hipemu::fmed3((a), (b), (c))
#define __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, x, y, z) hipemu::mfma_f32_32x32x2f32((a), (b), (c), (x), (y), (z))
// every active lane of the wavefront arrives before any goes on (a scheduling barrier on the hardware, where the
// lanes of a wavefront move in lockstep anyway; here the lanes are fibres and must really wait)
#define __builtin_amdgcn_wave_barrier() ((void)hipemu::ballot(true))
#define __builtin_amdgcn_fence(order, scope) ((void)0)
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) hipemu::mfma_f32_32x32x16_bf16((a), (b), (c), (x), (y), (z))

static inline float __fmaf_rn(float a, float b, float c) { return std::fmaf(a, b, c); }
static inline uint32_t __float_as_uint(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
static inline int __float_as_int(float f) { int u; std::memcpy(&u, &f, 4); return u; }
static inline float __uint_as_float(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }
static inline float __int_as_float(int u) { float f; std::memcpy(&f, &u, 4); return f; }
static inline void unsafeAtomicAdd(float* p, float v) { hipemu::atomic_add_f32(p, v); }
