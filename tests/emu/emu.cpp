// Lockstep CPU emulator for the gfx950 kernels of thrust_amd/csrc (see include/hip/hip_runtime.h
// in this directory for what a kernel sees).  TEST INFRASTRUCTURE ONLY.
//
// Execution model
//   * By default a launch runs its workgroups one after the other on the calling thread (in launch
//     order; emu_set_workgroup_order can reverse or shuffle it for kernels that never wait without
//     bound for another workgroup).
//   * emu_set_resident_workgroups(k, seed) with k > 1 keeps k workgroups in flight, dispatched in
//     launch order as the hardware does: each runs on a thread of its own (LDS is thread-local
//     storage), ONE thread runs at a time, and the turn passes to a workgroup chosen by the seeded
//     generator whenever the running one has released a barrier or slept.  This is how the tests see
//     tiles whose predecessors have published a partial result, or nothing yet.
//   * Every lane of a workgroup is a fiber with a stack of its own.  A lane runs until it reaches an
//     operation that involves other lanes, parks there, and the scheduler goes on with the next lane.
//   * When every lane of a wavefront is parked (or has returned), the scheduler serves ONE group of
//     parked lanes — the lanes parked at the same instruction (same call site) — and lets them run on:
//       - atomics first, lowest address first: an atomic needs nothing from lanes that do not execute
//         it, and the lanes of one instruction are served in lane order;
//       - last the cross-lane operation with the lowest code address.  Lanes that left a loop early or
//         skipped a branch are parked further down the code, so the group that is still inside goes
//         first, with exactly the lanes the hardware would have enabled in EXEC;
//       - s_sleep parks the wavefront until every other wavefront of the workgroup (and, with several
//         workgroups in flight, another workgroup) has had a turn.  Lanes that sleep are polling in
//         a loop that the rest of the wavefront has left already; the rest waits for them at the
//         point where the hardware would reconverge, so sleepers go before cross-lane operations;
//       - a workgroup barrier is released when every lane that has not returned is parked at one.
//   * A cross-lane read from a lane that does not take part (it is outside the group) behaves like a
//     read from a lane that EXEC disables: DPP keeps `old`, ds_bpermute and readlane give 0.
//
// Not modelled: interleavings finer than a barrier interval, memory ordering, timing, LDS capacity,
// registers.
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>

#include <algorithm>
#include <condition_variable>
#include <mutex>
#include <thread>
#include <vector>

#include <hip/hip_runtime.h>

#if !defined(__x86_64__) || !defined(__linux__)
#error "the emulator's context switch is written for x86-64 Linux (System V calling convention)"
#endif
// ---- context switch: callee-saved registers on the fiber's own stack (SysV x86-64) ----
extern "C" void emu_switch(void** save_sp, void* load_sp);
asm(R"(
.text
.globl emu_switch
.type emu_switch,@function
emu_switch:
  pushq %rbp
  pushq %rbx
  pushq %r12
  pushq %r13
  pushq %r14
  pushq %r15
  movq %rsp, (%rdi)
  movq %rsi, %rsp
  popq %r15
  popq %r14
  popq %r13
  popq %r12
  popq %rbx
  popq %rbp
  ret
.size emu_switch, .-emu_switch
)");

// ---- race detection (a build with -fsanitize=thread) ----
// ThreadSanitizer sees every WAVEFRONT of the running workgroup as a thread of its own (a "fiber" of
// its interface; the lanes of a wavefront share it, so accesses inside a wavefront are ordered as
// the hardware orders them, by program order).  Switching between lanes tells it nothing
// (no_sync); the only happens-before edges are the ones the kernel itself creates: a workgroup
// barrier, the start and the end of a workgroup (a launch orders everything before it and after
// it), and atomics, which the emulator performs as real atomic operations.  Two wavefronts that
// touch the same LDS or global location without a barrier between them are then a reported race,
// whatever order the emulator happened to run them in.
// (This file itself is compiled WITHOUT the sanitizer, with -DEMU_TSAN: the scheduler's own
// bookkeeping is no part of what is checked, and the atomics it performs for the lanes need no
// report.  Only the calls into the sanitizer's fiber interface are made from here.)
#if defined(EMU_TSAN)
extern "C" {
void* __tsan_get_current_fiber(void);
void* __tsan_create_fiber(unsigned flags);
void __tsan_destroy_fiber(void* fiber);
void __tsan_switch_to_fiber(void* fiber, unsigned flags);
void __tsan_acquire(void* addr);
void __tsan_release(void* addr);
}
#define EMU_TSAN_ONLY(...) __VA_ARGS__
#else
#define EMU_TSAN_ONLY(...)
#endif

namespace emu {

enum Op : int {
  kRun = 0,  // not parked
  kDpp,
  kBpermute,
  kReadlane,
  kReadfirst,
  kBallot,
  kShuffle,
  kWaveBarrier,
  kAtomicAdd32,
  kAtomicAdd64,
  kAtomicOr32,
  kLoad,
  kStore,
  kSleep,
  kWorkgroupBarrier,
  kDone,
};
static bool is_atomic(int op) { return op >= kAtomicAdd32 && op <= kStore; }
static bool is_cross_lane(int op) { return op >= kDpp && op <= kWaveBarrier; }

struct Lane {
  void* sp = nullptr;
  void* stack_top = nullptr;
  LaneView view;
  int op = kRun;
  const void* site = nullptr;  // return address of the call that parked the lane
  long depth = 0;              // and how deep in its stack the lane was: the same call of the source, reached
                               // through another caller of a function that was not inlined, is another operation
  int a[5] = {0, 0, 0, 0, 0};
  bool flag = false;
  void* ptr = nullptr;
  uint64_t val = 0;
  uint64_t result = 0;
  bool slept = false;  // parked at s_sleep and already counted for this round
};

constexpr size_t kStackBytes = 256 << 10;
constexpr int kMaxLanes = 1024;
constexpr int kWave = 64;

// per thread: the workgroup that the thread runs
static thread_local char* g_stacks = nullptr;
static thread_local Lane* g_lanes = nullptr;
static thread_local Lane* g_cur = nullptr;
static thread_local void* g_sched_sp = nullptr;
static LaneView g_host_view = {};
static void (*g_trampoline)(void*) = nullptr;
static void* g_closure = nullptr;
static uint64_t g_clock = 0;
static int g_order = 0;          // 0 launch order, 1 reversed, 2 shuffled
static uint64_t g_order_seed = 1;
static int g_resident = 1;       // workgroups in flight
static bool g_resident_set = false;
static uint64_t g_resident_seed = 1;

// the turn among the threads of a launch with several workgroups in flight
static std::mutex g_turn_mu;
static std::condition_variable g_turn_cv;
static int g_turn = -1;               // index of the thread that may run
static std::vector<char> g_alive;     // per thread of the launch
static thread_local int g_self = -1;  // index of this thread in the launch, -1 on the caller's thread
static uint64_t g_turn_rng = 1;
static uint64_t g_turns_passed = 0;

static void wait_for_turn() {
  std::unique_lock<std::mutex> lk(g_turn_mu);
  g_turn_cv.wait(lk, [] { return g_turn == g_self; });
}
// hands the turn to a live thread chosen at random (possibly this one); `leaving` when this thread
// has no workgroup left
static void pass_turn(bool leaving) {
  if (g_self < 0) return;
  {
    std::lock_guard<std::mutex> lk(g_turn_mu);
    if (leaving) g_alive[(size_t)g_self] = 0;
    int live = 0;
    for (char a : g_alive) live += a;
    if (live == 0) {
      g_turn = -1;
    } else {
      g_turn_rng = g_turn_rng * 6364136223846793005ull + 1442695040888963407ull;
      int pick = (int)((g_turn_rng >> 33) % (uint64_t)live);
      for (size_t i = 0; i < g_alive.size(); i++)
        if (g_alive[i] && pick-- == 0) g_turn = (int)i;
    }
    g_turns_passed++;
  }
  g_turn_cv.notify_all();
  if (!leaving) wait_for_turn();
}
static uint64_t g_divergent_cross_lane = 0;  // cross-lane groups served while other lanes waited elsewhere
static uint64_t g_launches = 0, g_workgroups = 0;

LaneView& view() { return g_cur ? g_cur->view : g_host_view; }
int lane() { return (int)(g_cur - g_lanes) % kWave; }
uint64_t clock() { return g_clock += 100; }

#if defined(EMU_TSAN)
constexpr unsigned kNoSync = 1u;  // __tsan_switch_to_fiber_no_sync
static thread_local void* g_sched_fiber = nullptr;
static thread_local void* g_wave_fiber[kMaxLanes / kWave];
// addresses that stand for the orderings: a barrier; the start of a workgroup (released by the
// scheduler, acquired by every lane); its end (released by every lane, acquired by the scheduler)
static thread_local char g_barrier_token, g_start_token, g_end_token;
static void* fiber_of(const Lane* l) { return g_wave_fiber[(l - g_lanes) / kWave]; }
#endif

static void park(int op, const void* site, const void* frame) {
  Lane* me = g_cur;
  me->op = op;
  me->site = site;
  me->depth = static_cast<const char*>(me->stack_top) - static_cast<const char*>(frame);
  EMU_TSAN_ONLY(if (op == kWorkgroupBarrier) __tsan_release(&g_barrier_token);)
  EMU_TSAN_ONLY(__tsan_switch_to_fiber(g_sched_fiber, kNoSync);)
  emu_switch(&me->sp, g_sched_sp);
  EMU_TSAN_ONLY(if (op == kWorkgroupBarrier) __tsan_acquire(&g_barrier_token);)
}

#define EMU_SITE __builtin_extract_return_addr(__builtin_return_address(0)), __builtin_frame_address(0)

__attribute__((noinline)) int dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
  Lane* me = g_cur;
  me->a[0] = old, me->a[1] = src, me->a[2] = ctrl, me->a[3] = row_mask, me->a[4] = bank_mask, me->flag = bound_ctrl;
  park(kDpp, EMU_SITE);
  return (int)me->result;
}
__attribute__((noinline)) int bpermute(int byte_address, int src) {
  Lane* me = g_cur;
  me->a[0] = byte_address, me->a[1] = src;
  park(kBpermute, EMU_SITE);
  return (int)me->result;
}
__attribute__((noinline)) int shuffle(int v, int src_lane) {
  Lane* me = g_cur;
  me->a[0] = v, me->a[1] = src_lane;
  park(kShuffle, EMU_SITE);
  return (int)me->result;
}
__attribute__((noinline)) int readlane(int v, int l) {
  Lane* me = g_cur;
  me->a[0] = v, me->a[1] = l;
  park(kReadlane, EMU_SITE);
  return (int)me->result;
}
__attribute__((noinline)) int readfirstlane(int v) {
  Lane* me = g_cur;
  me->a[0] = v;
  park(kReadfirst, EMU_SITE);
  return (int)me->result;
}
__attribute__((noinline)) uint64_t ballot(bool pred) {
  Lane* me = g_cur;
  me->flag = pred;
  park(kBallot, EMU_SITE);
  return me->result;
}
__attribute__((noinline)) void wave_barrier() { park(kWaveBarrier, EMU_SITE); }
__attribute__((noinline)) void workgroup_barrier() { park(kWorkgroupBarrier, EMU_SITE); }
__attribute__((noinline)) void sleep() { park(kSleep, EMU_SITE); }
__attribute__((noinline)) uint32_t atomic_add_u32(uint32_t* p, uint32_t v) {
  if (!g_cur) {  // host code
    const uint32_t o = *p;
    *p = o + v;
    return o;
  }
  Lane* me = g_cur;
  me->ptr = p, me->val = v;
  park(kAtomicAdd32, EMU_SITE);
  return (uint32_t)me->result;
}
__attribute__((noinline)) uint64_t atomic_add_u64(uint64_t* p, uint64_t v) {
  if (!g_cur) {
    const uint64_t o = *p;
    *p = o + v;
    return o;
  }
  Lane* me = g_cur;
  me->ptr = p, me->val = v;
  park(kAtomicAdd64, EMU_SITE);
  return me->result;
}
__attribute__((noinline)) uint32_t atomic_or_u32(uint32_t* p, uint32_t v) {
  if (!g_cur) {
    const uint32_t o = *p;
    *p = o | v;
    return o;
  }
  Lane* me = g_cur;
  me->ptr = p, me->val = v;
  park(kAtomicOr32, EMU_SITE);
  return (uint32_t)me->result;
}

__attribute__((noinline)) uint64_t lockstep_load(const void* p, int bytes) {
  Lane* me = g_cur;
  me->ptr = const_cast<void*>(p), me->a[0] = bytes;
  park(kLoad, EMU_SITE);
  return me->result;
}
__attribute__((noinline)) void lockstep_store(void* p, uint64_t v, int bytes) {
  Lane* me = g_cur;
  me->ptr = p, me->val = v, me->a[0] = bytes;
  park(kStore, EMU_SITE);
}

// ---- serving one group of lanes of a wavefront ----
static int dpp_source(int l, int ctrl) {  // source lane of lane l, or -1 when there is none
  const int row = l & ~15, in_row = l & 15;
  if (ctrl >= 0x000 && ctrl <= 0x0ff) return (l & ~3) | ((ctrl >> (2 * (l & 3))) & 3);
  if (ctrl >= 0x101 && ctrl <= 0x10f) return in_row + (ctrl & 15) < 16 ? l + (ctrl & 15) : -1;
  if (ctrl >= 0x111 && ctrl <= 0x11f) return in_row - (ctrl & 15) >= 0 ? l - (ctrl & 15) : -1;
  if (ctrl >= 0x121 && ctrl <= 0x12f) return row | ((in_row - (ctrl & 15)) & 15);
  switch (ctrl) {
    case 0x130: return l + 1 < kWave ? l + 1 : -1;  // wave_shl:1
    case 0x134: return (l + 1) & 63;                 // wave_rol:1
    case 0x138: return l - 1;                        // wave_shr:1 (-1 for lane 0)
    case 0x13c: return (l - 1) & 63;                 // wave_ror:1
    case 0x140: return row | (15 - in_row);          // row_mirror
    case 0x141: return (l & ~7) | (7 - (l & 7));     // row_half_mirror
    case 0x142: return l >= 16 ? row - 1 : -1;       // row_bcast:15
    case 0x143: return l >= 32 ? 31 : -1;            // row_bcast:31
  }
  fprintf(stderr, "emu: DPP control 0x%x is not modelled\n", ctrl);
  abort();
}

static void serve(Lane* w, int nl, int op, const void* site, long depth) {
  bool in[kWave];
  for (int l = 0; l < kWave; l++) in[l] = l < nl && w[l].op == op && w[l].site == site && w[l].depth == depth;
  EMU_TSAN_ONLY(__tsan_switch_to_fiber(fiber_of(w), kNoSync);)  // the memory operations below are the wavefront's
  switch (op) {
    case kDpp:
      for (int l = 0; l < kWave; l++) {
        if (!in[l]) continue;
        const int s = dpp_source(l, w[l].a[2]);
        const bool enabled = ((w[l].a[3] >> (l >> 4)) & 1) && ((w[l].a[4] >> ((l >> 2) & 3)) & 1);
        if (!enabled) w[l].result = (uint32_t)w[l].a[0];
        else if (s >= 0 && in[s]) w[l].result = (uint32_t)w[s].a[1];
        else w[l].result = w[l].flag ? 0u : (uint32_t)w[l].a[0];
      }
      break;
    case kBpermute:
      for (int l = 0; l < kWave; l++) {
        if (!in[l]) continue;
        const int s = (w[l].a[0] >> 2) & 63;
        w[l].result = in[s] ? (uint32_t)w[s].a[1] : 0u;
      }
      break;
    case kReadlane:
      for (int l = 0; l < kWave; l++) {
        if (!in[l]) continue;
        const int s = w[l].a[1] & 63;
        // v_readlane reads the register of the lane whatever EXEC says; a lane that is not parked
        // here has no value to give, which the emulator reports as 0
        w[l].result = in[s] ? (uint32_t)w[s].a[0] : 0u;
      }
      break;
    case kShuffle:
      for (int l = 0; l < kWave; l++) {
        if (!in[l]) continue;
        const int s = w[l].a[1] & 63;
        w[l].result = (uint32_t)(in[s] ? w[s].a[0] : w[l].a[0]);
      }
      break;
    case kReadfirst: {
      int first = 0;
      while (!in[first]) first++;
      for (int l = 0; l < kWave; l++)
        if (in[l]) w[l].result = (uint32_t)w[first].a[0];
      break;
    }
    case kBallot: {
      uint64_t m = 0;
      for (int l = 0; l < kWave; l++)
        if (in[l] && w[l].flag) m |= 1ull << l;
      for (int l = 0; l < kWave; l++)
        if (in[l]) w[l].result = m;
      break;
    }
    case kWaveBarrier:
    case kSleep:
      break;
    case kAtomicAdd32:
      for (int l = 0; l < kWave; l++) {
        if (!in[l]) continue;
        w[l].result = __atomic_fetch_add(static_cast<uint32_t*>(w[l].ptr), (uint32_t)w[l].val, __ATOMIC_RELAXED);
      }
      break;
    case kAtomicAdd64:
      for (int l = 0; l < kWave; l++) {
        if (!in[l]) continue;
        w[l].result = __atomic_fetch_add(static_cast<uint64_t*>(w[l].ptr), w[l].val, __ATOMIC_RELAXED);
      }
      break;
    case kLoad:
      for (int l = 0; l < kWave; l++) {
        if (!in[l]) continue;
        w[l].result = 0;
        memcpy(&w[l].result, w[l].ptr, (size_t)w[l].a[0]);
      }
      break;
    case kStore:
      for (int l = 0; l < kWave; l++)
        if (in[l]) memcpy(w[l].ptr, &w[l].val, (size_t)w[l].a[0]);
      break;
    case kAtomicOr32:
      for (int l = 0; l < kWave; l++) {
        if (!in[l]) continue;
        w[l].result = __atomic_fetch_or(static_cast<uint32_t*>(w[l].ptr), (uint32_t)w[l].val, __ATOMIC_RELAXED);
      }
      break;
  }
  EMU_TSAN_ONLY(__tsan_switch_to_fiber(g_sched_fiber, kNoSync);)
  for (int l = 0; l < kWave; l++)
    if (in[l]) w[l].op = kRun;
}

extern "C" void emu_lane_main() {
  EMU_TSAN_ONLY(__tsan_acquire(&g_start_token);)  // everything before the launch happened before this lane
  g_trampoline(g_closure);
  Lane* me = g_cur;
  me->op = kDone;
  EMU_TSAN_ONLY(__tsan_release(&g_end_token);)
  EMU_TSAN_ONLY(__tsan_switch_to_fiber(g_sched_fiber, kNoSync);)
  emu_switch(&me->sp, g_sched_sp);
  abort();  // a finished lane is never resumed
}

static void run_lane(Lane* l) {
  g_cur = l;
  EMU_TSAN_ONLY(__tsan_switch_to_fiber(fiber_of(l), kNoSync);)
  emu_switch(&g_sched_sp, l->sp);
  g_cur = nullptr;
}

static void run_workgroup(dim3 grid, dim3 block, unsigned bx, unsigned by, unsigned bz) {
  if (!g_stacks) {
    void* m = mmap(nullptr, kStackBytes * kMaxLanes, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (m == MAP_FAILED) { perror("emu: mmap"); abort(); }
    g_stacks = static_cast<char*>(m);
    g_lanes = new Lane[kMaxLanes];
  }
  const int nthreads = (int)(block.x * block.y * block.z);
  const int nwaves = (nthreads + kWave - 1) / kWave;
#if defined(EMU_TSAN)
  g_sched_fiber = __tsan_get_current_fiber();
  for (int wv = 0; wv < nwaves; wv++) g_wave_fiber[wv] = __tsan_create_fiber(0);
  __tsan_release(&g_start_token);
#endif
  for (int t = 0; t < nthreads; t++) {
    Lane& l = g_lanes[t];
    l = Lane();
    l.view.thread = {t % block.x, (t / block.x) % block.y, t / (block.x * block.y)};
    l.view.block = {bx, by, bz};
    l.view.block_dim = {block.x, block.y, block.z};
    l.view.grid_dim = {grid.x, grid.y, grid.z};
    // a fresh fiber: six zeroed callee-saved registers, then the entry point as return address;
    // the stack pointer is 8 modulo 16 when emu_lane_main starts, as after a call
    uint64_t* top = reinterpret_cast<uint64_t*>(g_stacks + (size_t)(t + 1) * kStackBytes);
    *--top = 0;  // a zero return address above the entry frame
    *--top = reinterpret_cast<uint64_t>(&emu_lane_main);
    for (int i = 0; i < 6; i++) *--top = 0;
    l.sp = top;
    l.stack_top = g_stacks + (size_t)(t + 1) * kStackBytes;
  }
  for (;;) {
    bool all_done = true;
    for (int wv = 0; wv < nwaves; wv++) {
      Lane* w = g_lanes + wv * kWave;
      const int nl = std::min(kWave, nthreads - wv * kWave);
      for (int l = 0; l < nl; l++)  // lanes that slept through the last round wake up together
        if (w[l].op == kSleep && w[l].slept) w[l].op = kRun, w[l].slept = false;
      for (;;) {
        for (int l = 0; l < nl; l++)
          while (w[l].op == kRun) run_lane(&w[l]);
        // every lane of the wavefront is parked or done: choose the group to serve
        int best = -1;
        for (int l = 0; l < nl; l++) {
          const int op = w[l].op;
          if (op == kDone || op == kWorkgroupBarrier) continue;
          if (best < 0) { best = l; continue; }
          // atomics before sleepers before cross-lane operations, lowest address within a class
          const int a = is_atomic(op) ? 0 : (op == kSleep ? 1 : 2);
          const int b = is_atomic(w[best].op) ? 0 : (w[best].op == kSleep ? 1 : 2);
          if (a != b ? a < b : w[l].site < w[best].site) best = l;
        }
        if (best < 0) break;  // the wavefront waits at the workgroup barrier, or has returned
        const int op = w[best].op;
        const void* site = w[best].site;
        const long depth = w[best].depth;
        if (op == kSleep) {
          for (int l = 0; l < nl; l++)
            if (w[l].op == kSleep && w[l].site == site && w[l].depth == depth) w[l].slept = true;
          break;  // the other wavefronts get their turn first
        }
        if (is_cross_lane(op))
          for (int l = 0; l < nl; l++)
            if (is_cross_lane(w[l].op) && (w[l].site != site || w[l].depth != depth)) { g_divergent_cross_lane++; break; }
        serve(w, nl, op, site, depth);
      }
      for (int l = 0; l < nl; l++) all_done &= w[l].op == kDone;
    }
    if (all_done) break;
    pass_turn(false);  // another workgroup in flight may run up to its next barrier or sleep
    bool asleep = false, at_barrier = false;
    for (int t = 0; t < nthreads; t++) asleep |= g_lanes[t].op == kSleep, at_barrier |= g_lanes[t].op == kWorkgroupBarrier;
    if (asleep) continue;  // sleepers go on before the barrier is looked at again
    if (at_barrier)
      for (int t = 0; t < nthreads; t++)
        if (g_lanes[t].op == kWorkgroupBarrier) g_lanes[t].op = kRun;
  }
#if defined(EMU_TSAN)
  __tsan_acquire(&g_end_token);  // what the workgroup did happened before whatever follows the launch
  for (int wv = 0; wv < nwaves; wv++) __tsan_destroy_fiber(g_wave_fiber[wv]);
#endif
}

void launch(dim3 grid, dim3 block, void (*trampoline)(void*), void* closure) {
  if (g_cur) { fprintf(stderr, "emu: launch from device code\n"); abort(); }
  const size_t nthreads = (size_t)block.x * block.y * block.z;
  if (nthreads == 0 || nthreads > kMaxLanes) { fprintf(stderr, "emu: workgroup of %zu lanes\n", nthreads); abort(); }
  g_trampoline = trampoline;
  g_closure = closure;
  g_launches++;
  const uint64_t total = (uint64_t)grid.x * grid.y * grid.z;
  std::vector<uint64_t> order(total);
  for (uint64_t i = 0; i < total; i++) order[i] = i;
  if (g_order == 1) std::reverse(order.begin(), order.end());
  if (g_order == 2) {
    uint64_t s = g_order_seed;
    for (uint64_t i = total; i > 1; i--) {
      s = s * 6364136223846793005ull + 1442695040888963407ull;
      std::swap(order[i - 1], order[(s >> 33) % i]);
    }
  }
  auto run = [&](uint64_t i) {
    const uint64_t b = order[i];
    run_workgroup(grid, block, (unsigned)(b % grid.x), (unsigned)((b / grid.x) % grid.y), (unsigned)(b / ((uint64_t)grid.x * grid.y)));
    g_workgroups++;
  };
  // programs that do not call emu_set_resident_workgroups (the C++ tests) take it from the environment
  static const bool from_environment = [] {
    const char* e = getenv("THRUST_CDNA4_EMULATED_RESIDENT");  // "k" or "k:seed"
    if (e && !g_resident_set) {
      g_resident = std::max(1, std::min(64, atoi(e)));
      const char* colon = strchr(e, ':');
      g_resident_seed = colon && atoll(colon + 1) ? (uint64_t)atoll(colon + 1) : 1;
    }
    return true;
  }();
  (void)from_environment;
  const int k = (int)std::min<uint64_t>((uint64_t)g_resident, total);
  if (k <= 1) {
    for (uint64_t i = 0; i < total; i++) run(i);
    return;
  }
  // The threads are kept from launch to launch: a new thread's first touch of LDS makes the C
  // library build the thread's copy of every kernel's LDS variables, tens of megabytes.
  struct Pool {
    std::mutex mu;
    std::condition_variable cv;
    std::vector<std::thread> threads;
    uint64_t generation = 0;
    int wanted = 0, finished = 0;
    void (*job)(void*, int) = nullptr;
    void* arg = nullptr;
  };
  static Pool* pool = new Pool;  // never destroyed: its threads outlive static destructors
  struct Job {
    uint64_t next = 0, total;  // `next` is touched by the thread whose turn it is only
    decltype(run)* run_one;
  } job_state{0, total, &run};
  auto body = [](void* a, int t) {
    Job* j = static_cast<Job*>(a);
    g_self = t;
    wait_for_turn();
    while (j->next < j->total) (*j->run_one)(j->next++);
    pass_turn(true);
    g_self = -1;
  };
  g_alive.assign((size_t)k, 1);
  g_turn_rng = g_resident_seed;
  g_turn = 0;
  {
    std::unique_lock<std::mutex> lk(pool->mu);
    while ((int)pool->threads.size() < k) {
      const int t = (int)pool->threads.size();
      pool->threads.emplace_back([t] {
        uint64_t seen = 0;
        for (;;) {
          void (*fn)(void*, int);
          void* arg;
          {
            std::unique_lock<std::mutex> lk2(pool->mu);
            pool->cv.wait(lk2, [&] { return pool->generation != seen && t < pool->wanted; });
            seen = pool->generation;
            fn = pool->job, arg = pool->arg;
          }
          fn(arg, t);
          {
            std::lock_guard<std::mutex> lk2(pool->mu);
            pool->finished++;
          }
          pool->cv.notify_all();
        }
      });
      pool->threads.back().detach();
    }
    pool->job = body, pool->arg = &job_state, pool->wanted = k, pool->finished = 0;
    pool->generation++;
    pool->cv.notify_all();
    pool->cv.wait(lk, [&] { return pool->finished == k; });
    pool->wanted = 0;
  }
}

}  // namespace emu

// ---- controls for the tests ----
extern "C" {
// 0: launch order; 1: last workgroup first; 2: shuffled with `seed`.  Only kernels that never wait
// without bound for another workgroup may be run out of order.
void emu_set_workgroup_order(int order, uint64_t seed) {
  emu::g_order = order;
  emu::g_order_seed = seed ? seed : 1;
}
// Workgroups in flight (1: one after the other on the calling thread) and the seed of the generator
// that chooses which of them runs next.
void emu_set_resident_workgroups(int k, uint64_t seed) {
  emu::g_resident = k < 1 ? 1 : (k > 64 ? 64 : k);
  emu::g_resident_set = true;
  emu::g_resident_seed = seed ? seed : 1;
}
uint64_t emu_turns_passed() { return emu::g_turns_passed; }
uint64_t emu_divergent_cross_lane_groups() { return emu::g_divergent_cross_lane; }
uint64_t emu_launches() { return emu::g_launches; }
uint64_t emu_workgroups() { return emu::g_workgroups; }
}
