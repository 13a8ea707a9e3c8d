// Host stand-in for csrc/blit_device.h: the blit kernels, compiled unchanged,
// run on the CPU with the lanes of a workgroup in lock step, and every address
// a lane touches is checked against the ranges the command may touch.
//
// Execution model.  A launch runs its workgroups one after the other.  Every
// work-item of a workgroup is a coroutine with a stack of its own; a lane runs
// until it reaches a move between lanes (wave_rotate_down1, lane_read,
// lane_read_up) or a workgroup barrier, deposits its operand and yields; when
// all live lanes of the wave (the workgroup, for a barrier) have arrived, they
// go on and pick up the operand of the lane they read from.  That is the
// meaning those instructions have on a 64-lane wavefront whose lanes are all
// active at the instruction, which is how the kernels use them; a lane that
// reads from one that did not take part in the move is reported as an error,
// and so is a workgroup in which lanes wait for each other for ever.
//
// Memory model.  The accessors go to host memory through check_load() and
// check_store(): the test registers what the command may read and what it may
// write, an access outside (or one that is not aligned the way its instruction
// needs) is counted and described, and is not performed.
//
// x86-64 only (the coroutine switch is a dozen instructions of assembly);
// built with g++, AddressSanitizer optional (the switch is announced to it).
#ifndef MI355_TESTS_LANE_EMULATION_H_
#define MI355_TESTS_LANE_EMULATION_H_

#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>

#include <algorithm>
#include <vector>

#include "blit_args.h"

#if defined(__SANITIZE_ADDRESS__)
#include <sanitizer/common_interface_defs.h>
#define LANE_EMU_ASAN 1
#else
#define LANE_EMU_ASAN 0
#endif

#define MI355_DEVICE static inline
#define MI355_KERNEL(max_wg) extern "C"
// one workgroup runs at a time, so one instance serves
#define MI355_LDS static

namespace lane_emu {

// ---- address checking --------------------------------------------------------

struct Range {
  uintptr_t lo, hi;
};

struct Checker {
  std::vector<Range> readable, writable;  // sorted by lo, disjoint after seal()
  uint64_t loads = 0, stores = 0, violations = 0;
  char first[320] = {0};
  // A deliberate fault for the self test: every dword load is moved by this
  // many bytes.
  intptr_t shift_dword_loads = 0;

  void clear() {
    readable.clear();
    writable.clear();
    loads = stores = violations = 0;
    first[0] = 0;
  }
  void allow_read(const void* p, uint64_t n) {
    if (n) readable.push_back({reinterpret_cast<uintptr_t>(p), reinterpret_cast<uintptr_t>(p) + n});
  }
  void allow_write(void* p, uint64_t n) {
    if (n) writable.push_back({reinterpret_cast<uintptr_t>(p), reinterpret_cast<uintptr_t>(p) + n});
  }
  static void merge(std::vector<Range>* v) {
    std::sort(v->begin(), v->end(), [](const Range& a, const Range& b) { return a.lo < b.lo; });
    size_t k = 0;
    for (size_t i = 0; i < v->size(); ++i) {
      if (k && (*v)[k - 1].hi >= (*v)[i].lo) (*v)[k - 1].hi = std::max((*v)[k - 1].hi, (*v)[i].hi);
      else (*v)[k++] = (*v)[i];
    }
    v->resize(k);
  }
  void seal() {
    merge(&readable);
    merge(&writable);
  }
  static bool inside(const std::vector<Range>& v, uintptr_t p, uint64_t n) {
    // the last range that starts at or below p
    size_t lo = 0, hi = v.size();
    while (lo < hi) {
      const size_t mid = (lo + hi) / 2;
      if (v[mid].lo <= p) lo = mid + 1; else hi = mid;
    }
    return lo && p + n <= v[lo - 1].hi;
  }
};

inline Checker g_check;

// ---- lanes as coroutines -----------------------------------------------------

extern "C" void lane_emu_switch(void** save_sp, void* next_sp);
asm(R"(
.text
.globl lane_emu_switch
.type lane_emu_switch,@function
lane_emu_switch:
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
.size lane_emu_switch,.-lane_emu_switch
)");

constexpr unsigned kMaxWorkgroup = 1024;
constexpr size_t kStackBytes = 128 << 10;

enum LaneState { kReady, kRunning, kAtLaneMove, kAtBarrier, kDone };

struct Lane {
  void* sp;
  LaneState state;
  uint64_t waits_for;  // generation of the wave / workgroup it arrived in
  size_t uniform_calls;
};

struct Wave {
  uint64_t gen;
  unsigned arrived, live;
  uint32_t operand[2][mi355::kWave];
  uint64_t deposited[2];  // lanes that took part in the move, by slot parity
  // values passed to wave_uniform, in call order, by the first lane to get there
  std::vector<uint32_t> uniform_log;
};

struct Machine {
  char* stacks = nullptr;
  Lane lanes[kMaxWorkgroup];
  Wave waves[kMaxWorkgroup / mi355::kWave];
  uint64_t barrier_gen = 0;
  unsigned barrier_arrived = 0, live = 0, size = 0;
  unsigned cur = 0;        // lane that is running
  unsigned workgroup = 0;  // its workgroup
  void* scheduler_sp = nullptr;
  void (*body)(const void*) = nullptr;
  const void* args = nullptr;
  uint64_t errors = 0;
  char first_error[200] = {0};
  uint64_t switches = 0;
#if LANE_EMU_ASAN
  const void* main_bottom = nullptr;
  size_t main_size = 0;
#endif
};

inline Machine g_m;

inline void machine_error(const char* what) {
  if (!g_m.errors++)
    snprintf(g_m.first_error, sizeof g_m.first_error, "%s (workgroup %u, lane %u)", what, g_m.workgroup, g_m.cur);
}

inline char* lane_stack(unsigned t) { return g_m.stacks + static_cast<size_t>(t) * kStackBytes; }

// from a lane back to the scheduler
inline void yield_to_scheduler(bool dying) {
  Lane& l = g_m.lanes[g_m.cur];
  ++g_m.switches;
#if LANE_EMU_ASAN
  void* fake = nullptr;
  __sanitizer_start_switch_fiber(dying ? nullptr : &fake, g_m.main_bottom, g_m.main_size);
#endif
  lane_emu_switch(&l.sp, g_m.scheduler_sp);
#if LANE_EMU_ASAN
  __sanitizer_finish_switch_fiber(fake, &g_m.main_bottom, &g_m.main_size);
#else
  (void)dying;
#endif
}

extern "C" inline void lane_emu_entry() {
#if LANE_EMU_ASAN
  __sanitizer_finish_switch_fiber(nullptr, &g_m.main_bottom, &g_m.main_size);
#endif
  g_m.body(g_m.args);
  g_m.lanes[g_m.cur].state = kDone;
  yield_to_scheduler(true);
  abort();  // a finished lane is never resumed
}

inline void resume_lane(unsigned t) {
  Lane& l = g_m.lanes[t];
  g_m.cur = t;
  if (l.state == kReady) {
    // a fresh stack that "returns" into lane_emu_entry
    uintptr_t top = reinterpret_cast<uintptr_t>(lane_stack(t) + kStackBytes) & ~static_cast<uintptr_t>(15);
    uint64_t* x = reinterpret_cast<uint64_t*>(top - 8);
    x[0] = 0;                                             // where lane_emu_entry would return to
    x[-1] = reinterpret_cast<uint64_t>(&lane_emu_entry);  // popped by the switch's ret
    for (int i = 2; i <= 7; ++i) x[-i] = 0;               // the six callee-saved registers
    l.sp = x - 7;
  }
  l.state = kRunning;
#if LANE_EMU_ASAN
  void* fake = nullptr;
  __sanitizer_start_switch_fiber(&fake, lane_stack(t), kStackBytes);
#endif
  lane_emu_switch(&g_m.scheduler_sp, l.sp);
#if LANE_EMU_ASAN
  __sanitizer_finish_switch_fiber(fake, nullptr, nullptr);
#endif
}

// The calling lane's operand goes into its wave's exchange; returns once all
// live lanes of the wave have deposited theirs, with the slot parity to read.
inline unsigned lane_move_arrive(uint32_t v) {
  const unsigned t = g_m.cur;
  Wave& w = g_m.waves[t / mi355::kWave];
  const uint64_t gen = w.gen;
  if (w.arrived == 0) w.deposited[gen & 1] = 0;
  w.operand[gen & 1][t % mi355::kWave] = v;
  w.deposited[gen & 1] |= 1ull << (t % mi355::kWave);
  if (++w.arrived == w.live) {
    w.arrived = 0;
    ++w.gen;
  } else {
    Lane& l = g_m.lanes[t];
    l.state = kAtLaneMove;
    l.waits_for = gen;
    yield_to_scheduler(false);
  }
  return static_cast<unsigned>(gen & 1);
}

inline uint32_t lane_move_read(unsigned parity, unsigned src_lane) {
  const Wave& w = g_m.waves[g_m.cur / mi355::kWave];
  if (!(w.deposited[parity] >> (src_lane % mi355::kWave) & 1)) {
    machine_error("a lane reads the operand of a lane that did not take part in the move");
    return 0;
  }
  return w.operand[parity][src_lane % mi355::kWave];
}

inline void barrier_arrive() {
  const uint64_t gen = g_m.barrier_gen;
  if (++g_m.barrier_arrived == g_m.live) {
    g_m.barrier_arrived = 0;
    ++g_m.barrier_gen;
  } else {
    Lane& l = g_m.lanes[g_m.cur];
    l.state = kAtBarrier;
    l.waits_for = gen;
    yield_to_scheduler(false);
  }
}

// A lane that returns may be the one the others were waiting for.
inline void retire_lane(unsigned t) {
  Wave& w = g_m.waves[t / mi355::kWave];
  --w.live;
  --g_m.live;
  if (w.live && w.arrived == w.live) {
    w.arrived = 0;
    ++w.gen;
  }
  if (g_m.live && g_m.barrier_arrived == g_m.live) {
    g_m.barrier_arrived = 0;
    ++g_m.barrier_gen;
  }
}

// Runs `grid` workgroups of `wg_size` work-items of kernel(args).
template <typename Args>
void launch(void (*kernel)(Args), const Args& args, unsigned grid, unsigned wg_size) {
  static void (*s_kernel)(Args);
  s_kernel = kernel;
  if (!g_m.stacks) {
    void* p = mmap(nullptr, kStackBytes * kMaxWorkgroup, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE,
                   -1, 0);
    if (p == MAP_FAILED) abort();
    g_m.stacks = static_cast<char*>(p);
  }
  if (wg_size == 0 || wg_size > kMaxWorkgroup || wg_size % mi355::kWave) {
    machine_error("workgroup size is not a multiple of 64 up to 1024");
    return;
  }
  g_m.body = [](const void* a) { s_kernel(*static_cast<const Args*>(a)); };
  g_m.args = &args;
  g_m.size = wg_size;
  for (unsigned b = 0; b < grid; ++b) {
    g_m.workgroup = b;
    g_m.live = wg_size;
    g_m.barrier_arrived = 0;
    for (unsigned t = 0; t < wg_size; ++t) {
      g_m.lanes[t].state = kReady;
      g_m.lanes[t].uniform_calls = 0;
    }
    for (unsigned w = 0; w < wg_size / mi355::kWave; ++w) {
      g_m.waves[w].arrived = 0;
      g_m.waves[w].live = mi355::kWave;
      g_m.waves[w].uniform_log.clear();
    }
    while (g_m.live) {
      bool progressed = false;
      for (unsigned t = 0; t < wg_size; ++t) {
        Lane& l = g_m.lanes[t];
        if (l.state == kDone) continue;
        if (l.state == kAtLaneMove && g_m.waves[t / mi355::kWave].gen == l.waits_for) continue;
        if (l.state == kAtBarrier && g_m.barrier_gen == l.waits_for) continue;
        resume_lane(t);
        progressed = true;
        if (l.state == kDone) retire_lane(t);
      }
      if (!progressed) {
        machine_error("lanes wait for each other for ever (a lane move or barrier not reached by all)");
        return;
      }
    }
  }
}

inline void access_violation(const char* what, uintptr_t p, uint64_t n, const std::vector<Range>& allowed) {
  Checker& c = g_check;
  if (!c.violations++) {
    // the nearest allowed range, for the message
    long long best = 0;
    bool have = false;
    for (const Range& r : allowed) {
      const long long d = p + n > r.hi ? static_cast<long long>(p + n - r.hi) : static_cast<long long>(p) - static_cast<long long>(r.lo);
      if (!have || llabs(d) < llabs(best)) best = d, have = true;
    }
    snprintf(c.first, sizeof c.first,
             "%s of %llu bytes at %#llx, %lld bytes %s the nearest allowed range (workgroup %u, lane %u of %u)", what,
             static_cast<unsigned long long>(n), static_cast<unsigned long long>(p), llabs(best),
             best > 0 ? "beyond the end of" : "below the start of", g_m.workgroup, g_m.cur, g_m.size);
  }
}

inline bool check_load(uintptr_t p, uint64_t n, unsigned align) {
  ++g_check.loads;
  if ((p & (align - 1)) || !Checker::inside(g_check.readable, p, n)) {
    access_violation(p & (align - 1) ? "misaligned load" : "load", p, n, g_check.readable);
    return false;
  }
  return true;
}
inline bool check_store(uintptr_t p, uint64_t n, unsigned align) {
  ++g_check.stores;
  if ((p & (align - 1)) || !Checker::inside(g_check.writable, p, n)) {
    access_violation(p & (align - 1) ? "misaligned store" : "store", p, n, g_check.writable);
    return false;
  }
  return true;
}

template <typename T>
inline T checked_load(const void* p, unsigned align) {
  T v;
  if (check_load(reinterpret_cast<uintptr_t>(p), sizeof(T), align)) memcpy(&v, p, sizeof(T));
  else memset(&v, 0xEB, sizeof(T));
  return v;
}
template <typename T>
inline void checked_store(void* p, const T& v, unsigned align) {
  if (check_store(reinterpret_cast<uintptr_t>(p), sizeof(T), align)) memcpy(p, &v, sizeof(T));
}

}  // namespace lane_emu

// ---- the names csrc/blit_device.h provides -----------------------------------

namespace mi355 {

struct v4u {
  unsigned x, y, z, w;
};
typedef v4u v4u_a4;
typedef v4u v4u_a1;

constexpr int kStoreCached = 0;
constexpr int kStoreNt = 1;
constexpr int kStoreAgentWt = 2;
constexpr int kStoreSystemWt = 3;

// global_load_dwordx4 / global_load_dword: dword aligned
template <bool NT>
MI355_DEVICE v4u ld_v4(const v4u_a4* p) { return lane_emu::checked_load<v4u>(p, 4); }
template <bool NT>
MI355_DEVICE unsigned ld_u32(const unsigned* p) {
  return lane_emu::checked_load<unsigned>(reinterpret_cast<const uint8_t*>(p) + lane_emu::g_check.shift_dword_loads, 4);
}
MI355_DEVICE uint8_t ld_u8(const uint8_t* p) { return lane_emu::checked_load<uint8_t>(p, 1); }
MI355_DEVICE void st_u8(uint8_t* p, uint8_t v) { lane_emu::checked_store(p, v, 1); }
MI355_DEVICE void st_u32(unsigned* p, unsigned v) { lane_emu::checked_store(p, v, 4); }

template <typename T>
MI355_DEVICE T ld_obj(const T* p) { return lane_emu::checked_load<T>(p, alignof(T)); }
template <typename T>
MI355_DEVICE void st_obj(T* p, const T& v) { lane_emu::checked_store(p, v, alignof(T)); }

MI355_DEVICE uint64_t ld_system_u64(const uint64_t* p) { return lane_emu::checked_load<uint64_t>(p, 8); }
MI355_DEVICE uint32_t ld_system_u32(const uint32_t* p) { return lane_emu::checked_load<uint32_t>(p, 4); }
MI355_DEVICE void st_system_u64(uint64_t* p, uint64_t v) { lane_emu::checked_store(p, v, 8); }

// the kernels' body stores are 16-byte aligned; the _at / _any forms take any address
template <int POLICY>
MI355_DEVICE void st_v4(v4u* p, v4u v) { lane_emu::checked_store(p, v, 16); }
template <int POLICY>
MI355_DEVICE void st_v4_at(uintptr_t p, v4u v) { lane_emu::checked_store(reinterpret_cast<void*>(p), v, 1); }
template <bool NT>
MI355_DEVICE v4u ld_v4_any(const uint8_t* p) { return lane_emu::checked_load<v4u>(p, 1); }
template <int POLICY>
MI355_DEVICE void st_v4_any(uintptr_t p, v4u v) { lane_emu::checked_store(reinterpret_cast<void*>(p), v, 1); }

MI355_DEVICE ChunkRecord ld_uniform_record(const ChunkRecord* p) { return lane_emu::checked_load<ChunkRecord>(p, 32); }
MI355_DEVICE BatchDesc ld_uniform_desc(const BatchDesc* p) { return lane_emu::checked_load<BatchDesc>(p, 8); }
MI355_DEVICE uint32_t ld_uniform_u32(const uint32_t* p) { return lane_emu::checked_load<uint32_t>(p, 4); }
MI355_DEVICE void keep_alive(unsigned) {}

MI355_DEVICE unsigned wave_rotate_down1(unsigned v) {
  const unsigned lane = lane_emu::g_m.cur % kWave;
  const unsigned parity = lane_emu::lane_move_arrive(v);
  return lane_emu::lane_move_read(parity, (lane + 1) % kWave);
}
MI355_DEVICE uint32_t lane_read(uint32_t v, unsigned src) {
  const unsigned parity = lane_emu::lane_move_arrive(v);
  return lane_emu::lane_move_read(parity, src);
}
MI355_DEVICE uint32_t lane_read_up(uint32_t v, unsigned delta) {
  const unsigned lane = lane_emu::g_m.cur % kWave;
  const unsigned parity = lane_emu::lane_move_arrive(v);
  return lane < delta ? v : lane_emu::lane_move_read(parity, lane - delta);
}
// A value that is the same in every lane of the wave, which is checked: the
// k-th call of a lane must pass what the wave's first lane to make its k-th
// call passed.  (v_readfirstlane_b32 of a value that differs between lanes is
// not something these kernels do.)
MI355_DEVICE uint32_t wave_uniform(uint32_t v) {
  lane_emu::Lane& l = lane_emu::g_m.lanes[lane_emu::g_m.cur];
  std::vector<uint32_t>& log = lane_emu::g_m.waves[lane_emu::g_m.cur / kWave].uniform_log;
  const size_t k = l.uniform_calls++;
  if (k == log.size()) log.push_back(v);
  else if (k > log.size() || log[k] != v) lane_emu::machine_error("wave_uniform of a value that differs between lanes");
  return v;
}

MI355_DEVICE unsigned shift_bytes(unsigned hi, unsigned lo, unsigned r) {
  return static_cast<unsigned>(((static_cast<uint64_t>(hi) << 32) | lo) >> (8 * (r & 3)));
}
MI355_DEVICE uint64_t mul_hi_u64(uint64_t a, uint64_t b) {
  return static_cast<uint64_t>((static_cast<unsigned __int128>(a) * b) >> 64);
}

MI355_DEVICE unsigned thread_in_workgroup() { return lane_emu::g_m.cur; }
MI355_DEVICE unsigned workgroup_index() { return lane_emu::g_m.workgroup; }
MI355_DEVICE void workgroup_barrier() { lane_emu::barrier_arrive(); }

// The completion of an HSA signal is not part of what runs here.
MI355_DEVICE uint64_t realtime_ticks() { return 0; }
MI355_DEVICE void send_interrupt(uint32_t) {}
MI355_DEVICE void signal_decrement_system(int64_t* value) { --*value; }
MI355_DEVICE void st_system_release_u64(uint64_t* p, uint64_t v) { *p = v; }

}  // namespace mi355

#endif  // MI355_TESTS_LANE_EMULATION_H_
