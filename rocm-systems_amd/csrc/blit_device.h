// Device primitives of the gfx950 blit kernels: every memory access, every
// move between lanes and every hardware id the kernels in blit_kernels.h use
// goes through a function of this header, and nothing else in the kernels names
// an instruction, an address space or a HIP built-in.
//
// That makes the kernels executable on a CPU: a host build defines
// MI355_BLIT_DEVICE_HEADER to a header of its own that provides the same names
// (the 16-byte vector type, the accessors, the lane moves, thread and workgroup
// index) over host memory, runs the lanes of a workgroup in lock step and checks
// every address a lane touches against the ranges the command may touch.  The
// kernels themselves are compiled unchanged.
#ifndef MI355_BLIT_DEVICE_H_
#define MI355_BLIT_DEVICE_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "blit_args.h"

#define MI355_DEVICE __device__ __forceinline__
// A kernel entry point for workgroups of up to `max_wg` work-items.
#define MI355_KERNEL(max_wg) extern "C" __global__ __launch_bounds__(max_wg)
// Workgroup-shared storage (LDS).
#define MI355_LDS __shared__

namespace mi355 {

typedef unsigned v4u __attribute__((ext_vector_type(4)));
// Same vector with only dword alignment promised: the compiler still emits one
// global_load_dwordx4, which the memory pipeline accepts at any dword address.
typedef v4u v4u_a4 __attribute__((aligned(4)));

// Every pointer these kernels dereference points into global memory, but one
// that was itself loaded from memory (the chunk records of a batch) reaches the
// compiler as a generic pointer and would be accessed with flat_* instructions,
// which go through the aperture check and count against both memory counters.
// The accessors below therefore state the address space.
#define MI355_GLOBAL __attribute__((address_space(1)))

template <typename T>
MI355_DEVICE const T MI355_GLOBAL* as_global(const T* p) {
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wold-style-cast"
  return (const T MI355_GLOBAL*)(p);
#pragma clang diagnostic pop
}
template <typename T>
MI355_DEVICE T MI355_GLOBAL* as_global(T* p) {
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wold-style-cast"
  return (T MI355_GLOBAL*)(p);
#pragma clang diagnostic pop
}

template <bool NT>
MI355_DEVICE v4u ld_v4(const v4u_a4* p) {
  if constexpr (NT) return __builtin_nontemporal_load(as_global(p));
  else return *as_global(p);
}
template <bool NT>
MI355_DEVICE unsigned ld_u32(const unsigned* p) {
  if constexpr (NT) return __builtin_nontemporal_load(as_global(p));
  else return *as_global(p);
}
MI355_DEVICE uint8_t ld_u8(const uint8_t* p) { return *as_global(p); }
MI355_DEVICE void st_u8(uint8_t* p, uint8_t v) { *as_global(p) = v; }
MI355_DEVICE void st_u32(unsigned* p, unsigned v) { *as_global(p) = v; }

// Plain cached access to one object of the kernels' own bookkeeping (a
// descriptor, a record).  These pointers come straight out of the kernel
// arguments, which the compiler knows to be global.
template <typename T>
MI355_DEVICE T ld_obj(const T* p) { return *p; }
template <typename T>
MI355_DEVICE void st_obj(T* p, const T& v) { *p = v; }

// Words the host wrote (into host memory, or across the bus into device
// memory) behind the GPU's caches, and words the host will read: system scope.
MI355_DEVICE uint64_t ld_system_u64(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
MI355_DEVICE uint32_t ld_system_u32(const uint32_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
MI355_DEVICE void st_system_u64(uint64_t* p, uint64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Store cache policies (values of mi355_blit_plan_t::store_policy).
constexpr int kStoreCached = 0;   // plain write-back L2
constexpr int kStoreNt = 1;       // non-temporal hint
constexpr int kStoreAgentWt = 2;  // sc1: written through L2 at agent scope
constexpr int kStoreSystemWt = 3; // sc0 sc1: written through at system scope

// The policies are spelled out in asm: the write-through forms have no builtin
// for a 16-byte store, and the non-temporal builtin's hint was seen to get lost
// on the way through the optimizer (the body store of one realigning variant
// came out as a plain store).  A store needs no wait of its own, and on gfx9
// the extra outstanding store only makes a compiler-placed s_waitcnt vmcnt(n)
// wait longer, never shorter.  A store of more than 8 bytes reads its data
// registers after issue: a VALU write to them within the next 2 wait states
// (gfx940 and later) corrupts the data.  The compiler pads its own stores but
// cannot see into the asm, so the s_nop is part of it.  The asm forms take any
// byte address.
template <int POLICY>
MI355_DEVICE void st_v4_at(uintptr_t p, v4u v) {
  if constexpr (POLICY == kStoreNt) {
    asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
  } else if constexpr (POLICY == kStoreAgentWt) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
  } else if constexpr (POLICY == kStoreSystemWt) {
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
  } else {
    typedef v4u v4u_any __attribute__((aligned(1)));
    *as_global(reinterpret_cast<v4u_any*>(p)) = v;
  }
}
template <int POLICY>
MI355_DEVICE void st_v4(v4u* p, v4u v) {
  if constexpr (POLICY == kStoreCached) *as_global(p) = v;
  else st_v4_at<POLICY>(reinterpret_cast<uintptr_t>(p), v);
}

// 16-byte accesses at any byte address: gfx950 under HSA runs with unaligned
// global access enabled, and the compiler emits one dwordx4 for these too.
typedef v4u v4u_a1 __attribute__((aligned(1)));

template <bool NT>
MI355_DEVICE v4u ld_v4_any(const uint8_t* p) {
  if constexpr (NT) return __builtin_nontemporal_load(as_global(reinterpret_cast<const v4u_a1*>(p)));
  else return *as_global(reinterpret_cast<const v4u_a1*>(p));
}

template <int POLICY>
MI355_DEVICE void st_v4_any(uintptr_t p, v4u v) {
  st_v4_at<POLICY>(p, v);
}

// One record, fetched with a scalar load.  The records were written by an
// earlier launch and are only read here; reading them through the constant
// address space tells the compiler so (a pointer taken out of the argument
// struct carries no such promise, and the record would otherwise be fetched by
// all 64 lanes with vector loads).  The address is the same for every lane.
MI355_DEVICE ChunkRecord ld_uniform_record(const ChunkRecord* p) {
  typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
  typedef const u32x8 __attribute__((address_space(4))) * ConstPtr;
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wold-style-cast"
  const u32x8 v = *(ConstPtr)(p);
#pragma clang diagnostic pop
  ChunkRecord r;
  __builtin_memcpy(&r, &v, sizeof(r));
  return r;
}

// A descriptor at an address that is the same for every lane, through the
// constant address space like a record.
MI355_DEVICE BatchDesc ld_uniform_desc(const BatchDesc* p) {
  typedef const uint64_t __attribute__((address_space(4))) * ConstPtr;
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wold-style-cast"
  ConstPtr q = (ConstPtr)(p);
#pragma clang diagnostic pop
  BatchDesc d;
  d.dst = reinterpret_cast<uint8_t*>(q[0]);
  d.src = reinterpret_cast<const uint8_t*>(q[1]);
  d.bytes = q[2];
  return d;
}

// A word at an address that is the same for every lane (scalar load).
MI355_DEVICE uint32_t ld_uniform_u32(const uint32_t* p) {
  typedef const uint32_t __attribute__((address_space(4))) * ConstPtr;
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wold-style-cast"
  return *(ConstPtr)(p);
#pragma clang diagnostic pop
}

// Keeps the compiler from dropping a load whose value is not used.
MI355_DEVICE void keep_alive(unsigned v) { asm volatile("" ::"v"(v)); }

// ---- moves between the lanes of a wave -------------------------------------

// Lane i receives the value lane (i + 1) % 64 passed in (DPP wave_rol:1).
MI355_DEVICE unsigned wave_rotate_down1(unsigned v) {
  return __builtin_amdgcn_update_dpp(0u, v, 0x134, 0xf, 0xf, false);
}
// The value lane `src` passed in.
MI355_DEVICE uint32_t lane_read(uint32_t v, unsigned src) { return __shfl(v, src, kWave); }
// The value lane (own index - delta) passed in; lanes below delta keep their own.
MI355_DEVICE uint32_t lane_read_up(uint32_t v, unsigned delta) { return __shfl_up(v, delta, kWave); }
// The value of the wave's first lane, as a wave-uniform (scalar) value.
MI355_DEVICE uint32_t wave_uniform(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

// Bytes r..r+3 of the little-endian pair {hi:lo}, r in 0..3.
MI355_DEVICE unsigned shift_bytes(unsigned hi, unsigned lo, unsigned r) {
  return __builtin_amdgcn_alignbyte(hi, lo, r);
}

MI355_DEVICE uint64_t mul_hi_u64(uint64_t a, uint64_t b) { return __umul64hi(a, b); }

// ---- ids and synchronisation ------------------------------------------------

MI355_DEVICE unsigned thread_in_workgroup() { return threadIdx.x; }
MI355_DEVICE unsigned workgroup_index() { return blockIdx.x; }
MI355_DEVICE void workgroup_barrier() { __syncthreads(); }

// The GPU's free-running 100 MHz counter (s_memrealtime): the clock the packet
// processor stamps completion signals with.
MI355_DEVICE uint64_t realtime_ticks() { return __builtin_amdgcn_s_memrealtime(); }

// MSG_INTERRUPT with an event id's low byte in m0.
MI355_DEVICE void send_interrupt(uint32_t event_id) {
  __builtin_amdgcn_s_sendmsg(1, __builtin_amdgcn_readfirstlane(event_id) & 0xff);
}
MI355_DEVICE void signal_decrement_system(int64_t* value) {
  __hip_atomic_fetch_sub(value, static_cast<int64_t>(1), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}
MI355_DEVICE void st_system_release_u64(uint64_t* p, uint64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

}  // namespace mi355

#endif  // MI355_BLIT_DEVICE_H_
