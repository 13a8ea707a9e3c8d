// Caller policy over the AQL blit engine: the decisions ROCr takes between the
// HSA API and core::Blit, restated with the public HSA API
// (projects/rocr-runtime/runtime/hsa-runtime/core/runtime/runtime.cpp:469-664,
// hsa.cpp:1170-1184, hsa_ext_amd.cpp:237-294).  Declarations:
// include/mi355_blit_aql.h.
#include <hsa/hsa.h>
#include <hsa/hsa_ext_amd.h>

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "aql_host_lock.h"
#include "blit_plan.h"
#include "mi355_blit_aql.h"

namespace {

using mi355::HostLockFns;
using mi355::HostLockLatch;
using mi355::ScopedHostLock;

enum class Where { kHost, kHostUnknown, kGpu };

// runtime.cpp:483-500: a pointer inside an allocation the runtime knows belongs
// to that allocation's owner; anything else is system memory that must be
// locked before a GPU can touch it.
struct Placement {
  Where where = Where::kHostUnknown;
  bool gpu_can_access = false;  // without locking
};

int classify(mi355_aql_t* h, const void* ptr, size_t size, Placement* out) {
  hsa_amd_pointer_info_t info;
  std::memset(&info, 0, sizeof(info));
  info.size = sizeof(info);
  uint32_t n_access = 0;
  hsa_agent_t* access = nullptr;
  hsa_status_t st = hsa_amd_pointer_info(ptr, &info, std::malloc, &n_access, &access);
  if (st != HSA_STATUS_SUCCESS) return static_cast<int>(st);
  const uint64_t gpu = mi355_aql_gpu_agent(h);
  Placement p;
  const char* base = static_cast<const char*>(info.agentBaseAddress);
  const char* cp = static_cast<const char*>(ptr);
  const bool known = info.type != HSA_EXT_POINTER_TYPE_UNKNOWN && base != nullptr && base <= cp &&
                     cp + size <= base + info.sizeInBytes;
  if (known) {
    hsa_agent_t owner = info.agentOwner;
    if (owner.handle == 0 && n_access) owner = access[0];
    hsa_device_type_t type = HSA_DEVICE_TYPE_CPU;
    if (owner.handle) hsa_agent_get_info(owner, HSA_AGENT_INFO_DEVICE, &type);
    p.where = type == HSA_DEVICE_TYPE_GPU ? Where::kGpu : Where::kHost;
    for (uint32_t i = 0; i < n_access; ++i)
      if (access[i].handle == gpu) p.gpu_can_access = true;
    if (owner.handle == gpu) p.gpu_can_access = true;
  }
  std::free(access);
  *out = p;
  return MI355_BLIT_SUCCESS;
}

// The blit a GPU<->host copy goes to (GetPcieBlit, amd_gpu_agent.cpp:2370-2377):
// host to device when the source is the host's, device to host otherwise.
uint32_t route_of(bool src_is_host, bool dst_is_host) {
  if (src_is_host && !dst_is_host) return MI355_BLIT_ROUTE_HOST_TO_DEVICE;
  if (dst_is_host) return MI355_BLIT_ROUTE_DEVICE_TO_HOST;
  return MI355_BLIT_ROUTE_DEVICE;
}

// Sizes from which the route changes the launch: below it a copy has too few
// tiles for the shapes to differ, and a pointer lookup would only add latency.
constexpr size_t kRouteLookupMinBytes = 1u << 20;

// Host memory the runtime does not know is locked for the GPU
// (runtime.cpp:521-535) through the runtime's own calls; which agents' systems
// refuse that is remembered for the process (aql_host_lock.h).
int runtime_lock(void* ptr, size_t size, uint64_t gpu_agent, void** mapped) {
  hsa_agent_t gpu;
  gpu.handle = gpu_agent;
  return static_cast<int>(hsa_amd_memory_lock(ptr, size, &gpu, 1, mapped));
}
int runtime_unlock(void* ptr) { return static_cast<int>(hsa_amd_memory_unlock(ptr)); }
const HostLockFns kRuntimeLock{runtime_lock, runtime_unlock};
HostLockLatch g_lock_refused;

// Host<->device copy through the engine's two GPU-visible bounce buffers, for
// host memory that can neither be reached by the GPU nor locked: while the
// blit moves one half the host fills (or drains) the other.  to_device says
// which side is the host's.
std::mutex g_bounce_lock;  // one bounced copy at a time per process

int bounced_copy(mi355_aql_t* h, void* dst, const void* src, size_t size, bool to_device) {
  std::lock_guard<std::mutex> g(g_bounce_lock);
  size_t half = 0;
  void* buf[2] = {nullptr, nullptr};
  int rc = mi355_aql_staging(h, &half, &buf[0], &buf[1]);
  if (rc != MI355_BLIT_SUCCESS) return rc;
  hsa_signal_t done[2];
  for (int i = 0; i < 2; ++i)
    if (hsa_signal_create(0, 0, nullptr, &done[i]) != HSA_STATUS_SUCCESS) {
      if (i) hsa_signal_destroy(done[0]);
      return MI355_BLIT_ERROR_OUT_OF_RESOURCES;
    }
  // Bounded waits that end with an error when the queue has reported one
  // (mi355_aql_wait_signal): a piece whose submission failed, or whose queue
  // died under it, must not leave this call waiting for its signal.
  auto wait = [&](int i) {
    const int w = mi355_aql_wait_signal(h, done[i].handle);
    if (w != MI355_BLIT_SUCCESS && rc == MI355_BLIT_SUCCESS) rc = w;
  };
  const char* s = static_cast<const char*>(src);
  char* d = static_cast<char*>(dst);
  size_t prev_off = 0, prev_len = 0;
  int piece = 0;
  for (size_t off = 0; off < size && rc == MI355_BLIT_SUCCESS; off += half, ++piece) {
    const int b = piece & 1;
    const size_t len = size - off < half ? size - off : half;
    wait(b);  // the blit that used this half two pieces ago
    if (rc != MI355_BLIT_SUCCESS) break;
    if (to_device) {
      std::memcpy(buf[b], s + off, len);
      hsa_signal_store_relaxed(done[b], 1);
      rc = mi355_aql_copy_route(h, d + off, buf[b], len, MI355_BLIT_ROUTE_HOST_TO_DEVICE, nullptr, 0, done[b].handle);
      if (rc != MI355_BLIT_SUCCESS) hsa_signal_store_relaxed(done[b], 0);  // nothing was queued that would
    } else {
      hsa_signal_store_relaxed(done[b], 1);
      rc = mi355_aql_copy_route(h, buf[b], s + off, len, MI355_BLIT_ROUTE_DEVICE_TO_HOST, nullptr, 0, done[b].handle);
      if (rc != MI355_BLIT_SUCCESS) {
        hsa_signal_store_relaxed(done[b], 0);
        break;
      }
      // drain the previous piece while this one is in flight
      if (piece > 0) {
        wait(b ^ 1);
        if (rc != MI355_BLIT_SUCCESS) break;
        std::memcpy(d + prev_off, buf[b ^ 1], prev_len);
      }
      prev_off = off;
      prev_len = len;
    }
  }
  // On an error the signals of pieces still in flight are waited for all the
  // same (bounded): the buffers are the engine's and the next call reuses them.
  wait(0);
  wait(1);
  if (!to_device && rc == MI355_BLIT_SUCCESS && piece > 0) std::memcpy(d + prev_off, buf[(piece - 1) & 1], prev_len);
  hsa_signal_destroy(done[0]);
  hsa_signal_destroy(done[1]);
  return rc;
}

}  // namespace

extern "C" {

int mi355_hsa_memory_copy(mi355_aql_t* h, void* dst, const void* src, size_t size) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  // hsa.cpp:1174-1180
  if (dst == nullptr || src == nullptr) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (size == 0) return MI355_BLIT_SUCCESS;
  Placement ps, pd;
  int rc = classify(h, src, size, &ps);
  if (rc == MI355_BLIT_SUCCESS) rc = classify(h, dst, size, &pd);
  if (rc != MI355_BLIT_SUCCESS) return rc;
  const bool src_sys = ps.where != Where::kGpu, dst_sys = pd.where != Where::kGpu;
  // CPU-CPU (runtime.cpp:507-510)
  if (src_sys && dst_sys) {
    std::memcpy(dst, src, size);
    return MI355_BLIT_SUCCESS;
  }
  // Same GPU, or GPU-CPU with the host side made visible to the GPU first.
  // Where existing host memory cannot be locked the copy is bounced instead.
  ScopedHostLock lock_src(kRuntimeLock, g_lock_refused), lock_dst(kRuntimeLock, g_lock_refused);
  void* d = dst;
  const void* s = src;
  if (src_sys && !ps.gpu_can_access) {
    void* mapped = nullptr;
    if (lock_src.Lock(mi355_aql_gpu_agent(h), src, size, &mapped) != MI355_BLIT_SUCCESS) return bounced_copy(h, dst, src, size, true);
    s = mapped;
  }
  if (dst_sys && !pd.gpu_can_access) {
    void* mapped = nullptr;
    if (lock_dst.Lock(mi355_aql_gpu_agent(h), dst, size, &mapped) != MI355_BLIT_SUCCESS) return bounced_copy(h, dst, src, size, false);
    d = mapped;
  }
  // Waits for this copy's own completion signal, not for the queue to drain
  // (amd_blit_kernel.cpp:614-639).  With the barrier bit clear, commands other
  // threads have parked behind unsatisfied dependencies do not hold the copy
  // up either; a copy of 4 MiB or more on an engine's own queue carries the
  // bit (mi355_aql_set_large_transfer_barrier) and does wait for them.
  return mi355_aql_copy_sync(h, d, s, size, route_of(src_sys, dst_sys));
}

int mi355_hsa_amd_memory_fill(mi355_aql_t* h, void* ptr, uint32_t value, size_t count) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  // hsa_ext_amd.cpp:241-247
  if (ptr == nullptr || (reinterpret_cast<uintptr_t>(ptr) % 4) != 0) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (count == 0) return MI355_BLIT_SUCCESS;
  Placement p;
  int rc = classify(h, ptr, count * sizeof(uint32_t), &p);
  if (rc != MI355_BLIT_SUCCESS) return rc;
  // runtime.cpp:640-655: any GPU that can reach the memory fills it
  if (p.where == Where::kGpu || p.gpu_can_access) {
    return mi355_aql_fill32_sync(h, ptr, value, count);
  }
  // host memory: the full pattern, dword by dword
  uint32_t* out = static_cast<uint32_t*>(ptr);
  for (size_t i = 0; i < count; ++i) out[i] = value;
  return MI355_BLIT_SUCCESS;
}

int mi355_hsa_amd_memory_async_copy(mi355_aql_t* h, void* dst, const void* src, size_t size,
                                    uint32_t num_dep_signals, const uint64_t* dep_signals,
                                    uint64_t completion_signal) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  // hsa_ext_amd.cpp:258-283
  if (dst == nullptr || src == nullptr) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if ((num_dep_signals == 0 && dep_signals != nullptr) || (num_dep_signals > 0 && dep_signals == nullptr))
    return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  for (uint32_t i = 0; i < num_dep_signals; ++i)
    if (dep_signals[i] == 0) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (completion_signal == 0) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  // hsa_ext_amd.cpp:285-293: size 0 succeeds and leaves the signal alone
  if (size == 0) return MI355_BLIT_SUCCESS;
  uint32_t route = MI355_BLIT_ROUTE_DEVICE;
  if (size >= kRouteLookupMinBytes) {
    Placement ps, pd;
    if (classify(h, src, size, &ps) == MI355_BLIT_SUCCESS && classify(h, dst, size, &pd) == MI355_BLIT_SUCCESS)
      route = route_of(ps.where != Where::kGpu, pd.where != Where::kGpu);
  }
  // GetBlitObject (amd_gpu_agent.cpp:2379-2442): within the GPU the size
  // decides between the SDMA-capable engine and the blit kernel; across the
  // host link it is blits_[BlitHostToDev] / [BlitDevToHost], SDMA when the GPU
  // has such engines.  The copy runs on this engine either way; the choice is
  // only reported.
  mi355_aql_note_reference_engine(
      h, route == MI355_BLIT_ROUTE_DEVICE ? mi355::policy_same_gpu_engine(size, mi355::policy_force_sdma_size())
                                          : static_cast<uint32_t>(MI355_ENGINE_SDMA));
  return mi355_aql_copy_route(h, dst, src, size, route, dep_signals, num_dep_signals, completion_signal);
}

namespace {
// SDMA engines of the GPU as the runtime reports them (what
// properties_.NumSdmaEngines / NumSdmaXgmiEngines hold in the reference).
void sdma_engine_counts(mi355_aql_t* h, uint32_t* sdma, uint32_t* xgmi) {
  hsa_agent_t gpu;
  gpu.handle = mi355_aql_gpu_agent(h);
  *sdma = *xgmi = 0;
  (void)hsa_agent_get_info(gpu, static_cast<hsa_agent_info_t>(HSA_AMD_AGENT_INFO_NUM_SDMA_ENG), sdma);
  (void)hsa_agent_get_info(gpu, static_cast<hsa_agent_info_t>(HSA_AMD_AGENT_INFO_NUM_SDMA_XGMI_ENG), xgmi);
}
}  // namespace

int mi355_hsa_amd_memory_async_copy_on_engine(mi355_aql_t* h, void* dst, const void* src, size_t size,
                                              uint32_t num_dep_signals, const uint64_t* dep_signals,
                                              uint64_t completion_signal, uint32_t engine_id,
                                              int force_copy_on_sdma) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  // hsa_ext_amd.cpp:303-327
  if (dst == nullptr || src == nullptr) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if ((num_dep_signals == 0 && dep_signals != nullptr) || (num_dep_signals > 0 && dep_signals == nullptr))
    return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  for (uint32_t i = 0; i < num_dep_signals; ++i)
    if (dep_signals[i] == 0) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (completion_signal == 0) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  // hsa_ext_amd.cpp:330-337: size 0 succeeds before the engine is looked at
  if (size == 0) return MI355_BLIT_SUCCESS;
  // runtime.cpp:593-597: exactly one bit names the engine
  if (engine_id == 0 || (engine_id & (engine_id - 1)) != 0) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  const uint32_t engine_offset = static_cast<uint32_t>(__builtin_ffs(static_cast<int>(engine_id)));
  // amd_gpu_agent.cpp:1123-1125
  uint32_t sdma = 0, xgmi = 0;
  sdma_engine_counts(h, &sdma, &xgmi);
  if (engine_offset > sdma + xgmi) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  // amd_gpu_agent.cpp:1159: within one GPU the named engine is set aside for
  // the blit kernel unless the caller insists on SDMA, which this library
  // does not drive.
  if (force_copy_on_sdma) return MI355_BLIT_ERROR_OUT_OF_RESOURCES;
  return mi355_aql_copy(h, dst, src, size, dep_signals, num_dep_signals, completion_signal);
}

int mi355_hsa_amd_memory_copy_engine_status(mi355_aql_t* h, int dst_is_gpu, int src_is_gpu, uint32_t* engine_ids_mask) {
  if (!h || !engine_ids_mask) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  *engine_ids_mask = 0;
  // runtime.cpp:608-610: the question is about two different agents.  With one
  // GPU behind the handle that leaves GPU <-> CPU (host <-> host never gets
  // here in the reference either: one of the two is a GPU agent, :605-606).
  if (dst_is_gpu && src_is_gpu) return HSA_STATUS_ERROR_INVALID_AGENT;
  if (!dst_is_gpu && !src_is_gpu) return HSA_STATUS_ERROR_INVALID_AGENT;
  // amd_gpu_agent.cpp:1181-1243 on an agent whose SDMA engines nobody has used
  // (this library never does): DmaEngineIsFree holds for all of them, so the
  // answer is the H2D engine, the D2H engine and every xGMI engine.
  uint32_t sdma = 0, xgmi = 0;
  sdma_engine_counts(h, &sdma, &xgmi);
  uint32_t mask = 0;
  if (sdma >= 1) mask |= HSA_AMD_SDMA_ENGINE_0;
  if (sdma >= 1) mask |= sdma > 1 ? HSA_AMD_SDMA_ENGINE_1 : HSA_AMD_SDMA_ENGINE_0;
  for (uint32_t i = 0; i < xgmi; ++i) mask |= HSA_AMD_SDMA_ENGINE_2 << i;
  *engine_ids_mask = mask;
  return mask ? MI355_BLIT_SUCCESS : MI355_BLIT_ERROR_OUT_OF_RESOURCES;
}

int mi355_hsa_amd_memory_async_copy_rect(mi355_aql_t* h, const mi355_pitched_ptr_t* dst,
                                         const mi355_dim3_t* dst_offset, const mi355_pitched_ptr_t* src,
                                         const mi355_dim3_t* src_offset, const mi355_dim3_t* range, int dir,
                                         uint32_t num_dep_signals, const uint64_t* dep_signals,
                                         uint64_t completion_signal) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  // hsa_ext_amd.cpp:372-381
  if (dst == nullptr || src == nullptr || dst_offset == nullptr || src_offset == nullptr || range == nullptr)
    return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if ((num_dep_signals == 0 && dep_signals != nullptr) || (num_dep_signals > 0 && dep_signals == nullptr))
    return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (dir == 0 /* hsaHostToHost */) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  for (uint32_t i = 0; i < num_dep_signals; ++i)
    if (dep_signals[i] == 0) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (completion_signal == 0) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  // hsa_ext_amd.cpp:400-405: an empty range succeeds and leaves the signal alone
  if (range->x == 0 || range->y == 0 || range->z == 0) return MI355_BLIT_SUCCESS;
  // hsa_amd_copy_direction_t: amd_gpu_agent.cpp:1265-1266 picks the blit by it
  const uint32_t route = dir == 1 /* hsaHostToDevice */   ? MI355_BLIT_ROUTE_HOST_TO_DEVICE
                         : dir == 2 /* hsaDeviceToHost */ ? MI355_BLIT_ROUTE_DEVICE_TO_HOST
                                                          : MI355_BLIT_ROUTE_DEVICE;
  return mi355_aql_copy_rect_route(h, dst, dst_offset, src, src_offset, range, route, dep_signals, num_dep_signals,
                                   completion_signal);
}

}  // extern "C"

extern "C" {
// The engine-choice policy of mi355_blit.h, exported by this library too so
// that a runtime linking only the AQL engine has it.
uint64_t mi355_policy_force_sdma_size(void) { return mi355::policy_force_sdma_size(); }
uint32_t mi355_policy_same_gpu_engine(uint64_t size, uint64_t force_sdma_size) {
  return mi355::policy_same_gpu_engine(size, force_sdma_size);
}
}
