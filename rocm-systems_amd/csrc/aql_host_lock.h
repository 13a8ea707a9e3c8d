// Locking host memory the runtime does not know for the GPU, the way
// Runtime::CopyMemory does before it hands a host<->device copy to a blit
// (projects/rocr-runtime/runtime/hsa-runtime/core/runtime/runtime.cpp:521-537:
// hsa_amd_memory_lock on the host side, the copy, hsa_amd_memory_unlock).
// The two runtime calls come in as function pointers so that the policy around
// them -- unlock exactly once, and stop asking a system that cannot lock -- is
// testable without a GPU.  Plain C++, no HSA headers: statuses are
// hsa_status_t values, agents hsa_agent_t.handle values.
#ifndef MI355_AQL_HOST_LOCK_H_
#define MI355_AQL_HOST_LOCK_H_

#include <stddef.h>
#include <stdint.h>

#include <mutex>
#include <vector>

#include "mi355_blit.h"

namespace mi355 {

struct HostLockFns {
  // hsa_amd_memory_lock(ptr, size, &agent, 1, mapped) / hsa_amd_memory_unlock(ptr)
  int (*lock)(void* ptr, size_t size, uint64_t gpu_agent, void** mapped);
  int (*unlock)(void* ptr);
};

// Agents whose system refuses to lock existing memory (the driver answers
// OUT_OF_RESOURCES or a plain ERROR, whatever the pointer): asking again for
// every copy costs a failed ioctl each time, so the refusal is remembered -- per
// agent, and only for those two answers.  A pointer-specific answer
// (INVALID_ARGUMENT, INVALID_ALLOCATION: this range cannot be locked) says
// nothing about the next pointer and is not remembered.
class HostLockLatch {
 public:
  bool refused(uint64_t gpu_agent) {
    std::lock_guard<std::mutex> g(lock_);
    for (uint64_t a : refused_)
      if (a == gpu_agent) return true;
    return false;
  }
  void note(uint64_t gpu_agent, int status) {
    if (status != MI355_BLIT_ERROR && status != MI355_BLIT_ERROR_OUT_OF_RESOURCES) return;
    std::lock_guard<std::mutex> g(lock_);
    for (uint64_t a : refused_)
      if (a == gpu_agent) return;
    refused_.push_back(gpu_agent);
  }

 private:
  std::mutex lock_;
  std::vector<uint64_t> refused_;
};

// Locks [ptr, ptr + size) for the GPU; unlocks on destruction.
class ScopedHostLock {
 public:
  ScopedHostLock(const HostLockFns& fns, HostLockLatch& latch) : fns_(fns), latch_(latch) {}
  ScopedHostLock(const ScopedHostLock&) = delete;
  ScopedHostLock& operator=(const ScopedHostLock&) = delete;
  ~ScopedHostLock() {
    if (host_) (void)fns_.unlock(host_);
  }
  // SUCCESS: *agent_ptr is the address the GPU uses for ptr.  Anything else:
  // nothing is locked and the caller takes another way (a bounce buffer).
  int Lock(uint64_t gpu_agent, const void* ptr, size_t size, void** agent_ptr) {
    if (host_) return MI355_BLIT_ERROR;  // one range per object
    if (latch_.refused(gpu_agent)) return MI355_BLIT_ERROR;
    void* mapped = nullptr;
    const int st = fns_.lock(const_cast<void*>(ptr), size, gpu_agent, &mapped);
    if (st != MI355_BLIT_SUCCESS) {
      latch_.note(gpu_agent, st);
      return st;
    }
    host_ = const_cast<void*>(ptr);
    *agent_ptr = mapped;
    return MI355_BLIT_SUCCESS;
  }

 private:
  const HostLockFns& fns_;
  HostLockLatch& latch_;
  void* host_ = nullptr;
};

}  // namespace mi355

#endif  // MI355_AQL_HOST_LOCK_H_
