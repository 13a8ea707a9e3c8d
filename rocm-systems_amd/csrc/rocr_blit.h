// The gfx950 blit engine behind ROCr's blit interface.
//
// rocr::core::Blit below repeats, member for member, the abstract interface of
// projects/rocr-runtime/runtime/hsa-runtime/core/inc/blit.h:52-122, and
// rocr::AMD::BlitKernelGfx950 is shaped like AMD::BlitKernel
// (core/inc/amd_blit_kernel.h:56-118): constructed over a queue, Initialize()d
// with the agent, owned by GpuAgent through lazy_ptr<core::Blit>
// (core/runtime/amd_gpu_agent.cpp:749-759, 858-863).
//
// ROCr's internal headers are not installed with ROCm, so the three internal
// types the interface mentions are given minimal stand-ins here, each with
// only members the real class has under the same name: core::Agent
// (public_handle(), profiling_enabled(): core/inc/agent.h:310, 320),
// core::Queue (public_handle(): core/inc/queue.h:373) and core::Signal, a thin
// view of an hsa_signal_t driven through the public hsa_signal_* API
// (Convert(): core/inc/signal.h:285-297).  Inside a ROCr tree
// MI355_ROCR_IN_TREE is defined: the stand-ins and the repeated core::Blit go
// away, the real core/inc/blit.h, agent.h, queue.h and signal.h come in, and
// nothing else changes (tests/test_rocr_in_tree.py compiles
// rocr_blit_aql.cpp that way against the reference's headers).
#ifndef MI355_ROCR_BLIT_H_
#define MI355_ROCR_BLIT_H_

#ifdef MI355_ROCR_IN_TREE
#include "core/inc/agent.h"
#include "core/inc/blit.h"
#include "core/inc/queue.h"
#include "core/inc/signal.h"
#else
#include <hsa/hsa.h>
#include <hsa/hsa_ext_amd.h>
#endif
#include <stdint.h>

#include <atomic>
#include <condition_variable>
#include <deque>
#include <mutex>
#include <thread>
#include <vector>

struct mi355_blit;
struct mi355_aql;

namespace rocr {
#ifndef MI355_ROCR_IN_TREE
namespace core {

class Agent {
 public:
  explicit Agent(hsa_agent_t public_handle, bool profiling = false)
      : public_handle_(public_handle), profiling_enabled_(profiling) {}
  virtual ~Agent() {}
  hsa_agent_t public_handle() const { return public_handle_; }
  bool profiling_enabled() const { return profiling_enabled_; }

 private:
  hsa_agent_t public_handle_;
  bool profiling_enabled_;
};

class Queue {
 public:
  explicit Queue(hsa_queue_t* public_handle) : public_handle_(public_handle) {}
  virtual ~Queue() {}
  hsa_queue_t* public_handle() const { return public_handle_; }

 private:
  hsa_queue_t* public_handle_;
};

class Signal {
 public:
  explicit Signal(hsa_signal_t handle) : handle_(handle) {}
  static hsa_signal_t Convert(const Signal* s) { return s->handle_; }
  hsa_signal_t handle() const { return handle_; }
  hsa_signal_value_t LoadRelaxed() const { return hsa_signal_load_relaxed(handle_); }
  void StoreRelaxed(hsa_signal_value_t v) { hsa_signal_store_relaxed(handle_, v); }
  void SubRelease(hsa_signal_value_t v) { hsa_signal_subtract_screlease(handle_, v); }

 private:
  hsa_signal_t handle_;
};

// core/inc/blit.h:52-122
class Blit {
 public:
  explicit Blit() {}
  virtual ~Blit() {}

  /// Blocks until all commands have executed, then releases the engine.
  virtual hsa_status_t Destroy(const core::Agent& agent) = 0;

  /// Blocking linear copy.
  virtual hsa_status_t SubmitLinearCopyCommand(void* dst, const void* src, size_t size) = 0;

  /// Non-blocking linear copy: starts after every dependent signal is 0,
  /// decrements out_signal once when done.
  virtual hsa_status_t SubmitLinearCopyCommand(void* dst, const void* src, size_t size,
                                               std::vector<core::Signal*>& dep_signals,
                                               core::Signal& out_signal,
                                               std::vector<core::Signal*>& gang_signals) = 0;

  /// Blocking fill of num uint32_t with value.
  virtual hsa_status_t SubmitLinearFillCommand(void* ptr, uint32_t value, size_t num) = 0;

  virtual hsa_status_t EnableProfiling(bool enable) = 0;

  virtual bool isSDMA() const { return false; }

  /// Approximate bytes still to copy or fill; a return of zero is exact.
  virtual uint64_t PendingBytes() = 0;

  virtual void GangLeader(bool gang_leader) = 0;
  virtual bool GangLeader() const { return false; }
};

}  // namespace core
#endif  // MI355_ROCR_IN_TREE

namespace AMD {

class BlitKernelGfx950 : public core::Blit {
 public:
  /// How out_signal is decremented when a command has finished.
  enum class Completion {
    kDeviceSignal,  ///< by a one-wave kernel queued behind the command
    kHostCallback,  ///< by hsa_signal_subtract_screlease from a host callback
  };

  /// This engine submits through a HIP stream: it has no use for the queue,
  /// and it is told which HIP device the agent is (the one thing HIP cannot
  /// learn from an hsa_agent_t).
  explicit BlitKernelGfx950(core::Queue* queue, Completion completion = Completion::kDeviceSignal,
                            int hip_device = 0);
  ~BlitKernelGfx950() override;

  /// Binds to the agent's GPU, loads the kernels, creates the completion
  /// signal used by the blocking calls (amd_blit_kernel.cpp:553-591).
  hsa_status_t Initialize(const core::Agent& agent);

  hsa_status_t Destroy(const core::Agent& agent) override;

  hsa_status_t SubmitLinearCopyCommand(void* dst, const void* src, size_t size) override;

  hsa_status_t SubmitLinearCopyCommand(void* dst, const void* src, size_t size,
                                       std::vector<core::Signal*>& dep_signals,
                                       core::Signal& out_signal,
                                       std::vector<core::Signal*>& gang_signals) override;

  hsa_status_t SubmitLinearFillCommand(void* ptr, uint32_t value, size_t count) override;

  /// Batched small copies: n independent copies in one submission, out_signal
  /// decremented once when all are done.  No counterpart in core::Blit.
  /// For device-resident descriptors, max_total_bytes != 0 vouches that the
  /// copies together move no more than that, which sizes a per-chunk grid
  /// (mi355_blit_copy_batch_bounded); 0 = no bound known.
  hsa_status_t SubmitBatchCopyCommand(const void* descs, size_t n, bool descs_on_device,
                                      std::vector<core::Signal*>& dep_signals,
                                      core::Signal& out_signal, uint64_t max_total_bytes = 0);

  hsa_status_t EnableProfiling(bool enable) override;

  uint64_t PendingBytes() override;

  void GangLeader(bool) override {}
  bool GangLeader() const override { return false; }

  /// The C ABI handle underneath (for the test driver).
  mi355_blit* c_handle() const { return blit_; }

 private:
  enum class Op { Copy, Fill, Batch };
  struct Command {
    Op op;
    void* dst;
    const void* src;
    size_t size;     // bytes, dwords (Fill) or descriptors (Batch)
    uint32_t value;  // Fill pattern / Batch: descriptors are device-resident
    uint64_t bound = 0;  // Batch, device-resident: most bytes the copies move together, 0 = unknown
    std::vector<hsa_signal_t> deps;
    hsa_signal_t out;
  };

  static bool DepsSatisfied(const std::vector<hsa_signal_t>& deps);
  hsa_status_t Launch(const Command& cmd);
  hsa_status_t Submit(Command&& cmd);
  void WorkerLoop();
  void DrainWorker();
  static void OnComplete(void* user);

  core::Queue* queue_;
  int hip_device_;
  mi355_blit* blit_;
  Completion completion_;

  /// Completion signal of the blocking calls; guarded by lock_.
  hsa_signal_t completion_signal_;
  std::mutex lock_;

  /// Commands whose dependencies were not yet satisfied at submission, and
  /// everything submitted behind them: executed in order by worker_.
  std::mutex queue_lock_;
  std::condition_variable queue_cv_;
  std::deque<Command> waiting_;
  bool worker_busy_;
  bool stopping_;
  std::thread worker_;
  uint64_t waiting_bytes_;

  std::atomic<bool> profiling_;
};

// The same interface over hand-built AQL packets (include/mi355_blit_aql.h):
// dependencies become BARRIER_AND packets, out_signal is the dispatch packet's
// completion signal and the packet processor decrements it, exactly as in
// AMD::BlitKernel (core/runtime/amd_blit_kernel.cpp:641-785).  No submission
// thread, no HIP.  This is the class that replaces AMD::BlitKernel in tree:
// like it, the object borrows the queue it is constructed over (the agent's
// utility queue, which other producers may share: core/inc/amd_blit_kernel.h:
// 58-66, core/runtime/amd_gpu_agent.cpp:692-701, 749-759) and runs on the
// agent Initialize() is given; it creates no queue and does not touch the
// runtime's reference count.
class BlitKernelGfx950Aql : public core::Blit {
 public:
  /// Which of GpuAgent's blits_ slots the object fills
  /// (core/inc/amd_gpu_agent.h:588): the linear copies of an object made for
  /// BlitHostToDev or BlitDevToHost are launched in the shape that suits the
  /// host link (MI355_BLIT_ROUTE_* in include/mi355_blit.h).
  enum class Slot : uint32_t { kDevToDev = 0, kHostToDev = 1, kDevToHost = 2 };

  explicit BlitKernelGfx950Aql(core::Queue* queue, Slot slot = Slot::kDevToDev);
  ~BlitKernelGfx950Aql() override;

  hsa_status_t Initialize(const core::Agent& agent);
  hsa_status_t Destroy(const core::Agent& agent) override;
  hsa_status_t SubmitLinearCopyCommand(void* dst, const void* src, size_t size) override;
  hsa_status_t SubmitLinearCopyCommand(void* dst, const void* src, size_t size,
                                       std::vector<core::Signal*>& dep_signals,
                                       core::Signal& out_signal,
                                       std::vector<core::Signal*>& gang_signals) override;
  hsa_status_t SubmitLinearFillCommand(void* ptr, uint32_t value, size_t count) override;
  /// Batched small copies, descriptors in host or device memory; no counterpart in core::Blit.
  /// max_total_bytes != 0: a bound on what device-resident descriptors move (0 = none known).
  hsa_status_t SubmitBatchCopyCommand(const void* descs, size_t n, bool descs_on_device,
                                      std::vector<core::Signal*>& dep_signals,
                                      core::Signal& out_signal, uint64_t max_total_bytes = 0);
  /// Pitched 3-D region copy with the signature of BlitSdmaBase::SubmitCopyRectCommand
  /// (core/inc/amd_blit_sdma.h:68-73), so that GpuAgent::DmaCopyRect
  /// (core/runtime/amd_gpu_agent.cpp:1255-1283) can call a shader blit where it
  /// now answers OUT_OF_RESOURCES.  Any byte alignment; the region must be a
  /// box inside both surfaces (amd_blit_sdma.cpp:577-585).
  hsa_status_t SubmitCopyRectCommand(const hsa_pitched_ptr_t* dst, const hsa_dim3_t* dst_offset,
                                     const hsa_pitched_ptr_t* src, const hsa_dim3_t* src_offset,
                                     const hsa_dim3_t* range, std::vector<core::Signal*>& dep_signals,
                                     core::Signal& out_signal);
  hsa_status_t EnableProfiling(bool enable) override;
  uint64_t PendingBytes() override;
  void GangLeader(bool) override {}
  bool GangLeader() const override { return false; }

  /// For the owner of the queue: its error callback forwards an asynchronous
  /// queue error here (what core::Queue::DefaultErrorHandler stands for,
  /// core/runtime/queue.cpp:52-59); blocking calls then return
  /// HSA_STATUS_ERROR instead of waiting for a signal nobody will complete.
  void ReportQueueError(hsa_status_t status);

  /// The C ABI handle underneath (for the test driver).
  mi355_aql* c_handle() const { return blit_; }

 private:
  core::Queue* queue_;
  Slot slot_;
  mi355_aql* blit_;
  /// Completion signal of the blocking calls; guarded by lock_.
  hsa_signal_t completion_signal_;
  std::mutex lock_;
};

}  // namespace AMD
}  // namespace rocr

#endif  // MI355_ROCR_BLIT_H_
