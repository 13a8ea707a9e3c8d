// rocr::AMD::BlitKernelGfx950Aql: ROCr's core::Blit interface over the AQL
// submission path.  Member for member the host side of AMD::BlitKernel
// (projects/rocr-runtime/runtime/hsa-runtime/core/runtime/amd_blit_kernel.cpp:
// 538-970); the packet building itself lives behind the C ABI
// (include/mi355_blit_aql.h).
#include "mi355_blit_aql.h"
#include "rocr_blit.h"

namespace rocr {
namespace AMD {

namespace {

hsa_status_t to_hsa(int st) { return static_cast<hsa_status_t>(st); }

std::vector<uint64_t> handles(const std::vector<core::Signal*>& signals) {
  std::vector<uint64_t> out;
  out.reserve(signals.size());
  for (core::Signal* s : signals) out.push_back(core::Signal::Convert(s).handle);
  return out;
}

}  // namespace

static_assert(static_cast<uint32_t>(BlitKernelGfx950Aql::Slot::kHostToDev) == MI355_BLIT_ROUTE_HOST_TO_DEVICE &&
                  static_cast<uint32_t>(BlitKernelGfx950Aql::Slot::kDevToHost) == MI355_BLIT_ROUTE_DEVICE_TO_HOST,
              "slots and routes count alike");

BlitKernelGfx950Aql::BlitKernelGfx950Aql(core::Queue* queue, Slot slot)
    : core::Blit(), queue_(queue), slot_(slot), blit_(nullptr) {
  completion_signal_.handle = 0;
}

BlitKernelGfx950Aql::~BlitKernelGfx950Aql() {}

hsa_status_t BlitKernelGfx950Aql::Initialize(const core::Agent& agent) {
  hsa_status_t status = hsa_signal_create(1, 0, NULL, &completion_signal_);
  if (status != HSA_STATUS_SUCCESS) return status;
  // the queue handed to the constructor and the agent handed here, as they are
  if (queue_ == nullptr) return HSA_STATUS_ERROR_INVALID_QUEUE;
  int st = mi355_aql_create_on(agent.public_handle().handle, queue_->public_handle(), &blit_);
  if (st != MI355_BLIT_SUCCESS) return to_hsa(st);
  if (agent.profiling_enabled()) return EnableProfiling(true);
  return HSA_STATUS_SUCCESS;
}

hsa_status_t BlitKernelGfx950Aql::Destroy(const core::Agent&) {
  std::lock_guard<std::mutex> guard(lock_);
  hsa_status_t result = HSA_STATUS_SUCCESS;
  if (blit_ != nullptr) {
    if (mi355_aql_destroy(blit_) != MI355_BLIT_SUCCESS) result = HSA_STATUS_ERROR;
    blit_ = nullptr;
  }
  if (completion_signal_.handle != 0) {
    hsa_signal_destroy(completion_signal_);
    completion_signal_.handle = 0;
  }
  return result;
}

hsa_status_t BlitKernelGfx950Aql::SubmitLinearCopyCommand(void* dst, const void* src, size_t size) {
  // Protect completion_signal_ (amd_blit_kernel.cpp:614-639).
  std::lock_guard<std::mutex> guard(lock_);
  if (blit_ == nullptr) return HSA_STATUS_ERROR_NOT_INITIALIZED;
  hsa_signal_store_relaxed(completion_signal_, 1);
  int st = mi355_aql_copy_route(blit_, dst, src, size, static_cast<uint32_t>(slot_), nullptr, 0,
                                completion_signal_.handle);
  if (st != MI355_BLIT_SUCCESS) return to_hsa(st);
  // Wait for the packet to finish: 0 is success, anything else (a negative
  // value, or a queue that has reported an error and will never decrement
  // the signal) is HSA_STATUS_ERROR (amd_blit_kernel.cpp:632-636).
  return to_hsa(mi355_aql_wait_signal(blit_, completion_signal_.handle));
}

hsa_status_t BlitKernelGfx950Aql::SubmitLinearCopyCommand(void* dst, const void* src, size_t size,
                                                          std::vector<core::Signal*>& dep_signals,
                                                          core::Signal& out_signal,
                                                          std::vector<core::Signal*>& /*gang_signals*/) {
  if (blit_ == nullptr) return HSA_STATUS_ERROR_NOT_INITIALIZED;
  const std::vector<uint64_t> deps = handles(dep_signals);
  return to_hsa(mi355_aql_copy_route(blit_, dst, src, size, static_cast<uint32_t>(slot_),
                                     deps.empty() ? nullptr : deps.data(), static_cast<uint32_t>(deps.size()),
                                     core::Signal::Convert(&out_signal).handle));
}

hsa_status_t BlitKernelGfx950Aql::SubmitLinearFillCommand(void* ptr, uint32_t value, size_t count) {
  std::lock_guard<std::mutex> guard(lock_);
  // Reject misaligned base address (amd_blit_kernel.cpp:791-794).
  if ((uintptr_t(ptr) & 0x3) != 0) return HSA_STATUS_ERROR;
  if (blit_ == nullptr) return HSA_STATUS_ERROR_NOT_INITIALIZED;
  hsa_signal_store_relaxed(completion_signal_, 1);
  int st = mi355_aql_fill32(blit_, ptr, value, count, nullptr, 0, completion_signal_.handle);
  if (st != MI355_BLIT_SUCCESS) return to_hsa(st);
  // Wait for the packet to finish: 0 is success, anything else (a negative
  // value, or a queue that has reported an error and will never decrement
  // the signal) is HSA_STATUS_ERROR (amd_blit_kernel.cpp:632-636).
  return to_hsa(mi355_aql_wait_signal(blit_, completion_signal_.handle));
}

hsa_status_t BlitKernelGfx950Aql::SubmitBatchCopyCommand(const void* descs, size_t n, bool descs_on_device,
                                                         std::vector<core::Signal*>& dep_signals,
                                                         core::Signal& out_signal, uint64_t max_total_bytes) {
  if (blit_ == nullptr) return HSA_STATUS_ERROR_NOT_INITIALIZED;
  const std::vector<uint64_t> deps = handles(dep_signals);
  if (descs_on_device && max_total_bytes != 0)
    return to_hsa(mi355_aql_copy_batch_bounded(blit_, static_cast<const mi355_blit_desc_t*>(descs), n, max_total_bytes,
                                               deps.empty() ? nullptr : deps.data(),
                                               static_cast<uint32_t>(deps.size()),
                                               core::Signal::Convert(&out_signal).handle));
  if (descs_on_device)
    return to_hsa(mi355_aql_copy_batch_device(blit_, static_cast<const mi355_blit_desc_t*>(descs), n,
                                              deps.empty() ? nullptr : deps.data(),
                                              static_cast<uint32_t>(deps.size()),
                                              core::Signal::Convert(&out_signal).handle));
  return to_hsa(mi355_aql_copy_batch(blit_, static_cast<const mi355_blit_desc_t*>(descs), n,
                                     deps.empty() ? nullptr : deps.data(), static_cast<uint32_t>(deps.size()),
                                     core::Signal::Convert(&out_signal).handle));
}

static_assert(sizeof(hsa_pitched_ptr_t) == sizeof(mi355_pitched_ptr_t) && sizeof(hsa_dim3_t) == sizeof(mi355_dim3_t),
              "the C ABI's pitched pointer and extent are laid out as HSA's");

hsa_status_t BlitKernelGfx950Aql::SubmitCopyRectCommand(const hsa_pitched_ptr_t* dst, const hsa_dim3_t* dst_offset,
                                                        const hsa_pitched_ptr_t* src, const hsa_dim3_t* src_offset,
                                                        const hsa_dim3_t* range,
                                                        std::vector<core::Signal*>& dep_signals,
                                                        core::Signal& out_signal) {
  if (blit_ == nullptr) return HSA_STATUS_ERROR_NOT_INITIALIZED;
  const std::vector<uint64_t> deps = handles(dep_signals);
  // DmaCopyRect has picked this object by the copy's direction
  // (amd_gpu_agent.cpp:1265-1266): the slot is the route.
  return to_hsa(mi355_aql_copy_rect_route(
      blit_, reinterpret_cast<const mi355_pitched_ptr_t*>(dst), reinterpret_cast<const mi355_dim3_t*>(dst_offset),
      reinterpret_cast<const mi355_pitched_ptr_t*>(src), reinterpret_cast<const mi355_dim3_t*>(src_offset),
      reinterpret_cast<const mi355_dim3_t*>(range), static_cast<uint32_t>(slot_), deps.empty() ? nullptr : deps.data(),
      static_cast<uint32_t>(deps.size()), core::Signal::Convert(&out_signal).handle));
}

hsa_status_t BlitKernelGfx950Aql::EnableProfiling(bool enable) {
  // amd_blit_kernel.cpp:839-842: the queue's profiling bit
  if (blit_ == nullptr) return HSA_STATUS_ERROR_NOT_INITIALIZED;
  return to_hsa(mi355_aql_enable_profiling(blit_, enable ? 1 : 0));
}

void BlitKernelGfx950Aql::ReportQueueError(hsa_status_t status) {
  if (blit_ != nullptr) mi355_aql_report_queue_error(blit_, static_cast<int>(status));
}

uint64_t BlitKernelGfx950Aql::PendingBytes() { return blit_ ? mi355_aql_pending_bytes(blit_) : 0; }

}  // namespace AMD
}  // namespace rocr
