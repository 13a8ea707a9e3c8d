// Compiled by tests/test_rocr_in_tree.py against ROCr's own core/inc headers
// (MI355_ROCR_IN_TREE): BlitKernelGfx950Aql must be a concrete core::Blit --
// every pure virtual of core/inc/blit.h:52-122 overridden with the exact
// signature -- and usable the way GpuAgent::CreateBlitKernel uses
// AMD::BlitKernel (core/runtime/amd_gpu_agent.cpp:749-759): constructed over
// the core::Queue*, initialised with the core::Agent, destroyed and dropped
// when initialisation fails, handed out as a core::Blit*.
#include "rocr_blit.h"

namespace rocr {
namespace AMD {

core::Blit* CreateBlitKernelGfx950(core::Queue* queue, const core::Agent& agent) {
  BlitKernelGfx950Aql* kernl = new BlitKernelGfx950Aql(queue);
  if (kernl->Initialize(agent) != HSA_STATUS_SUCCESS) {
    kernl->Destroy(agent);
    delete kernl;
    kernl = NULL;
  }
  return kernl;
}

// The calls GpuAgent makes through the interface (amd_gpu_agent.cpp:913-917,
// 951, 1080-1097, 1165-1176, 1185-1186, 1285-1293).
hsa_status_t UseLikeGpuAgent(core::Blit* blit, const core::Agent& agent, void* dst, const void* src, size_t size,
                             std::vector<core::Signal*>& dep_signals, core::Signal& out_signal) {
  std::vector<core::Signal*> gang_signals;
  hsa_status_t st = blit->SubmitLinearCopyCommand(dst, src, size);
  if (st != HSA_STATUS_SUCCESS) return st;
  st = blit->SubmitLinearCopyCommand(dst, src, size, dep_signals, out_signal, gang_signals);
  if (st != HSA_STATUS_SUCCESS) return st;
  st = blit->SubmitLinearFillCommand(dst, 0u, size / sizeof(uint32_t));
  if (st != HSA_STATUS_SUCCESS) return st;
  st = blit->EnableProfiling(agent.profiling_enabled());
  if (st != HSA_STATUS_SUCCESS) return st;
  if (blit->isSDMA() || blit->GangLeader()) return HSA_STATUS_ERROR;
  blit->GangLeader(false);
  return blit->PendingBytes() == 0 ? blit->Destroy(agent) : HSA_STATUS_SUCCESS;
}

}  // namespace AMD
}  // namespace rocr
