/*
 * mi355_blit_aql -- the gfx950 blit engine submitted the way ROCr's own
 * BlitKernel submits: AQL packets on an HSA queue, kernels from a stand-alone
 * code object, dependencies as BARRIER_AND packets and the caller's
 * hsa_signal_t as the dispatch packet's completion signal.  No HIP: the
 * library depends on libhsa-runtime64 only.
 *
 * Same kernels and the same dispatch sizing as mi355_blit.h; what differs is
 * the submission half.  Citations are relative to
 * projects/rocr-runtime/runtime/hsa-runtime/ in ROCm/rocm-systems.
 *
 * Signals are passed as hsa_signal_t.handle values (uint64_t), 0 meaning "no
 * signal".  Status values are hsa_status_t values.  Every entry point may be
 * called from any thread.
 *
 * MI355_BLIT_LOG_PKTS=1 in the environment of mi355_aql_create[_on] prints one
 * line per barrier and dispatch packet on stderr, with the fields that
 * LogPrint(HSA_AMD_LOG_FLAG_BLIT_KERNEL_PKTS, ...) prints in the reference
 * (core/runtime/amd_blit_kernel.cpp:681-702, 903-923).
 */
#ifndef MI355_BLIT_AQL_H_
#define MI355_BLIT_AQL_H_

#include <stddef.h>
#include <stdint.h>

#include "mi355_blit.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mi355_aql mi355_aql_t;

/* Replaces BlitKernel::BlitKernel + Initialize
 * (core/runtime/amd_blit_kernel.cpp:538-591), GpuAgent::AssembleShader
 * (core/runtime/amd_gpu_agent.cpp:251-426: here one gfx950 code object is
 * loaded with hsa_executable_load_agent_code_object instead of wrapping raw
 * ISA in a hand-filled amd_kernel_code_t) and the creation of the utility
 * queue (amd_gpu_agent.cpp:692-701).  gpu_ordinal counts GPU agents in
 * hsa_iterate_agents order.  Calls hsa_init (reference counted). */
int mi355_aql_create(int gpu_ordinal, mi355_aql_t** out);

/* The same engine on the caller's agent and the caller's queue: what
 * BlitKernel::BlitKernel(core::Queue*) + Initialize(const core::Agent&) take
 * (core/inc/amd_blit_kernel.h:58-66, core/runtime/amd_blit_kernel.cpp:553-591),
 * the queue being the agent's utility queue that GpuAgent made
 * (core/runtime/amd_gpu_agent.cpp:692-701: 64 packets, HSA_QUEUE_TYPE_MULTI)
 * and hands to CreateBlitKernel (:749-759).  hsa_agent_handle is
 * hsa_agent_t.handle of a GPU agent (core::Agent::public_handle()), hsa_queue
 * an hsa_queue_t* (core::Queue::public_handle()).  Calls neither hsa_init nor
 * hsa_shut_down and creates no queue: the runtime must be up, and both it and
 * the queue stay the caller's and must outlive the engine.  The kernarg ring
 * and the pending-bytes ledger have queue->size entries, indexed by packet
 * index like the reference's (amd_blit_kernel.cpp:554-569, 926-941).  Other
 * producers may use the queue at the same time: slots are reserved with an
 * atomic add on the write index and nothing else (amd_blit_kernel.cpp:
 * 844-861), and packets of others are never touched.  Two things follow from
 * sharing: mi355_aql_wait_idle and mi355_aql_destroy wait, behind a barrier
 * packet, also for what others queued earlier; and the queue's error callback
 * is its creator's, who forwards an error with mi355_aql_report_queue_error.
 * NULL or a queue whose size is not a power of two, or an agent that is not a
 * GPU -> INVALID_ARGUMENT. */
int mi355_aql_create_on(uint64_t hsa_agent_handle, void* hsa_queue, mi355_aql_t** out);

/* Replaces BlitKernel::Destroy (amd_blit_kernel.cpp:593-612).  Blocks until
 * every submitted packet has executed (the reference does not wait; its
 * caller must).  A borrowed queue and a borrowed runtime are left alone. */
int mi355_aql_destroy(mi355_aql_t* h);

/* The kernels of one GPU agent.  The reference's agent owns the blit shaders:
 * GpuAgent::AssembleShader makes the code once and every BlitKernel of the
 * agent's blits_[] slots runs it, GpuAgent::ReleaseShader frees it
 * (core/runtime/amd_gpu_agent.cpp:251-428, core/runtime/amd_blit_kernel.cpp:
 * 574-590, 600-604).  Here the gfx950 code object is loaded once per agent and
 * process: every engine created on the agent (mi355_aql_create,
 * mi355_aql_create_on) takes a reference to the same executable and gives it
 * back in mi355_aql_destroy, and the last reference unloads it, whatever the
 * order.  An owner that wants the executable to outlive its engines -- the
 * agent itself, which creates its blits lazily and drops them at will -- holds
 * a reference of its own with _acquire / _release; the runtime must be up for
 * both.  _info tells which executable (hsa_executable_t.handle) an engine runs
 * and how many references it has at the moment. */
typedef struct mi355_aql_code_object mi355_aql_code_object_t;
int mi355_aql_code_object_acquire(uint64_t hsa_agent_handle, mi355_aql_code_object_t** out);
int mi355_aql_code_object_release(mi355_aql_code_object_t* code);
int mi355_aql_code_object_info(mi355_aql_t* h, uint64_t* executable_handle, uint32_t* users);

/* Tells the engine that its queue has stopped on an asynchronous error: what
 * the error callback of a queue the engine created does by itself, and what
 * the owner of a borrowed queue forwards from its own callback (the role of
 * core::Queue::DefaultErrorHandler, core/runtime/queue.cpp:52-59).  From then
 * on submissions answer HSA_STATUS_ERROR and every wait inside the library
 * ends with HSA_STATUS_ERROR instead of waiting for signals that nobody will
 * complete.  status == 0 is ignored.  Tests of the error path use it to force
 * the condition from the host. */
int mi355_aql_report_queue_error(mi355_aql_t* h, int status);

/* Waits, actively and in slices of about a millisecond, until the signal's
 * value is below 1: the wait of BlitKernel's blocking calls
 * (amd_blit_kernel.cpp:632-636, 830-834).  0 -> SUCCESS; a negative value
 * (a failed command, inc/hsa_ext_amd.h:1735-1739) -> HSA_STATUS_ERROR; a
 * reported queue error while the value is still 1 or more -> HSA_STATUS_ERROR
 * where the reference would wait forever. */
int mi355_aql_wait_signal(mi355_aql_t* h, uint64_t signal);

/* Blocking forms: BlitKernel::SubmitLinearCopyCommand(dst, src, size) and
 * SubmitLinearFillCommand (amd_blit_kernel.cpp:614-639, 787-837).  They hold
 * the engine's blocking-call lock, arm its private completion signal with 1,
 * submit, and wait for that signal only (not for the queue to drain), as
 * mi355_aql_wait_signal waits.  Argument rules of mi355_aql_copy_route /
 * mi355_aql_fill32. */
int mi355_aql_copy_sync(mi355_aql_t* h, void* dst, const void* src, size_t bytes, uint32_t route);
int mi355_aql_fill32_sync(mi355_aql_t* h, void* ptr, uint32_t value, size_t num_dwords);

/* Replaces BlitKernel::SubmitLinearCopyCommand, asynchronous overload
 * (amd_blit_kernel.cpp:641-785): ceil(num_deps / 5) BARRIER_AND packets, then
 * one KERNEL_DISPATCH packet whose completion_signal is `completion_signal`
 * (decremented once by the packet processor when the copy is done).
 * dst or src NULL -> INVALID_ARGUMENT.  bytes == 0: a barrier packet carries
 * the dependencies and the completion signal, nothing is copied.
 * The dispatch packet's barrier bit: set behind dependency barriers (the copy
 * must not start before them); otherwise clear, as in the reference
 * (amd_blit_kernel.cpp:870-882: consecutive blits may overlap), with one
 * exception on an engine that runs on a queue of its own (mi355_aql_create):
 * there a copy, fill or region copy of 4 MiB or more carries the bit, because
 * two large transfers that overlap slow each other down
 * (mi355_aql_set_large_transfer_barrier).  An engine on a borrowed queue
 * (mi355_aql_create_on) keeps the reference's packets. */
int mi355_aql_copy(mi355_aql_t* h, void* dst, const void* src, size_t bytes,
                   const uint64_t* dep_signals, uint32_t num_deps, uint64_t completion_signal);

/* mi355_aql_copy for a copy that crosses the host link, launched in the
 * shape that suits the link (mi355_blit.h, MI355_BLIT_ROUTE_*): what the
 * reference submits to blits_[BlitHostToDev] / blits_[BlitDevToHost]
 * (amd_gpu_agent.cpp:761-841, :2370-2377).  MI355_BLIT_ROUTE_DEVICE is
 * mi355_aql_copy itself; any other value -> INVALID_ARGUMENT. */
int mi355_aql_copy_route(mi355_aql_t* h, void* dst, const void* src, size_t bytes, uint32_t route,
                         const uint64_t* dep_signals, uint32_t num_deps, uint64_t completion_signal);

/* Replaces the dispatch half of BlitKernel::SubmitLinearFillCommand
 * (amd_blit_kernel.cpp:787-837), asynchronous like the copy.  ptr NULL or not
 * 4-byte aligned -> INVALID_ARGUMENT. */
int mi355_aql_fill32(mi355_aql_t* h, void* ptr, uint32_t value, size_t num_dwords,
                     const uint64_t* dep_signals, uint32_t num_deps, uint64_t completion_signal);

/* Batched small copies (no counterpart in the reference): n host-resident
 * descriptors in one submission, the last packet carrying the completion
 * signal: two dispatch packets when the host walks the descriptors (record
 * kernel, copy), four when it stages them as they are for the GPU to do the
 * prefix sum (chosen for thousands of short copies, and whenever no batch is
 * running on the engine), behind ceil(num_deps / 5) barrier packets -- all with
 * the barrier bit set.  That matters on a borrowed 64-packet queue. */
int mi355_aql_copy_batch(mi355_aql_t* h, const mi355_blit_desc_t* descs, size_t n,
                         const uint64_t* dep_signals, uint32_t num_deps, uint64_t completion_signal);

/* The same with device-resident descriptors (read in place; they must stay
 * valid until completion and be ready when the dependencies are).  The host
 * cannot know the work's size: see mi355_blit_copy_batch in mi355_blit.h.
 * Four packets (two for the prefix sum, the records, the copy). */
int mi355_aql_copy_batch_device(mi355_aql_t* h, const mi355_blit_desc_t* device_descs, size_t n,
                                const uint64_t* dep_signals, uint32_t num_deps, uint64_t completion_signal);

/* Device-resident descriptors that together move at most max_total_bytes
 * bytes (see mi355_blit_copy_batch_bounded in mi355_blit.h: the bound sizes
 * the grid and the record buffer; what exceeds it is slower, not lost).  Four
 * packets.
 * max_total_bytes == 0 with n > 0 -> INVALID_ARGUMENT. */
int mi355_aql_copy_batch_bounded(mi355_aql_t* h, const mi355_blit_desc_t* device_descs, size_t n,
                                 uint64_t max_total_bytes, const uint64_t* dep_signals, uint32_t num_deps,
                                 uint64_t completion_signal);

/* Pitched 3-D region copy, asynchronous like mi355_aql_copy: the shader
 * counterpart of BlitSdmaBase::SubmitCopyRectCommand
 * (core/inc/amd_blit_sdma.h:68-73), which the reference reaches through
 * hsa_amd_memory_async_copy_rect -> GpuAgent::DmaCopyRect
 * (core/runtime/hsa_ext_amd.cpp:367-410, amd_gpu_agent.cpp:1255-1283) on SDMA
 * engines only.  One dispatch packet behind the dependency barriers.
 * Argument rules as for mi355_blit_copy_rect; with a zero in range the
 * dependencies and the completion signal ride on a barrier packet. */
int mi355_aql_copy_rect(mi355_aql_t* h, const mi355_pitched_ptr_t* dst, const mi355_dim3_t* dst_offset,
                        const mi355_pitched_ptr_t* src, const mi355_dim3_t* src_offset,
                        const mi355_dim3_t* range, const uint64_t* dep_signals, uint32_t num_deps,
                        uint64_t completion_signal);

/* mi355_aql_copy_rect for a region one side of which is host memory
 * (mi355_blit_copy_rect_route in mi355_blit.h): the direction argument of
 * hsa_amd_memory_async_copy_rect, which GpuAgent::DmaCopyRect turns into the
 * choice between blits_[BlitHostToDev] and blits_[BlitDevToHost]
 * (amd_gpu_agent.cpp:1265-1266). */
int mi355_aql_copy_rect_route(mi355_aql_t* h, const mi355_pitched_ptr_t* dst, const mi355_dim3_t* dst_offset,
                              const mi355_pitched_ptr_t* src, const mi355_dim3_t* src_offset,
                              const mi355_dim3_t* range, uint32_t route, const uint64_t* dep_signals,
                              uint32_t num_deps, uint64_t completion_signal);

/* Blocks until the queue has drained: the wait BlitKernel's blocking calls do
 * on their completion signal (amd_blit_kernel.cpp:632, 830). */
int mi355_aql_wait_idle(mi355_aql_t* h);

/* Replaces BlitKernel::PendingBytes (amd_blit_kernel.cpp:943-970), with the
 * same ledger: bytes queued before each packet index, compared with the
 * queue's read index.  0 is exact. */
uint64_t mi355_aql_pending_bytes(mi355_aql_t* h);

/* Replaces BlitKernel::EnableProfiling (amd_blit_kernel.cpp:839-842): sets the
 * queue's profiling bit, after which the packet processor writes start and end
 * timestamps into each completion signal.  While it is on, a copy of 1.5 GiB
 * or more is not cut into pieces (mi355_aql_copy): the stamps are those of one
 * dispatch, and they are to cover the command. */
int mi355_aql_enable_profiling(mi355_aql_t* h, int enable);

/* Start and end of the command whose completion signal is given, as stamped
 * by the packet processor while profiling is enabled, in ticks of the system
 * timestamp (ticks_per_second of them in a second): what
 * hsa_amd_profiling_get_async_copy_time reports for a copy
 * (core/runtime/hsa_ext_amd.cpp:474-502). */
int mi355_aql_get_command_time(mi355_aql_t* h, uint64_t completion_signal, uint64_t* start_ticks,
                               uint64_t* end_ticks, uint64_t* ticks_per_second);

int mi355_aql_set_tuning(mi355_aql_t* h, const mi355_blit_tuning_t* tuning);
int mi355_aql_last_launch_info(mi355_aql_t* h, mi355_blit_plan_t* out);
/* Records MI355_ENGINE_* for mi355_aql_last_launch_info to report (the caller
 * policy does, for every asynchronous copy it judges). */
int mi355_aql_note_reference_engine(mi355_aql_t* h, uint32_t engine);
int mi355_aql_num_cus(mi355_aql_t* h);

/* Fence scope of the dispatch packets' acquire and release: 1 = system (the
 * reference's choice, amd_blit_kernel.cpp:870-873; the default), 0 = agent,
 * enough when no other device or the host reads the result without a later
 * system-scope release. */
int mi355_aql_set_system_scope_fences(mi355_aql_t* h, int enable);

/* Whether a copy, fill or region copy of 4 MiB or more carries the barrier bit
 * although no dependency asks for it (1) or is queued like the reference's
 * blits, bit clear (0).  With the bit clear the packet processor starts a
 * transfer while the one before still drains; the two then work on stretches
 * of memory far apart and both slow down (back-to-back 1 GiB copies: 334 us
 * apiece overlapping, 317 us one after the other).  With the bit set a transfer
 * waits for every earlier packet on the queue, other producers' included,
 * which is why the default is 1 on a queue of the engine's own
 * (mi355_aql_create) and 0 on a borrowed one (mi355_aql_create_on).  A
 * stronger order than core::Blit promises, never a weaker one. */
int mi355_aql_set_large_transfer_barrier(mi355_aql_t* h, int enable);

/* hsa_agent_t.handle of the engine's GPU. */
uint64_t mi355_aql_gpu_agent(mi355_aql_t* h);

/* Two host buffers of `half_bytes` each that the GPU can access, owned by the
 * engine (allocated on first use from the fine-grained host pool, kept until
 * destroy): the bounce buffers of host<->device copies whose host side cannot
 * be locked.  The caller serialises their use. */
int mi355_aql_staging(mi355_aql_t* h, size_t* half_bytes, void** half0, void** half1);

/* ---- caller policy: what sits between the HSA API and the blit ------------
 * The three entry points below restate, over this engine, the decisions ROCr
 * takes before it reaches core::Blit, so that they can stand in for
 * hsa_memory_copy, hsa_amd_memory_fill and hsa_amd_memory_async_copy on one
 * GPU.  Pointers are classified with hsa_amd_pointer_info, as
 * Runtime::CopyMemory does (core/runtime/runtime.cpp:469-552). */

/* hsa_memory_copy (core/runtime/hsa.cpp:1170-1184 + Runtime::CopyMemory,
 * runtime.cpp:469-552).  Blocking.  NULL -> INVALID_ARGUMENT; size 0 ->
 * SUCCESS; host<->host is one memcpy on the calling thread (:507-510); when
 * one side is host memory unknown to the runtime it is locked for the GPU for
 * the duration of the copy (:521-537), or, where the system refuses to lock
 * existing memory, bounced through the engine's staging buffers in 4 MiB
 * pieces; everything else goes to the blit, on the route the two placements
 * give (the reference picks blits_[BlitHostToDev] or blits_[BlitDevToHost]
 * there, amd_gpu_agent.cpp:2370-2377). */
int mi355_hsa_memory_copy(mi355_aql_t* h, void* dst, const void* src, size_t size);

/* hsa_amd_memory_fill (core/runtime/hsa_ext_amd.cpp:237-251 + Runtime::FillMemory,
 * runtime.cpp:627-664).  Blocking.  NULL or ptr % 4 -> INVALID_ARGUMENT;
 * count 0 -> SUCCESS; memory the GPU can reach is filled by the blit; plain
 * host memory is filled on the host with the full 32-bit pattern (the
 * reference's memset(ptr, value, count*4) there keeps only the low byte,
 * runtime.cpp:657-661: a defect, not reproduced). */
int mi355_hsa_amd_memory_fill(mi355_aql_t* h, void* ptr, uint32_t value, size_t count);

/* hsa_amd_memory_async_copy for copies this GPU executes
 * (core/runtime/hsa_ext_amd.cpp:253-294).  NULL pointers, or a dependency count
 * that disagrees with the array pointer, or a zero completion signal ->
 * INVALID_ARGUMENT; size 0 -> SUCCESS without touching the signal (:285-291);
 * both ranges must already be accessible to the GPU (device memory, or host
 * memory allocated or locked through the runtime), as the API demands.  The
 * reference learns the direction from the two agents it is handed
 * (GetBlitObject, amd_gpu_agent.cpp:2379-2442); this signature has none, so
 * copies of 1 MiB and more, the sizes whose launch shape depends on it, look
 * the two pointers up (hsa_amd_pointer_info) and take the route they give.
 * The copy always runs on this engine; which engine GetBlitObject would have
 * picked for it (amd_gpu_agent.cpp:2379-2398, HSA_FORCE_SDMA_SIZE) is left in
 * mi355_blit_plan_t::reference_engine of mi355_aql_last_launch_info. */
int mi355_hsa_amd_memory_async_copy(mi355_aql_t* h, void* dst, const void* src, size_t size,
                                    uint32_t num_dep_signals, const uint64_t* dep_signals,
                                    uint64_t completion_signal);

/* hsa_amd_memory_async_copy_on_engine for copies within this GPU's memory
 * (core/runtime/hsa_ext_amd.cpp:296-339, Runtime::CopyMemoryOnEngine
 * runtime.cpp:585-601, GpuAgent::DmaCopyOnEngine amd_gpu_agent.cpp:1110-1179).
 * The argument checks of the asynchronous copy; size 0 -> SUCCESS; engine_id
 * (hsa_amd_sdma_engine_id_t) must be exactly one bit and name an engine the GPU
 * has (HSA_AMD_AGENT_INFO_NUM_SDMA_ENG + ..._XGMI_ENG), else INVALID_ARGUMENT.
 * Within one GPU the reference sets the named engine aside for the blit kernel
 * unless force_copy_on_sdma: so does this.  With force_copy_on_sdma the copy
 * would need an SDMA engine, which this library does not drive ->
 * OUT_OF_RESOURCES. */
int mi355_hsa_amd_memory_async_copy_on_engine(mi355_aql_t* h, void* dst, const void* src, size_t size,
                                              uint32_t num_dep_signals, const uint64_t* dep_signals,
                                              uint64_t completion_signal, uint32_t engine_id,
                                              int force_copy_on_sdma);

/* hsa_amd_memory_copy_engine_status between this GPU and the host
 * (core/runtime/hsa_ext_amd.cpp:341-352, Runtime::CopyMemoryStatus
 * runtime.cpp:603-613, GpuAgent::DmaCopyStatus amd_gpu_agent.cpp:1181-1243).
 * dst_is_gpu / src_is_gpu say which side is this GPU; both or neither ->
 * HSA_STATUS_ERROR_INVALID_AGENT (0x1004) as for equal agents.  The mask is
 * what the reference answers on an agent whose SDMA engines are all unused
 * (this library never occupies one): the H2D and the D2H engine and every
 * xGMI engine; OUT_OF_RESOURCES with a mask of 0 on a GPU without engines. */
int mi355_hsa_amd_memory_copy_engine_status(mi355_aql_t* h, int dst_is_gpu, int src_is_gpu,
                                            uint32_t* engine_ids_mask);

/* hsa_amd_memory_async_copy_rect for copies this GPU executes
 * (core/runtime/hsa_ext_amd.cpp:367-410): NULL pointers, a dependency count
 * that disagrees with the array pointer, a zero completion signal or
 * dir == 0 (hsaHostToHost) -> INVALID_ARGUMENT; a zero in range -> SUCCESS
 * without touching the signal (:400-402).  Where the reference then fails with
 * OUT_OF_RESOURCES unless an SDMA engine is available, this runs the shader,
 * on the route dir names (hsaHostToDevice = 1, hsaDeviceToHost = 2; any other
 * value, hsaDeviceToDevice = 3 included, within the device). */
int mi355_hsa_amd_memory_async_copy_rect(mi355_aql_t* h, const mi355_pitched_ptr_t* dst,
                                         const mi355_dim3_t* dst_offset, const mi355_pitched_ptr_t* src,
                                         const mi355_dim3_t* src_offset, const mi355_dim3_t* range, int dir,
                                         uint32_t num_dep_signals, const uint64_t* dep_signals,
                                         uint64_t completion_signal);

#ifdef __cplusplus
}
#endif
#endif /* MI355_BLIT_AQL_H_ */
