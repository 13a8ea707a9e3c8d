/*
 * mi355_blit -- C ABI of the gfx950 blit engine (linear copy, dword fill and
 * batched small copies done by compute kernels on one MI355X).
 *
 * This is the boundary a ROCr build binds to in place of the body of
 * AMD::BlitKernel.  Citations are relative to
 * projects/rocr-runtime/runtime/hsa-runtime/ in ROCm/rocm-systems.
 *
 * Conventions: plain C, opaque handle, every call returns an int status whose
 * values equal the hsa_status_t values of the same meaning (inc/hsa.h), so a
 * caller inside ROCr can return them unchanged.  Every entry point may be
 * called from any thread; calls on one handle are submitted in call order per
 * stream.  Pointers must be device-accessible on the handle's GPU and stay
 * valid until the work has completed; overlapping source and destination are
 * undefined, as in inc/hsa_ext_amd.h:1712-1714.
 */
#ifndef MI355_BLIT_H_
#define MI355_BLIT_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_BLIT_ABI_VERSION 4

/* Same numeric values as HSA_STATUS_* (inc/hsa.h). */
enum {
  MI355_BLIT_SUCCESS = 0x0,
  MI355_BLIT_ERROR = 0x1000,                  /* HSA_STATUS_ERROR */
  MI355_BLIT_ERROR_INVALID_ARGUMENT = 0x1001, /* HSA_STATUS_ERROR_INVALID_ARGUMENT */
  MI355_BLIT_ERROR_OUT_OF_RESOURCES = 0x1008, /* HSA_STATUS_ERROR_OUT_OF_RESOURCES */
  MI355_BLIT_ERROR_NOT_INITIALIZED = 0x100B   /* HSA_STATUS_ERROR_NOT_INITIALIZED */
};

/* Kernel families.  The reference picks between CopyAligned and CopyMisaligned
 * on (src & 3) == (dst & 3) (core/runtime/amd_blit_kernel.cpp:716); here the
 * same predicate picks between the plain vector copy and the one that realigns
 * source dwords in registers. */
enum {
  MI355_BLIT_KERNEL_COPY = 0,         /* (src - dst) % 4 == 0 */
  MI355_BLIT_KERNEL_COPY_REALIGN = 1, /* (src - dst) % 4 != 0 */
  MI355_BLIT_KERNEL_FILL = 2,
  MI355_BLIT_KERNEL_COPY_BATCH = 3,
  MI355_BLIT_KERNEL_COPY_RECT = 4
};

typedef struct mi355_blit mi355_blit_t;

/* How one command is cut up and launched.  Replaces the phase bounds the
 * reference writes into BlitKernel::KernelArgs (core/inc/amd_blit_kernel.h:
 * 122-154) and its fixed grids (amd_blit_kernel.cpp:723, 759, 797).
 *   bytes == head_bytes + 16 * body_vecs + tail_bytes
 *   (dst + head_bytes) % 16 == 0 whenever body_vecs > 0
 *   head_bytes <= 15 and tail_bytes <= 15
 * For a fill the same fields count bytes of whole dwords. */
typedef struct {
  uint32_t kernel;      /* MI355_BLIT_KERNEL_* */
  uint32_t wg_size;     /* work-items per workgroup, multiple of 64 */
  uint32_t grid;        /* workgroups */
  uint32_t unroll;      /* 16-byte vectors each lane keeps in flight */
  uint32_t nt_load;     /* non-temporal loads */
  uint32_t store_policy;/* MI355_BLIT_STORE_* */
  uint32_t byte_shift;  /* (src - dst) & 3 */
  uint32_t lead_vecs;   /* ((dst + head_bytes) & 255) / 16: tiles are anchored at
                           256-byte boundaries of the destination, the first one
                           starts this many vector slots below the body */
  uint64_t head_bytes;
  uint64_t body_vecs;
  uint64_t tail_bytes;
  uint32_t xcd_run;     /* 0: workgroups take tiles in launch order.  N > 1: the
                           hardware deals consecutive workgroups to the 8 XCDs
                           (each with its own L2) in turn; the launch is
                           permuted so that every XCD works on runs of N
                           neighbouring workgroups' tiles, and a cache line two
                           neighbouring tiles share is fetched into one L2 */
  uint32_t route;       /* MI355_BLIT_ROUTE_* the launch was shaped for */
  uint32_t reference_engine; /* MI355_ENGINE_*: the engine GpuAgent::GetBlitObject
                           (core/runtime/amd_gpu_agent.cpp:2379-2398) would have
                           sent the last mi355_hsa_amd_memory_async_copy to;
                           0 when no such call has been judged.  Reported by
                           mi355_aql_last_launch_info only */
  uint32_t pieces;      /* launches the command was cut into: 1, or more for a
                           copy of 1.5 GiB and beyond within the device, which is
                           submitted as consecutive copies of at most 512 MiB
                           (the other fields then describe the last of them) */
} mi355_blit_plan_t;

/* The engine choice of GpuAgent::GetBlitObject for an asynchronous copy within
 * one GPU's memory (core/runtime/amd_gpu_agent.cpp:2379-2398): below
 * HSA_FORCE_SDMA_SIZE the SDMA-capable engine of blits_[BlitDevToHost], "to
 * avoid cache flushing", from there on the blit kernel. */
enum {
  MI355_ENGINE_NONE = 0,
  MI355_ENGINE_BLIT_KERNEL = 1, /* blits_[BlitDevToDev] */
  MI355_ENGINE_SDMA = 2         /* blits_[BlitDevToHost] */
};

/* Flag::force_sdma_size() (core/util/flag.h:206-207): HSA_FORCE_SDMA_SIZE read
 * with atoi, 1 MiB when unset or empty.  Read on every call. */
uint64_t mi355_policy_force_sdma_size(void);

/* MI355_ENGINE_SDMA when size < force_sdma_size, else MI355_ENGINE_BLIT_KERNEL
 * (amd_gpu_agent.cpp:2390-2397).  Pure.  With this engine behind BlitDevToDev
 * the measured crossover against the DMA engine on MI355X is 128 KiB with
 * system-scope fences and 0 with agent-scope fences: a deployment would set
 * HSA_FORCE_SDMA_SIZE to that. */
uint32_t mi355_policy_same_gpu_engine(uint64_t size, uint64_t force_sdma_size);

/* Which memories a linear copy connects.  The reference keeps one blit object
 * per direction (core/inc/amd_gpu_agent.h:588, BlitDevToDev / BlitHostToDev /
 * BlitDevToHost; amd_gpu_agent.cpp:846-867, GetPcieBlit :2370-2377) and may put
 * a blit kernel behind each; here the direction shapes the launch.  A copy
 * one side of which is host memory is bound by the host link (64 GB/s
 * nominal), not by HBM: it wants a few hundred waves walking the buffer in
 * address order, not a wave per KiB.  The kernels and the results are the
 * same on every route. */
enum {
  MI355_BLIT_ROUTE_DEVICE = 0,         /* both sides in the GPU's memory */
  MI355_BLIT_ROUTE_HOST_TO_DEVICE = 1, /* src is host memory the GPU can read */
  MI355_BLIT_ROUTE_DEVICE_TO_HOST = 2  /* dst is host memory the GPU can write */
};

/* Cache policy of the body's 16-byte stores. */
enum {
  MI355_BLIT_STORE_CACHED = 0,    /* write-back L2 */
  MI355_BLIT_STORE_NT = 1,        /* non-temporal hint */
  MI355_BLIT_STORE_AGENT_WT = 2,  /* sc1: written through L2 */
  MI355_BLIT_STORE_SYSTEM_WT = 3  /* sc0 sc1: written through, system scope */
};

/* Overrides for the sizing heuristics; 0 in a field keeps the heuristic.
 * nt_load: 0 = heuristic, 1 = force off, 2 = force on.
 * store_policy: 0 = heuristic, otherwise MI355_BLIT_STORE_* + 1.
 * xcd_run: 0 = heuristic, 1 = launch order, N > 1 = runs of N workgroups per XCD. */
typedef struct {
  uint32_t wg_size;
  uint32_t unroll;
  uint32_t max_grid;   /* cap on workgroups; beyond it waves stride over tiles */
  uint32_t nt_load;
  uint32_t store_policy;
  uint32_t xcd_run;
  uint32_t batch_prefetch; /* batched copies: 0 = heuristic, 1 = no record prefetch,
                              N > 1 = touch the record N workgroups ahead */
  uint32_t batch_staging;  /* batches of host-resident descriptors: 0 = heuristic, 1 = the host
                              walks the descriptors, 2 = they are staged as they are and the
                              GPU does the prefix sum */
  uint32_t copy_piece_mib; /* copies within the device: 0 = heuristic (pieces of 512 MiB from
                              1.5 GiB on), 1 = always one launch, N > 1 = a copy of more than
                              N MiB goes out in pieces of N MiB */
} mi355_blit_tuning_t;

/* One element of a batched submission.  No counterpart in the reference. */
typedef struct {
  void* dst;
  const void* src;
  uint64_t bytes;
} mi355_blit_desc_t;

/* A pitched pointer and a 3-D extent, laid out as hsa_pitched_ptr_t and
 * hsa_dim3_t (inc/hsa_ext_amd.h:1842-1846, inc/hsa.h hsa_dim3_s): pitch is the
 * byte distance between rows, slice between layers; x counts bytes, y rows
 * and z layers. */
typedef struct {
  void* base;
  size_t pitch;
  size_t slice;
} mi355_pitched_ptr_t;

typedef struct {
  uint32_t x;
  uint32_t y;
  uint32_t z;
} mi355_dim3_t;

/* Replaces BlitKernel::BlitKernel + Initialize (core/runtime/amd_blit_kernel.cpp:
 * 538-591): binds to a GPU, reads its CU count, loads the kernels' code object
 * (what GpuAgent::AssembleShader does for the reference,
 * core/runtime/amd_gpu_agent.cpp:251-426) and creates the submission stream. */
int mi355_blit_create(int device_ordinal, mi355_blit_t** out);

/* Replaces BlitKernel::Destroy (amd_blit_kernel.cpp:593-612).  Blocks until all
 * submitted commands have executed. */
int mi355_blit_destroy(mi355_blit_t* h);

/* Replaces the dispatch half of BlitKernel::SubmitLinearCopyCommand
 * (amd_blit_kernel.cpp:641-785) and the CopyAligned / CopyMisaligned shaders
 * (core/runtime/blit_shaders/blit_copyAligned.s, blit_copyMisaligned.s).
 * Non-blocking.  stream is a hipStream_t, or NULL for the handle's own stream.
 * dst or src NULL -> INVALID_ARGUMENT; bytes == 0 -> SUCCESS without a launch
 * (core/runtime/hsa.cpp:1170-1184).
 * Copy, fill and region copy are one kernel launch each and allocate nothing,
 * so they may be issued on a stream under HIP graph capture; such commands
 * are not counted by mi355_blit_pending_bytes.  The batched copy stages its
 * descriptors and may not. */
int mi355_blit_copy(mi355_blit_t* h, void* dst, const void* src, size_t bytes, void* stream);

/* mi355_blit_copy for a copy that crosses the host link: what the reference
 * submits to blits_[BlitHostToDev] / blits_[BlitDevToHost] when a blit kernel
 * serves them (amd_gpu_agent.cpp:761-841 DmaCopy, :2370-2377).  route is
 * MI355_BLIT_ROUTE_*; MI355_BLIT_ROUTE_DEVICE is mi355_blit_copy itself, any
 * other value -> INVALID_ARGUMENT.  The host side must be memory the GPU can
 * access (allocated through the runtime or locked). */
int mi355_blit_copy_route(mi355_blit_t* h, void* dst, const void* src, size_t bytes, uint32_t route,
                          void* stream);

/* Replaces the dispatch half of BlitKernel::SubmitLinearFillCommand
 * (amd_blit_kernel.cpp:787-837) and the Fill shader (blit_shaders/blit_fill.s).
 * Non-blocking.  ptr NULL or not 4-byte aligned -> INVALID_ARGUMENT;
 * num_dwords == 0 -> SUCCESS without a launch
 * (core/runtime/hsa_ext_amd.cpp:237-251). */
int mi355_blit_fill32(mi355_blit_t* h, void* ptr, uint32_t value, size_t num_dwords, void* stream);

/* Batched small-copy descriptor path: n independent copies in one submission.
 * No counterpart in the reference (it submits one AQL packet per copy).
 * descs may live in host memory (descs_on_device == 0: the library checks and
 * stages them before it returns, so the array may be reused at once) or be
 * device-resident (descs_on_device != 0: read in place, must stay
 * valid until completion).  Host-resident descriptors are either walked by the
 * host (their chunks counted and summed: one small kernel before the copy) or,
 * from 4096 copies on, staged as they are for the GPU's own prefix sum when
 * the copies are short or no batch is running that would hide the walk
 * (mi355_blit_tuning_t::batch_staging overrides the choice).  The host cannot see the lengths of
 * device-resident descriptors: it sizes the launch by the bytes per copy of
 * the last such batch on the handle (which the copy kernel leaves in host
 * memory; 32 KiB a copy before any has run), the kernels read the real chunk
 * count on the device, and a batch that differs from the guess is slower,
 * never wrong (a caller that knows a bound says so through
 * mi355_blit_copy_batch_bounded).  A batch may have at most 2^32-1
 * chunks of 4 KiB.  Regions must not overlap one another.  A stream
 * under HIP graph capture -> INVALID_ARGUMENT (both batched entry points). */
int mi355_blit_copy_batch(mi355_blit_t* h, const mi355_blit_desc_t* descs, size_t n,
                          int descs_on_device, void* stream);

/* The batched path for device-resident descriptors whose sizes the host does
 * not know but can bound (a previous kernel wrote them): the n copies together
 * move at most max_total_bytes bytes.  No counterpart in the reference.  The
 * bound sizes the record buffer (max_total_bytes / 4096 + 2 n records of 32
 * bytes, 512 MiB at most) and the grid (a workgroup per likely chunk) in
 * place of the library's assumption.  It is a hint, not a contract: a loose
 * bound costs idle waves, and chunks beyond a bound that the descriptors
 * exceed have no record and are found through the prefix sums by the copy
 * kernel itself, several times slower but complete.  max_total_bytes == 0
 * with n > 0, or a bound that needs 2^32 records or more -> INVALID_ARGUMENT. */
int mi355_blit_copy_batch_bounded(mi355_blit_t* h, const mi355_blit_desc_t* device_descs, size_t n,
                                  uint64_t max_total_bytes, void* stream);

/* mi355_blit_copy_batch_bounded for callers that cannot allocate: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It
 * has no counterpart in the reference.  Same arguments, same kernels and same
 * results, but the prefix sums and chunk records live in a fixed array in the
 * library's device code (16.25 MiB per GPU, held from the load of the library
 * to the end of the process) instead of buffers the handle grows on demand,
 * and the call makes no hipMalloc, hipFree or other allocating call: four
 * kernel launches on the stream and nothing else -- no event, no wait, no
 * write to host memory (and a hipSetDevice pair only when the calling thread's
 * current device is not the handle's).  For the same reason the command is not
 * entered in the pending-bytes ledger: mi355_blit_pending_bytes does not see
 * it, and the caller, who owns the stream, waits on the stream.
 * Limits: n <= MI355_BLIT_NOALLOC_MAX_COPIES, more -> OUT_OF_RESOURCES and
 * nothing is launched.  The bytes are not limited: the array has room for
 * 2^19 chunk records (2 GiB of copies) and chunks beyond them are found
 * through the prefix sums by the copy kernel, as when a bound is exceeded.
 * The array is one per GPU, shared by every handle and every call on that GPU,
 * and keeps the last call's contents (each call rewrites all it reads, so
 * nothing needs clearing): calls that may overlap on one GPU -- on different
 * streams or handles without an ordering between them -- race and must be
 * ordered by the caller; calls on one stream are ordered by the stream.  The
 * engine does not size later batches by this one (nothing is written to host
 * memory). */
#define MI355_BLIT_NOALLOC_MAX_COPIES 65536
int mi355_blit_copy_batch_bounded_noalloc(mi355_blit_t* h, const mi355_blit_desc_t* device_descs, size_t n,
                                          uint64_t max_total_bytes, void* stream);

/* Pitched 3-D region copy as a shader: range->z layers of range->y rows of
 * range->x bytes, from src at src_offset to dst at dst_offset.  The reference
 * has this on its SDMA engines only: GpuAgent::DmaCopyRect answers
 * OUT_OF_RESOURCES when the agent's blits are shader blits
 * (core/runtime/amd_gpu_agent.cpp:1255-1283), and BlitSdma's
 * SubmitCopyRectCommand needs 4-byte aligned elements
 * (inc/hsa_ext_amd.h:1840).  Here any byte alignment of bases, offsets,
 * pitches and widths is accepted.  One launch, no staging memory.
 * NULL argument or base -> INVALID_ARGUMENT; a zero in range -> SUCCESS
 * without a launch (core/runtime/hsa_ext_amd.cpp:367-410); a region that is
 * not a box inside both surfaces (offset.x + range.x > pitch, offset.y +
 * range.y > slice / pitch when slice != 0, range.z > 1 with slice == 0:
 * core/runtime/amd_blit_sdma.cpp:577-585) or more than 2^32-1 rows in all ->
 * INVALID_ARGUMENT.  Source and destination regions must not
 * overlap. */
int mi355_blit_copy_rect(mi355_blit_t* h, const mi355_pitched_ptr_t* dst, const mi355_dim3_t* dst_offset,
                         const mi355_pitched_ptr_t* src, const mi355_dim3_t* src_offset,
                         const mi355_dim3_t* range, void* stream);

/* mi355_blit_copy_rect for a region one side of which is host memory the GPU
 * can access: route is MI355_BLIT_ROUTE_*, the hsa_amd_copy_direction_t of
 * hsa_amd_memory_async_copy_rect (inc/hsa_ext_amd.h, hsaHostToDevice = 1,
 * hsaDeviceToHost = 2) with 0 for a copy within the device. */
int mi355_blit_copy_rect_route(mi355_blit_t* h, const mi355_pitched_ptr_t* dst, const mi355_dim3_t* dst_offset,
                               const mi355_pitched_ptr_t* src, const mi355_dim3_t* src_offset,
                               const mi355_dim3_t* range, uint32_t route, void* stream);

/* How mi355_blit_copy_rect launches a region: pure host arithmetic, for
 * harnesses.  Rows (and layers) that are contiguous on both sides are merged
 * first; a region that merges into one run is a linear copy (linear = 1,
 * width = its bytes).  Otherwise a row is cut into units of 64 * unroll
 * 16-byte vectors anchored at 256-byte boundaries of its destination, the
 * last unit of a row taking up to 15 vectors more; `slots` is the largest unit
 * count of any row and the grid has one wave for each of rows * layers *
 * slots unit slots.  Rows that touch at most 64 16-byte slots of the
 * destination are packed instead: lanes_per_row lanes per row (one per slot),
 * rows * layers * lanes_per_row lanes in all, 64 to a wave; slots and unroll
 * are 0 then. */
typedef struct {
  uint32_t empty;
  uint32_t linear;
  uint64_t dst;   /* first byte of the region on each side */
  uint64_t src;
  uint64_t width; /* bytes per merged row */
  uint64_t dst_pitch, dst_slice, src_pitch, src_slice;
  uint32_t rows, layers;
  uint32_t slots;
  uint32_t unroll;
  uint32_t lanes_per_row;
  uint32_t xcd_run; /* as in mi355_blit_plan_t */
  uint32_t wg_size, grid, nt_load, store_policy;
  uint64_t total_bytes;
  uint32_t plain_rows; /* rows tiled like a linear copy (128-byte aligned on the
                          destination side, whole lines long, a multiple of 4
                          bytes from their source): the kernel's short path */
  uint32_t route;      /* MI355_BLIT_ROUTE_* the launch was shaped for */
} mi355_blit_rect_plan_t;

int mi355_blit_plan_rect(const mi355_pitched_ptr_t* dst, const mi355_dim3_t* dst_offset,
                         const mi355_pitched_ptr_t* src, const mi355_dim3_t* src_offset,
                         const mi355_dim3_t* range, const mi355_blit_tuning_t* tuning,
                         mi355_blit_rect_plan_t* out);
int mi355_blit_plan_rect_route(const mi355_pitched_ptr_t* dst, const mi355_dim3_t* dst_offset,
                               const mi355_pitched_ptr_t* src, const mi355_dim3_t* src_offset,
                               const mi355_dim3_t* range, const mi355_blit_tuning_t* tuning, uint32_t route,
                               mi355_blit_rect_plan_t* out);

/* Decrements an HSA signal by 1 from the GPU once every command submitted
 * before it on the stream has completed, and wakes its waiters: replaces the
 * completion_signal field of the reference's dispatch packet
 * (amd_blit_kernel.cpp:777-779, 884).  hsa_signal_handle is hsa_signal_t.handle
 * of a signal created by hsa_signal_create / hsa_amd_signal_create (its memory
 * is visible to every GPU); it must stay alive until it has been decremented. */
int mi355_blit_signal_complete(mi355_blit_t* h, uint64_t hsa_signal_handle, void* stream);

/* Timestamps for a command on a stream, in the signal's start_ts / end_ts:
 * replaces what the packet processor writes into the completion signal of a
 * dispatch on a queue whose profiling bit BlitKernel::EnableProfiling has set
 * (amd_blit_kernel.cpp:839-842; read by hsa_amd_profiling_get_async_copy_time,
 * hsa_ext_amd.cpp:474-502).  A HIP stream has no such bit, so a one-lane kernel
 * queued in front of the command stamps start_ts and the completion kernel
 * behind it stamps end_ts before it decrements the signal.  The stamps are
 * ticks of the GPU's own clock, as the packet processor's are;
 * hsa_amd_profiling_convert_tick_to_system_domain converts them. */
#define MI355_BLIT_STAMP_START 1u            /* start_ts = now */
#define MI355_BLIT_STAMP_END_AND_COMPLETE 2u /* end_ts = now, then as mi355_blit_signal_complete */
#define MI355_BLIT_STAMP_END 3u              /* end_ts = now; the signal's value is left alone */
int mi355_blit_signal_stamp(mi355_blit_t* h, uint64_t hsa_signal_handle, uint32_t which, void* stream);

/* Runs fn(user) on a host thread once every command submitted before it on the
 * stream has completed: the host-side alternative to
 * mi355_blit_signal_complete, slower by a thread wake-up.  fn must not call
 * back into this library. */
typedef void (*mi355_blit_callback_t)(void* user);
int mi355_blit_add_callback(mi355_blit_t* h, mi355_blit_callback_t fn, void* user, void* stream);

/* Blocks until every command submitted on the handle's own stream is done;
 * the wait BlitKernel does on its completion signal
 * (amd_blit_kernel.cpp:632, 830). */
int mi355_blit_synchronize(mi355_blit_t* h);

/* Replaces BlitKernel::PendingBytes (amd_blit_kernel.cpp:943-970): approximate
 * bytes not yet copied or filled; a return of 0 is exact. */
uint64_t mi355_blit_pending_bytes(mi355_blit_t* h);

/* The plan used by the most recent copy / fill / batch on this handle. */
int mi355_blit_last_launch_info(mi355_blit_t* h, mi355_blit_plan_t* out);

/* Dispatch sizing heuristics as pure host functions (no GPU needed): replace
 * the phase arithmetic of amd_blit_kernel.cpp:714-775 and 796-813.  num_cus is
 * the compute-unit count (amd_blit_kernel.cpp:572); tuning may be NULL. */
int mi355_blit_plan_copy(uint64_t dst, uint64_t src, uint64_t bytes, uint32_t num_cus,
                         const mi355_blit_tuning_t* tuning, mi355_blit_plan_t* out);
int mi355_blit_plan_fill(uint64_t ptr, uint64_t num_dwords, uint32_t num_cus,
                         const mi355_blit_tuning_t* tuning, mi355_blit_plan_t* out);
/* mi355_blit_plan_copy for a route other than within the device. */
int mi355_blit_plan_copy_route(uint64_t dst, uint64_t src, uint64_t bytes, uint32_t num_cus,
                               const mi355_blit_tuning_t* tuning, uint32_t route, mi355_blit_plan_t* out);

/* How a copy of `bytes` is cut into consecutive launches (no counterpart in the
 * reference, whose copy is one dispatch of a fixed grid that strides over any
 * size, amd_blit_kernel.cpp:796-813): returns the number of launches, at most
 * max_pieces, and writes the bytes of each but the last.  1 below 1.5 GiB and
 * for routes over the bus; tuning (may be NULL) can say otherwise. */
uint32_t mi355_blit_plan_copy_pieces(uint64_t bytes, uint32_t route, uint32_t max_pieces,
                                     const mi355_blit_tuning_t* tuning, uint64_t* piece_bytes);

/* Installs overrides used by every later command on the handle (NULL clears).
 * For tuning sweeps; replaces the reference's string-parsed kernel parameters
 * (amd_blit_kernel.cpp:499-532). */
int mi355_blit_set_tuning(mi355_blit_t* h, const mi355_blit_tuning_t* tuning);

/* Compute units of the handle's GPU (amd_blit_kernel.cpp:572). */
int mi355_blit_num_cus(mi355_blit_t* h);

/* The handle's own stream as a hipStream_t. */
void* mi355_blit_stream(mi355_blit_t* h);

const char* mi355_blit_status_string(int status);
int mi355_blit_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MI355_BLIT_H_ */
