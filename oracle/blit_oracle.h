/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of ROCr's blit-kernel data path
 * (linear copy, aligned and misaligned, and dword fill).  Nothing in the
 * product library links, loads or calls this file; it is the checker that the
 * parity tests, the smoke test and the CPU-baseline leg of the benchmark use.
 *
 * Paths are relative to projects/rocr-runtime/runtime/hsa-runtime/ in the
 * reference tree.
 *
 * How each function is pinned (see tests/test_oracle.py):
 *   oracle_copy           libc memcpy, which is literally the reference's
 *                         host path (core/runtime/runtime.cpp:507-510).
 *   oracle_fill32         the API contract "set count uint32_t to value"
 *                         (inc/hsa_ext_amd.h:2261-2281) and the fill-then-
 *                         verify-every-dword known-answer tests of
 *                         rocrtst/samples/async_mem_copy/async_mem_copy.cc:62-65,
 *                         348-354 (patterns 0xabcdef12 0xba5eba11 0xfeed5a1e,
 *                         init 0xbaadf00d).
 *   oracle_ref_plan_*     closed-form invariants of the phase split
 *                         (phases tile [0,size) exactly, p1 < 256, p2 a
 *                         multiple of its block, p3 a multiple of 4, p4 < 4)
 *                         brute-forced over all residues.
 *   oracle_ref_exec_*     lane-by-lane emulation of the three shaders; pinned
 *                         by requiring its output to equal oracle_copy /
 *                         oracle_fill32 with guard bytes untouched, for every
 *                         (src & 255, dst & 255) residue class that selects
 *                         each kernel.  Misaligned offsets and odd lengths are
 *                         not covered by any test the reference holds, so for
 *                         those the memcpy closed form is the only pin.
 *   oracle_copy_rect      row-by-row memcpy of a pitched 3-D region, the
 *                         meaning inc/hsa_ext_amd.h:1859-1872 gives the SDMA
 *                         rect copy ("offsets and range carry x in bytes, y
 *                         and z in rows and layers").  The reference holds no
 *                         golden vector for it; pinned against numpy slice
 *                         assignment on 3-D byte arrays and against guard
 *                         bytes around the region.
 *   oracle_ref_validate_rect  the argument checks of
 *                         hsa_amd_memory_async_copy_rect and
 *                         BlitSdma::SubmitCopyRectCommand, case by case.
 *   oracle_ref_host_fill  restates the reference's host fallback
 *                         memset(ptr, value, count*4) (runtime.cpp:657-661),
 *                         which keeps only the low byte of the pattern.  It is
 *                         documented as a reference quirk, NOT used as the
 *                         expected result of any parity test.
 */
#ifndef BLIT_ORACLE_H_
#define BLIT_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Kernel the reference would pick for a copy (core/runtime/amd_blit_kernel.cpp:716). */
enum { ORACLE_KERNEL_COPY_ALIGNED = 0, ORACLE_KERNEL_COPY_MISALIGNED = 1, ORACLE_KERNEL_FILL = 2 };

/* Byte-for-byte image of BlitKernel::KernelArgs (core/inc/amd_blit_kernel.h:122-154).
 * One slot is AlignUp(sizeof, 16) = 96 bytes. */
typedef union {
  struct {
    uint64_t phase1_src_start, phase1_dst_start;
    uint64_t phase2_src_start, phase2_dst_start;
    uint64_t phase3_src_start, phase3_dst_start;
    uint64_t phase4_src_start, phase4_dst_start;
    uint64_t phase4_src_end, phase4_dst_end;
    uint32_t num_workitems;
  } copy_aligned;
  struct {
    uint64_t phase1_src_start, phase1_dst_start;
    uint64_t phase2_src_start, phase2_dst_start;
    uint64_t phase2_src_end, phase2_dst_end;
    uint32_t num_workitems;
  } copy_misaligned;
  struct {
    uint64_t phase1_dst_start, phase2_dst_start, phase2_dst_end;
    uint32_t fill_value;
    uint32_t num_workitems;
  } fill;
  uint8_t raw[96];
} oracle_kernargs_t;

/* --- the semantic oracle: what every path must produce ------------------- */

/* Host copy, core/runtime/runtime.cpp:507-510. */
void oracle_copy(void* dst, const void* src, size_t size);

/* count dwords set to value, inc/hsa_ext_amd.h:2261-2281. */
void oracle_fill32(void* ptr, uint32_t value, size_t count);

/* hsa_pitched_ptr_t / hsa_dim3_t (inc/hsa_ext_amd.h:1842-1846). */
typedef struct {
  void* base;
  size_t pitch;
  size_t slice;
} oracle_pitched_ptr_t;
typedef struct {
  uint32_t x, y, z;
} oracle_dim3_t;

/* Pitched 3-D region copy: range.z layers of range.y rows of range.x bytes
 * (inc/hsa_ext_amd.h:1859-1872). */
void oracle_copy_rect(const oracle_pitched_ptr_t* dst, const oracle_dim3_t* dst_offset,
                      const oracle_pitched_ptr_t* src, const oracle_dim3_t* src_offset,
                      const oracle_dim3_t* range);

/* Status of hsa_amd_memory_async_copy_rect's and SubmitCopyRectCommand's
 * argument checks (core/runtime/hsa_ext_amd.cpp:372-405,
 * core/runtime/amd_blit_sdma.cpp:577-585; the SDMA packet's dword-alignment
 * checks, :570-575, are reported separately in *sdma_alignment_ok).
 * Returns hsa_status_t values; *does_work is 0 when the call returns SUCCESS
 * without submitting anything. */
int oracle_ref_validate_rect(const oracle_pitched_ptr_t* dst, const oracle_dim3_t* dst_offset,
                             const oracle_pitched_ptr_t* src, const oracle_dim3_t* src_offset,
                             const oracle_dim3_t* range, int dir, int* does_work, int* sdma_alignment_ok);

/* The reference's host fill fallback, runtime.cpp:657-661 (low byte only). */
void oracle_ref_host_fill(void* ptr, uint32_t value, size_t count);

/* Multi-threaded versions of the two above for the CPU baseline: the buffer is
 * cut into nthreads contiguous 64-byte-aligned slices. */
void oracle_copy_mt(void* dst, const void* src, size_t size, int nthreads);
void oracle_fill32_mt(void* ptr, uint32_t value, size_t count, int nthreads);

/* The same host path on a pool of worker threads that outlive the call, for
 * the benchmark's CPU baseline: `nthreads` threads, each pinned to one CPU of
 * the process's affinity mask (where the system allows it) and owning one
 * contiguous slice, a multiple of 64 bytes, of every buffer.
 * oracle_pool_first_touch makes every thread write zeros over its own slice,
 * so that a freshly allocated buffer's pages are placed by their owner;
 * oracle_pool_copy and oracle_pool_fill32 are memcpy / the dword loop on the
 * same slices.  Pinned by: output equal to oracle_copy / oracle_fill32 for
 * thread counts 1..33 and sizes that do not divide evenly (tests/test_oracle.py). */
typedef struct oracle_pool oracle_pool_t;
oracle_pool_t* oracle_pool_create(int nthreads);
void oracle_pool_destroy(oracle_pool_t* pool);
int oracle_pool_threads(const oracle_pool_t* pool);
int oracle_pool_pinned(const oracle_pool_t* pool); /* threads that could be pinned */
void oracle_pool_first_touch(oracle_pool_t* pool, void* buf, size_t size);
void oracle_pool_copy(oracle_pool_t* pool, void* dst, const void* src, size_t size);
void oracle_pool_fill32(oracle_pool_t* pool, void* ptr, uint32_t value, size_t count);

/* --- argument validation at the API edge -------------------------------- */
/* Status codes follow inc/hsa.h: SUCCESS 0, ERROR 0x1000, INVALID_ARGUMENT 0x1001. */
enum { ORACLE_STATUS_SUCCESS = 0, ORACLE_STATUS_ERROR = 0x1000, ORACLE_STATUS_INVALID_ARGUMENT = 0x1001 };

/* hsa_memory_copy, core/runtime/hsa.cpp:1170-1184.  *does_work = 0 when the
 * call returns before reaching the copy engine. */
int oracle_ref_validate_copy(uint64_t dst, uint64_t src, uint64_t size, int* does_work);
/* hsa_amd_memory_fill, core/runtime/hsa_ext_amd.cpp:237-251. */
int oracle_ref_validate_fill(uint64_t ptr, uint64_t count, int* does_work);
/* BlitKernel::SubmitLinearFillCommand's own check, amd_blit_kernel.cpp:791-794. */
int oracle_ref_blit_fill_status(uint64_t ptr);

/* --- the reference's host-side phase split ------------------------------ */

/* amd_blit_kernel.cpp:714-775.  Returns the kernel chosen; fills *args. */
int oracle_ref_plan_copy(uint64_t dst, uint64_t src, uint64_t size, int num_cus,
                         oracle_kernargs_t* args);
/* amd_blit_kernel.cpp:796-813. */
void oracle_ref_plan_fill(uint64_t ptr, uint32_t value, uint64_t count, int num_cus,
                          oracle_kernargs_t* args);
/* Grid of the dispatch packet, amd_blit_kernel.cpp:880-885: AlignUp(num_workitems, 64). */
uint32_t oracle_ref_grid_size(uint32_t num_workitems);

/* --- the reference's device shaders, one work-item at a time ------------- */
/* Addresses in args are host addresses here.  base/limit bound every access:
 * a store outside [dst_lo, dst_hi) or a load outside [src_lo, src_hi) makes the
 * function return -1 (nothing is written for that access). */
typedef struct {
  uint64_t dst_lo, dst_hi;
  uint64_t src_lo, src_hi;
} oracle_bounds_t;

/* core/runtime/blit_shaders/blit_copyAligned.s:76-259 */
int oracle_ref_exec_copy_aligned(const oracle_kernargs_t* args, const oracle_bounds_t* b);
/* core/runtime/blit_shaders/blit_copyMisaligned.s:90-182 */
int oracle_ref_exec_copy_misaligned(const oracle_kernargs_t* args, const oracle_bounds_t* b);
/* core/runtime/blit_shaders/blit_fill.s:91-185 */
int oracle_ref_exec_fill(const oracle_kernargs_t* args, const oracle_bounds_t* b);

/* plan + exec, i.e. what BlitKernel::SubmitLinearCopyCommand /
 * SubmitLinearFillCommand leave in memory.  Return the kernel used, or -1. */
int oracle_ref_blit_copy(void* dst, const void* src, size_t size, int num_cus,
                         const oracle_bounds_t* b);
int oracle_ref_blit_fill(void* ptr, uint32_t value, size_t count, int num_cus,
                         const oracle_bounds_t* b);

/* --- caller policy ------------------------------------------------------- */
/* GpuAgent::GetBlitObject for a same-GPU async copy, amd_gpu_agent.cpp:2379-2398:
 * returns 1 when the shader blit (BlitDevToDev) serves the copy, 0 when the
 * SDMA-capable engine does.  force_sdma_size is HSA_FORCE_SDMA_SIZE
 * (core/util/flag.h:206-207, default 1 MiB). */
int oracle_ref_same_gpu_uses_blit_kernel(uint64_t size, uint64_t force_sdma_size);

/* --- seeded inputs shared by tests and benchmark ------------------------- */
/* splitmix64-seeded xoshiro256**; bytes are the little-endian bytes of
 * successive 64-bit outputs. */
void oracle_fill_random(void* buf, size_t size, uint64_t seed);
/* FNV-1a 64 of a buffer: used to pin generator streams in golden fixtures. */
uint64_t oracle_fnv1a64(const void* buf, size_t size);

#ifdef __cplusplus
}
#endif
#endif /* BLIT_ORACLE_H_ */
