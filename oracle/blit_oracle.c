/*
 * TEST INFRASTRUCTURE ONLY -- see blit_oracle.h.  CPU restatement of ROCr's
 * blit-kernel data path.  Paths cited are relative to
 * projects/rocr-runtime/runtime/hsa-runtime/ in the reference tree.
 */
#ifndef _GNU_SOURCE
#define _GNU_SOURCE /* CPU_SET, sched_getaffinity, pthread_setaffinity_np */
#endif
#include "blit_oracle.h"

#include <pthread.h>
#include <sched.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------ */
/* Semantic oracle                                                          */
/* ------------------------------------------------------------------------ */

/* core/runtime/runtime.cpp:507-510: CPU<->CPU hsa_memory_copy is one memcpy. */
void oracle_copy(void* dst, const void* src, size_t size) { memcpy(dst, src, size); }

/* inc/hsa_ext_amd.h:2261-2281: "sets count uint32_t to value". */
void oracle_fill32(void* ptr, uint32_t value, size_t count) {
  uint32_t* p = (uint32_t*)ptr;
  for (size_t i = 0; i < count; ++i) p[i] = value;
}

/* inc/hsa_ext_amd.h:1859-1872 */
void oracle_copy_rect(const oracle_pitched_ptr_t* dst, const oracle_dim3_t* dst_offset,
                      const oracle_pitched_ptr_t* src, const oracle_dim3_t* src_offset,
                      const oracle_dim3_t* range) {
  for (uint32_t z = 0; z < range->z; ++z) {
    for (uint32_t y = 0; y < range->y; ++y) {
      uint8_t* d = (uint8_t*)dst->base + (size_t)(dst_offset->z + z) * dst->slice +
                   (size_t)(dst_offset->y + y) * dst->pitch + dst_offset->x;
      const uint8_t* s = (const uint8_t*)src->base + (size_t)(src_offset->z + z) * src->slice +
                         (size_t)(src_offset->y + y) * src->pitch + src_offset->x;
      memcpy(d, s, range->x);
    }
  }
}

/* core/runtime/hsa_ext_amd.cpp:372-405, core/runtime/amd_blit_sdma.cpp:570-585 */
int oracle_ref_validate_rect(const oracle_pitched_ptr_t* dst, const oracle_dim3_t* dst_offset,
                             const oracle_pitched_ptr_t* src, const oracle_dim3_t* src_offset,
                             const oracle_dim3_t* range, int dir, int* does_work, int* sdma_alignment_ok) {
  enum { kSuccess = 0, kInvalidArgument = 0x1001 };
  if (does_work) *does_work = 0;
  if (sdma_alignment_ok) *sdma_alignment_ok = 1;
  if (!dst || !src || !dst_offset || !src_offset || !range) return kInvalidArgument;
  if (dir == 0) return kInvalidArgument; /* hsaHostToHost */
  if (range->x == 0 || range->y == 0 || range->z == 0) return kSuccess;
  if (sdma_alignment_ok)
    *sdma_alignment_ok = ((uintptr_t)dst->base % 4 == 0 && (uintptr_t)src->base % 4 == 0 && dst->pitch % 4 == 0 &&
                          src->pitch % 4 == 0 && dst->slice % 4 == 0 && src->slice % 4 == 0);
  if ((uint64_t)src_offset->x + range->x > src->pitch || (uint64_t)dst_offset->x + range->x > dst->pitch)
    return kInvalidArgument;
  if (src->slice != 0 && (uint64_t)src_offset->y + range->y > src->slice / src->pitch) return kInvalidArgument;
  if (dst->slice != 0 && (uint64_t)dst_offset->y + range->y > dst->slice / dst->pitch) return kInvalidArgument;
  if (range->z > 1 && (src->slice == 0 || dst->slice == 0)) return kInvalidArgument;
  if (does_work) *does_work = 1;
  return kSuccess;
}

/* core/runtime/runtime.cpp:657-661: memset(ptr, value, count * sizeof(uint32_t)). */
void oracle_ref_host_fill(void* ptr, uint32_t value, size_t count) {
  memset(ptr, (int)value, count * sizeof(uint32_t));
}

typedef struct {
  uint8_t* dst;
  const uint8_t* src;
  size_t size;
  uint32_t value;
  int is_fill;
} mt_slice_t;

static void* mt_worker(void* p) {
  mt_slice_t* s = (mt_slice_t*)p;
  if (s->is_fill)
    oracle_fill32(s->dst, s->value, s->size / 4);
  else
    oracle_copy(s->dst, s->src, s->size);
  return NULL;
}

static void run_mt(uint8_t* dst, const uint8_t* src, size_t size, uint32_t value, int is_fill,
                   int nthreads) {
  if (nthreads < 1) nthreads = 1;
  if (nthreads > 256) nthreads = 256;
  pthread_t tid[256];
  mt_slice_t sl[256];
  /* contiguous slices, each a multiple of 64 bytes except the last */
  size_t per = ((size / (size_t)nthreads) + 63) & ~(size_t)63;
  int started = 0;
  size_t off = 0;
  for (int t = 0; t < nthreads && off < size; ++t) {
    size_t n = (t == nthreads - 1 || off + per > size) ? size - off : per;
    sl[t].dst = dst + off;
    sl[t].src = src ? src + off : NULL;
    sl[t].size = n;
    sl[t].value = value;
    sl[t].is_fill = is_fill;
    off += n;
    if (pthread_create(&tid[t], NULL, mt_worker, &sl[t]) != 0) {
      mt_worker(&sl[t]);
      tid[t] = 0;
    }
    started = t + 1;
  }
  for (int t = 0; t < started; ++t)
    if (tid[t]) pthread_join(tid[t], NULL);
}

void oracle_copy_mt(void* dst, const void* src, size_t size, int nthreads) {
  run_mt((uint8_t*)dst, (const uint8_t*)src, size, 0, 0, nthreads);
}

void oracle_fill32_mt(void* ptr, uint32_t value, size_t count, int nthreads) {
  run_mt((uint8_t*)ptr, NULL, count * 4, value, 1, nthreads);
}

/* ------------------------------------------------------------------------ */
/* The host path on T cores, for the benchmark's CPU baseline: worker threads  */
/* that live as long as the pool, each pinned to one CPU of the process's      */
/* affinity mask and owning one contiguous slice (a multiple of 64 bytes) of   */
/* every buffer, which it also touches first, so that its pages sit on its     */
/* own memory node.                                                            */
/* ------------------------------------------------------------------------ */

enum { POOL_JOB_NONE = 0, POOL_JOB_COPY, POOL_JOB_FILL, POOL_JOB_TOUCH, POOL_JOB_EXIT };

struct oracle_pool {
  int nthreads;
  int pinned; /* threads that could be pinned */
  pthread_t tid[256];
  pthread_mutex_t lock;
  pthread_cond_t go, done;
  unsigned long generation; /* bumped for every job */
  int job;
  int remaining;
  uint8_t* dst;
  const uint8_t* src;
  size_t size;
  uint32_t value;
};

typedef struct {
  struct oracle_pool* pool;
  int index;
} pool_arg_t;

/* Slice `index` of `size` bytes cut for n threads. */
static void pool_slice(size_t size, int n, int index, size_t* off, size_t* len) {
  size_t per = ((size / (size_t)n) + 63) & ~(size_t)63;
  size_t lo = per * (size_t)index;
  if (lo > size) lo = size;
  size_t hi = (index == n - 1) ? size : lo + per;
  if (hi > size) hi = size;
  *off = lo;
  *len = hi - lo;
}

static void* pool_worker(void* p) {
  pool_arg_t* a = (pool_arg_t*)p;
  struct oracle_pool* pool = a->pool;
  const int index = a->index;
  free(a);
  unsigned long seen = 0;
  for (;;) {
    pthread_mutex_lock(&pool->lock);
    while (pool->generation == seen) pthread_cond_wait(&pool->go, &pool->lock);
    seen = pool->generation;
    const int job = pool->job;
    uint8_t* dst = pool->dst;
    const uint8_t* src = pool->src;
    const size_t size = pool->size;
    const uint32_t value = pool->value;
    pthread_mutex_unlock(&pool->lock);
    if (job == POOL_JOB_EXIT) return NULL;
    size_t off, len;
    pool_slice(size, pool->nthreads, index, &off, &len);
    if (len) {
      if (job == POOL_JOB_COPY) oracle_copy(dst + off, src + off, len);
      else if (job == POOL_JOB_FILL) oracle_fill32(dst + off, value, len / 4);
      else if (job == POOL_JOB_TOUCH) memset(dst + off, 0, len);
    }
    pthread_mutex_lock(&pool->lock);
    if (--pool->remaining == 0) pthread_cond_signal(&pool->done);
    pthread_mutex_unlock(&pool->lock);
  }
}

static void pool_run(struct oracle_pool* pool, int job, void* dst, const void* src, size_t size, uint32_t value) {
  pthread_mutex_lock(&pool->lock);
  pool->job = job;
  pool->dst = (uint8_t*)dst;
  pool->src = (const uint8_t*)src;
  pool->size = size;
  pool->value = value;
  pool->remaining = pool->nthreads;
  ++pool->generation;
  pthread_cond_broadcast(&pool->go);
  while (pool->remaining) pthread_cond_wait(&pool->done, &pool->lock);
  pthread_mutex_unlock(&pool->lock);
}

oracle_pool_t* oracle_pool_create(int nthreads) {
  if (nthreads < 1) nthreads = 1;
  if (nthreads > 256) nthreads = 256;
  struct oracle_pool* pool = (struct oracle_pool*)calloc(1, sizeof(*pool));
  if (!pool) return NULL;
  pool->nthreads = nthreads;
  pthread_mutex_init(&pool->lock, NULL);
  pthread_cond_init(&pool->go, NULL);
  pthread_cond_init(&pool->done, NULL);
  cpu_set_t allowed;
  CPU_ZERO(&allowed);
  const int have_mask = sched_getaffinity(0, sizeof(allowed), &allowed) == 0;
  int next_cpu = 0;
  for (int t = 0; t < nthreads; ++t) {
    pool_arg_t* a = (pool_arg_t*)malloc(sizeof(*a));
    if (!a || (a->pool = pool, a->index = t, pthread_create(&pool->tid[t], NULL, pool_worker, a) != 0)) {
      free(a);
      pool->nthreads = t;
      break;
    }
    if (have_mask) {
      /* the t-th allowed CPU, wrapping when there are more threads than CPUs */
      int cpu = -1;
      for (int tries = 0; tries < 2 * CPU_SETSIZE; ++tries) {
        const int c = next_cpu++ % CPU_SETSIZE;
        if (CPU_ISSET(c, &allowed)) {
          cpu = c;
          break;
        }
      }
      if (cpu >= 0) {
        cpu_set_t one;
        CPU_ZERO(&one);
        CPU_SET(cpu, &one);
        if (pthread_setaffinity_np(pool->tid[t], sizeof(one), &one) == 0) ++pool->pinned;
      }
    }
  }
  if (pool->nthreads == 0) {
    free(pool);
    return NULL;
  }
  return pool;
}

void oracle_pool_destroy(oracle_pool_t* pool) {
  if (!pool) return;
  pthread_mutex_lock(&pool->lock);
  pool->job = POOL_JOB_EXIT;
  ++pool->generation;
  pthread_cond_broadcast(&pool->go);
  pthread_mutex_unlock(&pool->lock);
  for (int t = 0; t < pool->nthreads; ++t) pthread_join(pool->tid[t], NULL);
  pthread_mutex_destroy(&pool->lock);
  pthread_cond_destroy(&pool->go);
  pthread_cond_destroy(&pool->done);
  free(pool);
}

int oracle_pool_threads(const oracle_pool_t* pool) { return pool ? pool->nthreads : 0; }
int oracle_pool_pinned(const oracle_pool_t* pool) { return pool ? pool->pinned : 0; }

void oracle_pool_first_touch(oracle_pool_t* pool, void* buf, size_t size) {
  pool_run(pool, POOL_JOB_TOUCH, buf, NULL, size, 0);
}

void oracle_pool_copy(oracle_pool_t* pool, void* dst, const void* src, size_t size) {
  pool_run(pool, POOL_JOB_COPY, dst, src, size, 0);
}

void oracle_pool_fill32(oracle_pool_t* pool, void* ptr, uint32_t value, size_t count) {
  pool_run(pool, POOL_JOB_FILL, ptr, NULL, count * 4, value);
}

/* ------------------------------------------------------------------------ */
/* API-edge validation                                                      */
/* ------------------------------------------------------------------------ */

/* core/runtime/hsa.cpp:1170-1184 */
int oracle_ref_validate_copy(uint64_t dst, uint64_t src, uint64_t size, int* does_work) {
  *does_work = 0;
  if (dst == 0 || src == 0) return ORACLE_STATUS_INVALID_ARGUMENT;
  if (size == 0) return ORACLE_STATUS_SUCCESS;
  *does_work = 1;
  return ORACLE_STATUS_SUCCESS;
}

/* core/runtime/hsa_ext_amd.cpp:237-251 */
int oracle_ref_validate_fill(uint64_t ptr, uint64_t count, int* does_work) {
  *does_work = 0;
  if (ptr == 0 || (ptr % 4) != 0) return ORACLE_STATUS_INVALID_ARGUMENT;
  if (count == 0) return ORACLE_STATUS_SUCCESS;
  *does_work = 1;
  return ORACLE_STATUS_SUCCESS;
}

/* core/runtime/amd_blit_kernel.cpp:791-794 */
int oracle_ref_blit_fill_status(uint64_t ptr) {
  return (ptr & 0x3) ? ORACLE_STATUS_ERROR : ORACLE_STATUS_SUCCESS;
}

/* ------------------------------------------------------------------------ */
/* Host-side phase split                                                    */
/* ------------------------------------------------------------------------ */

/* Tunables string-parsed from the shader source at run time,
 * amd_blit_kernel.cpp:84-85, 291, 397-398. */
enum {
  kCopyAlignedVecWidth = 4,
  kCopyAlignedUnroll = 1,
  kCopyMisalignedUnroll = 4,
  kFillVecWidth = 4,
  kFillUnroll = 1
};

static uint64_t min_u64(uint64_t a, uint64_t b) { return a < b ? a : b; }

/* core/runtime/amd_blit_kernel.cpp:714-775 */
int oracle_ref_plan_copy(uint64_t dst, uint64_t src, uint64_t size, int num_cus,
                         oracle_kernargs_t* args) {
  memset(args, 0, sizeof(*args));
  const int aligned = ((src & 0x3) == (dst & 0x3)); /* :716 */
  const uint32_t num_workitems = 64u * 4u * (uint32_t)num_cus; /* :723, :759 */
  if (aligned) {
    /* phase 1: bytes until dst is 0x100-aligned (:728-729) */
    uint64_t p1 = min_u64(size, (uint64_t)(0x100 - (dst & 0xFF)) & 0xFF);
    /* phase 2: whole blocks of W * 4 B * unroll * vec (:732-734) */
    uint64_t blk = (uint64_t)num_workitems * 4u * kCopyAlignedUnroll * kCopyAlignedVecWidth;
    uint64_t p2 = ((size - p1) / blk) * blk;
    /* phase 3: whole dwords (:737-739) */
    uint64_t p3 = ((size - p1 - p2) / 4u) * 4u;
    args->copy_aligned.phase1_src_start = src;
    args->copy_aligned.phase1_dst_start = dst;
    args->copy_aligned.phase2_src_start = src + p1;
    args->copy_aligned.phase2_dst_start = dst + p1;
    args->copy_aligned.phase3_src_start = src + p1 + p2;
    args->copy_aligned.phase3_dst_start = dst + p1 + p2;
    args->copy_aligned.phase4_src_start = src + p1 + p2 + p3;
    args->copy_aligned.phase4_dst_start = dst + p1 + p2 + p3;
    args->copy_aligned.phase4_src_end = src + size;
    args->copy_aligned.phase4_dst_end = dst + size;
    args->copy_aligned.num_workitems = num_workitems;
    return ORACLE_KERNEL_COPY_ALIGNED;
  }
  /* :754-775 */
  uint64_t blk = (uint64_t)num_workitems * 1u * kCopyMisalignedUnroll;
  uint64_t p1 = (size / blk) * blk;
  args->copy_misaligned.phase1_src_start = src;
  args->copy_misaligned.phase1_dst_start = dst;
  args->copy_misaligned.phase2_src_start = src + p1;
  args->copy_misaligned.phase2_dst_start = dst + p1;
  args->copy_misaligned.phase2_src_end = src + size;
  args->copy_misaligned.phase2_dst_end = dst + size;
  args->copy_misaligned.num_workitems = num_workitems;
  return ORACLE_KERNEL_COPY_MISALIGNED;
}

/* core/runtime/amd_blit_kernel.cpp:796-813 */
void oracle_ref_plan_fill(uint64_t ptr, uint32_t value, uint64_t count, int num_cus,
                          oracle_kernargs_t* args) {
  memset(args, 0, sizeof(*args));
  const uint32_t num_workitems = 64u * (uint32_t)num_cus; /* :797 */
  uint64_t fill_size = count * 4u;
  uint64_t blk = (uint64_t)num_workitems * 4u * kFillUnroll * kFillVecWidth; /* :803-805 */
  uint64_t p1 = (fill_size / blk) * blk;
  args->fill.phase1_dst_start = ptr;
  args->fill.phase2_dst_start = ptr + p1;
  args->fill.phase2_dst_end = ptr + fill_size;
  args->fill.fill_value = value;
  args->fill.num_workitems = num_workitems;
}

/* core/runtime/amd_blit_kernel.cpp:880: AlignUp(grid_size_x, 64) */
uint32_t oracle_ref_grid_size(uint32_t num_workitems) { return (num_workitems + 63u) & ~63u; }

/* ------------------------------------------------------------------------ */
/* Device shaders, emulated one work-item at a time                          */
/* ------------------------------------------------------------------------ */
/* Work-item id t = workgroup_id * 64 + lane runs over the packet's grid.  All
 * loops below are written per work-item: the shaders' EXEC masking only
 * retires lanes whose own address ran past the phase end, and a wave leaves a
 * loop when no lane is left, which is the same as each work-item running its
 * own "while (addr < end)" loop. */

static int ld_ok(const oracle_bounds_t* b, uint64_t a, uint64_t n) {
  return !b || (a >= b->src_lo && a + n <= b->src_hi);
}
static int st_ok(const oracle_bounds_t* b, uint64_t a, uint64_t n) {
  return !b || (a >= b->dst_lo && a + n <= b->dst_hi);
}

/* core/runtime/blit_shaders/blit_copyAligned.s:76-259 */
int oracle_ref_exec_copy_aligned(const oracle_kernargs_t* ka, const oracle_bounds_t* b) {
  const uint64_t W = ka->copy_aligned.num_workitems;
  const uint32_t grid = oracle_ref_grid_size((uint32_t)W);
  int rc = 0;
  for (uint64_t t = 0; t < grid; ++t) {
    /* phase 1, :108-128: byte at src+t, stride W bytes, until phase2_src_start */
    uint64_t s = ka->copy_aligned.phase1_src_start + t;
    uint64_t d = ka->copy_aligned.phase1_dst_start + t;
    while (s < ka->copy_aligned.phase2_src_start) {
      if (ld_ok(b, s, 1) && st_ok(b, d, 1)) *(uint8_t*)(uintptr_t)d = *(const uint8_t*)(uintptr_t)s; else rc = -1;
      s += W; d += W;
    }
    /* phase 2, :132-203: dwordx4 at +16t, stride 16W, until phase3_src_start.
     * No EXEC masking here: the host guarantees whole blocks. */
    s = ka->copy_aligned.phase2_src_start + 16u * t;
    d = ka->copy_aligned.phase2_dst_start + 16u * t;
    while (s < ka->copy_aligned.phase3_src_start) {
      for (int u = 0; u < kCopyAlignedUnroll; ++u) {
        if (ld_ok(b, s, 16) && st_ok(b, d, 16)) memcpy((void*)(uintptr_t)d, (const void*)(uintptr_t)s, 16); else rc = -1;
        s += 16u * W; d += 16u * W;
      }
    }
    /* phase 3, :205-232: dword at +4t, stride 4W, until phase4_src_start */
    s = ka->copy_aligned.phase3_src_start + 4u * t;
    d = ka->copy_aligned.phase3_dst_start + 4u * t;
    while (s < ka->copy_aligned.phase4_src_start) {
      if (ld_ok(b, s, 4) && st_ok(b, d, 4)) memcpy((void*)(uintptr_t)d, (const void*)(uintptr_t)s, 4); else rc = -1;
      s += 4u * W; d += 4u * W;
    }
    /* phase 4, :236-256: one byte at +t if below phase4_src_end */
    s = ka->copy_aligned.phase4_src_start + t;
    d = ka->copy_aligned.phase4_dst_start + t;
    if (s < ka->copy_aligned.phase4_src_end) {
      if (ld_ok(b, s, 1) && st_ok(b, d, 1)) *(uint8_t*)(uintptr_t)d = *(const uint8_t*)(uintptr_t)s; else rc = -1;
    }
  }
  return rc;
}

/* core/runtime/blit_shaders/blit_copyMisaligned.s:90-182 */
int oracle_ref_exec_copy_misaligned(const oracle_kernargs_t* ka, const oracle_bounds_t* b) {
  const uint64_t W = ka->copy_misaligned.num_workitems;
  const uint32_t grid = oracle_ref_grid_size((uint32_t)W);
  int rc = 0;
  for (uint64_t t = 0; t < grid; ++t) {
    /* phase 1, :119-151: 4 byte loads at stride W, then 4 byte stores;
     * unmasked, the host guarantees whole blocks */
    uint64_t s = ka->copy_misaligned.phase1_src_start + t;
    uint64_t d = ka->copy_misaligned.phase1_dst_start + t;
    while (s < ka->copy_misaligned.phase2_src_start) {
      uint8_t v[kCopyMisalignedUnroll];
      int ok = 1;
      for (int u = 0; u < kCopyMisalignedUnroll; ++u) {
        if (ld_ok(b, s, 1)) v[u] = *(const uint8_t*)(uintptr_t)s; else { ok = 0; v[u] = 0; }
        s += W;
      }
      for (int u = 0; u < kCopyMisalignedUnroll; ++u) {
        if (ok && st_ok(b, d, 1)) *(uint8_t*)(uintptr_t)d = v[u]; else rc = -1;
        d += W;
      }
    }
    /* phase 2, :153-179: masked single bytes, stride W */
    s = ka->copy_misaligned.phase2_src_start + t;
    d = ka->copy_misaligned.phase2_dst_start + t;
    while (s < ka->copy_misaligned.phase2_src_end) {
      if (ld_ok(b, s, 1) && st_ok(b, d, 1)) *(uint8_t*)(uintptr_t)d = *(const uint8_t*)(uintptr_t)s; else rc = -1;
      s += W; d += W;
    }
  }
  return rc;
}

/* core/runtime/blit_shaders/blit_fill.s:91-185 */
int oracle_ref_exec_fill(const oracle_kernargs_t* ka, const oracle_bounds_t* b) {
  const uint64_t W = ka->fill.num_workitems;
  const uint32_t grid = oracle_ref_grid_size((uint32_t)W);
  const uint32_t v4[4] = {ka->fill.fill_value, ka->fill.fill_value, ka->fill.fill_value,
                          ka->fill.fill_value};
  int rc = 0;
  for (uint64_t t = 0; t < grid; ++t) {
    /* phase 1, :138-160: dwordx4 at +16t, stride 16W, until phase2_dst_start */
    uint64_t d = ka->fill.phase1_dst_start + 16u * t;
    while (d < ka->fill.phase2_dst_start) {
      for (int u = 0; u < kFillUnroll; ++u) {
        if (st_ok(b, d, 16)) memcpy((void*)(uintptr_t)d, v4, 16); else rc = -1;
        d += 16u * W;
      }
    }
    /* phase 2, :164-182: dword at +4t, stride 4W, masked, until phase2_dst_end */
    d = ka->fill.phase2_dst_start + 4u * t;
    while (d < ka->fill.phase2_dst_end) {
      if (st_ok(b, d, 4)) memcpy((void*)(uintptr_t)d, v4, 4); else rc = -1;
      d += 4u * W;
    }
  }
  return rc;
}

int oracle_ref_blit_copy(void* dst, const void* src, size_t size, int num_cus,
                         const oracle_bounds_t* b) {
  oracle_kernargs_t ka;
  int k = oracle_ref_plan_copy((uint64_t)(uintptr_t)dst, (uint64_t)(uintptr_t)src, size, num_cus, &ka);
  int rc = (k == ORACLE_KERNEL_COPY_ALIGNED) ? oracle_ref_exec_copy_aligned(&ka, b)
                                             : oracle_ref_exec_copy_misaligned(&ka, b);
  return rc < 0 ? rc : k;
}

int oracle_ref_blit_fill(void* ptr, uint32_t value, size_t count, int num_cus,
                         const oracle_bounds_t* b) {
  if (oracle_ref_blit_fill_status((uint64_t)(uintptr_t)ptr) != ORACLE_STATUS_SUCCESS) return -1;
  oracle_kernargs_t ka;
  oracle_ref_plan_fill((uint64_t)(uintptr_t)ptr, value, count, num_cus, &ka);
  int rc = oracle_ref_exec_fill(&ka, b);
  return rc < 0 ? rc : ORACLE_KERNEL_FILL;
}

/* core/runtime/amd_gpu_agent.cpp:2388-2398 */
int oracle_ref_same_gpu_uses_blit_kernel(uint64_t size, uint64_t force_sdma_size) {
  return size < force_sdma_size ? 0 : 1;
}

/* ------------------------------------------------------------------------ */
/* Seeded inputs                                                            */
/* ------------------------------------------------------------------------ */

static uint64_t splitmix64(uint64_t* x) {
  uint64_t z = (*x += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
static uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

void oracle_fill_random(void* buf, size_t size, uint64_t seed) {
  uint64_t sm = seed;
  uint64_t s[4];
  for (int i = 0; i < 4; ++i) s[i] = splitmix64(&sm);
  uint8_t* p = (uint8_t*)buf;
  size_t i = 0;
  while (i < size) {
    uint64_t r = rotl64(s[1] * 5, 7) * 9; /* xoshiro256** */
    uint64_t t = s[1] << 17;
    s[2] ^= s[0]; s[3] ^= s[1]; s[1] ^= s[2]; s[0] ^= s[3];
    s[2] ^= t; s[3] = rotl64(s[3], 45);
    for (int k = 0; k < 8 && i < size; ++k, ++i) p[i] = (uint8_t)(r >> (8 * k));
  }
}

uint64_t oracle_fnv1a64(const void* buf, size_t size) {
  const uint8_t* p = (const uint8_t*)buf;
  uint64_t h = 0xcbf29ce484222325ull;
  for (size_t i = 0; i < size; ++i) { h ^= p[i]; h *= 0x100000001b3ull; }
  return h;
}
