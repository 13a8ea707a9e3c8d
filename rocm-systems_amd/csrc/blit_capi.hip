// C ABI of the gfx950 blit engine over HIP (declarations and the reference
// interfaces they replace: include/mi355_blit.h).  Host work per command is
// O(1): one plan, one kernel launch, one ledger addition -- like the ~100 bytes
// of kernargs plus one AQL packet ROCr's BlitKernel writes per command
// (projects/rocr-runtime/runtime/hsa-runtime/core/runtime/amd_blit_kernel.cpp:
// 641-785).
#include <hip/hip_runtime.h>

#include <xmmintrin.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "blit_kernels.h"
#include "blit_batch_host.h"
#include "blit_plan.h"
#include "blit_rect.h"
#include "mi355_blit.h"

namespace {

using namespace mi355;

// Markers remembered for PendingBytes.  Recording an event after every command
// costs ~4 us of queue time per command on MI355X, so a marker is only
// recorded when somebody asks (or when a command goes to another stream than
// the one before): it then stands for all bytes submitted since the previous
// marker.  ROCr's ledger has one record per AQL queue slot and its utility
// queue has 64 (amd_gpu_agent.h:507-508).
constexpr unsigned kLedgerSlots = 64;

struct LedgerSlot {
  hipEvent_t done = nullptr;
  uint64_t bytes = 0;  // submitted between the previous marker and this one
  bool in_flight = false;
};

// What the allocation-free batched copy (mi355_blit_copy_batch_bounded_noalloc)
// may hold: descriptors per call, and chunk records before chunks are looked up
// in the prefix sums instead.
constexpr uint64_t kNoAllocMaxCopies = MI355_BLIT_NOALLOC_MAX_COPIES;
constexpr uint64_t kNoAllocRecords = 1ull << 19;
// Layout of its scratch memory: the prefix sum within groups of 1024 copies
// (one word per copy and one for the total), the prefix sum across groups, the
// chunk records; each part at a multiple of 256 bytes.
constexpr size_t kScratchChunkStart = 0;
constexpr size_t kScratchBlockSum = (kScratchChunkStart + (kNoAllocMaxCopies + 1) * sizeof(uint32_t) + 255) / 256 * 256;
constexpr size_t kScratchRecords = (kScratchBlockSum + (kNoAllocMaxCopies / 1024 + 1) * sizeof(uint32_t) + 255) / 256 * 256;
constexpr size_t kScratchBytes = kScratchRecords + kNoAllocRecords * sizeof(ChunkRecord);
static_assert(kScratchBytes <= (17u << 20), "the scratch array is meant to stay modest");

}  // namespace

// Scratch memory of the allocation-free batched copy: 16.25 MiB that every GPU
// this library runs on holds from the load of the library's code object to the
// end of the process.  In host code this name is only a stand-in for the
// symbol, not a device address: host code reaches the memory through the
// per-device pointer scratch_for_device() keeps (hipGetSymbolAddress), and the
// kernels take that pointer as an argument.
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {

// Each GPU holds its own copy of `scratch` at its own address.  Looked up once
// per device, with that device current, and kept.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
void* g_scratch_ptr[kMaxDevices];
bool g_scratch_known[kMaxDevices];
hipError_t g_scratch_err[kMaxDevices];

// The calling thread's current device must be `device`.
hipError_t scratch_for_device(int device, void** out) {
  *out = nullptr;
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> g(g_scratch_lock);
  if (!g_scratch_known[device]) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    g_scratch_err[device] = e;
    g_scratch_ptr[device] = e == hipSuccess ? p : nullptr;
    g_scratch_known[device] = true;
  }
  *out = g_scratch_ptr[device];
  return g_scratch_err[device];
}

}  // namespace

struct mi355_blit {
  int device = 0;
  int num_cus = 0;
  hipStream_t stream = nullptr;
  // This GPU's copy of `scratch` (a device address), or null with the error
  // that the lookup gave.
  unsigned char* scratch_dev = nullptr;
  hipError_t scratch_err = hipSuccess;

  std::mutex lock;  // guards everything below
  mi355_blit_tuning_t tuning{};
  bool has_tuning = false;
  mi355_blit_plan_t last_plan{};

  LedgerSlot ledger[kLedgerSlots];
  uint64_t ledger_head = 0;      // next slot to use
  uint64_t unmarked_bytes = 0;   // submitted after the newest marker
  bool unmarked = false;         // commands were submitted after the newest marker
  hipStream_t last_stream = nullptr;

  // batched path staging (grown on demand, never shrunk)
  // Two staging buffers for host-resident descriptors, used alternately.  On a
  // device whose memory the host can write (large BAR) they are device memory:
  // the host's copy lands in HBM while the batch before still runs (measured:
  // 1.5 MiB in 35 us of host time) and the first kernel reads it at HBM speed
  // instead of fetching it across the bus (32 us at the head of every batch).
  // Pinned host memory otherwise.
  bool stage_in_device_memory = false;
  BatchDesc* descs_host[2] = {nullptr, nullptr};
  BatchImage stage_image;  // built in ordinary memory, then copied to a staging buffer
  // One event per batch, recorded behind its copy kernel, alternating like the
  // staging buffers: it frees the batch's staging buffer for the host, and it
  // is what a batch on another stream, or a reallocation, waits for.  (An
  // event between the two kernels of a batch costs ~5 us of queue time.)
  hipEvent_t batch_done[2] = {nullptr, nullptr};
  bool batch_busy[2] = {false, false};
  unsigned next_host = 0;
  hipStream_t last_batch_stream = nullptr;
  uint32_t* chunk_start_dev = nullptr;
  uint32_t* block_sum_dev = nullptr;
  BatchDesc* descs_private_dev = nullptr;  // the GPU's own copy of descriptors the host staged as they were
  ChunkRecord* records_dev = nullptr;  // one per chunk
  // Pinned host memory where the copy kernel of a device-resident batch leaves
  // its numbers of copies and chunks (batch_device_sizing); made with the
  // first such batch.
  uint64_t* batch_seen = nullptr;
  size_t records_capacity = 0;
  size_t batch_capacity = 0;
};

namespace {

int status_of(hipError_t e) {
  switch (e) {
    case hipSuccess: return MI355_BLIT_SUCCESS;
    case hipErrorOutOfMemory: return MI355_BLIT_ERROR_OUT_OF_RESOURCES;
    case hipErrorInvalidValue: return MI355_BLIT_ERROR_INVALID_ARGUMENT;
    default: return MI355_BLIT_ERROR;
  }
}

#define BLIT_HIP(expr)                       \
  do {                                       \
    hipError_t e_ = (expr);                  \
    if (e_ != hipSuccess) return status_of(e_); \
  } while (0)

struct DeviceScope {
  int prev = -1;
  bool switched = false;
  hipError_t err = hipSuccess;
  explicit DeviceScope(int dev) {
    err = hipGetDevice(&prev);
    if (err == hipSuccess && prev != dev) {
      err = hipSetDevice(dev);
      switched = (err == hipSuccess);
    }
  }
  ~DeviceScope() {
    if (switched) (void)hipSetDevice(prev);
  }
};

typedef void (*copy_kernel_t)(CopyArgs);
typedef void (*fill_kernel_t)(FillArgs);
typedef void (*batch_kernel_t)(BatchCopyArgs);
typedef void (*batch_lookup_kernel_t)(BatchLookupArgs);
typedef void (*rect_kernel_t)(RectArgs);
typedef void (*rect_narrow_kernel_t)(RectNarrowArgs);

// One row per kernel variant, generated from the same list as the kernels.
struct CopyVariant { unsigned unroll, nt_load, store, realign; copy_kernel_t fn; };
struct FillVariant { unsigned unroll, store; fill_kernel_t fn; };
struct BatchVariant { unsigned split, nt_load, store; batch_kernel_t fn; };
struct BatchLookupVariant { unsigned nt_load, store; batch_lookup_kernel_t fn; };
struct RectVariant { unsigned unroll, nt_load, store; rect_kernel_t fn; };
struct RectNarrowVariant { unsigned nt_load, store; rect_narrow_kernel_t fn; };

#define MI355_COPY_ROW(U, L, S, R) {U, L, S, R, mi355_copy_u##U##_l##L##_s##S##_r##R},
const CopyVariant kCopyVariants[] = {MI355_FOR_EACH_COPY_KERNEL(MI355_COPY_ROW)};
#define MI355_FILL_ROW(U, S) {U, S, mi355_fill_u##U##_s##S},
const FillVariant kFillVariants[] = {MI355_FOR_EACH_FILL_KERNEL(MI355_FILL_ROW)};
#define MI355_BATCH_ROW(P, L, S) {P, L, S, mi355_batch_records_p##P##_l##L##_s##S},
const BatchVariant kBatchVariants[] = {MI355_FOR_EACH_BATCH_RECORDS_KERNEL(MI355_BATCH_ROW)};
#define MI355_BATCH_LOOKUP_ROW(L, S) {L, S, mi355_batch_lookup_l##L##_s##S},
const BatchLookupVariant kBatchLookupVariants[] = {MI355_FOR_EACH_BATCH_LOOKUP_KERNEL(MI355_BATCH_LOOKUP_ROW)};
#define MI355_RECT_ROW(U, L, S) {U, L, S, mi355_rect_u##U##_l##L##_s##S},
const RectVariant kRectVariants[] = {MI355_FOR_EACH_RECT_KERNEL(MI355_RECT_ROW)};
#define MI355_RECT_NARROW_ROW(L, S) {L, S, mi355_rect_narrow_l##L##_s##S},
const RectNarrowVariant kRectNarrowVariants[] = {MI355_FOR_EACH_RECT_NARROW_KERNEL(MI355_RECT_NARROW_ROW)};

copy_kernel_t select_copy_kernel(const mi355_blit_plan_t& p) {
  for (const CopyVariant& v : kCopyVariants)
    if (v.unroll == p.unroll && v.nt_load == p.nt_load && v.store == p.store_policy &&
        v.realign == (p.byte_shift ? 1u : 0u))
      return v.fn;
  return nullptr;
}

fill_kernel_t select_fill_kernel(const mi355_blit_plan_t& p) {
  for (const FillVariant& v : kFillVariants)
    if (v.unroll == p.unroll && v.store == p.store_policy) return v.fn;
  return nullptr;
}

batch_kernel_t select_batch_kernel(unsigned split, bool ntl, unsigned policy) {
  for (const BatchVariant& v : kBatchVariants)
    if (v.split == split && v.nt_load == (ntl ? 1u : 0u) && v.store == policy) return v.fn;
  return nullptr;
}

rect_kernel_t select_rect_kernel(unsigned unroll, bool ntl, unsigned policy) {
  for (const RectVariant& v : kRectVariants)
    if (v.unroll == unroll && v.nt_load == (ntl ? 1u : 0u) && v.store == policy) return v.fn;
  return nullptr;
}

// Puts a marker behind everything submitted so far.  Caller holds h->lock.
// When the ledger is full the oldest marker is waited for, the back-pressure
// ROCr applies when its AQL ring is full (amd_blit_kernel.cpp:844-854).
int ledger_mark(mi355_blit* h) {
  if (!h->unmarked) return MI355_BLIT_SUCCESS;
  LedgerSlot& slot = h->ledger[h->ledger_head % kLedgerSlots];
  if (slot.in_flight) {
    BLIT_HIP(hipEventSynchronize(slot.done));
    slot.in_flight = false;
  }
  BLIT_HIP(hipEventRecord(slot.done, h->last_stream));
  slot.bytes = h->unmarked_bytes;
  slot.in_flight = true;
  ++h->ledger_head;
  h->unmarked = false;
  h->unmarked_bytes = 0;
  return MI355_BLIT_SUCCESS;
}

bool stream_is_capturing(hipStream_t s) {
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  return hipStreamIsCapturing(s, &capture) == hipSuccess && capture == hipStreamCaptureStatusActive;
}

// Notes `bytes` as queued on `s`.  Caller holds h->lock.
int ledger_record(mi355_blit* h, hipStream_t s, uint64_t bytes) {
  // A command recorded into a graph under stream capture is not queued
  // anywhere: nothing is pending because of it, and no marker event may be
  // recorded on the capturing stream.  (The handle's own stream is never
  // captured by a caller that does not know it.)
  if (s != h->stream && stream_is_capturing(s)) return MI355_BLIT_SUCCESS;
  if (h->unmarked && h->last_stream != s) {
    // a marker only orders against its own stream
    int rc = ledger_mark(h);
    if (rc != MI355_BLIT_SUCCESS) return rc;
  }
  h->last_stream = s;
  h->unmarked = true;
  h->unmarked_bytes += bytes;
  return MI355_BLIT_SUCCESS;
}

void free_batch_buffers(mi355_blit* h) {
  for (int i = 0; i < 2; ++i) {
    if (h->descs_host[i]) {
      if (h->stage_in_device_memory) (void)hipFree(h->descs_host[i]);
      else (void)hipHostFree(h->descs_host[i]);
    }
    h->descs_host[i] = nullptr;
  }
  if (h->chunk_start_dev) (void)hipFree(h->chunk_start_dev);
  if (h->block_sum_dev) (void)hipFree(h->block_sum_dev);
  if (h->descs_private_dev) (void)hipFree(h->descs_private_dev);
  h->chunk_start_dev = nullptr;
  h->block_sum_dev = nullptr;
  h->descs_private_dev = nullptr;
  h->batch_capacity = 0;
}

// Buffers for n descriptors and, when n_records != 0, that many chunk records.
// Caller holds h->lock.
int ensure_batch_capacity(mi355_blit* h, size_t n, size_t n_records) {
  if (n <= h->batch_capacity && n_records <= h->records_capacity) return MI355_BLIT_SUCCESS;
  // the old buffers may still be read by a batch in flight
  for (int i = 0; i < 2; ++i) {
    if (h->batch_busy[i]) {
      BLIT_HIP(hipEventSynchronize(h->batch_done[i]));
      h->batch_busy[i] = false;
    }
  }
  if (n > h->batch_capacity) {
    size_t cap = h->batch_capacity ? h->batch_capacity : 1024;
    while (cap < n) cap *= 2;
    free_batch_buffers(h);
    for (int i = 0; i < 2; ++i) {
      if (h->stage_in_device_memory)
        BLIT_HIP(hipMalloc(reinterpret_cast<void**>(&h->descs_host[i]), batch_stage_bytes(cap)));
      else
        BLIT_HIP(hipHostMalloc(reinterpret_cast<void**>(&h->descs_host[i]), batch_stage_bytes(cap), hipHostMallocDefault));
    }
    BLIT_HIP(hipMalloc(reinterpret_cast<void**>(&h->chunk_start_dev), (cap + 1) * sizeof(uint32_t)));
    BLIT_HIP(hipMalloc(reinterpret_cast<void**>(&h->block_sum_dev), (cap / 1024 + 1) * sizeof(uint32_t)));
    BLIT_HIP(hipMalloc(reinterpret_cast<void**>(&h->descs_private_dev), cap * sizeof(BatchDesc)));
    h->batch_capacity = cap;
  }
  if (n_records > h->records_capacity) {
    size_t cap = h->records_capacity ? h->records_capacity : 65536;
    while (cap < n_records) cap *= 2;
    if (h->records_dev) (void)hipFree(h->records_dev);
    h->records_dev = nullptr;
    h->records_capacity = 0;
    BLIT_HIP(hipMalloc(reinterpret_cast<void**>(&h->records_dev), cap * sizeof(ChunkRecord)));
    h->records_capacity = cap;
  }
  return MI355_BLIT_SUCCESS;
}

}  // namespace

static_assert(sizeof(mi355_blit_desc_t) == sizeof(mi355::BatchDesc), "descriptor layout");
static_assert(mi355::kBatchChunkVecs == mi355::kChunkVecs, "chunk size");
static_assert(MI355_BLIT_STORE_SYSTEM_WT == mi355::kStoreSystemWt && MI355_BLIT_STORE_NT == mi355::kStoreNt &&
              MI355_BLIT_STORE_AGENT_WT == mi355::kStoreAgentWt, "store policy values");

extern "C" {

int mi355_blit_abi_version(void) { return MI355_BLIT_ABI_VERSION; }

const char* mi355_blit_status_string(int status) {
  switch (status) {
    case MI355_BLIT_SUCCESS: return "success";
    case MI355_BLIT_ERROR: return "error";
    case MI355_BLIT_ERROR_INVALID_ARGUMENT: return "invalid argument";
    case MI355_BLIT_ERROR_OUT_OF_RESOURCES: return "out of resources";
    case MI355_BLIT_ERROR_NOT_INITIALIZED: return "not initialized";
    default: return "unknown status";
  }
}

int mi355_blit_plan_copy(uint64_t dst, uint64_t src, uint64_t bytes, uint32_t num_cus,
                         const mi355_blit_tuning_t* tuning, mi355_blit_plan_t* out) {
  return plan_copy(dst, src, bytes, num_cus, tuning, out);
}

int mi355_blit_plan_copy_route(uint64_t dst, uint64_t src, uint64_t bytes, uint32_t num_cus,
                               const mi355_blit_tuning_t* tuning, uint32_t route, mi355_blit_plan_t* out) {
  return plan_copy(dst, src, bytes, num_cus, tuning, out, route);
}

int mi355_blit_plan_fill(uint64_t ptr, uint64_t num_dwords, uint32_t num_cus,
                         const mi355_blit_tuning_t* tuning, mi355_blit_plan_t* out) {
  return plan_fill(ptr, num_dwords, num_cus, tuning, out);
}

uint32_t mi355_blit_plan_copy_pieces(uint64_t bytes, uint32_t route, uint32_t max_pieces,
                                     const mi355_blit_tuning_t* tuning, uint64_t* piece_bytes) {
  uint64_t unused;
  return copy_pieces(bytes, route, max_pieces, tuning, piece_bytes ? piece_bytes : &unused);
}

uint64_t mi355_policy_force_sdma_size(void) { return policy_force_sdma_size(); }

uint32_t mi355_policy_same_gpu_engine(uint64_t size, uint64_t force_sdma_size) {
  return policy_same_gpu_engine(size, force_sdma_size);
}

int mi355_blit_create(int device_ordinal, mi355_blit_t** out) {
  if (!out) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  *out = nullptr;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) return MI355_BLIT_ERROR_NOT_INITIALIZED;
  if (device_ordinal < 0 || device_ordinal >= count) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  DeviceScope scope(device_ordinal);
  if (scope.err != hipSuccess) return status_of(scope.err);

  mi355_blit* h = new (std::nothrow) mi355_blit;
  if (!h) return MI355_BLIT_ERROR_OUT_OF_RESOURCES;
  h->device = device_ordinal;
  int cus = 0;
  hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device_ordinal);
  if (e == hipSuccess && cus > 0) e = hipStreamCreateWithFlags(&h->stream, hipStreamNonBlocking);
  for (unsigned i = 0; e == hipSuccess && i < kLedgerSlots; ++i)
    e = hipEventCreateWithFlags(&h->ledger[i].done, hipEventDisableTiming);
  for (int i = 0; e == hipSuccess && i < 2; ++i)
    e = hipEventCreateWithFlags(&h->batch_done[i], hipEventDisableTiming);
  if (e != hipSuccess || cus <= 0) {
    mi355_blit_destroy(h);
    return e == hipSuccess ? MI355_BLIT_ERROR : status_of(e);
  }
  h->num_cus = cus;
  {
    void* p = nullptr;
    h->scratch_err = scratch_for_device(device_ordinal, &p);
    h->scratch_dev = static_cast<unsigned char*>(p);
  }
  int large_bar = 0;
  if (hipDeviceGetAttribute(&large_bar, hipDeviceAttributeIsLargeBar, device_ordinal) == hipSuccess && large_bar &&
      !std::getenv("MI355_BLIT_HOST_STAGING"))
    h->stage_in_device_memory = true;
  *out = h;
  return MI355_BLIT_SUCCESS;
}

int mi355_blit_destroy(mi355_blit_t* h) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  int rc = MI355_BLIT_SUCCESS;
  {
    std::lock_guard<std::mutex> g(h->lock);
    DeviceScope scope(h->device);
    // every command, on whichever stream it went, is behind a marker
    if (h->ledger[0].done && ledger_mark(h) != MI355_BLIT_SUCCESS) rc = MI355_BLIT_ERROR;
    for (unsigned i = 0; i < kLedgerSlots; ++i) {
      LedgerSlot& s = h->ledger[i];
      if (s.done) {
        if (s.in_flight && hipEventSynchronize(s.done) != hipSuccess) rc = MI355_BLIT_ERROR;
        (void)hipEventDestroy(s.done);
      }
    }
    if (h->stream) {
      if (hipStreamSynchronize(h->stream) != hipSuccess) rc = MI355_BLIT_ERROR;
      (void)hipStreamDestroy(h->stream);
    }
    for (int i = 0; i < 2; ++i)
      if (h->batch_done[i]) (void)hipEventDestroy(h->batch_done[i]);
    free_batch_buffers(h);
    if (h->records_dev) (void)hipFree(h->records_dev);
    if (h->batch_seen) (void)hipHostFree(h->batch_seen);
  }
  delete h;
  return rc;
}

int mi355_blit_num_cus(mi355_blit_t* h) { return h ? h->num_cus : 0; }

void* mi355_blit_stream(mi355_blit_t* h) { return h ? static_cast<void*>(h->stream) : nullptr; }

int mi355_blit_set_tuning(mi355_blit_t* h, const mi355_blit_tuning_t* tuning) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> g(h->lock);
  h->has_tuning = tuning != nullptr;
  if (tuning) h->tuning = *tuning;
  return MI355_BLIT_SUCCESS;
}

int mi355_blit_last_launch_info(mi355_blit_t* h, mi355_blit_plan_t* out) {
  if (!h || !out) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> g(h->lock);
  *out = h->last_plan;
  return MI355_BLIT_SUCCESS;
}

int mi355_blit_copy(mi355_blit_t* h, void* dst, const void* src, size_t bytes, void* stream) {
  return mi355_blit_copy_route(h, dst, src, bytes, MI355_BLIT_ROUTE_DEVICE, stream);
}

int mi355_blit_copy_route(mi355_blit_t* h, void* dst, const void* src, size_t bytes, uint32_t route,
                          void* stream) {
  if (!h || !dst || !src || route > MI355_BLIT_ROUTE_DEVICE_TO_HOST) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (bytes == 0) return MI355_BLIT_SUCCESS;
  std::lock_guard<std::mutex> g(h->lock);
  DeviceScope scope(h->device);
  if (scope.err != hipSuccess) return status_of(scope.err);
  hipStream_t s = stream ? static_cast<hipStream_t>(stream) : h->stream;
  // one launch, or several for a copy of several GiB (copy_pieces)
  uint64_t piece_bytes;
  const uint32_t pieces = copy_pieces(bytes, route, kCopyMaxPieces, h->has_tuning ? &h->tuning : nullptr, &piece_bytes);
  mi355_blit_plan_t p;
  for (uint32_t i = 0; i < pieces; ++i) {
    const uint64_t off = i * piece_bytes;
    const uint64_t n = bytes - off < piece_bytes ? bytes - off : piece_bytes;
    uint8_t* d = static_cast<uint8_t*>(dst) + off;
    const uint8_t* sp = static_cast<const uint8_t*>(src) + off;
    int rc = plan_copy(reinterpret_cast<uint64_t>(d), reinterpret_cast<uint64_t>(sp), n, h->num_cus,
                       h->has_tuning ? &h->tuning : nullptr, &p, route);
    if (rc != MI355_BLIT_SUCCESS) return rc;
    copy_kernel_t k = select_copy_kernel(p);
    if (!k) return MI355_BLIT_ERROR;
    const CopyArgs a = make_copy_args(p, d, sp, n);
    hipLaunchKernelGGL(k, dim3(p.grid), dim3(p.wg_size), 0, s, a);
    BLIT_HIP(hipGetLastError());
  }
  p.pieces = pieces;
  h->last_plan = p;
  return ledger_record(h, s, bytes);
}

int mi355_blit_fill32(mi355_blit_t* h, void* ptr, uint32_t value, size_t num_dwords, void* stream) {
  if (!h || !ptr || (reinterpret_cast<uintptr_t>(ptr) & 3)) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (num_dwords == 0) return MI355_BLIT_SUCCESS;
  std::lock_guard<std::mutex> g(h->lock);
  DeviceScope scope(h->device);
  if (scope.err != hipSuccess) return status_of(scope.err);
  mi355_blit_plan_t p;
  int rc = plan_fill(reinterpret_cast<uint64_t>(ptr), num_dwords, h->num_cus,
                     h->has_tuning ? &h->tuning : nullptr, &p);
  if (rc != MI355_BLIT_SUCCESS) return rc;
  fill_kernel_t k = select_fill_kernel(p);
  if (!k) return MI355_BLIT_ERROR;
  const FillArgs a = make_fill_args(p, ptr, value, num_dwords);
  hipStream_t s = stream ? static_cast<hipStream_t>(stream) : h->stream;
  hipLaunchKernelGGL(k, dim3(p.grid), dim3(p.wg_size), 0, s, a);
  BLIT_HIP(hipGetLastError());
  h->last_plan = p;
  return ledger_record(h, s, num_dwords * 4);
}

namespace {
int copy_batch(mi355_blit_t* h, const mi355_blit_desc_t* descs, size_t n, int descs_on_device,
               uint64_t max_total_bytes, void* stream);
}

int mi355_blit_copy_batch(mi355_blit_t* h, const mi355_blit_desc_t* descs, size_t n,
                          int descs_on_device, void* stream) {
  return copy_batch(h, descs, n, descs_on_device, 0, stream);
}

int mi355_blit_copy_batch_bounded(mi355_blit_t* h, const mi355_blit_desc_t* device_descs, size_t n,
                                  uint64_t max_total_bytes, void* stream) {
  if (max_total_bytes == 0) return n ? MI355_BLIT_ERROR_INVALID_ARGUMENT : MI355_BLIT_SUCCESS;
  return copy_batch(h, device_descs, n, 1, max_total_bytes, stream);
}

namespace {
// The two launches of the device-side prefix sum over the copies' chunk
// counts: chunk_start within groups of 1024 copies, block_sum across groups.
// The device memory a batch of device-resident descriptors works in: the
// handle's own buffers, or the parts of the static scratch array.
struct BatchDeviceBuffers {
  uint32_t* chunk_start;
  uint32_t* block_sum;
  ChunkRecord* records;
  uint64_t* seen;  // host memory for the batch's numbers of copies and chunks; may be null
};

void launch_scans(const BatchDeviceBuffers& b, hipStream_t s, const BatchDesc* dev_descs, size_t n,
                  BatchDesc* private_copy) {
  const uint32_t n_blocks = static_cast<uint32_t>((n + 1023) / 1024);
  ScanLocalArgs sl{dev_descs, static_cast<uint64_t>(n), b.chunk_start, b.block_sum, private_copy};
  hipLaunchKernelGGL(mi355_batch_scan_local, dim3(n_blocks), dim3(1024), 0, s, sl);
  ScanTopArgs st{b.block_sum, b.chunk_start, static_cast<uint64_t>(n), n_blocks};
  hipLaunchKernelGGL(mi355_batch_scan_top, dim3(1), dim3(1024), 0, s, st);
}

// The copy over h->records_dev, launched as *p says (plan_batch_records).
int launch_records_copy(mi355_blit* h, hipStream_t s, const mi355_blit_plan_t& p, const BatchLaunch& l,
                        uint64_t total_chunks) {
  batch_kernel_t k = select_batch_kernel(l.split, p.nt_load != 0, p.store_policy);
  if (!k) return MI355_BLIT_ERROR;
  BatchCopyArgs bc{h->records_dev, total_chunks, nullptr, l.waves_per_wg, l.n_waves, make_xcd_runs(p.grid, p.xcd_run),
                   l.prefetch_waves, 0};
  hipLaunchKernelGGL(k, dim3(p.grid), dim3(p.wg_size), 0, s, bc);
  return MI355_BLIT_SUCCESS;
}

// The same for device-resident descriptors: `records` is what the record
// buffer has room for, the number of chunks is behind the prefix sums.
int launch_lookup_copy(const BatchDeviceBuffers& b, hipStream_t s, const mi355_blit_plan_t& p, const BatchLaunch& l,
                       uint64_t records, const BatchDesc* dev_descs, size_t n) {
  batch_lookup_kernel_t k = nullptr;
  for (const BatchLookupVariant& v : kBatchLookupVariants)
    if (v.nt_load == p.nt_load && v.store == p.store_policy) k = v.fn;
  if (!k || l.split != 4) return MI355_BLIT_ERROR;
  BatchLookupArgs a{{b.records, records, b.chunk_start + n, l.waves_per_wg, l.n_waves,
                     make_xcd_runs(p.grid, p.xcd_run), l.prefetch_waves, 0},
                    dev_descs, b.chunk_start, b.block_sum, static_cast<uint64_t>(n), b.seen};
  hipLaunchKernelGGL(k, dim3(p.grid), dim3(p.wg_size), 0, s, a);
  return MI355_BLIT_SUCCESS;
}

// Prefix sums, records and the copy for n device-resident descriptors, in the
// buffers *b: four launches, nothing else.
int launch_device_batch(const BatchDeviceBuffers& b, hipStream_t s, const mi355_blit_plan_t& p, const BatchLaunch& l,
                        uint64_t records, const BatchDesc* scanned, const BatchDesc* dev_descs,
                        BatchDesc* private_copy, size_t n) {
  launch_scans(b, s, scanned, n, private_copy);
  EmitRecordsDeviceArgs er{dev_descs, b.chunk_start, b.block_sum, static_cast<uint64_t>(n), b.records, records};
  hipLaunchKernelGGL(mi355_batch_emit_records_lookup, dim3(static_cast<uint32_t>((records + 255) / 256)),
                     dim3(256), 0, s, er);
  BLIT_HIP(hipGetLastError());
  return launch_lookup_copy(b, s, p, l, records, dev_descs, n);
}

int copy_batch(mi355_blit_t* h, const mi355_blit_desc_t* descs, size_t n, int descs_on_device,
               uint64_t max_total_bytes, void* stream) {
  if (!h || (!descs && n)) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (n == 0) return MI355_BLIT_SUCCESS;
  if (n > 0xffffffffull) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> g(h->lock);
  DeviceScope scope(h->device);
  if (scope.err != hipSuccess) return status_of(scope.err);
  hipStream_t s = stream ? static_cast<hipStream_t>(stream) : h->stream;
  if (stream_is_capturing(s)) {
    // A batch stages descriptors, may allocate, and shares its record buffer
    // with the batches around it through events: none of that can be
    // recorded into a graph.
    return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  }

  // Host-resident descriptors go one of two ways: the host walks them (the
  // exact chunk total, one small kernel before the copy), or, when the walk
  // would take longer than the copies themselves, they are staged as they are
  // and taken from there like device-resident ones.
  // Idle means nothing of this engine is in flight: the batch before has
  // finished (its event is the last thing it left in its stream) and so has
  // whatever was submitted since (a 1 GiB copy hides the walk as well as a
  // batch does).
  auto engine_idle = [h]() {
    const unsigned before = h->next_host ^ 1;
    if (h->batch_busy[before] && hipEventQuery(h->batch_done[before]) == hipSuccess) h->batch_busy[before] = false;
    if (h->batch_busy[before]) return false;
    return !h->unmarked || hipStreamQuery(h->last_stream) == hipSuccess;
  };
  const bool raw = !descs_on_device &&
                   batch_prefers_raw_staging(descs, n, engine_idle, h->has_tuning ? &h->tuning : nullptr);
  const bool walk = !descs_on_device && !raw;
  BatchShape shape;
  BatchDeviceSizing sizing{};
  int rc;
  if (walk) {
    rc = batch_build(descs, n, &h->stage_image, &shape);
    if (rc != MI355_BLIT_SUCCESS) return rc;
    if (shape.total_chunks == 0) return MI355_BLIT_SUCCESS;
    rc = ensure_batch_capacity(h, shape.pieces, shape.total_chunks);
    if (rc != MI355_BLIT_SUCCESS) return rc;
  } else {
    rc = ensure_batch_capacity(h, n, 0);
    if (rc != MI355_BLIT_SUCCESS) return rc;
  }

  // The two staging buffers alternate, so staging one batch overlaps the
  // execution of the one before; a buffer is only waited for until the batch
  // that used it, two batches ago, has finished.
  const unsigned b = h->next_host;
  if (!descs_on_device && h->batch_busy[b]) {
    BLIT_HIP(hipEventSynchronize(h->batch_done[b]));
    h->batch_busy[b] = false;
  }
  size_t staged_bytes = 0;
  if (walk) {
    staged_bytes = batch_stage_bytes(shape.pieces);
    batch_stage(h->stage_image, h->descs_host[b]);
  } else if (raw) {
    uint64_t total_bytes = 0;
    uint64_t likely_chunks = 0;
    rc = batch_stage_raw(descs, n, h->descs_host[b], &total_bytes, &likely_chunks);
    if (rc != MI355_BLIT_SUCCESS) return rc;
    if (total_bytes == 0) return MI355_BLIT_SUCCESS;
    staged_bytes = n * sizeof(BatchDesc);
    // the bytes are known exactly: they size the record buffer as a caller's
    // bound would, and the grid follows the host's estimate of the chunk count
    sizing = batch_device_sizing(n, total_bytes, 0, likely_chunks);
  } else {
    // lengths are only known on the device
    if (!h->batch_seen) {
      BLIT_HIP(hipHostMalloc(reinterpret_cast<void**>(&h->batch_seen), 64, hipHostMallocDefault));
      *h->batch_seen = 0;
    }
    sizing = batch_device_sizing(n, max_total_bytes, *static_cast<volatile uint64_t*>(h->batch_seen));
  }
  if (!walk) {
    if (sizing.records == 0) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
    shape.pieces = n;
    shape.total_chunks = sizing.grid_chunks;
    shape.total_bytes = sizing.bytes;
    rc = ensure_batch_capacity(h, n, sizing.records);
    if (rc != MI355_BLIT_SUCCESS) return rc;
  }
  if (staged_bytes && h->stage_in_device_memory) {
    // posted writes across the bus: order them, then read one back so that
    // they have landed before the launch below can reach the GPU
    _mm_sfence();
    (void)*(reinterpret_cast<volatile uint32_t*>(reinterpret_cast<uint8_t*>(h->descs_host[b]) + staged_bytes) - 1);
  }

  // The device-side buffers (records, prefix sums) are shared by consecutive
  // batches: the next batch waits for the previous one, which stream order
  // does by itself unless the two are on different streams.
  h->next_host ^= 1;
  if (h->batch_busy[b ^ 1] && h->last_batch_stream != s) BLIT_HIP(hipStreamWaitEvent(s, h->batch_done[b ^ 1], 0));

  const mi355_blit_tuning_t* t = h->has_tuning ? &h->tuning : nullptr;
  // Descriptors whose lengths the host has not walked are taken to be a large
  // batch.  Only walked ones leave the copy's shape open to tuning.
  mi355_blit_plan_t p;
  const BatchLaunch l = plan_batch_records(shape.total_chunks, shape.total_bytes,
                                           !walk || shape.total_bytes >= (4ull << 20), t, walk, &p);

  if (walk) {
    // The image the host staged (the descriptors, cut into pieces of at most 64
    // chunks, and each piece's first record index) is all the GPU needs to
    // write the records, a wave for kEmitPiecesPerWave pieces.
    const BatchDesc* staged = h->descs_host[b];
    EmitRecordsArgs er{staged, reinterpret_cast<const uint32_t*>(staged + shape.pieces), shape.pieces, h->records_dev};
    hipLaunchKernelGGL(mi355_batch_emit_records, dim3(emit_records_grid(shape.pieces)), dim3(256), 0, s, er);
    BLIT_HIP(hipGetLastError());

    rc = launch_records_copy(h, s, p, l, shape.total_chunks);
    if (rc != MI355_BLIT_SUCCESS) return rc;
  } else {
    // The prefix sum over the chunk counts and the records are made on the
    // device; the grid and the record buffer are sized by the bytes the host
    // added up, by the caller's bound or, without either, by an assumption
    // (batch_device_sizing).  The copy kernel reads the number of chunks on the
    // device: surplus waves end at once, missing ones are made up for by
    // striding, and chunks without a record are looked up in the prefix sums.
    // Descriptors the host staged are read once, by the first kernel, which
    // leaves a copy of them for the others.
    const BatchDesc* scanned = raw ? h->descs_host[b] : reinterpret_cast<const BatchDesc*>(descs);
    const BatchDesc* dev_descs = raw ? h->descs_private_dev : scanned;
    const BatchDeviceBuffers bufs{h->chunk_start_dev, h->block_sum_dev, h->records_dev, h->batch_seen};
    rc = launch_device_batch(bufs, s, p, l, sizing.records, scanned, dev_descs, raw ? h->descs_private_dev : nullptr, n);
    if (rc != MI355_BLIT_SUCCESS) return rc;
  }
  BLIT_HIP(hipGetLastError());
  BLIT_HIP(hipEventRecord(h->batch_done[b], s));
  h->batch_busy[b] = true;
  h->last_batch_stream = s;
  h->last_plan = p;
  return ledger_record(h, s, shape.total_bytes);
}
}  // namespace

int mi355_blit_copy_batch_bounded_noalloc(mi355_blit_t* h, const mi355_blit_desc_t* device_descs, size_t n,
                                          uint64_t max_total_bytes, void* stream) {
  if (!h || (!device_descs && n)) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (max_total_bytes == 0) return n ? MI355_BLIT_ERROR_INVALID_ARGUMENT : MI355_BLIT_SUCCESS;
  if (n == 0) return MI355_BLIT_SUCCESS;
  if (n > kNoAllocMaxCopies) return MI355_BLIT_ERROR_OUT_OF_RESOURCES;
  std::lock_guard<std::mutex> g(h->lock);
  DeviceScope scope(h->device);
  if (scope.err != hipSuccess) return status_of(scope.err);
  if (!h->scratch_dev) return h->scratch_err != hipSuccess ? status_of(h->scratch_err) : MI355_BLIT_ERROR;
  hipStream_t s = stream ? static_cast<hipStream_t>(stream) : h->stream;
  BatchDeviceSizing sizing = batch_device_sizing(n, max_total_bytes);
  if (sizing.records == 0) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  // Chunks beyond the records the scratch has room for are looked up in the
  // prefix sums by the copy kernel: the scratch bounds the number of copies,
  // not their bytes.
  if (sizing.records > kNoAllocRecords) sizing.records = kNoAllocRecords;
  mi355_blit_plan_t p;
  const BatchLaunch l = plan_batch_records(sizing.grid_chunks, sizing.bytes, true,
                                           h->has_tuning ? &h->tuning : nullptr, false, &p);
  // Every word of the scratch that the kernels read was written by a kernel of
  // this same call before (the prefix sums in full, the records up to the
  // smaller of the chunk total and the capacity): nothing has to start at zero.
  const BatchDeviceBuffers bufs{reinterpret_cast<uint32_t*>(h->scratch_dev + kScratchChunkStart),
                                reinterpret_cast<uint32_t*>(h->scratch_dev + kScratchBlockSum),
                                reinterpret_cast<ChunkRecord*>(h->scratch_dev + kScratchRecords), nullptr};
  const BatchDesc* descs = reinterpret_cast<const BatchDesc*>(device_descs);
  const int rc = launch_device_batch(bufs, s, p, l, sizing.records, descs, descs, nullptr, n);
  if (rc != MI355_BLIT_SUCCESS) return rc;
  BLIT_HIP(hipGetLastError());
  h->last_plan = p;
  // No entry in the pending-bytes ledger: a command on another stream than the
  // last one makes the ledger record an event there, and a full ledger waits
  // for its oldest one -- neither belongs in a call that is four launches.
  return MI355_BLIT_SUCCESS;
}

int mi355_blit_copy_rect(mi355_blit_t* h, const mi355_pitched_ptr_t* dst, const mi355_dim3_t* dst_offset,
                         const mi355_pitched_ptr_t* src, const mi355_dim3_t* src_offset,
                         const mi355_dim3_t* range, void* stream) {
  return mi355_blit_copy_rect_route(h, dst, dst_offset, src, src_offset, range, MI355_BLIT_ROUTE_DEVICE, stream);
}

int mi355_blit_copy_rect_route(mi355_blit_t* h, const mi355_pitched_ptr_t* dst, const mi355_dim3_t* dst_offset,
                               const mi355_pitched_ptr_t* src, const mi355_dim3_t* src_offset,
                               const mi355_dim3_t* range, uint32_t route, void* stream) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  RectPlan rp;
  {
    std::lock_guard<std::mutex> g(h->lock);
    int rc = plan_rect(dst, dst_offset, src, src_offset, range, h->has_tuning ? &h->tuning : nullptr, &rp, route);
    if (rc != MI355_BLIT_SUCCESS) return rc;
  }
  if (rp.empty) return MI355_BLIT_SUCCESS;
  if (rp.linear) return mi355_blit_copy_route(h, rp.args.dst, rp.args.src, rp.args.width, route, stream);
  std::lock_guard<std::mutex> g(h->lock);
  DeviceScope scope(h->device);
  if (scope.err != hipSuccess) return status_of(scope.err);
  hipStream_t s = stream ? static_cast<hipStream_t>(stream) : h->stream;
  if (rp.narrow) {
    rect_narrow_kernel_t k = nullptr;
    for (const RectNarrowVariant& v : kRectNarrowVariants)
      if (v.nt_load == rp.streaming && v.store == rp.store_policy) k = v.fn;
    if (!k) return MI355_BLIT_ERROR;
    hipLaunchKernelGGL(k, dim3(rp.grid), dim3(rp.wg_size), 0, s, rp.nargs);
  } else {
    rect_kernel_t k = select_rect_kernel(rp.unroll, rp.streaming != 0, rp.store_policy);
    if (!k) return MI355_BLIT_ERROR;
    hipLaunchKernelGGL(k, dim3(rp.grid), dim3(rp.wg_size), 0, s, rp.args);
  }
  BLIT_HIP(hipGetLastError());
  rect_launch_info(rp, &h->last_plan);
  return ledger_record(h, s, rp.total_bytes);
}

int mi355_blit_plan_rect(const mi355_pitched_ptr_t* dst, const mi355_dim3_t* dst_offset,
                         const mi355_pitched_ptr_t* src, const mi355_dim3_t* src_offset,
                         const mi355_dim3_t* range, const mi355_blit_tuning_t* tuning,
                         mi355_blit_rect_plan_t* out) {
  return mi355_blit_plan_rect_route(dst, dst_offset, src, src_offset, range, tuning, MI355_BLIT_ROUTE_DEVICE, out);
}

int mi355_blit_plan_rect_route(const mi355_pitched_ptr_t* dst, const mi355_dim3_t* dst_offset,
                               const mi355_pitched_ptr_t* src, const mi355_dim3_t* src_offset,
                               const mi355_dim3_t* range, const mi355_blit_tuning_t* tuning, uint32_t route,
                               mi355_blit_rect_plan_t* out) {
  if (!out) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  RectPlan rp;
  int rc = plan_rect(dst, dst_offset, src, src_offset, range, tuning, &rp, route);
  if (rc != MI355_BLIT_SUCCESS) return rc;
  *out = mi355_blit_rect_plan_t{};
  out->empty = rp.empty;
  out->linear = rp.linear;
  out->dst = reinterpret_cast<uint64_t>(rp.args.dst);
  out->src = reinterpret_cast<uint64_t>(rp.args.src);
  out->width = rp.args.width;
  out->total_bytes = rp.total_bytes;
  out->route = rp.route;
  if (rp.empty || rp.linear) return MI355_BLIT_SUCCESS;
  out->dst_pitch = rp.args.dst_pitch;
  out->dst_slice = rp.args.dst_slice;
  out->src_pitch = rp.args.src_pitch;
  out->src_slice = rp.args.src_slice;
  out->rows = rp.args.rows;
  if (rp.narrow) {
    out->layers = rp.nargs.lines / rp.nargs.rows;
    out->lanes_per_row = rp.nargs.lanes_per_row;
  } else {
    out->slots = rp.args.slots;
    out->layers = rp.args.total_slots / (rp.args.slots * rp.args.rows);
    out->unroll = rp.unroll;
    out->plain_rows = rp.args.plain_rows;
  }
  out->wg_size = rp.wg_size;
  out->grid = rp.grid;
  out->nt_load = rp.streaming;
  out->store_policy = rp.store_policy;
  out->xcd_run = rp.xcd_run;
  return MI355_BLIT_SUCCESS;
}

namespace {
int launch_signal_kernel(mi355_blit_t* h, uint64_t hsa_signal_handle, uint32_t mode, void* stream) {
  if (!h || !hsa_signal_handle || (hsa_signal_handle & 63)) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> g(h->lock);
  DeviceScope scope(h->device);
  if (scope.err != hipSuccess) return status_of(scope.err);
  hipStream_t s = stream ? static_cast<hipStream_t>(stream) : h->stream;
  SignalArgs sa{reinterpret_cast<HsaSignalAbi*>(hsa_signal_handle), mode, 0};
  hipLaunchKernelGGL(mi355_signal_complete, dim3(1), dim3(64), 0, s, sa);
  BLIT_HIP(hipGetLastError());
  return MI355_BLIT_SUCCESS;
}
}  // namespace

int mi355_blit_signal_complete(mi355_blit_t* h, uint64_t hsa_signal_handle, void* stream) {
  return launch_signal_kernel(h, hsa_signal_handle, kSignalComplete, stream);
}

int mi355_blit_signal_stamp(mi355_blit_t* h, uint64_t hsa_signal_handle, uint32_t which, void* stream) {
  if (which != MI355_BLIT_STAMP_START && which != MI355_BLIT_STAMP_END && which != MI355_BLIT_STAMP_END_AND_COMPLETE)
    return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  return launch_signal_kernel(h, hsa_signal_handle, which, stream);
}

int mi355_blit_add_callback(mi355_blit_t* h, mi355_blit_callback_t fn, void* user, void* stream) {
  if (!h || !fn) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> g(h->lock);
  DeviceScope scope(h->device);
  if (scope.err != hipSuccess) return status_of(scope.err);
  hipStream_t s = stream ? static_cast<hipStream_t>(stream) : h->stream;
  BLIT_HIP(hipLaunchHostFunc(s, fn, user));
  return MI355_BLIT_SUCCESS;
}

int mi355_blit_synchronize(mi355_blit_t* h) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  hipStream_t s;
  {
    std::lock_guard<std::mutex> g(h->lock);
    s = h->stream;
  }
  DeviceScope scope(h->device);
  if (scope.err != hipSuccess) return status_of(scope.err);
  BLIT_HIP(hipStreamSynchronize(s));
  return MI355_BLIT_SUCCESS;
}

uint64_t mi355_blit_pending_bytes(mi355_blit_t* h) {
  if (!h) return 0;
  std::lock_guard<std::mutex> g(h->lock);
  DeviceScope scope(h->device);
  // Bytes after the newest marker count as pending until a marker behind
  // them has completed, so a return of 0 means every command has finished.
  uint64_t pending = 0;
  if (h->unmarked && hipStreamQuery(h->last_stream) == hipSuccess) {
    // the stream has drained: nothing submitted to it is left, no marker needed
    h->unmarked = false;
    h->unmarked_bytes = 0;
  }
  if (ledger_mark(h) != MI355_BLIT_SUCCESS) pending += h->unmarked_bytes ? h->unmarked_bytes : 1;
  for (unsigned i = 0; i < kLedgerSlots; ++i) {
    LedgerSlot& s = h->ledger[i];
    if (!s.in_flight) continue;
    if (hipEventQuery(s.done) == hipSuccess) s.in_flight = false;
    else pending += s.bytes ? s.bytes : 1;
  }
  return pending;
}

}  // extern "C"
