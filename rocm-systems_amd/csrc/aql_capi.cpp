// The gfx950 blit engine on a raw HSA queue (declarations and the reference
// interfaces they replace: include/mi355_blit_aql.h).  This is the submission
// half of ROCr's BlitKernel done with the same means
// (projects/rocr-runtime/runtime/hsa-runtime/core/runtime/amd_blit_kernel.cpp:
// 641-924): reserve packet slots with an atomic add on the write index, fill
// the kernarg slot and the packet body, publish the header with one atomic
// store, ring the doorbell with the index of the last packet.  Uses the public
// HSA API only.
#include <hsa/hsa.h>
#include <hsa/hsa_ext_amd.h>
#include <sched.h>
#include <xmmintrin.h>

#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "aql_wait.h"
#include "blit_args.h"
#include "blit_kernel_list.h"
#include "blit_batch_host.h"
#include "blit_plan.h"
#include "blit_rect.h"
#include "mi355_blit_aql.h"

// The gfx950 code object with every kernel variant, linked in as data.
extern "C" const unsigned char mi355_blit_hsaco[];
extern "C" const unsigned char mi355_blit_hsaco_end[];

namespace {

using namespace mi355;

// Packets in a queue this library creates for itself (mi355_aql_create).  The
// reference shares the agent's 64-packet utility queue (amd_gpu_agent.h:
// 507-508), which mi355_aql_create_on adopts as it is; a batch here is two to
// four packets, so a queue of the library's own is a little larger.
constexpr uint32_t kQueuePackets = 256;
// One kernarg slot per packet slot, as in the reference (amd_blit_kernel.cpp:
// 565-569): the slot of packet index i is i & mask, so it is free again
// exactly when the packet slot is.
constexpr size_t kKernargSlotBytes = 128;
// Dispatches of up to this many workgroups take their kernarg slot from the
// ring in host memory even when there is one in device memory.
constexpr uint32_t kHostKernargMaxWorkgroups = 16;

struct Kernel {
  uint64_t object = 0;
  uint32_t kernarg_size = 0;
  uint32_t group_size = 0;
  uint32_t private_size = 0;
};

struct CopyKernel { unsigned unroll, nt_load, store, realign; const char* name; Kernel k; };
struct FillKernel { unsigned unroll, store; const char* name; Kernel k; };
struct BatchKernel { unsigned split, nt_load, store; const char* name; Kernel k; };
struct RectKernel { unsigned unroll, nt_load, store; const char* name; Kernel k; };  // unroll 0: the narrow-row kernel

#define MI355_COPY_NAME(U, L, S, R) {U, L, S, R, "mi355_copy_u" #U "_l" #L "_s" #S "_r" #R, {}},
#define MI355_FILL_NAME(U, S) {U, S, "mi355_fill_u" #U "_s" #S, {}},
#define MI355_BATCH_NAME(P, L, S) {P, L, S, "mi355_batch_records_p" #P "_l" #L "_s" #S, {}},
#define MI355_RECT_NAME(U, L, S) {U, L, S, "mi355_rect_u" #U "_l" #L "_s" #S, {}},
#define MI355_BATCH_LOOKUP_NAME(L, S) {0, L, S, "mi355_batch_lookup_l" #L "_s" #S, {}},
#define MI355_RECT_NARROW_NAME(L, S) {0, L, S, "mi355_rect_narrow_l" #L "_s" #S, {}},

struct BytesWritten {
  uint64_t index;
  uint64_t bytes;
};

int to_status(hsa_status_t s) { return static_cast<int>(s); }

#define AQL_HSA(expr)                                   \
  do {                                                  \
    hsa_status_t s_ = (expr);                           \
    if (s_ != HSA_STATUS_SUCCESS) return to_status(s_); \
  } while (0)

}  // namespace

// The kernels of one GPU agent: one loaded executable and the kernel objects
// found in it, shared by every engine on that agent and released with the last
// reference.  In the reference the agent owns the blit shaders
// (GpuAgent::AssembleShader / ReleaseShader, core/runtime/amd_gpu_agent.cpp:
// 251-428) and hands the same code to each of its blits_[] slots.
struct mi355_aql_code_object {
  hsa_agent_t gpu{};
  hsa_executable_t exe{};
  hsa_code_object_reader_t reader{};
  bool have_exe = false, have_reader = false;
  std::vector<CopyKernel> copy_kernels{MI355_FOR_EACH_COPY_KERNEL(MI355_COPY_NAME)};
  std::vector<FillKernel> fill_kernels{MI355_FOR_EACH_FILL_KERNEL(MI355_FILL_NAME)};
  std::vector<BatchKernel> batch_kernels{MI355_FOR_EACH_BATCH_RECORDS_KERNEL(MI355_BATCH_NAME)};
  std::vector<RectKernel> rect_kernels{MI355_FOR_EACH_RECT_KERNEL(MI355_RECT_NAME)};
  std::vector<RectKernel> rect_narrow_kernels{MI355_FOR_EACH_RECT_NARROW_KERNEL(MI355_RECT_NARROW_NAME)};
  std::vector<RectKernel> batch_lookup_kernels{MI355_FOR_EACH_BATCH_LOOKUP_KERNEL(MI355_BATCH_LOOKUP_NAME)};
  Kernel scan_local, scan_top, emit_records, emit_records_lookup;
  uint32_t users = 0;  // guarded by g_code_objects_lock

  ~mi355_aql_code_object() {
    if (have_exe) hsa_executable_destroy(exe);
    if (have_reader) hsa_code_object_reader_destroy(reader);
  }
};

struct mi355_aql {
  hsa_agent_t gpu{};
  hsa_agent_t cpu{};
  bool have_gpu = false, have_cpu = false;
  int wanted_ordinal = 0, seen_gpus = 0;
  uint32_t num_cus = 0;

  hsa_amd_memory_pool_t kernarg_pool{};  // host memory the packet processor reads kernargs from
  hsa_amd_memory_pool_t host_pool{};     // fine-grained host memory (descriptor staging)
  hsa_amd_memory_pool_t local_pool{};    // device memory
  bool have_kernarg = false, have_host = false, have_local = false;

  hsa_queue_t* queue = nullptr;
  uint32_t queue_mask = 0;
  // mi355_aql_create makes the runtime reference and the queue and gives both
  // back; mi355_aql_create_on borrows the caller's.
  bool owns_runtime = false, owns_queue = false;
  uint64_t wait_slice_ticks = 100000;  // one slice of a bounded wait: about a millisecond
  bool log_packets = false;            // MI355_BLIT_LOG_PKTS=1
  uint8_t* kernargs = nullptr;
  // The kernarg ring lives in device memory when the host can write there
  // (large BAR): a wave then reads its arguments from HBM instead of from
  // host memory across the bus, which on MI355X takes ~11 us off a dispatch
  // of a few hundred workgroups.  Host memory otherwise, as in the reference
  // (amd_blit_kernel.cpp:565-569).
  bool kernargs_in_device_memory = false;
  // With the ring in device memory there is a second one in host memory for
  // dispatches of a few workgroups: writing a slot across the bus and reading
  // it back before the doorbell costs the host 1.5 us, more than the handful
  // of waves of a small copy lose by fetching their arguments from the host
  // (blocking 4 KiB copy: 9.9 us with the slot in device memory, 8.5 us with it
  // in host memory; 64 KiB: equal; 1 MiB: 10.9 against 21.4 us).
  uint8_t* kernargs_host = nullptr;

  // the agent's kernels: a reference taken at creation, given back by destroy
  mi355_aql_code_object* code = nullptr;

  hsa_signal_t idle_signal{};  // completion signal of wait_idle's barrier packet
  // Completion signal of the blocking calls, guarded by sync_lock
  // (completion_signal_ and lock_ of the reference, amd_blit_kernel.h:199-204).
  hsa_signal_t sync_signal{};
  std::mutex sync_lock;

  // Orders packet indices and ledger updates (reservation_lock_ of the
  // reference, amd_blit_kernel.h:209-210).
  std::mutex reservation_lock;
  std::vector<BytesWritten> bytes_written;
  uint64_t bytes_queued = 0;
  uint64_t last_queued = 0;
  bool anything_queued = false;
  // Packets below this index are known to have completed (a wait_idle barrier
  // behind them was seen to complete).  The queue's read index says the same
  // but the packet processor publishes it with a delay.
  std::atomic<uint64_t> known_complete{0};

  std::mutex lock;  // tuning, last plan, batch buffers, wait_idle
  mi355_blit_tuning_t tuning{};
  bool has_tuning = false;
  mi355_blit_plan_t last_plan{};
  uint32_t reference_engine = 0;  // MI355_ENGINE_* of the last asynchronous copy the caller policy judged
  uint16_t fence_scope = HSA_FENCE_SCOPE_SYSTEM;
  // Transfers of 4 MiB and more carry the barrier bit (serialise()): set for an
  // engine on a queue of its own, clear on a borrowed queue.
  std::atomic<bool> serialise_large{false};
  // mi355_aql_enable_profiling: the packet processor stamps a dispatch's
  // completion signal, so a command whose times are asked for stays one dispatch.
  std::atomic<bool> profiling{false};
  std::atomic<bool> queue_error{false};

  // batched path: two staging buffers used alternately, device buffers.  The
  // staging buffers sit in device memory when the host can write there (as
  // the kernarg ring does): the host's copy of the descriptors then lands in
  // HBM while the batch before still runs, and the GPU does not fetch 24 bytes
  // per copy across the bus at the head of the batch.
  bool stage_in_device_memory[2] = {false, false};
  BatchDesc* stage[2] = {nullptr, nullptr};
  BatchImage stage_image;  // built in ordinary memory, then copied to a staging buffer
  hsa_signal_t stage_free[2] = {{0}, {0}};  // 0 when the kernel that reads stage[i] has finished
  unsigned next_stage = 0;
  uint32_t* chunk_start_dev = nullptr;
  uint32_t* block_sum_dev = nullptr;
  BatchDesc* descs_private_dev = nullptr;  // the GPU's own copy of descriptors the host staged as they were
  ChunkRecord* records_dev = nullptr;
  size_t batch_capacity = 0, records_capacity = 0;
  uint64_t* batch_seen = nullptr;  // host memory: copies << 32 | chunks of the last device-resident batch
  // Index of the last packet of the latest batch; the engine is taken to be
  // idle, as far as batches go, once the queue's read index has passed it.
  uint64_t last_batch_index = 0;
  bool any_batch = false;

  // bounce buffers of host<->device copies (mi355_aql_staging)
  void* bounce[2] = {nullptr, nullptr};
};

namespace {

hsa_status_t find_pools_cb(hsa_amd_memory_pool_t pool, void* data) {
  auto* pr = static_cast<std::pair<mi355_aql*, bool>*>(data);
  mi355_aql* h = pr->first;
  const bool is_gpu = pr->second;
  hsa_amd_segment_t seg;
  if (hsa_amd_memory_pool_get_info(pool, HSA_AMD_MEMORY_POOL_INFO_SEGMENT, &seg) != HSA_STATUS_SUCCESS ||
      seg != HSA_AMD_SEGMENT_GLOBAL)
    return HSA_STATUS_SUCCESS;
  bool can_alloc = false;
  hsa_amd_memory_pool_get_info(pool, HSA_AMD_MEMORY_POOL_INFO_RUNTIME_ALLOC_ALLOWED, &can_alloc);
  if (!can_alloc) return HSA_STATUS_SUCCESS;
  uint32_t flags = 0;
  hsa_amd_memory_pool_get_info(pool, HSA_AMD_MEMORY_POOL_INFO_GLOBAL_FLAGS, &flags);
  if (is_gpu) {
    if (!h->have_local && (flags & HSA_AMD_MEMORY_POOL_GLOBAL_FLAG_COARSE_GRAINED)) {
      h->local_pool = pool;
      h->have_local = true;
    }
  } else {
    if (!h->have_kernarg && (flags & HSA_AMD_MEMORY_POOL_GLOBAL_FLAG_KERNARG_INIT)) {
      h->kernarg_pool = pool;
      h->have_kernarg = true;
    }
    if (!h->have_host && (flags & HSA_AMD_MEMORY_POOL_GLOBAL_FLAG_FINE_GRAINED)) {
      h->host_pool = pool;
      h->have_host = true;
    }
  }
  return HSA_STATUS_SUCCESS;
}

hsa_status_t find_agents_cb(hsa_agent_t agent, void* data) {
  mi355_aql* h = static_cast<mi355_aql*>(data);
  hsa_device_type_t type;
  if (hsa_agent_get_info(agent, HSA_AGENT_INFO_DEVICE, &type) != HSA_STATUS_SUCCESS) return HSA_STATUS_SUCCESS;
  if (type == HSA_DEVICE_TYPE_GPU) {
    if (h->wanted_ordinal >= 0 && h->seen_gpus++ == h->wanted_ordinal) {
      h->gpu = agent;
      h->have_gpu = true;
    }
  } else if (type == HSA_DEVICE_TYPE_CPU && !h->have_cpu) {
    h->cpu = agent;
    h->have_cpu = true;
  }
  return HSA_STATUS_SUCCESS;
}

void queue_error_cb(hsa_status_t status, hsa_queue_t*, void* data) {
  mi355_aql* h = static_cast<mi355_aql*>(data);
  h->queue_error.store(true);
  const char* msg = nullptr;
  hsa_status_string(status, &msg);
  std::fprintf(stderr, "mi355_blit_aql: queue error 0x%x (%s)\n", status, msg ? msg : "?");
}

// Waits until `signal` drops below 1, in bounded slices, giving up with an
// error when the queue has reported one (aql_wait.h).
int wait_signal(mi355_aql* h, hsa_signal_t signal) {
  return wait_below_one(
      [signal](uint64_t ticks) {
        return static_cast<int64_t>(
            hsa_signal_wait_scacquire(signal, HSA_SIGNAL_CONDITION_LT, 1, ticks, HSA_WAIT_STATE_ACTIVE));
      },
      h->queue_error, h->wait_slice_ticks);
}

bool env_is_one(const char* name) {
  const char* v = std::getenv(name);
  return v && v[0] == '1';
}

// What LogPrint(HSA_AMD_LOG_FLAG_BLIT_KERNEL_PKTS, ...) prints for every
// packet in the reference (amd_blit_kernel.cpp:681-702, 903-923), on stderr
// when MI355_BLIT_LOG_PKTS=1.
unsigned header_bits(uint16_t header, unsigned pos, unsigned width) { return (header >> pos) & ((1u << width) - 1); }

void log_barrier_packet(mi355_aql* h, uint16_t header, const hsa_barrier_and_packet_t& pkt, uint64_t index) {
  std::fprintf(stderr,
               "HWq=%p, id=%lu, Barrier Header = 0x%x (type=%u, barrier=%u, acquire=%u, release=%u), "
               "dep_signal=[0x%zx 0x%zx 0x%zx 0x%zx 0x%zx], completion_signal=0x%zx rptr=%lu, wptr=%lu\n",
               h->queue->base_address, static_cast<unsigned long>(h->queue->id), header,
               header_bits(header, HSA_PACKET_HEADER_TYPE, HSA_PACKET_HEADER_WIDTH_TYPE),
               header_bits(header, HSA_PACKET_HEADER_BARRIER, HSA_PACKET_HEADER_WIDTH_BARRIER),
               header_bits(header, HSA_PACKET_HEADER_SCACQUIRE_FENCE_SCOPE, HSA_PACKET_HEADER_WIDTH_SCACQUIRE_FENCE_SCOPE),
               header_bits(header, HSA_PACKET_HEADER_SCRELEASE_FENCE_SCOPE, HSA_PACKET_HEADER_WIDTH_SCRELEASE_FENCE_SCOPE),
               static_cast<size_t>(pkt.dep_signal[0].handle), static_cast<size_t>(pkt.dep_signal[1].handle),
               static_cast<size_t>(pkt.dep_signal[2].handle), static_cast<size_t>(pkt.dep_signal[3].handle),
               static_cast<size_t>(pkt.dep_signal[4].handle), static_cast<size_t>(pkt.completion_signal.handle),
               static_cast<unsigned long>(hsa_queue_load_read_index_relaxed(h->queue)),
               static_cast<unsigned long>(index));
}

void log_dispatch_packet(mi355_aql* h, uint16_t header, uint16_t setup, const hsa_kernel_dispatch_packet_t& pkt,
                         uint64_t index) {
  std::fprintf(stderr,
               "HWq=%p, id=%lu, Dispatch Header = 0x%x (type=%u, barrier=%u, acquire=%u, release=%u), "
               "setup=%d, grid=[%zu, %zu, %zu], workgroup=[%zu, %zu, %zu], private_seg_size=%zu, "
               "group_seg_size=%zu, kernel_obj=0x%zx, kernarg_address=0x%zx, completion_signal=0x%zx "
               "rptr=%lu, wptr=%lu\n",
               h->queue->base_address, static_cast<unsigned long>(h->queue->id), header,
               header_bits(header, HSA_PACKET_HEADER_TYPE, HSA_PACKET_HEADER_WIDTH_TYPE),
               header_bits(header, HSA_PACKET_HEADER_BARRIER, HSA_PACKET_HEADER_WIDTH_BARRIER),
               header_bits(header, HSA_PACKET_HEADER_SCACQUIRE_FENCE_SCOPE, HSA_PACKET_HEADER_WIDTH_SCACQUIRE_FENCE_SCOPE),
               header_bits(header, HSA_PACKET_HEADER_SCRELEASE_FENCE_SCOPE, HSA_PACKET_HEADER_WIDTH_SCRELEASE_FENCE_SCOPE),
               setup, static_cast<size_t>(pkt.grid_size_x), static_cast<size_t>(pkt.grid_size_y),
               static_cast<size_t>(pkt.grid_size_z), static_cast<size_t>(pkt.workgroup_size_x),
               static_cast<size_t>(pkt.workgroup_size_y), static_cast<size_t>(pkt.workgroup_size_z),
               static_cast<size_t>(pkt.private_segment_size), static_cast<size_t>(pkt.group_segment_size),
               static_cast<size_t>(pkt.kernel_object), reinterpret_cast<size_t>(pkt.kernarg_address),
               static_cast<size_t>(pkt.completion_signal.handle),
               static_cast<unsigned long>(hsa_queue_load_read_index_relaxed(h->queue)),
               static_cast<unsigned long>(index));
}

// MI355_BLIT_HOST_KERNARGS=1 keeps the kernarg ring in host memory (for
// measurements and for systems whose BAR writes misbehave).
bool force_host_kernargs() { return env_is_one("MI355_BLIT_HOST_KERNARGS"); }

int lookup(mi355_aql_code_object* c, const char* name, Kernel* out) {
  const std::string sym = std::string(name) + ".kd";
  hsa_executable_symbol_t s;
  AQL_HSA(hsa_executable_get_symbol_by_name(c->exe, sym.c_str(), &c->gpu, &s));
  AQL_HSA(hsa_executable_symbol_get_info(s, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_OBJECT, &out->object));
  AQL_HSA(hsa_executable_symbol_get_info(s, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_KERNARG_SEGMENT_SIZE,
                                         &out->kernarg_size));
  AQL_HSA(hsa_executable_symbol_get_info(s, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_GROUP_SEGMENT_SIZE,
                                         &out->group_size));
  AQL_HSA(hsa_executable_symbol_get_info(s, HSA_EXECUTABLE_SYMBOL_INFO_KERNEL_PRIVATE_SEGMENT_SIZE,
                                         &out->private_size));
  if (out->kernarg_size > kKernargSlotBytes || out->private_size != 0) return MI355_BLIT_ERROR;
  return MI355_BLIT_SUCCESS;
}

// What AssembleShader does for the reference, with a real code object.
int load_code_object(mi355_aql_code_object* c) {
  const size_t size = static_cast<size_t>(mi355_blit_hsaco_end - mi355_blit_hsaco);
  AQL_HSA(hsa_code_object_reader_create_from_memory(mi355_blit_hsaco, size, &c->reader));
  c->have_reader = true;
  AQL_HSA(hsa_executable_create_alt(HSA_PROFILE_FULL, HSA_DEFAULT_FLOAT_ROUNDING_MODE_DEFAULT, nullptr, &c->exe));
  c->have_exe = true;
  AQL_HSA(hsa_executable_load_agent_code_object(c->exe, c->gpu, c->reader, nullptr, nullptr));
  AQL_HSA(hsa_executable_freeze(c->exe, nullptr));
  int rc;
  for (auto& k : c->copy_kernels)
    if ((rc = lookup(c, k.name, &k.k)) != MI355_BLIT_SUCCESS) return rc;
  for (auto& k : c->fill_kernels)
    if ((rc = lookup(c, k.name, &k.k)) != MI355_BLIT_SUCCESS) return rc;
  for (auto& k : c->batch_kernels)
    if ((rc = lookup(c, k.name, &k.k)) != MI355_BLIT_SUCCESS) return rc;
  for (auto& k : c->rect_kernels)
    if ((rc = lookup(c, k.name, &k.k)) != MI355_BLIT_SUCCESS) return rc;
  for (auto& k : c->rect_narrow_kernels)
    if ((rc = lookup(c, k.name, &k.k)) != MI355_BLIT_SUCCESS) return rc;
  if ((rc = lookup(c, "mi355_batch_scan_local", &c->scan_local)) != MI355_BLIT_SUCCESS) return rc;
  if ((rc = lookup(c, "mi355_batch_scan_top", &c->scan_top)) != MI355_BLIT_SUCCESS) return rc;
  if ((rc = lookup(c, "mi355_batch_emit_records", &c->emit_records)) != MI355_BLIT_SUCCESS) return rc;
  if ((rc = lookup(c, "mi355_batch_emit_records_lookup", &c->emit_records_lookup)) != MI355_BLIT_SUCCESS) return rc;
  for (auto& k : c->batch_lookup_kernels)
    if ((rc = lookup(c, k.name, &k.k)) != MI355_BLIT_SUCCESS) return rc;
  return MI355_BLIT_SUCCESS;
}

// One code object per agent in this process, found by the agent's handle.
std::mutex g_code_objects_lock;
std::vector<mi355_aql_code_object*> g_code_objects;

int code_object_acquire(hsa_agent_t gpu, mi355_aql_code_object** out) {
  std::lock_guard<std::mutex> g(g_code_objects_lock);
  for (mi355_aql_code_object* c : g_code_objects)
    if (c->gpu.handle == gpu.handle) {
      ++c->users;
      *out = c;
      return MI355_BLIT_SUCCESS;
    }
  mi355_aql_code_object* c = new (std::nothrow) mi355_aql_code_object;
  if (!c) return MI355_BLIT_ERROR_OUT_OF_RESOURCES;
  c->gpu = gpu;
  const int rc = load_code_object(c);
  if (rc != MI355_BLIT_SUCCESS) {
    delete c;
    return rc;
  }
  c->users = 1;
  g_code_objects.push_back(c);
  *out = c;
  return MI355_BLIT_SUCCESS;
}

int code_object_release(mi355_aql_code_object* c) {
  std::lock_guard<std::mutex> g(g_code_objects_lock);
  for (size_t i = 0; i < g_code_objects.size(); ++i)
    if (g_code_objects[i] == c) {
      if (--c->users == 0) {
        g_code_objects.erase(g_code_objects.begin() + static_cast<long>(i));
        delete c;  // destroys the executable
      }
      return MI355_BLIT_SUCCESS;
    }
  return MI355_BLIT_ERROR_INVALID_ARGUMENT;
}


// amd_blit_kernel.cpp:844-854: reserve num_packet slots; yield while the ring
// is full.  False when the queue has reported an error: before the write index
// was touched, or, if the report came while waiting for room, once the read
// index has stood still for two milliseconds more -- a queue that has stopped
// never frees a slot.  The caller then writes no packet and rings no doorbell:
// slots that were never freed may hold packets of other producers.  (While the
// read index still moves the wait goes on: on a queue that works, a reserved
// slot left unwritten would stop the packet processor for everybody.)
bool acquire_write_index(mi355_aql* h, uint32_t num_packet, uint64_t* out) {
  if (h->queue_error.load(std::memory_order_acquire)) return false;
  const uint64_t index = hsa_queue_add_write_index_scacq_screl(h->queue, num_packet);
  *out = index;
  uint64_t last_read = hsa_queue_load_read_index_relaxed(h->queue);
  auto last_progress = std::chrono::steady_clock::now();
  while (index + num_packet - hsa_queue_load_read_index_relaxed(h->queue) > h->queue->size) {
    if (h->queue_error.load(std::memory_order_acquire)) {
      const uint64_t rd = hsa_queue_load_read_index_relaxed(h->queue);
      const auto now = std::chrono::steady_clock::now();
      if (rd != last_read) {
        last_read = rd;
        last_progress = now;
      } else if (now - last_progress > std::chrono::milliseconds(2)) {
        return false;
      }
    }
    sched_yield();
  }
  return true;
}

// amd_blit_kernel.cpp:935-941
void record_blit_history(mi355_aql* h, uint64_t size, uint64_t index) {
  const uint64_t queued = h->bytes_queued;
  h->bytes_queued += size;
  h->bytes_written[index & h->queue_mask].bytes = queued;
  h->bytes_written[index & h->queue_mask].index = index;
  h->last_queued = index;
  h->anything_queued = true;
}

// amd_blit_kernel.cpp:856-861: doorbell = index of the last packet written.
void release_write_index(mi355_aql* h, uint64_t index, uint32_t num_packet) {
  hsa_signal_store_screlease(h->queue->doorbell_signal, static_cast<hsa_signal_value_t>(index + num_packet - 1));
}

void publish(void* slot, uint16_t header, uint16_t setup) {
  // body first, then the header in one atomic store (amd_blit_kernel.cpp:893-901)
  std::atomic_thread_fence(std::memory_order_release);
  __atomic_store_n(static_cast<uint32_t*>(slot), static_cast<uint32_t>(header) | (static_cast<uint32_t>(setup) << 16),
                   __ATOMIC_RELEASE);
}

// BARRIER_AND packets for the dependencies, five signals each, fences NONE
// (amd_blit_kernel.cpp:645-709).  `completion` goes on the last one.
void write_barriers(mi355_aql* h, uint64_t index, const uint64_t* deps, uint32_t num_deps, uint32_t num_packets,
                    uint64_t completion, bool barrier_bit) {
  auto* ring = static_cast<hsa_barrier_and_packet_t*>(h->queue->base_address);
  uint32_t d = 0;
  for (uint32_t p = 0; p < num_packets; ++p) {
    hsa_barrier_and_packet_t pkt;
    std::memset(&pkt, 0, sizeof(pkt));
    for (int k = 0; k < 5 && d < num_deps; ++k, ++d) pkt.dep_signal[k].handle = deps[d];
    if (p + 1 == num_packets) pkt.completion_signal.handle = completion;
    hsa_barrier_and_packet_t* slot = &ring[(index + p) & h->queue_mask];
    std::memcpy(reinterpret_cast<uint8_t*>(slot) + 4, reinterpret_cast<uint8_t*>(&pkt) + 4, sizeof(pkt) - 4);
    uint16_t header = (HSA_PACKET_TYPE_BARRIER_AND << HSA_PACKET_HEADER_TYPE) |
                      (HSA_FENCE_SCOPE_NONE << HSA_PACKET_HEADER_SCACQUIRE_FENCE_SCOPE) |
                      (HSA_FENCE_SCOPE_NONE << HSA_PACKET_HEADER_SCRELEASE_FENCE_SCOPE);
    if (barrier_bit) header |= 1 << HSA_PACKET_HEADER_BARRIER;
    publish(slot, header, 0);
    if (h->log_packets) log_barrier_packet(h, header, pkt, index + p);
  }
}

// One KERNEL_DISPATCH packet (amd_blit_kernel.cpp:863-924): 1-D grid, kernarg
// slot of the same index, acquire and release fences at the configured scope.
// Where a dispatch stands in a command made of several packets, each waiting
// for the one before: what one packet leaves for the next is only read on this
// GPU, so only the command's first acquire and its last release need the
// configured (system) scope and the fences between its packets are at agent
// scope (the reference's commands are one packet each, amd_blit_kernel.cpp:
// 870-873).  The caller's data is covered as for a single packet: acquired
// before the first kernel, released behind the last.
enum class Chain { kAlone, kFirst, kMiddle, kLast };

void write_dispatch(mi355_aql* h, uint64_t index, const Kernel& k, const void* args, size_t args_size,
                    uint32_t grid_wgs, uint32_t wg_size, uint64_t completion, bool barrier_bit,
                    Chain chain = Chain::kAlone) {
  const bool host_slot = h->kernargs_host != nullptr && grid_wgs <= kHostKernargMaxWorkgroups;
  uint8_t* karg = (host_slot ? h->kernargs_host : h->kernargs) + (index & h->queue_mask) * kKernargSlotBytes;
  std::memcpy(karg, args, args_size);
  if (h->kernargs_in_device_memory && !host_slot) {
    // Writes across the bus are posted: order them, then read one back so
    // that they have landed before the doorbell lets a wave read them (the
    // reference fences its packet writes the same way when the ring is in
    // device memory, amd_blit_kernel.cpp:896-899).
    _mm_sfence();
    (void)*reinterpret_cast<volatile uint32_t*>(karg + ((args_size - 1) & ~size_t(3)));
  }
  hsa_kernel_dispatch_packet_t pkt;
  std::memset(&pkt, 0, sizeof(pkt));
  pkt.workgroup_size_x = static_cast<uint16_t>(wg_size);
  pkt.workgroup_size_y = pkt.workgroup_size_z = 1;
  pkt.grid_size_x = grid_wgs * wg_size;
  pkt.grid_size_y = pkt.grid_size_z = 1;
  pkt.private_segment_size = k.private_size;
  pkt.group_segment_size = k.group_size;
  pkt.kernel_object = k.object;
  pkt.kernarg_address = karg;
  pkt.completion_signal.handle = completion;
  auto* ring = static_cast<hsa_kernel_dispatch_packet_t*>(h->queue->base_address);
  hsa_kernel_dispatch_packet_t* slot = &ring[index & h->queue_mask];
  std::memcpy(reinterpret_cast<uint8_t*>(slot) + 4, reinterpret_cast<uint8_t*>(&pkt) + 4, sizeof(pkt) - 4);
  const uint16_t outer = h->fence_scope, inner = HSA_FENCE_SCOPE_AGENT;
  const uint16_t acquire = (chain == Chain::kAlone || chain == Chain::kFirst) ? outer : inner;
  const uint16_t release = (chain == Chain::kAlone || chain == Chain::kLast) ? outer : inner;
  uint16_t header = (HSA_PACKET_TYPE_KERNEL_DISPATCH << HSA_PACKET_HEADER_TYPE) |
                    (acquire << HSA_PACKET_HEADER_SCACQUIRE_FENCE_SCOPE) |
                    (release << HSA_PACKET_HEADER_SCRELEASE_FENCE_SCOPE);
  if (barrier_bit) header |= 1 << HSA_PACKET_HEADER_BARRIER;
  publish(slot, header, 1 << HSA_KERNEL_DISPATCH_PACKET_SETUP_DIMENSIONS);
  if (h->log_packets) log_dispatch_packet(h, header, 1 << HSA_KERNEL_DISPATCH_PACKET_SETUP_DIMENSIONS, pkt, index);
}

uint32_t barrier_packets(uint32_t num_deps) { return (num_deps + 4) / 5; }

// Whether a transfer's dispatch packet carries the barrier bit although no
// dependency asks for it.  The reference leaves the bit clear on every blit
// (amd_blit_kernel.cpp:870-882): consecutive blits may overlap, which hides
// the launch latency of small ones.  Large ones lose by it: while one transfer
// drains, the next one's waves start on another stretch of memory and the two
// streams disturb each other in DRAM (back-to-back 1 GiB copies: 334 us apiece
// overlapping, 317 us one after the other, the gap between them included).  So
// transfers that stream past the caches wait for the queue to drain; that is a
// stronger order than the interface promises, never a weaker one.
// On a queue the engine borrowed the reference's packet format is kept (bit
// clear): with the bit set a large blit would also wait for every earlier
// packet of the queue's other producers.  mi355_aql_set_large_transfer_barrier
// overrides either default.
constexpr uint64_t kSerialiseMinBytes = 4ull << 20;
bool serialise(const mi355_aql* h, uint64_t bytes) { return h->serialise_large.load() && bytes >= kSerialiseMinBytes; }

void free_device(void* p) {
  if (p) (void)hsa_amd_memory_pool_free(p);
}

int alloc(mi355_aql* h, hsa_amd_memory_pool_t pool, size_t bytes, void** out, bool host) {
  AQL_HSA(hsa_amd_memory_pool_allocate(pool, bytes, 0, out));
  if (host) {
    hsa_status_t s = hsa_amd_agents_allow_access(1, &h->gpu, nullptr, *out);
    if (s != HSA_STATUS_SUCCESS) {
      (void)hsa_amd_memory_pool_free(*out);
      *out = nullptr;
      return to_status(s);
    }
  }
  return MI355_BLIT_SUCCESS;
}

// One staging buffer of the batched path: device memory the host can write
// when the kernarg ring found that to work, host memory the GPU can read
// otherwise.
int alloc_stage(mi355_aql* h, size_t bytes, int i) {
  h->stage[i] = nullptr;
  h->stage_in_device_memory[i] = false;
  if (h->kernargs_in_device_memory) {
    void* p = nullptr;
    if (hsa_amd_memory_pool_allocate(h->local_pool, bytes, 0, &p) == HSA_STATUS_SUCCESS) {
      if (hsa_amd_agents_allow_access(1, &h->cpu, nullptr, p) == HSA_STATUS_SUCCESS) {
        h->stage[i] = static_cast<BatchDesc*>(p);
        h->stage_in_device_memory[i] = true;
        return MI355_BLIT_SUCCESS;
      }
      (void)hsa_amd_memory_pool_free(p);
    }
  }
  return alloc(h, h->host_pool, bytes, reinterpret_cast<void**>(&h->stage[i]), true);
}

int wait_idle_locked(mi355_aql* h) {
  hsa_signal_store_relaxed(h->idle_signal, 1);
  uint64_t index;
  {
    std::lock_guard<std::mutex> r(h->reservation_lock);
    if (!acquire_write_index(h, 1, &index)) {
      hsa_signal_store_relaxed(h->idle_signal, 0);
      return MI355_BLIT_ERROR;
    }
    record_blit_history(h, 0, index);
  }
  write_barriers(h, index, nullptr, 0, 1, h->idle_signal.handle, true);
  release_write_index(h, index, 1);
  if (wait_signal(h, h->idle_signal) != MI355_BLIT_SUCCESS) return MI355_BLIT_ERROR;
  // the barrier had its barrier bit set: everything up to it has completed
  uint64_t seen = h->known_complete.load();
  while (seen < index + 1 && !h->known_complete.compare_exchange_weak(seen, index + 1)) {
  }
  return h->queue_error.load() ? MI355_BLIT_ERROR : MI355_BLIT_SUCCESS;
}

int ensure_batch_capacity(mi355_aql* h, size_t n, size_t n_records) {
  if (n <= h->batch_capacity && n_records <= h->records_capacity) return MI355_BLIT_SUCCESS;
  // buffers may be in use by a batch in flight
  int rc = wait_idle_locked(h);
  if (rc != MI355_BLIT_SUCCESS) return rc;
  if (n > h->batch_capacity) {
    size_t cap = h->batch_capacity ? h->batch_capacity : 1024;
    while (cap < n) cap *= 2;
    for (int i = 0; i < 2; ++i) {
      free_device(h->stage[i]);
      h->stage[i] = nullptr;
    }
    free_device(h->chunk_start_dev);
    free_device(h->block_sum_dev);
    free_device(h->descs_private_dev);
    h->chunk_start_dev = nullptr;
    h->block_sum_dev = nullptr;
    h->descs_private_dev = nullptr;
    h->batch_capacity = 0;
    for (int i = 0; i < 2; ++i) {
      if ((rc = alloc_stage(h, batch_stage_bytes(cap), i)) != MI355_BLIT_SUCCESS) return rc;
      hsa_signal_store_relaxed(h->stage_free[i], 0);
    }
    if ((rc = alloc(h, h->local_pool, (cap + 1) * sizeof(uint32_t), reinterpret_cast<void**>(&h->chunk_start_dev), false)))
      return rc;
    if ((rc = alloc(h, h->local_pool, (cap / 1024 + 1) * sizeof(uint32_t), reinterpret_cast<void**>(&h->block_sum_dev), false)))
      return rc;
    if ((rc = alloc(h, h->local_pool, cap * sizeof(BatchDesc), reinterpret_cast<void**>(&h->descs_private_dev), false)))
      return rc;
    h->batch_capacity = cap;
  }
  if (n_records > h->records_capacity) {
    size_t cap = h->records_capacity ? h->records_capacity : 65536;
    while (cap < n_records) cap *= 2;
    free_device(h->records_dev);
    h->records_dev = nullptr;
    h->records_capacity = 0;
    if ((rc = alloc(h, h->local_pool, cap * sizeof(ChunkRecord), reinterpret_cast<void**>(&h->records_dev), false))) return rc;
    h->records_capacity = cap;
  }
  return MI355_BLIT_SUCCESS;
}

const Kernel* find_copy(mi355_aql* h, const mi355_blit_plan_t& p) {
  for (const auto& v : h->code->copy_kernels)
    if (v.unroll == p.unroll && v.nt_load == p.nt_load && v.store == p.store_policy &&
        v.realign == (p.byte_shift ? 1u : 0u))
      return &v.k;
  return nullptr;
}

const Kernel* find_batch(mi355_aql* h, const BatchLaunch& l, const mi355_blit_plan_t& p) {
  for (const auto& v : h->code->batch_kernels)
    if (v.split == l.split && v.nt_load == p.nt_load && v.store == p.store_policy) return &v.k;
  return nullptr;
}

}  // namespace

extern "C" {

namespace {

// Everything an engine needs beyond its GPU agent and its queue, which the
// caller has put into *h: pools, the code object, the kernarg ring and the
// ledger (both sized by the queue), the signals of its own waits.
int init_engine(mi355_aql* h) {
  int rc = MI355_BLIT_SUCCESS;
  if (hsa_iterate_agents(find_agents_cb, h) != HSA_STATUS_SUCCESS || !h->have_cpu) return MI355_BLIT_ERROR;
  if (!h->have_gpu) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  std::pair<mi355_aql*, bool> ctx{h, false};
  hsa_amd_agent_iterate_memory_pools(h->cpu, find_pools_cb, &ctx);
  ctx.second = true;
  hsa_amd_agent_iterate_memory_pools(h->gpu, find_pools_cb, &ctx);
  if (!h->have_kernarg || !h->have_host || !h->have_local) return MI355_BLIT_ERROR;
  if (hsa_agent_get_info(h->gpu, static_cast<hsa_agent_info_t>(HSA_AMD_AGENT_INFO_COMPUTE_UNIT_COUNT), &h->num_cus) !=
          HSA_STATUS_SUCCESS || h->num_cus == 0)
    return MI355_BLIT_ERROR;
  uint64_t freq = 0;
  if (hsa_system_get_info(HSA_SYSTEM_INFO_TIMESTAMP_FREQUENCY, &freq) == HSA_STATUS_SUCCESS && freq >= 1000)
    h->wait_slice_ticks = freq / 1000;
  h->log_packets = env_is_one("MI355_BLIT_LOG_PKTS");
  if ((rc = code_object_acquire(h->gpu, &h->code)) != MI355_BLIT_SUCCESS) return rc;
  if (!h->queue) {
    hsa_status_t st = hsa_queue_create(h->gpu, kQueuePackets, HSA_QUEUE_TYPE_MULTI, queue_error_cb, h, UINT32_MAX,
                                       UINT32_MAX, &h->queue);
    if (st != HSA_STATUS_SUCCESS) return to_status(st);
    h->owns_queue = true;
    h->serialise_large.store(true);
  }
  // amd_blit_kernel.cpp:554-569: the ledger and the kernarg ring have one
  // entry per packet slot of the queue, whoever made it
  h->queue_mask = h->queue->size - 1;
  h->bytes_written.assign(h->queue->size, BytesWritten{~0ull, ~0ull});
  void* ka = nullptr;
  hsa_amd_memory_pool_access_t host_access = HSA_AMD_MEMORY_POOL_ACCESS_NEVER_ALLOWED;
  hsa_amd_agent_memory_pool_get_info(h->cpu, h->local_pool, HSA_AMD_AGENT_MEMORY_POOL_INFO_ACCESS, &host_access);
  if (host_access != HSA_AMD_MEMORY_POOL_ACCESS_NEVER_ALLOWED && !force_host_kernargs() &&
      hsa_amd_memory_pool_allocate(h->local_pool, h->queue->size * kKernargSlotBytes, 0, &ka) == HSA_STATUS_SUCCESS) {
    if (hsa_amd_agents_allow_access(1, &h->cpu, nullptr, ka) == HSA_STATUS_SUCCESS) {
      h->kernargs_in_device_memory = true;
    } else {
      (void)hsa_amd_memory_pool_free(ka);
      ka = nullptr;
    }
  }
  if (!ka && (rc = alloc(h, h->kernarg_pool, h->queue->size * kKernargSlotBytes, &ka, true)) != MI355_BLIT_SUCCESS)
    return rc;
  h->kernargs = static_cast<uint8_t*>(ka);
  if (h->kernargs_in_device_memory && !env_is_one("MI355_BLIT_DEVICE_KERNARGS_ONLY")) {
    void* kh = nullptr;
    if ((rc = alloc(h, h->kernarg_pool, h->queue->size * kKernargSlotBytes, &kh, true)) != MI355_BLIT_SUCCESS) return rc;
    h->kernargs_host = static_cast<uint8_t*>(kh);
  }
  if (hsa_signal_create(1, 0, nullptr, &h->idle_signal) != HSA_STATUS_SUCCESS) return MI355_BLIT_ERROR_OUT_OF_RESOURCES;
  if (hsa_signal_create(1, 0, nullptr, &h->sync_signal) != HSA_STATUS_SUCCESS) return MI355_BLIT_ERROR_OUT_OF_RESOURCES;
  for (int i = 0; i < 2; ++i)
    if (hsa_signal_create(0, 0, nullptr, &h->stage_free[i]) != HSA_STATUS_SUCCESS) return MI355_BLIT_ERROR_OUT_OF_RESOURCES;
  return MI355_BLIT_SUCCESS;
}

}  // namespace

int mi355_aql_create(int gpu_ordinal, mi355_aql_t** out) {
  if (!out || gpu_ordinal < 0) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  *out = nullptr;
  hsa_status_t st = hsa_init();
  if (st != HSA_STATUS_SUCCESS) return MI355_BLIT_ERROR_NOT_INITIALIZED;
  mi355_aql* h = new (std::nothrow) mi355_aql;
  if (!h) {
    hsa_shut_down();
    return MI355_BLIT_ERROR_OUT_OF_RESOURCES;
  }
  h->owns_runtime = true;
  h->wanted_ordinal = gpu_ordinal;
  const int rc = init_engine(h);
  if (rc != MI355_BLIT_SUCCESS) {
    mi355_aql_destroy(h);
    return rc;
  }
  *out = h;
  return MI355_BLIT_SUCCESS;
}

int mi355_aql_create_on(uint64_t hsa_agent_handle, void* hsa_queue, mi355_aql_t** out) {
  if (!out) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  *out = nullptr;
  hsa_queue_t* queue = static_cast<hsa_queue_t*>(hsa_queue);
  if (!hsa_agent_handle || !queue || !queue->base_address || queue->size == 0 || (queue->size & (queue->size - 1)))
    return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  hsa_agent_t gpu;
  gpu.handle = hsa_agent_handle;
  hsa_device_type_t type;
  // also what tells a runtime that is not initialised: the caller owns that
  hsa_status_t st = hsa_agent_get_info(gpu, HSA_AGENT_INFO_DEVICE, &type);
  if (st != HSA_STATUS_SUCCESS) return to_status(st);
  if (type != HSA_DEVICE_TYPE_GPU) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  mi355_aql* h = new (std::nothrow) mi355_aql;
  if (!h) return MI355_BLIT_ERROR_OUT_OF_RESOURCES;
  h->gpu = gpu;
  h->have_gpu = true;
  h->wanted_ordinal = -1;  // the agent walk only looks for the host's agent
  h->queue = queue;
  const int rc = init_engine(h);
  if (rc != MI355_BLIT_SUCCESS) {
    mi355_aql_destroy(h);
    return rc;
  }
  *out = h;
  return MI355_BLIT_SUCCESS;
}

int mi355_aql_destroy(mi355_aql_t* h) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  int rc = MI355_BLIT_SUCCESS;
  const bool owns_runtime = h->owns_runtime;
  {
    std::lock_guard<std::mutex> g(h->lock);
    // The kernarg ring and the batch buffers go away below: everything this
    // engine has queued must have run.  On a borrowed queue the barrier also
    // waits for what other producers queued before it.
    if (h->queue && h->idle_signal.handle && !h->queue_error.load()) rc = wait_idle_locked(h);
    if (h->queue && h->owns_queue) hsa_queue_destroy(h->queue);
    h->queue = nullptr;
    free_device(h->kernargs);
    free_device(h->kernargs_host);
    for (int i = 0; i < 2; ++i) {
      free_device(h->stage[i]);
      if (h->stage_free[i].handle) hsa_signal_destroy(h->stage_free[i]);
    }
    free_device(h->chunk_start_dev);
    free_device(h->block_sum_dev);
    free_device(h->descs_private_dev);
    free_device(h->records_dev);
    free_device(h->batch_seen);
    free_device(h->bounce[0]);
    free_device(h->bounce[1]);
    if (h->idle_signal.handle) hsa_signal_destroy(h->idle_signal);
    if (h->sync_signal.handle) hsa_signal_destroy(h->sync_signal);
    if (h->code) code_object_release(h->code);
    h->code = nullptr;
  }
  delete h;
  if (owns_runtime) hsa_shut_down();
  return rc;
}

int mi355_aql_code_object_acquire(uint64_t hsa_agent_handle, mi355_aql_code_object_t** out) {
  if (!out || !hsa_agent_handle) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  *out = nullptr;
  hsa_agent_t gpu;
  gpu.handle = hsa_agent_handle;
  hsa_device_type_t type;
  hsa_status_t st = hsa_agent_get_info(gpu, HSA_AGENT_INFO_DEVICE, &type);
  if (st != HSA_STATUS_SUCCESS) return to_status(st);
  if (type != HSA_DEVICE_TYPE_GPU) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  return code_object_acquire(gpu, out);
}

int mi355_aql_code_object_release(mi355_aql_code_object_t* code) {
  if (!code) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  return code_object_release(code);
}

int mi355_aql_code_object_info(mi355_aql_t* h, uint64_t* executable_handle, uint32_t* users) {
  if (!h || !h->code) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> g(g_code_objects_lock);
  if (executable_handle) *executable_handle = h->code->exe.handle;
  if (users) *users = h->code->users;
  return MI355_BLIT_SUCCESS;
}

int mi355_aql_report_queue_error(mi355_aql_t* h, int status) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (status != MI355_BLIT_SUCCESS) h->queue_error.store(true, std::memory_order_release);
  return MI355_BLIT_SUCCESS;
}

int mi355_aql_wait_signal(mi355_aql_t* h, uint64_t signal) {
  if (!h || !signal) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  hsa_signal_t s;
  s.handle = signal;
  return wait_signal(h, s);
}

int mi355_aql_num_cus(mi355_aql_t* h) { return h ? static_cast<int>(h->num_cus) : 0; }

uint64_t mi355_aql_gpu_agent(mi355_aql_t* h) { return h ? h->gpu.handle : 0; }

int mi355_aql_staging(mi355_aql_t* h, size_t* half_bytes, void** half0, void** half1) {
  if (!h || !half_bytes || !half0 || !half1) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  constexpr size_t kHalf = 4u << 20;
  std::lock_guard<std::mutex> g(h->lock);
  for (int i = 0; i < 2; ++i) {
    if (!h->bounce[i]) {
      int rc = alloc(h, h->host_pool, kHalf, &h->bounce[i], true);
      if (rc != MI355_BLIT_SUCCESS) return rc;
    }
  }
  *half_bytes = kHalf;
  *half0 = h->bounce[0];
  *half1 = h->bounce[1];
  return MI355_BLIT_SUCCESS;
}

int mi355_aql_set_tuning(mi355_aql_t* h, const mi355_blit_tuning_t* tuning) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> g(h->lock);
  h->has_tuning = tuning != nullptr;
  if (tuning) h->tuning = *tuning;
  return MI355_BLIT_SUCCESS;
}

int mi355_aql_last_launch_info(mi355_aql_t* h, mi355_blit_plan_t* out) {
  if (!h || !out) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> g(h->lock);
  *out = h->last_plan;
  out->reference_engine = h->reference_engine;
  return MI355_BLIT_SUCCESS;
}

int mi355_aql_note_reference_engine(mi355_aql_t* h, uint32_t engine) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> g(h->lock);
  h->reference_engine = engine;
  return MI355_BLIT_SUCCESS;
}

int mi355_aql_set_system_scope_fences(mi355_aql_t* h, int enable) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> g(h->lock);
  h->fence_scope = enable ? HSA_FENCE_SCOPE_SYSTEM : HSA_FENCE_SCOPE_AGENT;
  return MI355_BLIT_SUCCESS;
}

int mi355_aql_set_large_transfer_barrier(mi355_aql_t* h, int enable) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  h->serialise_large.store(enable != 0);
  return MI355_BLIT_SUCCESS;
}

int mi355_aql_enable_profiling(mi355_aql_t* h, int enable) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  AQL_HSA(hsa_amd_profiling_set_profiler_enabled(h->queue, enable ? 1 : 0));
  h->profiling.store(enable != 0);
  return MI355_BLIT_SUCCESS;
}

int mi355_aql_get_command_time(mi355_aql_t* h, uint64_t completion_signal, uint64_t* start_ticks,
                               uint64_t* end_ticks, uint64_t* ticks_per_second) {
  if (!h || !completion_signal || !start_ticks || !end_ticks) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  hsa_signal_t s;
  s.handle = completion_signal;
  hsa_amd_profiling_dispatch_time_t t{0, 0};
  AQL_HSA(hsa_amd_profiling_get_dispatch_time(h->gpu, s, &t));
  *start_ticks = t.start;
  *end_ticks = t.end;
  if (ticks_per_second) AQL_HSA(hsa_system_get_info(HSA_SYSTEM_INFO_TIMESTAMP_FREQUENCY, ticks_per_second));
  return MI355_BLIT_SUCCESS;
}

int mi355_aql_copy(mi355_aql_t* h, void* dst, const void* src, size_t bytes, const uint64_t* dep_signals,
                   uint32_t num_deps, uint64_t completion_signal) {
  return mi355_aql_copy_route(h, dst, src, bytes, MI355_BLIT_ROUTE_DEVICE, dep_signals, num_deps, completion_signal);
}

int mi355_aql_copy_route(mi355_aql_t* h, void* dst, const void* src, size_t bytes, uint32_t route,
                         const uint64_t* dep_signals, uint32_t num_deps, uint64_t completion_signal) {
  if (!h || !dst || !src || (num_deps && !dep_signals) || route > MI355_BLIT_ROUTE_DEVICE_TO_HOST)
    return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (h->queue_error.load()) return MI355_BLIT_ERROR;
  const uint32_t nb = barrier_packets(num_deps);
  // One dispatch, or several for a copy of several GiB (copy_pieces) where the
  // engine shapes large transfers (its own queue, or asked to): every piece after
  // the first carries the barrier bit, which is the point of cutting.
  struct Piece {
    mi355_blit_plan_t p;
    const Kernel* k;
    CopyArgs a;
  };
  Piece piece[kCopyMaxPieces];
  uint32_t pieces = 0;
  {
    std::lock_guard<std::mutex> g(h->lock);
    if (bytes) {
      const uint32_t room = h->queue->size / 2 > nb ? h->queue->size / 2 - nb : 1;
      uint64_t piece_bytes;
      const bool cut = h->serialise_large.load() && !h->profiling.load();
      pieces = copy_pieces(bytes, route, cut ? room : 1, h->has_tuning ? &h->tuning : nullptr, &piece_bytes);
      for (uint32_t i = 0; i < pieces; ++i) {
        const uint64_t off = i * piece_bytes;
        const uint64_t n = bytes - off < piece_bytes ? bytes - off : piece_bytes;
        uint8_t* d = static_cast<uint8_t*>(dst) + off;
        const uint8_t* s = static_cast<const uint8_t*>(src) + off;
        Piece& q = piece[i];
        int rc = plan_copy(reinterpret_cast<uint64_t>(d), reinterpret_cast<uint64_t>(s), n, h->num_cus,
                           h->has_tuning ? &h->tuning : nullptr, &q.p, route);
        if (rc != MI355_BLIT_SUCCESS) return rc;
        q.k = find_copy(h, q.p);
        if (!q.k) return MI355_BLIT_ERROR;
        q.a = make_copy_args(q.p, d, s, n);
      }
      h->last_plan = piece[pieces - 1].p;
      h->last_plan.pieces = pieces;
    }
  }
  if (bytes == 0) {
    // nothing to move: the dependencies and the completion ride on barriers
    const uint32_t n = nb ? nb : 1;
    if (!num_deps && !completion_signal) return MI355_BLIT_SUCCESS;
    uint64_t index;
    {
      std::lock_guard<std::mutex> r(h->reservation_lock);
      if (!acquire_write_index(h, n, &index)) return MI355_BLIT_ERROR;
      record_blit_history(h, 0, index + n - 1);
    }
    write_barriers(h, index, dep_signals, num_deps, n, completion_signal, false);
    release_write_index(h, index, n);
    return MI355_BLIT_SUCCESS;
  }
  const uint32_t total = nb + pieces;
  uint64_t index;
  {
    std::lock_guard<std::mutex> r(h->reservation_lock);
    if (!acquire_write_index(h, total, &index)) return MI355_BLIT_ERROR;
    record_blit_history(h, bytes, index + total - 1);
  }
  write_barriers(h, index, dep_signals, num_deps, nb, 0, false);
  // Barrier bit clear, as in the reference: consecutive blits may overlap
  // unless linked by signals.  After dependency barriers the bit is set so
  // that the copy cannot start before them.  The completion signal goes on the
  // last piece, which the barrier bit orders behind the others.
  for (uint32_t i = 0; i < pieces; ++i) {
    const Piece& q = piece[i];
    const Chain chain = pieces == 1 ? Chain::kAlone
                        : i == 0 ? Chain::kFirst
                        : i + 1 == pieces ? Chain::kLast
                                          : Chain::kMiddle;
    write_dispatch(h, index + nb + i, *q.k, &q.a, sizeof(q.a), q.p.grid, q.p.wg_size,
                   i + 1 == pieces ? completion_signal : 0, i != 0 || nb != 0 || serialise(h, bytes), chain);
  }
  release_write_index(h, index, total);
  return MI355_BLIT_SUCCESS;
}

int mi355_aql_fill32(mi355_aql_t* h, void* ptr, uint32_t value, size_t num_dwords, const uint64_t* dep_signals,
                     uint32_t num_deps, uint64_t completion_signal) {
  if (!h || !ptr || (reinterpret_cast<uintptr_t>(ptr) & 3) || (num_deps && !dep_signals))
    return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (h->queue_error.load()) return MI355_BLIT_ERROR;
  if (num_dwords == 0) {
    // same as a zero-size copy: only the signals matter
    return mi355_aql_copy(h, ptr, ptr, 0, dep_signals, num_deps, completion_signal);
  }
  mi355_blit_plan_t p;
  const Kernel* k = nullptr;
  {
    std::lock_guard<std::mutex> g(h->lock);
    int rc = plan_fill(reinterpret_cast<uint64_t>(ptr), num_dwords, h->num_cus, h->has_tuning ? &h->tuning : nullptr, &p);
    if (rc != MI355_BLIT_SUCCESS) return rc;
    for (const auto& v : h->code->fill_kernels)
      if (v.unroll == p.unroll && v.store == p.store_policy) k = &v.k;
    if (!k) return MI355_BLIT_ERROR;
    h->last_plan = p;
  }
  const FillArgs a = make_fill_args(p, ptr, value, num_dwords);
  const uint32_t nb = barrier_packets(num_deps);
  const uint32_t total = nb + 1;
  uint64_t index;
  {
    std::lock_guard<std::mutex> r(h->reservation_lock);
    if (!acquire_write_index(h, total, &index)) return MI355_BLIT_ERROR;
    record_blit_history(h, num_dwords * 4, index + total - 1);
  }
  write_barriers(h, index, dep_signals, num_deps, nb, 0, false);
  write_dispatch(h, index + nb, *k, &a, sizeof(a), p.grid, p.wg_size, completion_signal, nb != 0 || serialise(h, num_dwords * 4));
  release_write_index(h, index, total);
  return MI355_BLIT_SUCCESS;
}

namespace {
int copy_batch_device_locked(mi355_aql_t* h, const BatchDesc* scanned, size_t n, uint64_t max_total_bytes,
                             uint64_t likely_chunks, uint64_t staged_free, const uint64_t* dep_signals,
                             uint32_t num_deps, uint64_t completion_signal);
}

int mi355_aql_copy_batch(mi355_aql_t* h, const mi355_blit_desc_t* descs, size_t n, const uint64_t* dep_signals,
                         uint32_t num_deps, uint64_t completion_signal) {
  if (!h || (!descs && n) || (num_deps && !dep_signals)) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (n > 0xffffffffull) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (h->queue_error.load()) return MI355_BLIT_ERROR;
  std::unique_lock<std::mutex> g(h->lock);
  // The packet processor publishes the read index with a delay: a batch that
  // has just finished may still count as running, which only means that the
  // host walks the descriptors as it would have anyway.
  // Idle means nothing of this engine is in flight, batch or not: behind a
  // running 1 GiB copy the walk is hidden just as it is behind a batch.
  auto engine_idle = [h]() {
    uint64_t last;
    {
      std::lock_guard<std::mutex> r(h->reservation_lock);
      if (!h->anything_queued) return true;
      last = h->last_queued;
    }
    return hsa_queue_load_read_index_scacquire(h->queue) > last || h->known_complete.load() > last;
  };
  if (batch_prefers_raw_staging(descs, n, engine_idle, h->has_tuning ? &h->tuning : nullptr)) {
    // The walk below would take longer than the copies: stage the descriptors
    // as they are and take them from there like device-resident ones.
    int rc = ensure_batch_capacity(h, n, 0);
    if (rc != MI355_BLIT_SUCCESS) return rc;
    const unsigned b = h->next_stage;
    if (wait_signal(h, h->stage_free[b]) != MI355_BLIT_SUCCESS) return MI355_BLIT_ERROR;
    uint64_t total_bytes = 0, likely_chunks = 0;
    rc = batch_stage_raw(descs, n, h->stage[b], &total_bytes, &likely_chunks);
    if (rc != MI355_BLIT_SUCCESS) return rc;
    if (total_bytes == 0) {
      g.unlock();
      return mi355_aql_copy(h, h, h, 0, dep_signals, num_deps, completion_signal);
    }
    if (h->stage_in_device_memory[b]) {
      _mm_sfence();
      (void)*(reinterpret_cast<volatile uint32_t*>(h->stage[b] + n) - 1);
    }
    h->next_stage ^= 1;
    hsa_signal_store_relaxed(h->stage_free[b], 1);
    // the bytes are known exactly: they size the launch as a caller's bound would
    rc = copy_batch_device_locked(h, h->stage[b], n, total_bytes, likely_chunks, h->stage_free[b].handle, dep_signals,
                                  num_deps, completion_signal);
    if (rc != MI355_BLIT_SUCCESS) hsa_signal_store_relaxed(h->stage_free[b], 0);
    return rc;
  }
  BatchShape shape;
  int rc = batch_build(descs, n, &h->stage_image, &shape);
  if (rc != MI355_BLIT_SUCCESS) return rc;
  const uint64_t total_bytes = shape.total_bytes, total_chunks = shape.total_chunks;
  if (total_chunks == 0) {
    g.unlock();
    return mi355_aql_copy(h, h, h, 0, dep_signals, num_deps, completion_signal);
  }
  rc = ensure_batch_capacity(h, shape.pieces, total_chunks);
  if (rc != MI355_BLIT_SUCCESS) return rc;
  const mi355_blit_tuning_t* t = h->has_tuning ? &h->tuning : nullptr;

  // Stage what the GPU needs: the descriptors, cut into pieces of at most
  // 64 chunks, and each piece's first record index (the host, which walks the
  // descriptors anyway, does the prefix sum).  The buffer is free again when
  // the kernel that read it last has finished.
  // The launch is planned before the staging buffer is armed, so that nothing
  // can fail between arming it and the packet that frees it again.
  mi355_blit_plan_t p;
  const BatchLaunch l = plan_batch_records(total_chunks, total_bytes, total_bytes >= (4ull << 20), t, true, &p);
  const Kernel* bk = find_batch(h, l, p);
  if (!bk) return MI355_BLIT_ERROR;
  const unsigned b = h->next_stage;
  if (wait_signal(h, h->stage_free[b]) != MI355_BLIT_SUCCESS) return MI355_BLIT_ERROR;
  h->next_stage ^= 1;
  const size_t image_bytes = batch_stage_bytes(shape.pieces);
  batch_stage(h->stage_image, h->stage[b]);
  if (h->stage_in_device_memory[b]) {
    // posted writes across the bus: order them and read one back, as for kernargs
    _mm_sfence();
    (void)*(reinterpret_cast<volatile uint32_t*>(reinterpret_cast<uint8_t*>(h->stage[b]) + image_bytes) - 1);
  }
  hsa_signal_store_relaxed(h->stage_free[b], 1);

  // 1. the chunk records, kEmitPiecesPerWave pieces to a wave
  EmitRecordsArgs er{h->stage[b], reinterpret_cast<const uint32_t*>(h->stage[b] + shape.pieces), shape.pieces,
                     h->records_dev};

  // 2. the copy
  BatchCopyArgs bc{h->records_dev, total_chunks, nullptr, l.waves_per_wg, l.n_waves, make_xcd_runs(p.grid, p.xcd_run),
                   l.prefetch_waves, 0};
  h->last_plan = p;

  const uint32_t nb = barrier_packets(num_deps);
  const uint32_t total = nb + 2;
  uint64_t index;
  {
    std::lock_guard<std::mutex> r(h->reservation_lock);
    if (!acquire_write_index(h, total, &index)) {
      hsa_signal_store_relaxed(h->stage_free[b], 0);  // armed above; nothing will read the staging buffer
      return MI355_BLIT_ERROR;
    }
    record_blit_history(h, total_bytes, index + total - 1);
  }
  write_barriers(h, index, dep_signals, num_deps, nb, 0, false);
  uint64_t i = index + nb;
  // Both packets wait for everything before them (barrier bit): the first for
  // whatever still reads the shared record buffer; it frees the staging buffer
  // when it is done with it.
  write_dispatch(h, i++, h->code->emit_records, &er, sizeof(er), emit_records_grid(shape.pieces), 256,
                 h->stage_free[b].handle, true, Chain::kFirst);
  write_dispatch(h, i++, *bk, &bc, sizeof(bc), p.grid, p.wg_size, completion_signal, true, Chain::kLast);
  release_write_index(h, index, total);
  h->last_batch_index = index + total - 1;
  h->any_batch = true;
  return MI355_BLIT_SUCCESS;
}

namespace {
// Device-resident descriptors, with a bound on the bytes they move or without
// (max_total_bytes == 0): four packets, each waiting for the one before --
// the two launches of the prefix sum, the records, and the copy, whose grid
// and record buffer follow batch_device_sizing and which reads the number of
// chunks on the device.
// With h->lock held.  staged_free != 0: the descriptors are ones the host
// staged; the first kernel, their only reader, leaves a copy for the others
// and sets that signal to 0 when it is done.
int copy_batch_device_locked(mi355_aql_t* h, const BatchDesc* scanned, size_t n, uint64_t max_total_bytes,
                             uint64_t likely_chunks, uint64_t staged_free, const uint64_t* dep_signals,
                             uint32_t num_deps, uint64_t completion_signal) {
  int rc;
  if (!h->batch_seen) {
    // where the copy kernel leaves its numbers of copies and chunks (batch_device_sizing)
    if ((rc = alloc(h, h->host_pool, 64, reinterpret_cast<void**>(&h->batch_seen), true)) != MI355_BLIT_SUCCESS)
      return rc;
    *h->batch_seen = 0;
  }
  const BatchDeviceSizing sizing =
      batch_device_sizing(n, max_total_bytes, *static_cast<volatile uint64_t*>(h->batch_seen), likely_chunks);
  if (sizing.records == 0) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  rc = ensure_batch_capacity(h, n, sizing.records);
  if (rc != MI355_BLIT_SUCCESS) return rc;
  const mi355_blit_tuning_t* t = h->has_tuning ? &h->tuning : nullptr;
  const BatchDesc* descs = staged_free ? h->descs_private_dev : scanned;
  const uint32_t n_blocks = static_cast<uint32_t>((n + 1023) / 1024);
  ScanLocalArgs sl{scanned, static_cast<uint64_t>(n), h->chunk_start_dev, h->block_sum_dev,
                   staged_free ? h->descs_private_dev : nullptr};
  ScanTopArgs stp{h->block_sum_dev, h->chunk_start_dev, static_cast<uint64_t>(n), n_blocks};
  EmitRecordsDeviceArgs er{descs, h->chunk_start_dev, h->block_sum_dev, static_cast<uint64_t>(n), h->records_dev,
                           sizing.records};

  // the lengths are only known on the device: a large batch, in the fixed shape
  mi355_blit_plan_t p;
  const BatchLaunch l = plan_batch_records(sizing.grid_chunks, sizing.bytes, true, t, false, &p);
  const Kernel* bk = nullptr;
  for (const auto& v : h->code->batch_lookup_kernels)
    if (v.nt_load == p.nt_load && v.store == p.store_policy) bk = &v.k;
  if (!bk || l.split != 4) return MI355_BLIT_ERROR;
  BatchLookupArgs bc{{h->records_dev, sizing.records, h->chunk_start_dev + n, l.waves_per_wg, l.n_waves,
                      make_xcd_runs(p.grid, p.xcd_run), l.prefetch_waves, 0},
                     descs, h->chunk_start_dev, h->block_sum_dev, static_cast<uint64_t>(n), h->batch_seen};
  h->last_plan = p;

  const uint32_t nb = barrier_packets(num_deps);
  const uint32_t total = nb + 4;
  uint64_t index;
  {
    std::lock_guard<std::mutex> r(h->reservation_lock);
    // (a caller that armed staged_free takes it back when this fails)
    if (!acquire_write_index(h, total, &index)) return MI355_BLIT_ERROR;
    // without a bound the lengths are unknown here: keep the record non-zero
    record_blit_history(h, max_total_bytes ? max_total_bytes : n, index + total - 1);
  }
  write_barriers(h, index, dep_signals, num_deps, nb, 0, false);
  uint64_t i = index + nb;
  // every packet waits for the one before; the first also for whatever still uses the shared buffers
  write_dispatch(h, i++, h->code->scan_local, &sl, sizeof(sl), n_blocks, 1024, staged_free, true, Chain::kFirst);
  write_dispatch(h, i++, h->code->scan_top, &stp, sizeof(stp), 1, 1024, 0, true, Chain::kMiddle);
  write_dispatch(h, i++, h->code->emit_records_lookup, &er, sizeof(er),
                 static_cast<uint32_t>((sizing.records + 255) / 256), 256, 0, true, Chain::kMiddle);
  write_dispatch(h, i++, *bk, &bc, sizeof(bc), p.grid, p.wg_size, completion_signal, true, Chain::kLast);
  release_write_index(h, index, total);
  h->last_batch_index = index + total - 1;
  h->any_batch = true;
  return MI355_BLIT_SUCCESS;
}

int copy_batch_device(mi355_aql_t* h, const mi355_blit_desc_t* device_descs, size_t n, uint64_t max_total_bytes,
                      const uint64_t* dep_signals, uint32_t num_deps, uint64_t completion_signal) {
  if (!h || (!device_descs && n) || (num_deps && !dep_signals)) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (n > 0xffffffffull) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (h->queue_error.load()) return MI355_BLIT_ERROR;
  if (n == 0) return mi355_aql_copy(h, h, h, 0, dep_signals, num_deps, completion_signal);
  std::lock_guard<std::mutex> g(h->lock);
  return copy_batch_device_locked(h, reinterpret_cast<const BatchDesc*>(device_descs), n, max_total_bytes, 0, 0,
                                  dep_signals, num_deps, completion_signal);
}
}  // namespace

int mi355_aql_copy_batch_device(mi355_aql_t* h, const mi355_blit_desc_t* device_descs, size_t n,
                                const uint64_t* dep_signals, uint32_t num_deps, uint64_t completion_signal) {
  return copy_batch_device(h, device_descs, n, 0, dep_signals, num_deps, completion_signal);
}

int mi355_aql_copy_batch_bounded(mi355_aql_t* h, const mi355_blit_desc_t* device_descs, size_t n,
                                 uint64_t max_total_bytes, const uint64_t* dep_signals, uint32_t num_deps,
                                 uint64_t completion_signal) {
  if (max_total_bytes == 0 && n != 0) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  return copy_batch_device(h, device_descs, n, max_total_bytes, dep_signals, num_deps, completion_signal);
}

int mi355_aql_copy_rect(mi355_aql_t* h, const mi355_pitched_ptr_t* dst, const mi355_dim3_t* dst_offset,
                        const mi355_pitched_ptr_t* src, const mi355_dim3_t* src_offset,
                        const mi355_dim3_t* range, const uint64_t* dep_signals, uint32_t num_deps,
                        uint64_t completion_signal) {
  return mi355_aql_copy_rect_route(h, dst, dst_offset, src, src_offset, range, MI355_BLIT_ROUTE_DEVICE, dep_signals,
                                   num_deps, completion_signal);
}

int mi355_aql_copy_rect_route(mi355_aql_t* h, const mi355_pitched_ptr_t* dst, const mi355_dim3_t* dst_offset,
                              const mi355_pitched_ptr_t* src, const mi355_dim3_t* src_offset,
                              const mi355_dim3_t* range, uint32_t route, const uint64_t* dep_signals,
                              uint32_t num_deps, uint64_t completion_signal) {
  if (!h || (num_deps && !dep_signals)) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (h->queue_error.load()) return MI355_BLIT_ERROR;
  RectPlan rp;
  const Kernel* k = nullptr;
  {
    std::lock_guard<std::mutex> g(h->lock);
    int rc = plan_rect(dst, dst_offset, src, src_offset, range, h->has_tuning ? &h->tuning : nullptr, &rp, route);
    if (rc != MI355_BLIT_SUCCESS) return rc;
    if (!rp.empty && !rp.linear) {
      if (rp.narrow) {
        for (const auto& v : h->code->rect_narrow_kernels)
          if (v.nt_load == rp.streaming && v.store == rp.store_policy) k = &v.k;
      } else {
        for (const auto& v : h->code->rect_kernels)
          if (v.unroll == rp.unroll && v.nt_load == rp.streaming && v.store == rp.store_policy) k = &v.k;
      }
      if (!k) return MI355_BLIT_ERROR;
      rect_launch_info(rp, &h->last_plan);
    }
  }
  if (rp.empty) return mi355_aql_copy(h, h, h, 0, dep_signals, num_deps, completion_signal);
  if (rp.linear)
    return mi355_aql_copy_route(h, rp.args.dst, rp.args.src, rp.args.width, route, dep_signals, num_deps,
                                completion_signal);
  const uint32_t nb = barrier_packets(num_deps);
  const uint32_t total = nb + 1;
  uint64_t index;
  {
    std::lock_guard<std::mutex> r(h->reservation_lock);
    if (!acquire_write_index(h, total, &index)) return MI355_BLIT_ERROR;
    record_blit_history(h, rp.total_bytes, index + total - 1);
  }
  write_barriers(h, index, dep_signals, num_deps, nb, 0, false);
  if (rp.narrow)
    write_dispatch(h, index + nb, *k, &rp.nargs, sizeof(rp.nargs), rp.grid, rp.wg_size, completion_signal,
                   nb != 0 || serialise(h, rp.total_bytes));
  else
    write_dispatch(h, index + nb, *k, &rp.args, sizeof(rp.args), rp.grid, rp.wg_size, completion_signal,
                   nb != 0 || serialise(h, rp.total_bytes));
  release_write_index(h, index, total);
  return MI355_BLIT_SUCCESS;
}

int mi355_aql_copy_sync(mi355_aql_t* h, void* dst, const void* src, size_t bytes, uint32_t route) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  // amd_blit_kernel.cpp:614-639: one blocking command at a time owns the signal
  std::lock_guard<std::mutex> g(h->sync_lock);
  hsa_signal_store_relaxed(h->sync_signal, 1);
  const int rc = mi355_aql_copy_route(h, dst, src, bytes, route, nullptr, 0, h->sync_signal.handle);
  if (rc != MI355_BLIT_SUCCESS) {
    hsa_signal_store_relaxed(h->sync_signal, 0);  // nothing was queued that would complete it
    return rc;
  }
  // a copy of no bytes completes the signal from a barrier packet
  return wait_signal(h, h->sync_signal);
}

int mi355_aql_fill32_sync(mi355_aql_t* h, void* ptr, uint32_t value, size_t num_dwords) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  // amd_blit_kernel.cpp:787-837
  std::lock_guard<std::mutex> g(h->sync_lock);
  hsa_signal_store_relaxed(h->sync_signal, 1);
  const int rc = mi355_aql_fill32(h, ptr, value, num_dwords, nullptr, 0, h->sync_signal.handle);
  if (rc != MI355_BLIT_SUCCESS) {
    hsa_signal_store_relaxed(h->sync_signal, 0);
    return rc;
  }
  return wait_signal(h, h->sync_signal);
}

int mi355_aql_wait_idle(mi355_aql_t* h) {
  if (!h) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> g(h->lock);
  return wait_idle_locked(h);
}

// amd_blit_kernel.cpp:943-970
uint64_t mi355_aql_pending_bytes(mi355_aql_t* h) {
  if (!h) return 0;
  std::lock_guard<std::mutex> r(h->reservation_lock);
  if (!h->anything_queued) return 0;
  uint64_t read = hsa_queue_load_read_index_relaxed(h->queue);
  const uint64_t known = h->known_complete.load();
  if (known > read) read = known;
  const uint64_t last = h->last_queued;
  // the queue has consumed the newest command's packet: nothing is pending
  if (read > last) return 0;
  for (uint64_t index = read; index <= last; ++index) {
    const BytesWritten& rec = h->bytes_written[index & h->queue_mask];
    // a record that was not overwritten by a later lap of the ring
    if (rec.index == index) {
      const uint64_t pending = h->bytes_queued - rec.bytes;
      return pending ? pending : 1;  // commands without bytes still count as work
    }
  }
  return 1;
}

}  // extern "C"
