// Native test driver for rocr::AMD::BlitKernelGfx950 (the core::Blit adapter).
// Runs on a GPU box; prints one "PASS <name>" or "FAIL <name>: why" line per
// case and exits non-zero if any case fails.  Expected bytes come from the CPU
// oracle (oracle/blit_oracle.h); the cases follow what the reference's own
// tests do with this interface through the HSA API: fill, copy, wait on the
// completion signal, compare every element
// (rocrtst/samples/async_mem_copy/async_mem_copy.cc:269-357).
#include <hip/hip_runtime_api.h>
#include <hsa/hsa.h>
#include <hsa/hsa_ext_amd.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <string>
#include <thread>
#include <vector>

#include "../../oracle/blit_oracle.h"
#include "blit_args.h"
#include "mi355_blit.h"
#include "mi355_blit_aql.h"
#include "rocr_blit.h"

using rocr::AMD::BlitKernelGfx950;
using rocr::AMD::BlitKernelGfx950Aql;
using rocr::core::Blit;
using rocr::core::Signal;

// SubmitBatchCopyCommand is not part of core::Blit; each engine supplies it.
typedef std::function<hsa_status_t(const void*, size_t, bool, uint64_t, std::vector<Signal*>&, Signal&)> BatchFn;

namespace {

int g_failures = 0;
std::string g_suffix;  // "_hip" or "_aql": which engine the cases run on
constexpr size_t kGuard = 256;
constexpr uint8_t kGuardByte = 0xEE;

#define REQUIRE(cond, ...)                         \
  do {                                             \
    if (!(cond)) {                                 \
      std::printf("FAIL %s%s: ", name, g_suffix.c_str()); \
      std::printf(__VA_ARGS__);                    \
      std::printf(" (line %d)\n", __LINE__);       \
      std::fflush(stdout);                         \
      ++g_failures;                                \
      return;                                      \
    }                                              \
  } while (0)

#define HIP_OK(expr) REQUIRE((expr) == hipSuccess, "%s failed", #expr)

struct DeviceBuf {
  uint8_t* p = nullptr;
  size_t n = 0;
  explicit DeviceBuf(size_t bytes) : n(bytes) {
    if (hipMalloc(reinterpret_cast<void**>(&p), bytes) != hipSuccess) p = nullptr;
  }
  ~DeviceBuf() {
    if (p) (void)hipFree(p);
  }
  bool upload(const std::vector<uint8_t>& h) { return hipMemcpy(p, h.data(), h.size(), hipMemcpyHostToDevice) == hipSuccess; }
  bool download(std::vector<uint8_t>& h) {
    h.resize(n);
    return hipMemcpy(h.data(), p, n, hipMemcpyDeviceToHost) == hipSuccess;
  }
};

hsa_signal_t make_signal(hsa_signal_value_t v) {
  hsa_signal_t s{0};
  if (hsa_signal_create(v, 0, nullptr, &s) != HSA_STATUS_SUCCESS) s.handle = 0;
  return s;
}

// The agent's utility queue as GpuAgent makes it (amd_gpu_agent.cpp:692-701:
// minAqlSize_ = 64 packets, HSA_QUEUE_TYPE_MULTI), with an error callback that
// forwards to whichever engine runs on the queue, as its owner would.
struct UtilityQueue {
  hsa_queue_t* q = nullptr;
  BlitKernelGfx950Aql* engine = nullptr;
  static void on_error(hsa_status_t status, hsa_queue_t*, void* data) {
    auto* self = static_cast<UtilityQueue*>(data);
    std::printf("INFO queue error 0x%x\n", status);
    if (self->engine) self->engine->ReportQueueError(status);
  }
  explicit UtilityQueue(hsa_agent_t gpu, uint32_t packets = 64) {
    if (hsa_queue_create(gpu, packets, HSA_QUEUE_TYPE_MULTI, on_error, this, UINT32_MAX, UINT32_MAX, &q) !=
        HSA_STATUS_SUCCESS)
      q = nullptr;
  }
  ~UtilityQueue() {
    if (q) hsa_queue_destroy(q);
  }
};

bool wait_zero(hsa_signal_t s, hsa_wait_state_t state, uint64_t timeout_ms = 20000) {
  // timeout in the system timestamp's units; read its frequency
  uint64_t freq = 0;
  hsa_system_get_info(HSA_SYSTEM_INFO_TIMESTAMP_FREQUENCY, &freq);
  const uint64_t ticks = freq ? freq / 1000 * timeout_ms : UINT64_MAX;
  const auto deadline = std::chrono::steady_clock::now() + std::chrono::milliseconds(timeout_ms);
  while (std::chrono::steady_clock::now() < deadline) {
    if (hsa_signal_wait_scacquire(s, HSA_SIGNAL_CONDITION_LT, 1, ticks, state) < 1) return true;
  }
  return false;
}

std::vector<uint8_t> seeded(size_t n, uint64_t seed) {
  std::vector<uint8_t> v(n);
  oracle_fill_random(v.data(), n, seed);
  return v;
}

// ---------------------------------------------------------------------------

void test_blocking_copy(Blit& blit) {
  const char* name = "blocking_copy_offsets_and_sizes";
  const size_t max_n = (3u << 20) + 77;
  std::vector<uint8_t> src_h = seeded(max_n + 64, 0xB1170003);
  DeviceBuf src(src_h.size()), dst(max_n + 2 * kGuard + 64);
  REQUIRE(src.p && dst.p, "hipMalloc");
  REQUIRE(src.upload(src_h), "upload");
  const size_t sizes[] = {1, 3, 4, 15, 16, 17, 255, 4096, 65537, (1u << 20), max_n};
  for (size_t n : sizes) {
    for (int pair = 0; pair < 4; ++pair) {
      const size_t so = (pair * 5 + 1) & 15, dof = (pair * 11 + 2) & 15;
      std::vector<uint8_t> want(dst.n, kGuardByte), got;
      REQUIRE(dst.upload(want), "upload");
      hsa_status_t st = blit.SubmitLinearCopyCommand(dst.p + kGuard + dof, src.p + so, n);
      REQUIRE(st == HSA_STATUS_SUCCESS, "status 0x%x", st);
      oracle_copy(want.data() + kGuard + dof, src_h.data() + so, n);
      REQUIRE(dst.download(got), "download");
      REQUIRE(got == want, "bytes differ n=%zu so=%zu do=%zu", n, so, dof);
    }
  }
  std::printf("PASS %s%s\n", name, g_suffix.c_str());
}

void test_blocking_fill(Blit& blit) {
  const char* name = "blocking_fill_reference_patterns";
  // rocrtst/samples/async_mem_copy/async_mem_copy.cc:62-65
  const uint32_t values[] = {0xabcdef12, 0xba5eba11, 0xfeed5a1e, 0xbaadf00d, 0xA5C30F1E};
  const size_t counts[] = {1, 3, 4, 5, 1023, 262144 + 3};
  DeviceBuf dst(4 * (262144 + 3) + 2 * kGuard + 16);
  REQUIRE(dst.p, "hipMalloc");
  for (uint32_t v : values) {
    for (size_t c : counts) {
      for (size_t off : {size_t(0), size_t(4), size_t(12)}) {
        std::vector<uint8_t> want(dst.n, kGuardByte), got;
        REQUIRE(dst.upload(want), "upload");
        hsa_status_t st = blit.SubmitLinearFillCommand(dst.p + kGuard + off, v, c);
        REQUIRE(st == HSA_STATUS_SUCCESS, "status 0x%x", st);
        oracle_fill32(want.data() + kGuard + off, v, c);
        REQUIRE(dst.download(got), "download");
        REQUIRE(got == want, "bytes differ value=%x count=%zu off=%zu", v, c, off);
      }
    }
  }
  // amd_blit_kernel.cpp:791-794: misaligned pointer -> HSA_STATUS_ERROR, nothing written
  std::vector<uint8_t> want(dst.n, kGuardByte), got;
  REQUIRE(dst.upload(want), "upload");
  for (size_t off : {size_t(1), size_t(2), size_t(3)}) {
    hsa_status_t st = blit.SubmitLinearFillCommand(dst.p + kGuard + off, 1, 4);
    REQUIRE(st == HSA_STATUS_ERROR, "misaligned fill returned 0x%x", st);
    REQUIRE(oracle_ref_blit_fill_status(reinterpret_cast<uintptr_t>(dst.p + kGuard + off)) == ORACLE_STATUS_ERROR,
            "oracle disagrees");
  }
  REQUIRE(dst.download(got), "download");
  REQUIRE(got == want, "rejected fill wrote memory");
  std::printf("PASS %s%s\n", name, g_suffix.c_str());
}

void test_async_copy_signal(Blit& blit, hsa_wait_state_t state, const char* name) {
  const size_t n = (8u << 20) + 5;
  std::vector<uint8_t> src_h = seeded(n + 16, 0xB1170002);
  DeviceBuf src(src_h.size()), dst(n + 2 * kGuard + 16);
  REQUIRE(src.p && dst.p, "hipMalloc");
  REQUIRE(src.upload(src_h), "upload");
  std::vector<uint8_t> want(dst.n, kGuardByte), got;
  REQUIRE(dst.upload(want), "upload");
  hsa_signal_t done = make_signal(1);
  REQUIRE(done.handle, "signal");
  Signal out(done);
  std::vector<Signal*> deps, gang;
  hsa_status_t st = blit.SubmitLinearCopyCommand(dst.p + kGuard + 3, src.p + 1, n, deps, out, gang);
  REQUIRE(st == HSA_STATUS_SUCCESS, "status 0x%x", st);
  REQUIRE(wait_zero(done, state), "completion signal never reached 0");
  REQUIRE(hsa_signal_load_relaxed(done) == 0, "signal value %ld", (long)hsa_signal_load_relaxed(done));
  oracle_copy(want.data() + kGuard + 3, src_h.data() + 1, n);
  REQUIRE(dst.download(got), "download");
  REQUIRE(got == want, "bytes differ");
  // the blit reports idle once everything has completed
  uint64_t pending = 1;
  for (int i = 0; i < 1000 && pending; ++i) {
    pending = blit.PendingBytes();
    if (pending) std::this_thread::sleep_for(std::chrono::milliseconds(1));
  }
  REQUIRE(pending == 0, "PendingBytes stuck at %llu", (unsigned long long)pending);
  hsa_signal_destroy(done);
  std::printf("PASS %s%s\n", name, g_suffix.c_str());
}

void test_dependencies(Blit& blit, size_t n_deps, const char* name) {
  const size_t n = (1u << 20) + 9;
  std::vector<uint8_t> src_h = seeded(n, 0xB1170004);
  DeviceBuf src(n), dst(n + 2 * kGuard);
  REQUIRE(src.p && dst.p, "hipMalloc");
  REQUIRE(src.upload(src_h), "upload");
  std::vector<uint8_t> before(dst.n, kGuardByte), got;
  REQUIRE(dst.upload(before), "upload");
  std::vector<hsa_signal_t> dep_handles;
  std::vector<Signal> dep_objs;
  for (size_t i = 0; i < n_deps; ++i) dep_handles.push_back(make_signal(1));
  for (hsa_signal_t h : dep_handles) {
    REQUIRE(h.handle, "signal");
    dep_objs.emplace_back(h);
  }
  std::vector<Signal*> deps, gang;
  for (Signal& s : dep_objs) deps.push_back(&s);
  hsa_signal_t done = make_signal(1);
  Signal out(done);
  hsa_status_t st = blit.SubmitLinearCopyCommand(dst.p + kGuard, src.p, n, deps, out, gang);
  REQUIRE(st == HSA_STATUS_SUCCESS, "status 0x%x", st);
  // a command submitted behind a blocked one must not overtake it
  hsa_signal_t done2 = make_signal(1);
  Signal out2(done2);
  std::vector<Signal*> no_deps;
  st = blit.SubmitLinearCopyCommand(dst.p + kGuard, src.p + 1, 16, no_deps, out2, gang);
  REQUIRE(st == HSA_STATUS_SUCCESS, "status 0x%x", st);
  REQUIRE(blit.PendingBytes() != 0, "PendingBytes is 0 with blocked commands");
  // satisfy all but the last dependency: nothing may run
  for (size_t i = 0; i + 1 < n_deps; ++i) hsa_signal_store_screlease(dep_handles[i], 0);
  std::this_thread::sleep_for(std::chrono::milliseconds(100));
  REQUIRE(hsa_signal_load_scacquire(done) == 1, "copy completed before its dependencies");
  REQUIRE(hsa_signal_load_scacquire(done2) == 1, "a later command overtook a blocked one");
  REQUIRE(dst.download(got), "download");
  REQUIRE(got == before, "destination written before dependencies were satisfied");
  hsa_signal_store_screlease(dep_handles[n_deps - 1], 0);
  REQUIRE(wait_zero(done, HSA_WAIT_STATE_BLOCKED), "copy never completed");
  REQUIRE(wait_zero(done2, HSA_WAIT_STATE_BLOCKED), "second copy never completed");
  std::vector<uint8_t> want(before);
  oracle_copy(want.data() + kGuard, src_h.data(), n);
  oracle_copy(want.data() + kGuard, src_h.data() + 1, 16);  // second command, in order
  REQUIRE(dst.download(got), "download");
  REQUIRE(got == want, "bytes differ");
  for (hsa_signal_t h : dep_handles) hsa_signal_destroy(h);
  hsa_signal_destroy(done);
  hsa_signal_destroy(done2);
  std::printf("PASS %s%s\n", name, g_suffix.c_str());
}

void test_chain(Blit& blit) {
  const char* name = "chain_a_to_b_to_c";
  const size_t n = (2u << 20) + 11;
  std::vector<uint8_t> a_h = seeded(n, 0xB1170005);
  DeviceBuf a(n), b(n + 32), c(n + 2 * kGuard + 32);
  REQUIRE(a.p && b.p && c.p, "hipMalloc");
  REQUIRE(a.upload(a_h), "upload");
  std::vector<uint8_t> want(c.n, kGuardByte), got;
  REQUIRE(c.upload(want), "upload");
  HIP_OK(hipMemset(b.p, 0, b.n));
  hsa_signal_t s1 = make_signal(1), s2 = make_signal(1);
  Signal sig1(s1), sig2(s2);
  std::vector<Signal*> none, after1{&sig1}, gang;
  REQUIRE(blit.SubmitLinearCopyCommand(b.p + 5, a.p, n, none, sig1, gang) == HSA_STATUS_SUCCESS, "submit 1");
  REQUIRE(blit.SubmitLinearCopyCommand(c.p + kGuard + 2, b.p + 5, n, after1, sig2, gang) == HSA_STATUS_SUCCESS,
          "submit 2");
  REQUIRE(wait_zero(s2, HSA_WAIT_STATE_BLOCKED), "chain never completed");
  REQUIRE(hsa_signal_load_relaxed(s1) == 0, "first signal not 0");
  oracle_copy(want.data() + kGuard + 2, a_h.data(), n);
  REQUIRE(c.download(got), "download");
  REQUIRE(got == want, "bytes differ");
  hsa_signal_destroy(s1);
  hsa_signal_destroy(s2);
  std::printf("PASS %s%s\n", name, g_suffix.c_str());
}

void test_zero_size_and_bad_args(Blit& blit) {
  const char* name = "zero_size_and_bad_arguments";
  DeviceBuf d(4096);
  REQUIRE(d.p, "hipMalloc");
  hsa_signal_t s = make_signal(1);
  Signal sig(s);
  std::vector<Signal*> none, gang;
  REQUIRE(blit.SubmitLinearCopyCommand(nullptr, d.p, 16, none, sig, gang) == HSA_STATUS_ERROR_INVALID_ARGUMENT, "null dst");
  REQUIRE(blit.SubmitLinearCopyCommand(d.p, nullptr, 16, none, sig, gang) == HSA_STATUS_ERROR_INVALID_ARGUMENT, "null src");
  REQUIRE(hsa_signal_load_relaxed(s) == 1, "signal touched by a rejected command");
  // size 0 completes the signal without moving anything
  REQUIRE(blit.SubmitLinearCopyCommand(d.p, d.p + 64, 0, none, sig, gang) == HSA_STATUS_SUCCESS, "zero size");
  REQUIRE(wait_zero(s, HSA_WAIT_STATE_BLOCKED), "zero-size copy never completed");
  REQUIRE(blit.SubmitLinearCopyCommand(d.p, d.p + 64, 0) == HSA_STATUS_SUCCESS, "blocking zero size");
  REQUIRE(blit.SubmitLinearFillCommand(d.p, 7, 0) == HSA_STATUS_SUCCESS, "zero-count fill");
  REQUIRE(!blit.isSDMA() && !blit.GangLeader(), "engine kind");
  REQUIRE(blit.EnableProfiling(true) == HSA_STATUS_SUCCESS && blit.EnableProfiling(false) == HSA_STATUS_SUCCESS,
          "EnableProfiling");
  hsa_signal_destroy(s);
  std::printf("PASS %s%s\n", name, g_suffix.c_str());
}

void test_batch(Blit& blit, const BatchFn& submit_batch) {
  const char* name = "batched_copies_with_signal";
  const size_t ncopy = 500;
  std::vector<size_t> len(ncopy), off(ncopy), so(ncopy), dof(ncopy);
  std::vector<uint8_t> rnd = seeded(ncopy * 4, 0xB1170055);
  size_t total = 256;
  for (size_t i = 0; i < ncopy; ++i) {
    len[i] = 1 + (size_t(rnd[4 * i]) | (size_t(rnd[4 * i + 1]) << 8)) % 40000;
    so[i] = rnd[4 * i + 2] & 15;
    dof[i] = rnd[4 * i + 3] & 15;
    off[i] = total;
    total += ((len[i] + 255) / 256) * 256 + 256;
  }
  std::vector<uint8_t> src_h = seeded(total, 0xB1170056);
  DeviceBuf src(total), dst(total);
  REQUIRE(src.p && dst.p, "hipMalloc");
  REQUIRE(src.upload(src_h), "upload");
  std::vector<uint8_t> want(total, kGuardByte), got;
  REQUIRE(dst.upload(want), "upload");
  std::vector<mi355_blit_desc_t> descs(ncopy);
  for (size_t i = 0; i < ncopy; ++i) {
    descs[i].dst = dst.p + off[i] + dof[i];
    descs[i].src = src.p + off[i] + so[i];
    descs[i].bytes = len[i];
    oracle_copy(want.data() + off[i] + dof[i], src_h.data() + off[i] + so[i], len[i]);
  }
  hsa_signal_t s = make_signal(1);
  Signal sig(s);
  std::vector<Signal*> none;
  REQUIRE(submit_batch(descs.data(), ncopy, false, 0, none, sig) == HSA_STATUS_SUCCESS, "submit");
  REQUIRE(wait_zero(s, HSA_WAIT_STATE_BLOCKED), "batch never completed");
  REQUIRE(dst.download(got), "download");
  REQUIRE(got == want, "bytes differ");
  std::printf("PASS %s%s\n", name, g_suffix.c_str());

  // the same descriptors, device-resident: without a bound on their sizes and with one
  name = "batched_copies_device_resident";
  std::vector<uint8_t> image(ncopy * sizeof(mi355_blit_desc_t));
  std::memcpy(image.data(), descs.data(), image.size());
  DeviceBuf descs_dev(image.size());
  REQUIRE(descs_dev.p, "hipMalloc");
  REQUIRE(descs_dev.upload(image), "upload");
  uint64_t sum = 0;
  for (size_t i = 0; i < ncopy; ++i) sum += len[i];
  for (uint64_t bound : {uint64_t(0), sum, 3 * sum}) {
    REQUIRE(dst.upload(std::vector<uint8_t>(total, kGuardByte)), "upload");
    hsa_signal_store_relaxed(s, 1);
    REQUIRE(submit_batch(descs_dev.p, ncopy, true, bound, none, sig) == HSA_STATUS_SUCCESS, "submit");
    REQUIRE(wait_zero(s, HSA_WAIT_STATE_BLOCKED), "batch never completed");
    REQUIRE(dst.download(got), "download");
    REQUIRE(got == want, "bytes differ");
  }
  hsa_signal_destroy(s);
  std::printf("PASS %s%s\n", name, g_suffix.c_str());
}

// A 3-D box out of one pitched surface into another, behind a dependency:
// what GpuAgent::DmaCopyRect would submit.
void test_copy_rect(BlitKernelGfx950Aql& blit) {
  const char* name = "copy_rect_with_signal";
  const size_t s_pitch = 5011, s_rows = 40, d_pitch = 6001, d_rows = 37, layers = 3;
  std::vector<uint8_t> src_h = seeded(s_pitch * s_rows * layers, 0xB1170061);
  DeviceBuf src(src_h.size()), dst(d_pitch * d_rows * layers);
  REQUIRE(src.p && dst.p, "hipMalloc");
  REQUIRE(src.upload(src_h), "upload");
  std::vector<uint8_t> want(dst.n, kGuardByte), got;
  REQUIRE(dst.upload(want), "upload");
  hsa_pitched_ptr_t sp{src.p, s_pitch, s_pitch * s_rows}, dp{dst.p, d_pitch, d_pitch * d_rows};
  hsa_dim3_t so{7, 3, 1}, dof{1001, 2, 0}, range{4999, 33, 2};
  oracle_pitched_ptr_t osp{src_h.data(), s_pitch, s_pitch * s_rows}, odp{want.data(), d_pitch, d_pitch * d_rows};
  oracle_dim3_t oso{so.x, so.y, so.z}, odo{dof.x, dof.y, dof.z}, orange{range.x, range.y, range.z};
  oracle_copy_rect(&odp, &odo, &osp, &oso, &orange);
  hsa_signal_t dep = make_signal(1), done = make_signal(1);
  Signal dep_sig(dep), done_sig(done);
  std::vector<Signal*> deps{&dep_sig};
  REQUIRE(blit.SubmitCopyRectCommand(&dp, &dof, &sp, &so, &range, deps, done_sig) == HSA_STATUS_SUCCESS, "submit");
  REQUIRE(hsa_signal_load_relaxed(done) == 1, "ran before its dependency");
  hsa_signal_store_screlease(dep, 0);
  REQUIRE(wait_zero(done, HSA_WAIT_STATE_BLOCKED), "rect copy never completed");
  REQUIRE(dst.download(got), "download");
  REQUIRE(got == want, "bytes differ");
  // not a box inside the surface: refused like amd_blit_sdma.cpp:577-579
  hsa_dim3_t wide{static_cast<uint32_t>(d_pitch), 1, 1};
  std::vector<Signal*> none;
  REQUIRE(blit.SubmitCopyRectCommand(&dp, &dof, &sp, &so, &wide, none, done_sig) == HSA_STATUS_ERROR_INVALID_ARGUMENT,
          "width out of range accepted");
  hsa_signal_destroy(dep);
  hsa_signal_destroy(done);
  std::printf("PASS %s%s\n", name, g_suffix.c_str());
}

// Objects made for GpuAgent's BlitHostToDev / BlitDevToHost slots
// (amd_gpu_agent.cpp:864-867) move a payload from pinned host memory into the
// device and back out, blocking and with a signal.
void test_host_link_slots(const rocr::core::Agent& agent) {
  const char* name = "host_link_slots";
  const size_t n = (6u << 20) + 13;
  uint8_t *in = nullptr, *out = nullptr;
  HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&in), n + 64, hipHostMallocDefault));
  HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&out), n + 2 * kGuard, hipHostMallocDefault));
  const std::vector<uint8_t> payload = seeded(n + 64, 0xB1170031);
  std::memcpy(in, payload.data(), n + 64);
  std::memset(out, kGuardByte, n + 2 * kGuard);
  DeviceBuf dev(n + 2 * kGuard);
  REQUIRE(dev.p, "hipMalloc");
  std::vector<uint8_t> want(dev.n, kGuardByte), got;
  REQUIRE(dev.upload(want), "upload");
  // both objects on one borrowed queue, as GpuAgent's blit_lambda puts them on queues_[QueueBlitOnly]
  UtilityQueue uq(agent.public_handle());
  REQUIRE(uq.q, "hsa_queue_create");
  rocr::core::Queue queue(uq.q);
  BlitKernelGfx950Aql h2d(&queue, BlitKernelGfx950Aql::Slot::kHostToDev);
  BlitKernelGfx950Aql d2h(&queue, BlitKernelGfx950Aql::Slot::kDevToHost);
  REQUIRE(h2d.Initialize(agent) == HSA_STATUS_SUCCESS && d2h.Initialize(agent) == HSA_STATUS_SUCCESS, "Initialize");
  hsa_status_t st = h2d.SubmitLinearCopyCommand(dev.p + kGuard + 5, in + 3, n);
  REQUIRE(st == HSA_STATUS_SUCCESS, "host to device: status 0x%x", st);
  oracle_copy(want.data() + kGuard + 5, payload.data() + 3, n);
  REQUIRE(dev.download(got), "download");
  REQUIRE(got == want, "host to device: bytes differ");
  hsa_signal_t done = make_signal(1);
  REQUIRE(done.handle, "signal");
  std::vector<Signal*> none;
  Signal out_signal(done);
  st = d2h.SubmitLinearCopyCommand(out + kGuard + 1, dev.p + kGuard + 5, n, none, out_signal, none);
  REQUIRE(st == HSA_STATUS_SUCCESS, "device to host: status 0x%x", st);
  REQUIRE(wait_zero(done, HSA_WAIT_STATE_ACTIVE), "device to host: signal never reached 0");
  std::vector<uint8_t> want_out(n + 2 * kGuard, kGuardByte);
  oracle_copy(want_out.data() + kGuard + 1, payload.data() + 3, n);
  REQUIRE(std::memcmp(out, want_out.data(), want_out.size()) == 0, "device to host: bytes differ");
  hsa_signal_destroy(done);
  REQUIRE(h2d.Destroy(agent) == HSA_STATUS_SUCCESS && d2h.Destroy(agent) == HSA_STATUS_SUCCESS, "Destroy");
  (void)hipHostFree(in);
  (void)hipHostFree(out);
  std::printf("PASS %s%s\n", name, g_suffix.c_str());
}

void test_threads(Blit& blit) {
  const char* name = "concurrent_submitters";
  const int kThreads = 4, kPer = 6;
  const size_t n = (1u << 18) + 13, region = ((n + 2 * kGuard + 255) / 256) * 256;
  std::vector<uint8_t> src_h = seeded(n + 64, 0xB1170077);
  DeviceBuf src(src_h.size()), dst(region * kThreads * kPer);
  REQUIRE(src.p && dst.p, "hipMalloc");
  REQUIRE(src.upload(src_h), "upload");
  std::vector<uint8_t> want(dst.n, kGuardByte), got;
  REQUIRE(dst.upload(want), "upload");
  std::vector<hsa_status_t> status(kThreads * kPer, HSA_STATUS_SUCCESS);
  std::vector<std::thread> ths;
  for (int t = 0; t < kThreads; ++t) {
    ths.emplace_back([&, t] {
      for (int j = 0; j < kPer; ++j) {
        const int slot = t * kPer + j;
        // alternate blocking copies and blocking fills followed by copies
        if (j & 1) status[slot] = blit.SubmitLinearFillCommand(dst.p + slot * region + kGuard, 0x01020304u * (slot + 1), n / 4);
        else status[slot] = blit.SubmitLinearCopyCommand(dst.p + slot * region + kGuard + (slot & 15), src.p + (slot % 7), n);
      }
    });
  }
  for (auto& th : ths) th.join();
  for (int slot = 0; slot < kThreads * kPer; ++slot) {
    REQUIRE(status[slot] == HSA_STATUS_SUCCESS, "slot %d status 0x%x", slot, status[slot]);
    if ((slot % kPer) & 1) oracle_fill32(want.data() + slot * region + kGuard, 0x01020304u * (slot + 1), n / 4);
    else oracle_copy(want.data() + slot * region + kGuard + (slot & 15), src_h.data() + (slot % 7), n);
  }
  REQUIRE(dst.download(got), "download");
  REQUIRE(got == want, "bytes differ");
  std::printf("PASS %s%s\n", name, g_suffix.c_str());
}

// The engine on a queue it shares with another producer: the driver writes
// BARRIER_AND packets of its own between the blit's commands, by the same
// protocol (atomic add on the write index, body, header, doorbell), each with a
// completion signal of its own.  64 packet slots and some 400 packets: the ring
// and the engine's kernarg ring, indexed by packet index, wrap several times.
void write_own_barrier(hsa_queue_t* q, hsa_signal_t completion) {
  const uint64_t index = hsa_queue_add_write_index_scacq_screl(q, 1);
  while (index - hsa_queue_load_read_index_relaxed(q) >= q->size) std::this_thread::yield();
  auto* ring = static_cast<hsa_barrier_and_packet_t*>(q->base_address);
  hsa_barrier_and_packet_t* slot = &ring[index & (q->size - 1)];
  hsa_barrier_and_packet_t pkt;
  std::memset(&pkt, 0, sizeof(pkt));
  pkt.completion_signal = completion;
  std::memcpy(reinterpret_cast<uint8_t*>(slot) + 4, reinterpret_cast<uint8_t*>(&pkt) + 4, sizeof(pkt) - 4);
  const uint16_t header = (HSA_PACKET_TYPE_BARRIER_AND << HSA_PACKET_HEADER_TYPE) |
                          (HSA_FENCE_SCOPE_NONE << HSA_PACKET_HEADER_SCACQUIRE_FENCE_SCOPE) |
                          (HSA_FENCE_SCOPE_NONE << HSA_PACKET_HEADER_SCRELEASE_FENCE_SCOPE);
  __atomic_store_n(reinterpret_cast<uint32_t*>(slot), static_cast<uint32_t>(header), __ATOMIC_RELEASE);
  hsa_signal_store_screlease(q->doorbell_signal, static_cast<hsa_signal_value_t>(index));
}

void test_shared_queue(BlitKernelGfx950Aql& blit, hsa_queue_t* q) {
  const char* name = "shared_queue_interleaved_packets";
  REQUIRE(q->size == 64, "the case is meant for the 64-packet utility queue, got %u", q->size);
  const int kRounds = 96;
  const size_t n = (96u << 10) + 7, region = ((n + 2 * kGuard + 255) / 256) * 256;
  std::vector<uint8_t> src_h = seeded(n + 64, 0xB1170088);
  DeviceBuf src(src_h.size()), dst(region * kRounds);
  REQUIRE(src.p && dst.p, "hipMalloc");
  REQUIRE(src.upload(src_h), "upload");
  std::vector<uint8_t> want(dst.n, kGuardByte), got;
  REQUIRE(dst.upload(want), "upload");
  hsa_signal_t mine = make_signal(3 * kRounds), copies = make_signal(kRounds);
  REQUIRE(mine.handle && copies.handle, "signal");
  Signal out(copies);
  std::vector<Signal*> none, gang;
  for (int i = 0; i < kRounds; ++i) {
    write_own_barrier(q, mine);
    uint8_t* d = dst.p + i * region + kGuard;
    hsa_status_t st;
    if (i % 3 == 2) {
      // a blocking fill between the asynchronous copies
      st = blit.SubmitLinearFillCommand(d, 0x01010101u * (i + 1), n / 4);
      oracle_fill32(want.data() + i * region + kGuard, 0x01010101u * (i + 1), n / 4);
      hsa_signal_subtract_screlease(copies, 1);
    } else {
      st = blit.SubmitLinearCopyCommand(d + (i & 15), src.p + (i % 7), n, none, out, gang);
      oracle_copy(want.data() + i * region + kGuard + (i & 15), src_h.data() + (i % 7), n);
    }
    REQUIRE(st == HSA_STATUS_SUCCESS, "round %d status 0x%x", i, st);
    write_own_barrier(q, mine);
    write_own_barrier(q, mine);
  }
  REQUIRE(wait_zero(copies, HSA_WAIT_STATE_ACTIVE), "the blit's commands never completed");
  REQUIRE(wait_zero(mine, HSA_WAIT_STATE_ACTIVE), "the driver's own packets never completed: %ld left",
          (long)hsa_signal_load_relaxed(mine));
  REQUIRE(dst.download(got), "download");
  REQUIRE(got == want, "bytes differ");
  uint64_t pending = 1;
  for (int i = 0; i < 1000 && pending; ++i) {
    pending = blit.PendingBytes();
    if (pending) std::this_thread::sleep_for(std::chrono::milliseconds(1));
  }
  REQUIRE(pending == 0, "PendingBytes stuck at %llu", (unsigned long long)pending);
  hsa_signal_destroy(mine);
  hsa_signal_destroy(copies);
  std::printf("PASS %s%s\n", name, g_suffix.c_str());
}

// A queue that has stopped on an error never completes a signal.  The error is
// forced from the host (the owner's callback forwarding it, without any fault
// on the GPU): a wait that is already in progress must end with
// HSA_STATUS_ERROR, and later blocking calls must answer it at once.
void test_queue_error_ends_waits(const rocr::core::Agent& agent) {
  const char* name = "queue_error_ends_waits";
  UtilityQueue uq(agent.public_handle());
  REQUIRE(uq.q, "hsa_queue_create");
  rocr::core::Queue queue(uq.q);
  BlitKernelGfx950Aql blit(&queue);
  REQUIRE(blit.Initialize(agent) == HSA_STATUS_SUCCESS, "Initialize");
  DeviceBuf a(4096), b(4096);
  REQUIRE(a.p && b.p, "hipMalloc");
  REQUIRE(blit.SubmitLinearCopyCommand(b.p, a.p, 4096) == HSA_STATUS_SUCCESS, "a copy on the healthy queue");
  hsa_signal_t never = make_signal(1);
  REQUIRE(never.handle, "signal");
  std::thread reporter([&] {
    std::this_thread::sleep_for(std::chrono::milliseconds(50));
    blit.ReportQueueError(HSA_STATUS_ERROR_EXCEPTION);
  });
  const auto t0 = std::chrono::steady_clock::now();
  const int st = mi355_aql_wait_signal(blit.c_handle(), never.handle);
  const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
  reporter.join();
  REQUIRE(st == HSA_STATUS_ERROR, "wait on a signal nobody completes returned 0x%x", st);
  REQUIRE(ms >= 40.0 && ms < 2000.0, "the wait took %.1f ms", ms);
  REQUIRE(blit.SubmitLinearCopyCommand(b.p, a.p, 4096) == HSA_STATUS_ERROR, "blocking copy on a failed queue");
  REQUIRE(blit.SubmitLinearFillCommand(b.p, 1, 16) == HSA_STATUS_ERROR, "blocking fill on a failed queue");
  hsa_signal_destroy(never);
  // the queue itself is healthy (the error was only reported): Destroy may
  // not wait on it, and does not
  REQUIRE(blit.Destroy(agent) == HSA_STATUS_SUCCESS, "Destroy");
  std::printf("PASS %s%s\n", name, g_suffix.c_str());
}

hsa_status_t first_gpu_cb(hsa_agent_t agent, void* data) {
  hsa_device_type_t type;
  if (hsa_agent_get_info(agent, HSA_AGENT_INFO_DEVICE, &type) == HSA_STATUS_SUCCESS && type == HSA_DEVICE_TYPE_GPU) {
    *static_cast<hsa_agent_t*>(data) = agent;
    return HSA_STATUS_INFO_BREAK;
  }
  return HSA_STATUS_SUCCESS;
}

// With profiling on, the packet processor stamps the completion signal
// (amd_blit_kernel.cpp:839-842; read back like hsa_ext_amd.cpp:474-502 does).
void test_profiling_timestamps(Blit& blit) {
  const char* name = "profiling_timestamps";
  hsa_agent_t gpu{0};
  hsa_iterate_agents(first_gpu_cb, &gpu);
  REQUIRE(gpu.handle, "no GPU agent");
  const size_t n = 64u << 20;
  DeviceBuf a(n), b(n);
  REQUIRE(a.p && b.p, "hipMalloc");
  REQUIRE(blit.EnableProfiling(true) == HSA_STATUS_SUCCESS, "EnableProfiling(true)");
  hsa_signal_t s = make_signal(1);
  Signal sig(s);
  std::vector<Signal*> none, gang;
  REQUIRE(blit.SubmitLinearCopyCommand(b.p, a.p, n, none, sig, gang) == HSA_STATUS_SUCCESS, "submit");
  REQUIRE(wait_zero(s, HSA_WAIT_STATE_BLOCKED), "copy never completed");
  hsa_amd_profiling_dispatch_time_t t{0, 0};
  hsa_status_t st = hsa_amd_profiling_get_dispatch_time(gpu, s, &t);
  REQUIRE(st == HSA_STATUS_SUCCESS, "get_dispatch_time 0x%x", st);
  REQUIRE(t.end > t.start, "timestamps not written: start %llu end %llu", (unsigned long long)t.start,
          (unsigned long long)t.end);
  uint64_t freq = 0;
  hsa_system_get_info(HSA_SYSTEM_INFO_TIMESTAMP_FREQUENCY, &freq);
  const double us = freq ? double(t.end - t.start) * 1e6 / double(freq) : 0.0;
  std::printf("INFO profiling_copy_64MiB_us %.1f\n", us);
  REQUIRE(us > 5.0 && us < 5000.0, "implausible copy time %.1f us", us);
  REQUIRE(blit.EnableProfiling(false) == HSA_STATUS_SUCCESS, "EnableProfiling(false)");
  hsa_signal_destroy(s);
  std::printf("PASS %s%s\n", name, g_suffix.c_str());
}

// The HIP-stream engine has no queue bit to flip: with profiling on it stamps
// the command's signal from the device (one-lane kernels in front of and behind
// the command).  The stamps are raw ticks of the GPU's clock, like the packet
// processor's; converted to the system domain with the public HSA call they
// must lie between the host's own readings of that clock around the copy.
void test_profiling_stamps_from_device(Blit& blit) {
  const char* name = "profiling_timestamps";
  hsa_agent_t gpu{0};
  hsa_iterate_agents(first_gpu_cb, &gpu);
  REQUIRE(gpu.handle, "no GPU agent");
  const size_t n = 64u << 20;
  DeviceBuf a(n), b(n);
  REQUIRE(a.p && b.p, "hipMalloc");
  REQUIRE(blit.EnableProfiling(true) == HSA_STATUS_SUCCESS, "EnableProfiling(true)");
  uint64_t freq = 0;
  hsa_system_get_info(HSA_SYSTEM_INFO_TIMESTAMP_FREQUENCY, &freq);
  REQUIRE(freq, "no timestamp frequency");
  for (int round = 0; round < 3; ++round) {
    hsa_signal_t s = make_signal(1);
    Signal sig(s);
    std::vector<Signal*> none, gang;
    uint64_t before = 0, after = 0;
    hsa_system_get_info(HSA_SYSTEM_INFO_TIMESTAMP, &before);
    REQUIRE(blit.SubmitLinearCopyCommand(b.p, a.p, n, none, sig, gang) == HSA_STATUS_SUCCESS, "submit");
    REQUIRE(wait_zero(s, HSA_WAIT_STATE_BLOCKED), "copy never completed");
    hsa_system_get_info(HSA_SYSTEM_INFO_TIMESTAMP, &after);
    const mi355::HsaSignalAbi* raw = reinterpret_cast<const mi355::HsaSignalAbi*>(s.handle);
    const uint64_t start_raw = raw->start_ts, end_raw = raw->end_ts;
    REQUIRE(start_raw != 0 && end_raw > start_raw, "stamps not written: start %llu end %llu",
            (unsigned long long)start_raw, (unsigned long long)end_raw);
    uint64_t start = 0, end = 0;
    REQUIRE(hsa_amd_profiling_convert_tick_to_system_domain(gpu, start_raw, &start) == HSA_STATUS_SUCCESS, "convert");
    REQUIRE(hsa_amd_profiling_convert_tick_to_system_domain(gpu, end_raw, &end) == HSA_STATUS_SUCCESS, "convert");
    const double us = double(end - start) * 1e6 / double(freq);
    // the conversion interpolates between two readings of both clocks: allow it a few microseconds
    const uint64_t slack = freq / 20000;  // 50 us
    std::printf("INFO profiling_copy_64MiB_us%s %.1f (submit to start %.1f us, end to seen %.1f us)\n", g_suffix.c_str(), us,
                (double(start) - double(before)) * 1e6 / double(freq), (double(after) - double(end)) * 1e6 / double(freq));
    REQUIRE(us > 5.0 && us < 5000.0, "implausible copy time %.1f us", us);
    REQUIRE(start + slack >= before && end <= after + slack,
            "stamps outside the host's window: before %llu start %llu end %llu after %llu", (unsigned long long)before,
            (unsigned long long)start, (unsigned long long)end, (unsigned long long)after);
    hsa_signal_destroy(s);
  }
  REQUIRE(blit.EnableProfiling(false) == HSA_STATUS_SUCCESS, "EnableProfiling(false)");
  // off again: the signal of the next command keeps its zeros
  hsa_signal_t s = make_signal(1);
  Signal sig(s);
  std::vector<Signal*> none, gang;
  REQUIRE(blit.SubmitLinearCopyCommand(b.p, a.p, n, none, sig, gang) == HSA_STATUS_SUCCESS, "submit");
  REQUIRE(wait_zero(s, HSA_WAIT_STATE_BLOCKED), "copy never completed");
  const mi355::HsaSignalAbi* raw = reinterpret_cast<const mi355::HsaSignalAbi*>(s.handle);
  REQUIRE(raw->start_ts == 0 && raw->end_ts == 0, "stamps written with profiling off");
  hsa_signal_destroy(s);
  std::printf("PASS %s%s\n", name, g_suffix.c_str());
}

void latency_report(Blit& blit, const char* mode) {
  // host-observed time per blocking call, submit -> completion seen
  // (the way memory_async_copy.cc:396-405 times a copy)
  DeviceBuf a(1 << 20), b(1 << 20);
  if (!a.p || !b.p) return;
  for (size_t n : {size_t(4096), size_t(65536), size_t(1 << 20)}) {
    std::vector<double> us;
    for (int i = 0; i < 120; ++i) {
      auto t0 = std::chrono::steady_clock::now();
      blit.SubmitLinearCopyCommand(b.p, a.p, n);
      auto t1 = std::chrono::steady_clock::now();
      if (i >= 20) us.push_back(std::chrono::duration<double, std::micro>(t1 - t0).count());
    }
    std::sort(us.begin(), us.end());
    std::printf("INFO blocking_copy_us mode=%s bytes=%zu median=%.2f min=%.2f\n", mode, n, us[us.size() / 2], us[0]);
  }
}

// Where the time of a small blocking copy goes on the AQL path, the way
// rocrtst times one (memory_async_copy.cc:396-405: submit, then spin on the
// completion signal), cut at the packet processor's own timestamps: host
// submit call | doorbell to start of the kernel | kernel | end of the kernel
// to the host seeing the signal.  The signal's stamps are in the system
// timestamp domain (the runtime translates them), like the host's readings.
uint64_t now_ticks() {
  uint64_t t = 0;
  hsa_system_get_info(HSA_SYSTEM_INFO_TIMESTAMP, &t);
  return t;
}

double median_of(std::vector<double>& v) {
  std::sort(v.begin(), v.end());
  return v[v.size() / 2];
}

void latency_breakdown(bool system_scope, const char* kernargs, const mi355_blit_tuning_t* tuning = nullptr,
                       const char* shape = "heuristic") {
  mi355_aql_t* h = nullptr;
  if (mi355_aql_create(0, &h) != MI355_BLIT_SUCCESS) {
    std::printf("FAIL latency_breakdown: mi355_aql_create\n");
    ++g_failures;
    return;
  }
  mi355_aql_set_tuning(h, tuning);
  mi355_aql_set_system_scope_fences(h, system_scope ? 1 : 0);
  mi355_aql_enable_profiling(h, 1);
  uint64_t freq = 0;
  hsa_system_get_info(HSA_SYSTEM_INFO_TIMESTAMP_FREQUENCY, &freq);
  const double us_per_tick = 1e6 / double(freq);
  DeviceBuf a(1 << 20), b(1 << 20);
  hsa_signal_t done = make_signal(1);
  if (!a.p || !b.p || !done.handle) return;
  for (size_t n : {size_t(4096), size_t(65536), size_t(1 << 20)}) {
    std::vector<double> submit, to_start, kernel, to_host, total;
    for (int i = 0; i < 320; ++i) {
      hsa_signal_store_relaxed(done, 1);
      const uint64_t t0 = now_ticks();
      if (mi355_aql_copy(h, b.p, a.p, n, nullptr, 0, done.handle) != MI355_BLIT_SUCCESS) return;
      const uint64_t t1 = now_ticks();
      while (hsa_signal_wait_scacquire(done, HSA_SIGNAL_CONDITION_LT, 1, UINT64_MAX, HSA_WAIT_STATE_ACTIVE) >= 1) {
      }
      const uint64_t t2 = now_ticks();
      uint64_t start = 0, end = 0;
      if (mi355_aql_get_command_time(h, done.handle, &start, &end, nullptr) != MI355_BLIT_SUCCESS) return;
      if (i < 20) continue;
      submit.push_back(double(t1 - t0) * us_per_tick);
      to_start.push_back((double(start) - double(t1)) * us_per_tick);
      kernel.push_back(double(end - start) * us_per_tick);
      to_host.push_back((double(t2) - double(end)) * us_per_tick);
      total.push_back(double(t2 - t0) * us_per_tick);
    }
    std::printf("INFO latency_breakdown fences=%s kernargs=%s shape=%s bytes=%zu total=%.2f submit_call=%.2f doorbell_to_start=%.2f "
                "kernel=%.2f end_to_host=%.2f (medians of %zu, us)\n",
                system_scope ? "system" : "agent", kernargs, shape, n, median_of(total), median_of(submit), median_of(to_start),
                median_of(kernel), median_of(to_host), total.size());
  }
  hsa_signal_destroy(done);
  mi355_aql_destroy(h);
}

}  // namespace

int main(int argc, char** argv) {
  if (argc > 1 && std::string(argv[1]) == "--list") {
    const char* cases[] = {"blocking_copy_offsets_and_sizes", "blocking_fill_reference_patterns",
                           "async_copy_active_wait", "async_copy_blocked_wait", "dependencies_1", "dependencies_6",
                           "chain_a_to_b_to_c", "zero_size_and_bad_arguments", "batched_copies_with_signal",
                           "concurrent_submitters", "destroy"};
    for (const char* engine : {"_hip", "_aql"})
      for (const char* c : cases) std::printf("%s%s\n", c, engine);
    std::printf("async_copy_blocked_wait_hip_callback\nchain_a_to_b_to_c_hip_callback\n"
                "profiling_timestamps_hip_callback\nprofiling_timestamps_hip\nprofiling_timestamps_aql\ncopy_rect_with_signal_aql\nhost_link_slots_aql\n"
                "shared_queue_interleaved_packets_aql\nqueue_error_ends_waits_aql\n");
    return 0;
  }
  if (hsa_init() != HSA_STATUS_SUCCESS) {
    std::printf("FAIL setup: hsa_init failed (no GPU?)\n");
    return 2;
  }
  if (argc > 1 && std::string(argv[1]) == "--latency") {
    // test_rocr_blit --latency: the breakdown only, for the placement of the
    // kernarg ring the environment asks for (MI355_BLIT_HOST_KERNARGS=1: host memory)
    const char* env = std::getenv("MI355_BLIT_HOST_KERNARGS");
    const char* where = env && env[0] == '1' ? "host" : "device";
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count < 1) return 2;
    latency_breakdown(true, where);
    latency_breakdown(false, where);
    if (argc > 2 && std::string(argv[2]) == "shapes") {
      // what the launch shape and the store policy of a small copy are worth under system-scope fences
      mi355_blit_tuning_t t{};
      t.store_policy = MI355_BLIT_STORE_AGENT_WT + 1;
      latency_breakdown(true, where, &t, "stores_sc1");
      t.store_policy = MI355_BLIT_STORE_SYSTEM_WT + 1;
      latency_breakdown(true, where, &t, "stores_sc0_sc1");
      t.store_policy = MI355_BLIT_STORE_NT + 1;
      latency_breakdown(true, where, &t, "stores_nt");
      t = mi355_blit_tuning_t{};
      t.wg_size = 1024;
      latency_breakdown(true, where, &t, "wg1024");
      t.wg_size = 64;
      latency_breakdown(true, where, &t, "wg64");
    }
    hsa_shut_down();
    return g_failures ? 1 : 0;
  }
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count < 1) {
    std::printf("FAIL setup: no HIP device\n");
    return 2;
  }
  hsa_agent_t gpu{0};
  hsa_iterate_agents(first_gpu_cb, &gpu);
  if (!gpu.handle) {
    std::printf("FAIL setup: no GPU agent\n");
    return 2;
  }
  // what GpuAgent hands to CreateBlitKernel: itself and its utility queue
  rocr::core::Agent agent(gpu);
  UtilityQueue utility(gpu);
  if (!utility.q) {
    std::printf("FAIL setup: hsa_queue_create\n");
    return 2;
  }
  rocr::core::Queue utility_queue(utility.q);
  {
    // the host-callback completion mode of the HIP-stream engine
    g_suffix = "_hip_callback";
    BlitKernelGfx950 cb(nullptr, BlitKernelGfx950::Completion::kHostCallback);
    if (cb.Initialize(agent) != HSA_STATUS_SUCCESS) {
      std::printf("FAIL setup: Initialize (host callback)\n");
      return 2;
    }
    test_async_copy_signal(cb, HSA_WAIT_STATE_BLOCKED, "async_copy_blocked_wait");
    test_chain(cb);
    test_profiling_stamps_from_device(cb);
    latency_report(cb, "hip_host_callback");
    if (cb.Destroy(agent) != HSA_STATUS_SUCCESS) {
      std::printf("FAIL destroy (host callback)\n");
      ++g_failures;
    }
  }
  for (int engine = 0; engine < 2; ++engine) {
    Blit* blit = nullptr;
    BatchFn batch;
    hsa_status_t init;
    if (engine == 0) {
      g_suffix = "_hip";
      auto* b = new BlitKernelGfx950(nullptr);
      init = b->Initialize(agent);
      batch = [b](const void* d, size_t n, bool on_device, uint64_t bound, std::vector<Signal*>& deps, Signal& out) {
        return b->SubmitBatchCopyCommand(d, n, on_device, deps, out, bound);
      };
      blit = b;
    } else {
      g_suffix = "_aql";
      auto* b = new BlitKernelGfx950Aql(&utility_queue);
      utility.engine = b;
      init = b->Initialize(agent);
      batch = [b](const void* d, size_t n, bool on_device, uint64_t bound, std::vector<Signal*>& deps, Signal& out) {
        return b->SubmitBatchCopyCommand(d, n, on_device, deps, out, bound);
      };
      blit = b;
    }
    if (init != HSA_STATUS_SUCCESS) {
      std::printf("FAIL setup%s: Initialize returned 0x%x\n", g_suffix.c_str(), init);
      return 2;
    }
    test_blocking_copy(*blit);
    test_blocking_fill(*blit);
    test_async_copy_signal(*blit, HSA_WAIT_STATE_ACTIVE, "async_copy_active_wait");
    test_async_copy_signal(*blit, HSA_WAIT_STATE_BLOCKED, "async_copy_blocked_wait");
    test_dependencies(*blit, 1, "dependencies_1");
    test_dependencies(*blit, 6, "dependencies_6");  // more than one barrier packet's worth
    test_chain(*blit);
    test_zero_size_and_bad_args(*blit);
    test_batch(*blit, batch);
    test_threads(*blit);
    if (engine == 0) test_profiling_stamps_from_device(*blit);
    if (engine == 1) {
      test_profiling_timestamps(*blit);
      test_copy_rect(*static_cast<BlitKernelGfx950Aql*>(blit));
      test_shared_queue(*static_cast<BlitKernelGfx950Aql*>(blit), utility.q);
      test_host_link_slots(agent);
      test_queue_error_ends_waits(agent);
    }
    latency_report(*blit, engine == 0 ? "hip_device_signal" : "aql");
    hsa_status_t st = blit->Destroy(agent);
    if (st != HSA_STATUS_SUCCESS) {
      std::printf("FAIL destroy%s: status 0x%x\n", g_suffix.c_str(), st);
      ++g_failures;
    } else {
      std::printf("PASS destroy%s\n", g_suffix.c_str());
    }
    delete blit;
    utility.engine = nullptr;
  }
  hsa_shut_down();
  std::printf("%s (%d failures)\n", g_failures ? "FAILED" : "OK", g_failures);
  return g_failures ? 1 : 0;
}
