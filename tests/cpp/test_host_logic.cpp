// Host arithmetic of the blit engine under AddressSanitizer and UBSan, at a
// volume the Python tests cannot reach: the copy / fill plans
// (csrc/blit_plan.h) and the region-copy plans (csrc/blit_rect.h) over
// hundreds of thousands of seeded cases.  Every plan is checked against
// invariants that do not restate its formulas: a plan must tile its byte range
// exactly, a region plan's units (or packed slots) must cover every row's bytes
// once, in order and inside the row, and the region validation must give the
// reference's verdict (oracle_ref_validate_rect), and the staging image of a
// batch must tile every copy into pieces with the right record indices.  No
// GPU, no device code.
//
//   test_host_logic [cases]      exit status 0 = all checks passed
#include <cinttypes>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <chrono>
#include <thread>
#include <vector>

#include "../../oracle/blit_oracle.h"
#include "aql_host_lock.h"
#include "aql_wait.h"
#include "blit_batch_host.h"
#include "blit_plan.h"
#include "blit_rect.h"

namespace {

using namespace mi355;

uint64_t g_state = 0x9E3779B97F4A7C15ull;
uint64_t rnd() {  // splitmix64
  uint64_t z = (g_state += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
uint64_t below(uint64_t n) { return n ? rnd() % n : 0; }

int g_failures = 0;
#define CHECK(cond, ...)                          \
  do {                                            \
    if (!(cond)) {                                \
      if (g_failures < 20) {                      \
        std::printf("FAIL %s:%d: ", __FILE__, __LINE__); \
        std::printf(__VA_ARGS__);                 \
        std::printf("\n");                        \
      }                                           \
      ++g_failures;                               \
      return;                                     \
    }                                             \
  } while (0)

mi355_blit_tuning_t random_tuning() {
  mi355_blit_tuning_t t{};
  const uint32_t wgs[] = {0, 64, 128, 256, 512, 1024, 100, 2048};
  const uint32_t unrolls[] = {0, 1, 2, 4, 3};
  t.wg_size = wgs[below(8)];
  t.unroll = unrolls[below(5)];
  t.max_grid = below(3) ? 0 : static_cast<uint32_t>(below(5000));
  t.nt_load = static_cast<uint32_t>(below(3));
  t.store_policy = static_cast<uint32_t>(below(6));
  const uint32_t prefetch[] = {0, 0, 1, 4224};
  t.batch_prefetch = prefetch[below(4)];
  return t;
}

uint64_t random_size() {
  switch (below(4)) {
    case 0: return below(600);
    case 1: return below(1u << 20);
    case 2: return (1ull << (20 + below(16))) + below(4096) - below(64);
    default: return rnd() >> (16 + below(40));
  }
}

void check_linear_plan(const mi355_blit_plan_t& p, uint64_t dst, uint64_t bytes, uint32_t kernel) {
  CHECK(p.kernel == kernel, "kernel %u", p.kernel);
  CHECK(p.head_bytes + 16 * p.body_vecs + p.tail_bytes == bytes, "plan does not tile %" PRIu64 " bytes", bytes);
  CHECK(p.head_bytes <= 15 && p.tail_bytes <= 15, "head %" PRIu64 " tail %" PRIu64, p.head_bytes, p.tail_bytes);
  CHECK(p.body_vecs == 0 || (dst + p.head_bytes) % 16 == 0, "body not 16-byte aligned");
  CHECK(p.lead_vecs == ((dst + p.head_bytes) & 255) / 16, "lead %u", p.lead_vecs);
  CHECK(p.wg_size >= 64 && p.wg_size <= 1024 && p.wg_size % 64 == 0, "wg %u", p.wg_size);
  CHECK(p.unroll == 1 || p.unroll == 2 || p.unroll == 4, "unroll %u", p.unroll);
  CHECK(p.grid >= 1 && static_cast<uint64_t>(p.grid) * p.wg_size <= 0x7fffffc0ull, "grid %u x %u", p.grid, p.wg_size);
  CHECK(p.store_policy <= 3 && p.nt_load <= 1, "policy");
}

void one_copy_plan() {
  const uint64_t dst = (1ull << 40) + below(1 << 20), src = (2ull << 40) + below(1 << 20);
  const uint64_t bytes = random_size();
  const bool tuned = below(2);
  mi355_blit_tuning_t t = random_tuning();
  mi355_blit_plan_t p;
  CHECK(plan_copy(dst, src, bytes, 256, tuned ? &t : nullptr, &p) == MI355_BLIT_SUCCESS, "plan_copy failed");
  // the reference's predicate for its two copy shaders (amd_blit_kernel.cpp:716)
  const bool same_dword_phase = (src & 3) == (dst & 3);
  check_linear_plan(p, dst, bytes, same_dword_phase ? MI355_BLIT_KERNEL_COPY : MI355_BLIT_KERNEL_COPY_REALIGN);
  CHECK(p.byte_shift == ((src - dst) & 3), "byte shift");
  if (!tuned || t.max_grid == 0) {
    // uncapped: one wave per tile and one for the edges
    const uint64_t tile = 64ull * p.unroll;
    const uint64_t tiles = (p.body_vecs + p.lead_vecs + tile - 1) / tile;
    const uint64_t waves = static_cast<uint64_t>(p.grid) * (p.wg_size / 64);
    CHECK(waves >= tiles + 1 || waves * 64 + p.wg_size > 0x7fffffc0ull, "grid %u too small for %" PRIu64 " tiles", p.grid, tiles);
  }
}

void one_fill_plan() {
  const uint64_t ptr = (1ull << 40) + 4 * below(1 << 18);
  const uint64_t dwords = random_size() / 4;
  mi355_blit_tuning_t t = random_tuning();
  mi355_blit_plan_t p;
  CHECK(plan_fill(ptr, dwords, 256, below(2) ? &t : nullptr, &p) == MI355_BLIT_SUCCESS, "plan_fill failed");
  check_linear_plan(p, ptr, dwords * 4, MI355_BLIT_KERNEL_FILL);
  CHECK(p.head_bytes % 4 == 0 && p.tail_bytes % 4 == 0, "fill edges are whole dwords");
  CHECK(plan_fill(ptr + 1 + below(3), dwords, 256, nullptr, &p) == MI355_BLIT_ERROR_INVALID_ARGUMENT, "misaligned fill accepted");
}

// Bytes [*lo, *hi) of a row that unit kq of the wide-row kernel moves.
void unit_range(uint64_t d, uint64_t width, uint64_t unit, uint64_t kq, uint64_t units, uint64_t* lo, uint64_t* hi,
                uint64_t* vectors) {
  uint64_t head = (16 - (d & 15)) & 15;
  if (head > width) head = width;
  const uint64_t n_vec = (width - head) / 16, lead = ((d + head) & 255) / 16, n_virtual = n_vec + lead;
  const bool last = kq + 1 == units;
  const uint64_t v_lo = kq * unit > lead ? kq * unit : lead;
  const uint64_t v_hi = last ? n_virtual : kq * unit + unit;
  *lo = kq == 0 ? 0 : head + 16 * (v_lo - lead);
  *hi = last ? width : head + 16 * (v_hi - lead);
  *vectors = v_hi - kq * unit;
}

void one_rect_plan() {
  mi355_pitched_ptr_t dst{}, src{};
  dst.base = reinterpret_cast<void*>((1ull << 40) + below(512));
  src.base = reinterpret_cast<void*>((2ull << 40) + below(512));
  const bool narrow = below(2);
  mi355_dim3_t range{static_cast<uint32_t>(1 + below(narrow ? 1200 : 40000)), static_cast<uint32_t>(1 + below(40)),
                     static_cast<uint32_t>(1 + below(4))};
  mi355_dim3_t doff{static_cast<uint32_t>(below(300)), static_cast<uint32_t>(below(8)), static_cast<uint32_t>(below(3))};
  mi355_dim3_t soff{static_cast<uint32_t>(below(300)), static_cast<uint32_t>(below(8)), static_cast<uint32_t>(below(3))};
  dst.pitch = below(8) ? doff.x + range.x + below(300) : range.x;
  src.pitch = below(8) ? soff.x + range.x + below(300) : range.x;
  if (below(16) == 0) dst.pitch = below(dst.pitch + 1);  // sometimes too small
  dst.slice = below(5) ? dst.pitch * (doff.y + range.y + below(5)) : (below(2) ? 0 : dst.pitch * below(range.y + 2));
  src.slice = below(5) ? src.pitch * (soff.y + range.y + below(5)) : (below(2) ? 0 : src.pitch * below(range.y + 2));
  if (below(50) == 0) range.x = 0;
  mi355_blit_tuning_t t = random_tuning();
  const bool tuned = below(3) == 0;
  RectPlan rp;
  const int st = plan_rect(&dst, &doff, &src, &soff, &range, tuned ? &t : nullptr, &rp);

  oracle_pitched_ptr_t od{dst.base, dst.pitch, dst.slice}, os{src.base, src.pitch, src.slice};
  oracle_dim3_t odo{doff.x, doff.y, doff.z}, oso{soff.x, soff.y, soff.z}, orange{range.x, range.y, range.z};
  int does_work = -1, aligned = -1;
  const int want = oracle_ref_validate_rect(&od, &odo, &os, &oso, &orange, 3, &does_work, &aligned);
  CHECK(st == want, "status 0x%x, the reference's checks say 0x%x", st, want);
  if (st != MI355_BLIT_SUCCESS) return;
  CHECK(rp.empty == (does_work == 0), "empty flag");
  if (rp.empty) return;

  const uint64_t d0 = reinterpret_cast<uint64_t>(dst.base) + doff.z * dst.slice + doff.y * dst.pitch + doff.x;
  const uint64_t s0 = reinterpret_cast<uint64_t>(src.base) + soff.z * src.slice + soff.y * src.pitch + soff.x;
  const uint64_t total = static_cast<uint64_t>(range.x) * range.y * range.z;
  CHECK(rp.total_bytes == total, "total bytes");
  CHECK(reinterpret_cast<uint64_t>(rp.args.dst) == d0 && reinterpret_cast<uint64_t>(rp.args.src) == s0, "region origin");
  if (rp.linear) {
    CHECK(rp.args.width == total, "a linear region is all of its bytes");
    // contiguous on both sides: the last byte of the box sits total - 1 bytes after the first
    const uint64_t last_d = d0 + (range.z - 1) * dst.slice + (range.y - 1) * dst.pitch + range.x - 1;
    const uint64_t last_s = s0 + (range.z - 1) * src.slice + (range.y - 1) * src.pitch + range.x - 1;
    CHECK(last_d - d0 == total - 1 && last_s - s0 == total - 1, "region merged into one run is not contiguous");
    return;
  }
  // merged rows: every merged row is a run of whole original rows
  const uint64_t width = rp.narrow ? rp.nargs.width : rp.args.width;
  const uint64_t rows = rp.args.rows;
  const uint64_t lines = rp.narrow ? rp.nargs.lines : rp.args.total_slots / rp.args.slots;
  CHECK(rows >= 1 && lines % rows == 0 && width * lines == total, "merged geometry");
  CHECK(width % range.x == 0, "merged width is not a multiple of the row width");
  const uint64_t per = width / range.x;  // original rows per merged row
  const uint64_t dp = rp.narrow ? rp.nargs.dst_pitch : rp.args.dst_pitch, ds = rp.narrow ? rp.nargs.dst_slice : rp.args.dst_slice;
  const uint64_t sp = rp.narrow ? rp.nargs.src_pitch : rp.args.src_pitch, ss = rp.narrow ? rp.nargs.src_slice : rp.args.src_slice;
  for (uint64_t line = 0; line < lines; ++line) {
    const uint64_t layer = line / rows, y = line % rows;
    const uint64_t d = d0 + layer * ds + y * dp, s = s0 + layer * ss + y * sp;
    // where the original geometry puts the first row of this merged row
    const uint64_t first = line * per;  // index among all original rows, layer-major
    const uint64_t oz = first / range.y, oy = first % range.y;
    CHECK(d == d0 + oz * dst.slice + oy * dst.pitch && s == s0 + oz * src.slice + oy * src.pitch, "row origin");
    if (per > 1) CHECK(dst.pitch == range.x && src.pitch == range.x, "rows merged across a gap");
    if (rp.narrow) {
      const uint64_t lpr = rp.nargs.lanes_per_row;
      CHECK(lpr >= 1 && lpr <= kRectNarrowRaggedSlots, "lanes per row %" PRIu64, lpr);
      uint64_t covered = d;  // bytes of the row below this address have been written
      for (uint64_t j = 0; j < lpr; ++j) {
        const uint64_t slot = (d & ~15ull) + 16 * j;
        if (slot >= d + width) continue;
        uint64_t lo, hi;
        if (width >= 16) {
          lo = slot > d ? slot : d;
          if (lo + 16 > d + width) lo = d + width - 16;
          hi = lo + 16;
        } else {
          lo = slot > d ? slot : d;
          hi = slot + 16 < d + width ? slot + 16 : d + width;
        }
        CHECK(lo >= d && hi <= d + width && lo <= covered, "slot %" PRIu64 " leaves a hole or the row", j);
        if (hi > covered) covered = hi;
      }
      CHECK(covered == d + width, "row not covered by its %" PRIu64 " slots", lpr);
      // the host's magic numbers divide as the kernel needs them to
      for (uint32_t n = 0; n < lpr + 64; ++n) CHECK(div_magic(n, rp.nargs.magic64) == n / lpr, "lane's row within the wave");
      if (lpr > 1) {
        const uint64_t probe = below(1ull << 38);
        CHECK(static_cast<uint64_t>((static_cast<unsigned __int128>(probe) * rp.nargs.magic64) >> 64) == probe / lpr,
              "64-bit magic");
      }
    } else {
      const uint64_t unit = 64ull * rp.unroll;
      uint64_t head = (16 - (d & 15)) & 15;
      if (head > width) head = width;
      const uint64_t n_virtual = (width - head) / 16 + ((d + head) & 255) / 16;
      const uint64_t units = n_virtual > 15 + unit ? (n_virtual - 15 + unit - 1) / unit : 1;
      CHECK(units <= rp.args.slots, "row needs %" PRIu64 " units, plan has %u slots", units, rp.args.slots);
      uint64_t at = 0;
      for (uint64_t kq = 0; kq < units; ++kq) {
        uint64_t lo, hi, vectors;
        unit_range(d, width, unit, kq, units, &lo, &hi, &vectors);
        CHECK(lo == at && hi >= lo && hi <= width, "unit %" PRIu64 " does not continue the row", kq);
        CHECK(vectors <= unit + 64, "a lane would need more than one extra vector");
        at = hi;
      }
      CHECK(at == width, "units stop short of the row's end");
    }
  }
  if (!rp.narrow) {
    CHECK(rp.args.n_waves == rp.grid * rp.args.waves_per_wg && rp.args.waves_per_wg == rp.wg_size / 64, "launch shape");
    if (!tuned || t.max_grid == 0) CHECK(rp.args.n_waves >= rp.args.total_slots, "grid smaller than the unit slots");
  } else {
    CHECK(rp.nargs.n_waves == rp.grid * rp.nargs.waves_per_wg, "launch shape");
    if (!tuned || t.max_grid == 0)
      CHECK(64ull * rp.nargs.n_waves >= static_cast<uint64_t>(rp.nargs.lines) * rp.nargs.lanes_per_row, "grid smaller than the slots");
  }
}

// The staging image of a batch: the pieces must tile every copy in order, a
// piece has at most 64 chunks and every piece but a copy's last has exactly 64,
// cutting adds no chunk to the copy, and the record indices must be the
// running sum of the pieces' chunk counts.
void one_batch_stage() {
  const size_t n = 1 + below(40);
  std::vector<mi355_blit_desc_t> descs(n);
  for (auto& d : descs) {
    d.dst = reinterpret_cast<void*>((1ull << 40) + below(1ull << 34));
    d.src = reinterpret_cast<const void*>((2ull << 40) + below(1ull << 34));
    switch (below(5)) {
      case 0: d.bytes = 0; break;
      case 1: d.bytes = 1 + below(5000); break;
      case 2: d.bytes = 1 + below(3u << 20); break;
      case 3: d.bytes = (1ull << 20) * below(5) + below(3) ; break;
      default: d.bytes = 1 + below(1ull << 28); break;
    }
  }
  BatchShape shape;
  static BatchImage image;  // reused, as the engine does
  CHECK(batch_build(descs.data(), n, &image, &shape) == MI355_BLIT_SUCCESS, "batch_build failed");
  const std::vector<BatchDesc>& pieces = image.pieces;
  const std::vector<uint32_t>& starts = image.first_record;
  CHECK(image.count == shape.pieces && pieces.size() >= image.count && starts.size() >= image.count, "image size");
  uint64_t p = 0, chunks = 0, bytes = 0;
  for (const auto& d : descs) {
    uint64_t at = 0, copy_chunks = 0;
    while (at < d.bytes) {
      CHECK(p < shape.pieces, "more pieces than counted");
      const BatchDesc& q = pieces[p];
      const uint64_t qd = reinterpret_cast<uint64_t>(q.dst), qs = reinterpret_cast<uint64_t>(q.src);
      CHECK(qd == reinterpret_cast<uint64_t>(d.dst) + at && qs == reinterpret_cast<uint64_t>(d.src) + at,
            "piece %" PRIu64 " does not continue its copy", p);
      CHECK(q.bytes >= 1 && q.bytes <= kBatchPieceBytes + 30 && at + q.bytes <= d.bytes, "piece length %" PRIu64, q.bytes);
      CHECK(starts[p] == chunks, "record index of piece %" PRIu64, p);
      // the chunk count, from the geometry of 256-byte anchored 4 KiB chunks
      const uint64_t head = q.bytes < ((16 - (qd & 15)) & 15) ? q.bytes : ((16 - (qd & 15)) & 15);
      const uint64_t body_lo = qd + head, body_hi = body_lo + (q.bytes - head) / 16 * 16;
      // 4 KiB steps from the 256-byte boundary below the body's first vector
      const uint64_t anchor = body_lo & ~255ull;
      const uint64_t c = body_hi > body_lo ? (body_hi - anchor + 4095) / 4096 : 1;
      CHECK(c <= kBatchPieceChunks, "a piece with %" PRIu64 " chunks", c);
      CHECK(at + q.bytes == d.bytes || (c == kBatchPieceChunks && (qd + q.bytes) % 256 == 0),
            "a piece of %" PRIu64 " chunks in the middle of a copy", c);
      CHECK(c == batch_desc_chunks(qd, q.bytes), "chunk count of a piece");
      copy_chunks += c;
      chunks += c;
      bytes += q.bytes;
      at += q.bytes;
      ++p;
    }
    CHECK(d.bytes == 0 || copy_chunks == batch_desc_chunks(reinterpret_cast<uint64_t>(d.dst), d.bytes),
          "cutting changed a copy's chunk count: %" PRIu64, copy_chunks);
  }
  CHECK(p == shape.pieces && chunks == shape.total_chunks && bytes == shape.total_bytes, "shape totals");
  mi355_blit_desc_t bad = descs[0];
  bad.bytes = 8;
  bad.dst = nullptr;
  CHECK(batch_build(&bad, 1, &image, &shape) == MI355_BLIT_ERROR_INVALID_ARGUMENT, "NULL destination accepted");

  // The bound on the records of uncut copies (device-resident descriptors, of
  // which the host only knows a bound on the total size) must cover their
  // actual chunk counts, also when the bound on the bytes is exact.
  uint64_t uncut_chunks = 0, uncut_bytes = 0;
  for (const auto& d : descs) {
    uncut_chunks += batch_desc_chunks(reinterpret_cast<uint64_t>(d.dst), d.bytes);
    uncut_bytes += d.bytes;
  }
  if (uncut_bytes) {
    const uint64_t bound = batch_bound_chunks(n, uncut_bytes);
    CHECK(bound >= uncut_chunks, "bound of %" PRIu64 " records for %" PRIu64, bound, uncut_chunks);
    CHECK(bound <= uncut_chunks + 2 * n + 1, "bound of %" PRIu64 " records is loose for %" PRIu64, bound, uncut_chunks);
  }
  CHECK(batch_bound_chunks(1, 1ull << 62) == 0, "a bound beyond 32-bit record indices accepted");
}

// What the host sizes for device-resident descriptors, whose lengths it cannot
// see: never more records than the cap, never a grid without a record behind
// each of its chunks, a bound followed exactly while it fits.
void one_batch_device_sizing() {
  const uint64_t n = 1 + below(1ull << (1 + below(32)));
  const BatchDeviceSizing u = batch_device_sizing(n, 0);
  CHECK(u.records >= kBatchMinDeviceRecords && u.records <= kBatchMaxDeviceRecords, "records %" PRIu64, u.records);
  CHECK(u.grid_chunks >= 1 && u.grid_chunks <= u.records, "grid of %" PRIu64 " chunks, %" PRIu64 " records",
        u.grid_chunks, u.records);
  CHECK(u.grid_chunks == 8 * n || u.grid_chunks == kBatchMaxDeviceRecords, "grid of %" PRIu64 " chunks for %" PRIu64,
        u.grid_chunks, n);
  CHECK(u.bytes == u.grid_chunks * 4096, "assumed bytes");
  const uint64_t bytes = 1 + below(1ull << (1 + below(50)));
  const BatchDeviceSizing b = batch_device_sizing(n, bytes);
  const uint64_t want = batch_bound_chunks(n, bytes);
  if (want == 0) {  // more chunks than 32-bit record indices count
    CHECK(b.records == 0, "records %" PRIu64 " for a bound beyond the record indices", b.records);
    return;
  }
  CHECK(b.grid_chunks >= 1 && b.grid_chunks <= b.records && b.bytes == bytes, "grid of %" PRIu64 " chunks, %" PRIu64 " records",
        b.grid_chunks, b.records);
  const uint64_t likely = bytes / 4096 + n / 2 + 1 > n ? bytes / 4096 + n / 2 + 1 : n;
  CHECK(b.grid_chunks == b.records || b.grid_chunks == likely, "grid of %" PRIu64 " chunks for a bound", b.grid_chunks);
  CHECK(b.records == (want < kBatchMaxDeviceRecords ? want : kBatchMaxDeviceRecords),
        "records %" PRIu64 " for a bound of %" PRIu64 " chunks", b.records, want);
  CHECK(batch_device_sizing(1, 1ull << 62).records == 0, "a bound beyond 32-bit record indices accepted");
}

// Division by an invariant through its magic number must be exact for every
// 32-bit dividend: divisors and dividends at the extremes and at random.
void one_magic_division() {
  const uint32_t ds[] = {1, 2, 3, 5, 7, 255, 256, 257, 65535, 65536, 0x7fffffffu, 0x80000000u, 0xfffffffeu, 0xffffffffu,
                         static_cast<uint32_t>(1 + below(0xffffffffull)), static_cast<uint32_t>(1 + below(100000))};
  for (uint32_t d : ds) {
    const uint64_t m = magic_divisor(d);
    const uint32_t ns[] = {0, 1, d - 1, d, d + 1, 2 * d - 1, 2 * d, 0x7fffffffu, 0x80000000u, 0xfffffffeu, 0xffffffffu,
                           static_cast<uint32_t>(below(1ull << 32)), static_cast<uint32_t>(below(1ull << 32)),
                           0xffffffffu / d * d, 0xffffffffu / d * d - 1};
    for (uint32_t n : ns) {
      const uint32_t q = div_magic(n, m);
      CHECK(q == n / d, "%u / %u through the magic number gives %u", n, d, q);
    }
  }
}

// Launch shape of the batched copy: a wave for every quarter chunk (or what the
// tuning says) unless the grid is capped; the fixed shape ignores the tuning's
// workgroup and unroll but keeps its grid cap and cache policy.
void one_batch_launch() {
  const uint64_t chunks = 1 + below(3000000);
  const uint64_t bytes = chunks * 4096;
  mi355_blit_tuning_t t = random_tuning();
  const bool tuned = below(2), tunable = below(2);
  mi355_blit_plan_t p;
  const BatchLaunch l = plan_batch_records(chunks, bytes, bytes >= (4ull << 20), tuned ? &t : nullptr, tunable, &p);
  CHECK(p.kernel == MI355_BLIT_KERNEL_COPY_BATCH && p.body_vecs == chunks, "kernel / chunk count");
  CHECK(l.split * p.unroll == 4 && l.waves_per_wg == p.wg_size / 64, "split %u unroll %u", l.split, p.unroll);
  CHECK(l.n_waves == static_cast<uint64_t>(p.grid) * l.waves_per_wg, "wave count");
  const bool capped = tuned && t.max_grid && t.max_grid < (chunks * l.split + l.waves_per_wg - 1) / l.waves_per_wg;
  if (capped) CHECK(p.grid == t.max_grid, "grid cap");
  else CHECK(l.n_waves >= chunks * l.split && l.n_waves < chunks * l.split + l.waves_per_wg, "one wave per part of a chunk");
  if (!tuned || !tunable) CHECK(p.wg_size == 64 && l.split == 4, "fixed shape");
  // the record touched ahead belongs to the same XCD: whole rounds of 8 workgroups away
  const bool no_prefetch = tuned && t.batch_prefetch == 1;
  CHECK(no_prefetch ? l.prefetch_waves == 0 : (l.prefetch_waves % (8 * l.waves_per_wg) == 0 || (tuned && t.batch_prefetch > 1)),
        "prefetch distance %u", l.prefetch_waves);
  if (!tuned) {
    CHECK(p.nt_load == (bytes >= (4ull << 20)) && p.store_policy == (p.nt_load ? MI355_BLIT_STORE_NT : MI355_BLIT_STORE_CACHED),
          "cache policy by size");
    CHECK(p.xcd_run == (bytes >= (64ull << 20) ? 4 * 528u : 0u), "XCD runs by size: %u", p.xcd_run);
  }
}

// The XCD permutation of a launch: workgroups below make_xcd_runs(grid, run).full swap
// places among themselves (a bijection), each XCD (b % 8) gets whole runs of
// neighbouring workgroups in launch order, the rest keep their place.
void one_xcd_permutation() {
  const uint32_t run = 2 + static_cast<uint32_t>(below(700));
  const uint32_t grid = static_cast<uint32_t>(below(40000));
  const XcdRuns x = make_xcd_runs(grid, run);
  const uint32_t full = x.full;
  CHECK(x.run == run && full <= grid && full % (8 * run) == 0 && grid - full < 8 * run, "runs of %u in a grid of %u: %u take part", run, grid, full);
  CHECK(make_xcd_runs(grid, 0).full == 0 && make_xcd_runs(grid, 1).full == 0 && make_xcd_runs(grid, 1).run == 0,
        "no permutation without a run");
  std::vector<uint8_t> seen(full, 0);
  std::vector<uint32_t> last(8, 0);
  for (uint32_t b = 0; b < full; ++b) {
    const uint32_t w = xcd_workgroup(b, x);
    CHECK(w < full && !seen[w], "workgroup %u -> %u (run %u) out of range or taken twice", b, w, run);
    if (w < full) seen[w] = 1;
    // within a round the work of XCD x is [x * run, (x + 1) * run), taken in launch order
    CHECK((w % (8 * run)) / run == (b & 7), "workgroup %u works on another XCD's run", b);
    if (b >= 8) CHECK(w == last[b & 7] + 1 || w == last[b & 7] + 1 + 7 * run, "XCD %u jumps from %u to %u", b & 7, last[b & 7], w);
    last[b & 7] = w;
  }
  const mi355_blit_tuning_t linear{0, 0, 0, 0, 0, 1, 0, 0}, forced{0, 0, 0, 0, 0, 99, 0, 0};
  CHECK(plan_xcd_run(288, nullptr) == 288 && plan_xcd_run(288, &linear) == 0 && plan_xcd_run(0, &forced) == 99,
        "tuning of the run");
}

// The bounded wait of the AQL engine (csrc/aql_wait.h) without a GPU: the
// slice is a callable, here a stand-in for hsa_signal_wait_scacquire on a
// signal that nobody completes (it sleeps the slice out and reports 1).
void wait_helper_cases() {
  using clock = std::chrono::steady_clock;
  int slices = 0;
  auto never = [&](uint64_t ticks) -> int64_t {
    ++slices;
    std::this_thread::sleep_for(std::chrono::microseconds(ticks));
    return 1;
  };
  // 1. the flag set from another thread ends a wait that is in progress
  {
    std::atomic<bool> error{false};
    std::thread setter([&] {
      std::this_thread::sleep_for(std::chrono::milliseconds(30));
      error.store(true, std::memory_order_release);
    });
    const auto t0 = clock::now();
    const int rc = wait_below_one(never, error, 1000);
    const double ms = std::chrono::duration<double, std::milli>(clock::now() - t0).count();
    setter.join();
    CHECK(rc == kWaitError, "a wait on a dead queue returned 0x%x", rc);
    CHECK(ms >= 25.0 && ms < 1000.0 && slices >= 5, "the wait took %.1f ms in %d slices", ms, slices);
  }
  // 2. a completed signal wins over the flag: the value is looked at first
  {
    std::atomic<bool> error{true};
    CHECK(wait_below_one([](uint64_t) -> int64_t { return 0; }, error, 1000) == kWaitSuccess, "0 with the flag set");
  }
  // 3. a negative value is a failed command, whatever the flag says
  {
    std::atomic<bool> error{false};
    CHECK(wait_below_one([](uint64_t) -> int64_t { return -1; }, error, 1000) == kWaitError, "negative value");
  }
  // 4. values above 0 keep the wait going until the signal gets there
  {
    std::atomic<bool> error{false};
    int64_t v = 5;
    int calls = 0;
    const int rc = wait_below_one([&](uint64_t) -> int64_t { ++calls; return --v; }, error, 1000);
    CHECK(rc == kWaitSuccess && calls == 5, "counted down in %d calls, rc 0x%x", calls, rc);
  }
  // 5. the flag already set and the signal never completing: one slice, then the error
  {
    std::atomic<bool> error{true};
    slices = 0;
    CHECK(wait_below_one(never, error, 100) == kWaitError && slices == 1, "%d slices", slices);
  }
}

// The engine choice of GetBlitObject restated in csrc/blit_plan.h against the
// oracle's restatement of the same lines (amd_gpu_agent.cpp:2390-2397).
void engine_policy_cases() {
  const uint64_t sizes[] = {0, 1, 4095, 4096, (128u << 10) - 1, 128u << 10, (1u << 20) - 1, 1u << 20, (1u << 20) + 1,
                            1ull << 30, ~0ull};
  const uint64_t flags[] = {0, 1, 128u << 10, 1u << 20, 1ull << 40, ~0ull};
  for (uint64_t size : sizes)
    for (uint64_t flag : flags) {
      const bool blit = oracle_ref_same_gpu_uses_blit_kernel(size, flag) != 0;
      CHECK(policy_same_gpu_engine(size, flag) == (blit ? uint32_t(MI355_ENGINE_BLIT_KERNEL) : uint32_t(MI355_ENGINE_SDMA)),
            "size %" PRIu64 " flag %" PRIu64, size, flag);
    }
  // core/util/flag.h:206-207: unset or empty -> 1 MiB, otherwise atoi
  unsetenv("HSA_FORCE_SDMA_SIZE");
  CHECK(policy_force_sdma_size() == 1024 * 1024, "default");
  setenv("HSA_FORCE_SDMA_SIZE", "", 1);
  CHECK(policy_force_sdma_size() == 1024 * 1024, "empty");
  setenv("HSA_FORCE_SDMA_SIZE", "131072", 1);
  CHECK(policy_force_sdma_size() == 131072, "128 KiB");
  setenv("HSA_FORCE_SDMA_SIZE", "0", 1);
  CHECK(policy_force_sdma_size() == 0 && policy_same_gpu_engine(1, 0) == MI355_ENGINE_BLIT_KERNEL, "0: always the blit kernel");
  setenv("HSA_FORCE_SDMA_SIZE", "-1", 1);  // atoi's int becomes a size_t: every size is below it
  CHECK(policy_same_gpu_engine(1ull << 40, policy_force_sdma_size()) == MI355_ENGINE_SDMA, "-1");
  unsetenv("HSA_FORCE_SDMA_SIZE");
}

}  // namespace

namespace {
using namespace mi355;

// The policy around hsa_amd_memory_lock (csrc/aql_host_lock.h), with the two
// runtime calls injected: the branch that succeeds -- which the GPU boxes of
// this pool never take, they refuse to lock existing memory -- must hand out
// the mapped address and unlock the host pointer exactly once; a refusal that
// speaks for the system is remembered for that agent only, one that speaks for
// the pointer is not remembered at all (runtime.cpp:521-537).
struct FakeLocker {
  static int mode;      // status the next lock() answers with
  static int locks, unlocks;
  static void* last_unlocked;
  static uint64_t last_agent;
  static int lock(void* ptr, size_t, uint64_t agent, void** mapped) {
    ++locks;
    last_agent = agent;
    if (mode != MI355_BLIT_SUCCESS) return mode;
    *mapped = static_cast<char*>(ptr) + 0x1000;  // the GPU's address of the range differs from the host's
    return MI355_BLIT_SUCCESS;
  }
  static int unlock(void* ptr) {
    ++unlocks;
    last_unlocked = ptr;
    return MI355_BLIT_SUCCESS;
  }
};
int FakeLocker::mode = 0, FakeLocker::locks = 0, FakeLocker::unlocks = 0;
void* FakeLocker::last_unlocked = nullptr;
uint64_t FakeLocker::last_agent = 0;

void host_lock_cases() {
  const HostLockFns fns{FakeLocker::lock, FakeLocker::unlock};
  HostLockLatch latch;
  char buffer[64];
  const uint64_t gpu_a = 0x1111, gpu_b = 0x2222;
  {
    // success: mapped address out, one unlock of the host pointer at scope end
    FakeLocker::mode = MI355_BLIT_SUCCESS;
    void* mapped = nullptr;
    {
      ScopedHostLock l(fns, latch);
      CHECK(l.Lock(gpu_a, buffer, sizeof buffer, &mapped) == MI355_BLIT_SUCCESS, "lock that succeeds");
      CHECK(mapped == buffer + 0x1000 && FakeLocker::last_agent == gpu_a, "mapped address / agent");
      CHECK(FakeLocker::unlocks == 0, "unlocked too early");
      void* again = nullptr;
      CHECK(l.Lock(gpu_a, buffer, sizeof buffer, &again) != MI355_BLIT_SUCCESS && FakeLocker::locks == 1,
            "one range per object");
    }
    CHECK(FakeLocker::locks == 1 && FakeLocker::unlocks == 1 && FakeLocker::last_unlocked == buffer, "unlock exactly once");
  }
  {
    // a refusal about this pointer: nothing unlocked, nothing remembered
    FakeLocker::mode = MI355_BLIT_ERROR_INVALID_ARGUMENT;
    void* mapped = nullptr;
    {
      ScopedHostLock l(fns, latch);
      CHECK(l.Lock(gpu_a, buffer, sizeof buffer, &mapped) == MI355_BLIT_ERROR_INVALID_ARGUMENT, "status passed on");
    }
    CHECK(FakeLocker::unlocks == 1, "a failed lock must not unlock");
    CHECK(!latch.refused(gpu_a), "a pointer's refusal was remembered");
    FakeLocker::mode = MI355_BLIT_SUCCESS;
    ScopedHostLock l(fns, latch);
    CHECK(l.Lock(gpu_a, buffer, sizeof buffer, &mapped) == MI355_BLIT_SUCCESS && FakeLocker::locks == 3, "asked again");
  }
  CHECK(FakeLocker::unlocks == 2, "second unlock");
  for (int status : {static_cast<int>(MI355_BLIT_ERROR_OUT_OF_RESOURCES), static_cast<int>(MI355_BLIT_ERROR)}) {
    // the system's refusal: remembered, for that agent only
    HostLockLatch fresh;
    const int before = FakeLocker::locks;
    FakeLocker::mode = status;
    void* mapped = nullptr;
    {
      ScopedHostLock l(fns, fresh);
      CHECK(l.Lock(gpu_a, buffer, sizeof buffer, &mapped) == status, "refusal passed on");
    }
    CHECK(fresh.refused(gpu_a) && !fresh.refused(gpu_b), "latched for the agent that was refused only");
    FakeLocker::mode = MI355_BLIT_SUCCESS;
    {
      ScopedHostLock l(fns, fresh);
      CHECK(l.Lock(gpu_a, buffer, sizeof buffer, &mapped) != MI355_BLIT_SUCCESS && FakeLocker::locks == before + 1,
            "a refused agent is not asked again");
    }
    {
      ScopedHostLock l(fns, fresh);
      CHECK(l.Lock(gpu_b, buffer, sizeof buffer, &mapped) == MI355_BLIT_SUCCESS && FakeLocker::locks == before + 2,
            "another agent is still asked");
    }
  }
  CHECK(FakeLocker::unlocks == 4, "unlock count at the end: %d", FakeLocker::unlocks);
}

}  // namespace

int main(int argc, char** argv) {
  wait_helper_cases();
  engine_policy_cases();
  host_lock_cases();
  const long cases = argc > 1 ? std::atol(argv[1]) : 200000;
  for (long i = 0; i < cases; ++i) {
    one_copy_plan();
    one_fill_plan();
    one_rect_plan();
    if (i % 8 == 0) one_batch_stage();
    if (i % 64 == 0) one_xcd_permutation();
    if (i % 16 == 0) one_magic_division();
    if (i % 8 == 0) one_batch_launch();
    if (i % 8 == 0) one_batch_device_sizing();
  }
  std::printf("%s: %ld cases each of copy, fill and region plans, %d failures\n", g_failures ? "FAILED" : "OK", cases,
              g_failures);
  return g_failures ? 1 : 0;
}
