// The blit kernels themselves (csrc/blit_kernels.h, compiled unchanged) run on
// the CPU, lane by lane in lock step (lane_emulation.h), launched with the
// argument blocks the product's own host code makes (plan_copy / plan_fill /
// make_copy_args, batch_build + plan_batch_records, plan_rect).  What it pins:
//
//  * no over-read: every load of a copy lies inside the aligned dwords that
//    hold a requested source byte, [src & ~3, (src + n + 3) & ~3) -- per copy of
//    a batch, per row of a region -- and every store inside [dst, dst + n).
//    The reference's shaders mask their edge accesses with EXEC and never
//    over-read either (projects/rocr-runtime/runtime/hsa-runtime/core/runtime/
//    blit_shaders/blit_copyAligned.s:108-128, 236-256); a GPU test cannot show
//    this without a fault, a CPU run can.  Sources and destinations also end
//    exactly where their heap blocks end, so that AddressSanitizer sees
//    anything that slipped past the accessors.
//  * the result: the destination holds the source's bytes and nothing around
//    it changed, for every kernel, unroll, grid cap and XCD permutation.
//
//   test_kernels_on_cpu [--shard I/N] [--self-test] [--quick]
//   exit status 0 = all checks passed (self test: the planted fault was found)
#include <cinttypes>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#define MI355_BLIT_DEVICE_HEADER "lane_emulation.h"
#include "blit_kernels.h"

#include "blit_batch_host.h"
#include "blit_plan.h"
#include "blit_rect.h"

namespace {

using namespace mi355;
using lane_emu::g_check;
using lane_emu::g_m;

uint64_t g_state = 0x9E3779B97F4A7C15ull;
uint64_t rnd() {  // splitmix64
  uint64_t z = (g_state += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
uint64_t below(uint64_t n) { return n ? rnd() % n : 0; }

uint64_t g_cases = 0, g_failures = 0, g_waves = 0;
unsigned g_shard = 0, g_shards = 1;

void fail(const char* what, const std::string& detail) {
  if (g_failures++ < 20) std::printf("FAIL %s: %s\n", what, detail.c_str());
}

std::string fmt(const char* f, ...) __attribute__((format(printf, 1, 2)));
std::string fmt(const char* f, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, f);
  vsnprintf(buf, sizeof buf, f, ap);
  va_end(ap);
  return buf;
}

// ---- kernel tables, from the same lists as the product's ---------------------

typedef void (*copy_kernel_t)(CopyArgs);
typedef void (*fill_kernel_t)(FillArgs);
typedef void (*batch_kernel_t)(BatchCopyArgs);
typedef void (*batch_lookup_kernel_t)(BatchLookupArgs);
typedef void (*rect_kernel_t)(RectArgs);
typedef void (*rect_narrow_kernel_t)(RectNarrowArgs);

struct CopyVariant { unsigned unroll, nt_load, store, realign; copy_kernel_t fn; };
struct FillVariant { unsigned unroll, store; fill_kernel_t fn; };
struct BatchVariant { unsigned split, nt_load, store; batch_kernel_t fn; };
struct BatchLookupVariant { unsigned nt_load, store; batch_lookup_kernel_t fn; };
struct RectVariant { unsigned unroll, nt_load, store; rect_kernel_t fn; };
struct RectNarrowVariant { unsigned nt_load, store; rect_narrow_kernel_t fn; };

#define ROW_COPY(U, L, S, R) {U, L, S, R, mi355_copy_u##U##_l##L##_s##S##_r##R},
const CopyVariant kCopyVariants[] = {MI355_FOR_EACH_COPY_KERNEL(ROW_COPY)};
#define ROW_FILL(U, S) {U, S, mi355_fill_u##U##_s##S},
const FillVariant kFillVariants[] = {MI355_FOR_EACH_FILL_KERNEL(ROW_FILL)};
#define ROW_BATCH(P, L, S) {P, L, S, mi355_batch_records_p##P##_l##L##_s##S},
const BatchVariant kBatchVariants[] = {MI355_FOR_EACH_BATCH_RECORDS_KERNEL(ROW_BATCH)};
#define ROW_LOOKUP(L, S) {L, S, mi355_batch_lookup_l##L##_s##S},
const BatchLookupVariant kBatchLookupVariants[] = {MI355_FOR_EACH_BATCH_LOOKUP_KERNEL(ROW_LOOKUP)};
#define ROW_RECT(U, L, S) {U, L, S, mi355_rect_u##U##_l##L##_s##S},
const RectVariant kRectVariants[] = {MI355_FOR_EACH_RECT_KERNEL(ROW_RECT)};
#define ROW_NARROW(L, S) {L, S, mi355_rect_narrow_l##L##_s##S},
const RectNarrowVariant kRectNarrowVariants[] = {MI355_FOR_EACH_RECT_NARROW_KERNEL(ROW_NARROW)};

// ---- buffers that end where their heap block ends ------------------------------

// n bytes whose address is `residue` modulo `modulus` (a power of two up to
// 4096) and whose heap block ends `slack_after` bytes behind them.
struct Block {
  uint8_t* raw = nullptr;
  uint8_t* p = nullptr;
  size_t n = 0;
  Block() {}
  Block(size_t bytes, size_t residue, size_t modulus, size_t slack_after = 0) { make(bytes, residue, modulus, slack_after); }
  Block(const Block&) = delete;
  Block& operator=(const Block&) = delete;
  void make(size_t bytes, size_t residue, size_t modulus, size_t slack_after = 0) {
    std::free(raw);
    const size_t total = residue + bytes + slack_after;
    void* q = nullptr;
    // AddressSanitizer ends the block exactly `total` bytes after its start
    if (posix_memalign(&q, modulus < 16 ? 16 : modulus, total ? total : 1) != 0) std::abort();
    raw = static_cast<uint8_t*>(q);
    p = raw + residue;
    n = bytes;
  }
  ~Block() { std::free(raw); }
};

void fill_random(uint8_t* p, size_t n) {
  size_t i = 0;
  for (; i + 8 <= n; i += 8) {
    const uint64_t v = rnd();
    std::memcpy(p + i, &v, 8);
  }
  for (; i < n; ++i) p[i] = static_cast<uint8_t>(rnd());
}

constexpr uint8_t kGuard = 0xEE;

// dword-granular extent of a source range
void allow_source(const uint8_t* s, uint64_t n) {
  const uintptr_t lo = reinterpret_cast<uintptr_t>(s) & ~static_cast<uintptr_t>(3);
  const uintptr_t hi = (reinterpret_cast<uintptr_t>(s) + n + 3) & ~static_cast<uintptr_t>(3);
  g_check.allow_read(reinterpret_cast<const void*>(lo), hi - lo);
}

bool machine_ok(const char* what, const std::string& detail) {
  bool ok = true;
  if (g_m.errors) {
    fail(what, detail + ": " + g_m.first_error);
    g_m.errors = 0;
    ok = false;
  }
  if (g_check.violations) {
    fail(what, detail + fmt(": %" PRIu64 " accesses outside what the command may touch; first: %s",
                             g_check.violations, g_check.first));
    ok = false;
  }
  return ok;
}

// ---- linear copy ---------------------------------------------------------------

struct CopyCase {
  uint64_t n;
  unsigned so, d256;  // source address mod 16, destination address mod 256
  mi355_blit_tuning_t t;
};

std::string describe(const CopyCase& c, const mi355_blit_plan_t& p) {
  return fmt("copy of %" PRIu64 " bytes, src&15=%u dst&255=%u, unroll %u wg %u grid %u xcd_run %u", c.n, c.so, c.d256,
             p.unroll, p.wg_size, p.grid, p.xcd_run);
}

// returns the number of violations found (for the self test)
uint64_t run_copy(const CopyCase& c, bool expect_clean = true) {
  ++g_cases;
  // 64 guard bytes on both sides of the destination, inside the block
  Block dst(c.n + 128, (c.d256 + 256 - 64) % 256, 256);
  // the source block ends at the end of the last dword that holds a source byte
  const size_t pad = (0 - (c.so + c.n)) & 3;
  Block src(c.n, 16 + c.so, 16, pad);
  fill_random(src.raw, 16 + c.so + c.n + pad);
  std::memset(dst.p, kGuard, c.n + 128);
  uint8_t* d = dst.p + 64;
  mi355_blit_plan_t p;
  if (plan_copy(reinterpret_cast<uint64_t>(d), reinterpret_cast<uint64_t>(src.p), c.n, 256, &c.t, &p) != 0) {
    fail("plan_copy", "refused");
    return 0;
  }
  copy_kernel_t k = nullptr;
  for (const CopyVariant& v : kCopyVariants)
    if (v.unroll == p.unroll && v.nt_load == p.nt_load && v.store == p.store_policy && v.realign == (p.byte_shift ? 1u : 0u))
      k = v.fn;
  if (!k) {
    fail("copy kernel", "no variant for the plan");
    return 0;
  }
  const CopyArgs a = make_copy_args(p, d, src.p, c.n);
  g_check.clear();
  allow_source(src.p, c.n);
  g_check.allow_write(d, c.n);
  g_check.seal();
  lane_emu::launch(k, a, p.grid, p.wg_size);
  g_waves += static_cast<uint64_t>(p.grid) * (p.wg_size / 64);
  const uint64_t found = g_check.violations + g_m.errors;
  if (!expect_clean) {
    g_m.errors = 0;
    return found;  // accesses only: wrong bytes are not what the self test looks for
  }
  if (!machine_ok("linear copy", describe(c, p))) return found;
  if (std::memcmp(d, src.p, c.n) != 0) fail("linear copy", describe(c, p) + ": destination differs from the source");
  for (unsigned i = 0; i < 64; ++i)
    if (dst.p[i] != kGuard || d[c.n + i] != kGuard) {
      fail("linear copy", describe(c, p) + ": bytes around the destination changed");
      break;
    }
  return found;
}

// Lengths around everything the kernels cut at: the 16-byte vector, the
// 256-byte anchor, the tile of 1, 2 and 4 KiB, and a few tiles.
std::vector<uint64_t> edge_lengths(bool quick) {
  std::vector<uint64_t> v;
  for (uint64_t n = 1; n <= (quick ? 80u : 1100u); ++n) v.push_back(n);
  const int deltas[] = {-33, -17, -16, -15, -4, -3, -1, 0, 1, 3, 4, 15, 16, 17, 33};
  for (uint64_t k : {1, 2, 3, 4, 5, 8, 9})
    for (int d : deltas)
      if (1024 * k + d > v.back()) v.push_back(1024 * k + d);
  return v;
}

void linear_copies(bool quick) {
  const std::vector<uint64_t> lens = edge_lengths(quick);
  uint64_t index = 0;
  for (unsigned so = 0; so < 16; ++so)
    for (unsigned dl = 0; dl < 16; ++dl) {
      for (size_t li = 0; li < lens.size(); ++li, ++index) {
        if (index % g_shards != g_shard) continue;
        const uint64_t n = lens[li];
        // every destination residue mod 256 comes up: the 16-byte slot within the line varies with the case
        const unsigned d256 = dl + 16 * static_cast<unsigned>((index * 7 + li) % 16);
        // the plan's own choice at this size ...
        CopyCase c{n, so, d256, mi355_blit_tuning_t{}};
        run_copy(c);
        // ... and, for the lengths around the tiles, every unroll, capped grids, other workgroup sizes and the
        // XCD permutation (which only takes effect on grids of 16 workgroups or more: runs of 2)
        if ((n < 700 || (n < 1100 && n % 16 != 1)) && (n % 16) != 3) continue;
        for (unsigned unroll : {1u, 2u, 4u}) {
          mi355_blit_tuning_t t{};
          t.unroll = unroll;
          t.wg_size = (index + unroll) % 3 == 0 ? 256 : 64;
          run_copy(CopyCase{n, so, d256, t});
          t.max_grid = 1 + static_cast<uint32_t>((index + unroll) % 3);
          run_copy(CopyCase{n, so, d256, t});
        }
      }
    }
  // longer copies on single-wave workgroups in XCD runs of 2 and 3, all pairs
  for (unsigned so = 0; so < 16; ++so)
    for (unsigned dl = 0; dl < 16; ++dl, ++index) {
      if (index % g_shards != g_shard) continue;
      mi355_blit_tuning_t t{};
      t.wg_size = 64;
      t.unroll = 1 + static_cast<uint32_t>(index % 2);
      t.xcd_run = 2 + static_cast<uint32_t>(index % 2);
      const uint64_t n = (quick ? 20000 : 60000) + below(9000);
      run_copy(CopyCase{n, so, dl + 16 * static_cast<unsigned>(below(16)), t});
    }
}

// ---- fill -------------------------------------------------------------------------

void fills(bool quick) {
  std::vector<uint64_t> dwords;
  for (uint64_t n = 1; n <= 90; ++n) dwords.push_back(n);
  for (uint64_t k : {1, 2, 4, 5})
    for (int d : {-5, -4, -3, -1, 0, 1, 3, 4, 5}) dwords.push_back(256 * k + d);
  uint64_t index = 0;
  for (unsigned res = 0; res < 256; res += 4)
    for (uint64_t n : dwords)
      for (unsigned variant = 0; variant < (quick ? 2u : 4u); ++variant, ++index) {
        if (index % g_shards != g_shard) continue;
        ++g_cases;
        mi355_blit_tuning_t t{};
        if (variant) {
          t.unroll = 1u << (variant - 1);
          t.wg_size = variant == 2 ? 128 : 64;
          if (index % 2) t.max_grid = 1 + index % 3;
        }
        Block dst(4 * n + 128, (res + 256 - 64) % 256, 256);
        std::memset(dst.p, kGuard, 4 * n + 128);
        uint8_t* d = dst.p + 64;
        const uint32_t value = static_cast<uint32_t>(rnd()) | 1;
        mi355_blit_plan_t p;
        if (plan_fill(reinterpret_cast<uint64_t>(d), n, 256, &t, &p) != 0) {
          fail("plan_fill", "refused");
          continue;
        }
        fill_kernel_t k = nullptr;
        for (const FillVariant& v : kFillVariants)
          if (v.unroll == p.unroll && v.store == p.store_policy) k = v.fn;
        if (!k) {
          fail("fill kernel", "no variant for the plan");
          continue;
        }
        const FillArgs a = make_fill_args(p, d, value, n);
        g_check.clear();
        g_check.allow_write(d, 4 * n);
        g_check.seal();
        lane_emu::launch(k, a, p.grid, p.wg_size);
        g_waves += static_cast<uint64_t>(p.grid) * (p.wg_size / 64);
        const std::string what = fmt("fill of %" PRIu64 " dwords at residue %u, unroll %u wg %u grid %u", n, res, p.unroll,
                                     p.wg_size, p.grid);
        if (!machine_ok("fill", what)) continue;
        if (g_check.loads) fail("fill", what + ": a fill has no business loading");
        bool good = true;
        for (uint64_t i = 0; i < n && good; ++i) {
          uint32_t w;
          std::memcpy(&w, d + 4 * i, 4);
          good = w == value;
        }
        for (unsigned i = 0; i < 64 && good; ++i) good = dst.p[i] == kGuard && d[4 * n + i] == kGuard;
        if (!good) fail("fill", what + ": wrong dwords or changed bytes around them");
      }
}

// ---- batched copies ----------------------------------------------------------------

struct BatchBuffers {
  std::vector<Block*> src, dst;
  std::vector<mi355_blit_desc_t> descs;
  ~BatchBuffers() {
    for (Block* b : src) delete b;
    for (Block* b : dst) delete b;
  }
};

// every copy in heap blocks of its own: a stray access cannot land in a neighbour
void make_batch(const std::vector<uint64_t>& lens, BatchBuffers* out) {
  for (uint64_t n : lens) {
    const unsigned so = static_cast<unsigned>(below(16)), d256 = static_cast<unsigned>(below(256));
    const size_t pad = (0 - (so + n)) & 3;
    Block* s = new Block(n, 16 + so, 16, pad);
    Block* d = new Block(n + 128, (d256 + 256 - 64) % 256, 256);
    fill_random(s->raw, 16 + so + n + pad);
    std::memset(d->p, kGuard, n + 128);
    out->src.push_back(s);
    out->dst.push_back(d);
    out->descs.push_back(mi355_blit_desc_t{d->p + 64, s->p, n});
  }
}

void allow_batch_data(const BatchBuffers& b) {
  for (const mi355_blit_desc_t& d : b.descs) {
    allow_source(static_cast<const uint8_t*>(d.src), d.bytes);
    g_check.allow_write(d.dst, d.bytes);
  }
}

void check_batch_result(const BatchBuffers& b, const char* what, const std::string& detail) {
  for (size_t i = 0; i < b.descs.size(); ++i) {
    const mi355_blit_desc_t& d = b.descs[i];
    const uint8_t* dp = static_cast<const uint8_t*>(d.dst);
    bool good = std::memcmp(dp, d.src, d.bytes) == 0;
    for (unsigned k = 0; k < 64 && good; ++k) good = dp[-64 + static_cast<int>(k)] == kGuard && dp[d.bytes + k] == kGuard;
    if (!good) {
      fail(what, detail + fmt(": copy %zu of %" PRIu64 " bytes differs or the bytes around it changed", i, d.bytes));
      return;
    }
  }
}

std::vector<uint64_t> batch_lengths(unsigned which, bool quick) {
  std::vector<uint64_t> v;
  if (which == 0) {
    // zero-length entries (whole waves of them), lengths around the vector and the 4 KiB chunk, and copies that
    // are cut into several pieces of 64 chunks
    v.assign(70, 0);
    for (uint64_t n = 1; n < 49; ++n) v.push_back(n);
    for (uint64_t n : {0, 4095, 4096, 4097, 4096 + 15, 8192, 8193, 12288 + 31, 0, 77, 0}) v.push_back(n);
    v.push_back(quick ? 270000 : 600003);
    v.insert(v.end(), 130, 0);
    v.push_back(9);
    v.push_back(262144 + 4096 - 17);
  } else if (which == 4) {
    // more than 1024 copies: the prefix sum's first level has several workgroups
    const unsigned n = quick ? 1100 : 2600;
    for (unsigned i = 0; i < n; ++i) v.push_back(below(7) == 0 ? 0 : 1 + below(i % 50 == 0 ? 9000 : 300));
  } else {
    const unsigned n = quick ? 150 : 700;
    for (unsigned i = 0; i < n; ++i) {
      // log-uniform 1 B .. 64 KiB, the benchmark's mix scaled down
      double u = static_cast<double>(below(1u << 20)) / (1u << 20);
      uint64_t len = 1;
      for (double x = 16 * u; x >= 1; x -= 1) len *= 2;
      len += below(len);
      v.push_back(below(9) == 0 ? 0 : len);
    }
  }
  return v;
}

// host-resident descriptors: the host's walk, the record kernel, the copy over records
void batch_walked(unsigned which, const mi355_blit_tuning_t& t, bool quick) {
  ++g_cases;
  BatchBuffers b;
  make_batch(batch_lengths(which, quick), &b);
  BatchImage image;
  BatchShape shape;
  if (batch_build(b.descs.data(), b.descs.size(), &image, &shape) != 0) {
    fail("batch_build", "refused");
    return;
  }
  if (shape.total_chunks == 0) return;
  // the staging image as the GPU reads it, and the records
  Block stage(batch_stage_bytes(shape.pieces), 0, 64);
  batch_stage(image, stage.p);
  Block records(shape.total_chunks * sizeof(ChunkRecord), 0, 64);
  std::memset(records.p, 0xCD, records.n);
  const BatchDesc* staged = reinterpret_cast<const BatchDesc*>(stage.p);
  EmitRecordsArgs er{staged, reinterpret_cast<const uint32_t*>(staged + shape.pieces), shape.pieces,
                     reinterpret_cast<ChunkRecord*>(records.p)};
  g_check.clear();
  g_check.allow_read(stage.p, stage.n);
  g_check.allow_write(records.p, records.n);
  g_check.seal();
  lane_emu::launch(mi355_batch_emit_records, er, emit_records_grid(shape.pieces), 256);
  const std::string what = fmt("batch %u of %zu copies (%" PRIu64 " pieces, %" PRIu64 " chunks), unroll %u wg %u max_grid %u xcd_run %u",
                               which, b.descs.size(), shape.pieces, shape.total_chunks, t.unroll, t.wg_size, t.max_grid,
                               t.xcd_run);
  if (!machine_ok("batch record kernel", what)) return;

  mi355_blit_plan_t p;
  const BatchLaunch l = plan_batch_records(shape.total_chunks, shape.total_bytes, true, &t, true, &p);
  batch_kernel_t k = nullptr;
  for (const BatchVariant& v : kBatchVariants)
    if (v.split == l.split && v.nt_load == p.nt_load && v.store == p.store_policy) k = v.fn;
  if (!k) {
    fail("batch kernel", "no variant for the plan");
    return;
  }
  BatchCopyArgs bc{reinterpret_cast<const ChunkRecord*>(records.p), shape.total_chunks, nullptr, l.waves_per_wg, l.n_waves,
                   make_xcd_runs(p.grid, p.xcd_run), l.prefetch_waves, 0};
  g_check.clear();
  g_check.allow_read(records.p, records.n);
  allow_batch_data(b);
  g_check.seal();
  lane_emu::launch(k, bc, p.grid, p.wg_size);
  g_waves += static_cast<uint64_t>(p.grid) * (p.wg_size / 64);
  if (!machine_ok("batch copy over records", what)) return;
  check_batch_result(b, "batch copy over records", what);
}

// device-resident descriptors: two prefix-sum launches, one lane per record for as many records as there is room
// for, and the copy that looks the other chunks up
void batch_device(unsigned which, uint64_t capacity_percent, const mi355_blit_tuning_t& t, bool quick) {
  ++g_cases;
  BatchBuffers b;
  make_batch(batch_lengths(which, quick), &b);
  const size_t n = b.descs.size();
  uint64_t chunks = 0, bytes = 0;
  for (const mi355_blit_desc_t& d : b.descs) {
    chunks += batch_desc_chunks(reinterpret_cast<uintptr_t>(d.dst), d.bytes);
    bytes += d.bytes;
  }
  const uint64_t capacity = chunks * capacity_percent / 100 + 1;
  const uint32_t n_blocks = static_cast<uint32_t>((n + 1023) / 1024);
  Block descs(n * sizeof(BatchDesc), 0, 64);
  std::memcpy(descs.p, b.descs.data(), descs.n);
  Block priv(n * sizeof(BatchDesc), 0, 64);
  Block chunk_start((n + 1) * 4, 0, 64);
  Block block_sum(n_blocks * 4, 0, 64);
  Block records(capacity * sizeof(ChunkRecord), 0, 64);
  Block seen(8, 0, 64);
  std::memset(chunk_start.p, 0xCD, chunk_start.n);
  std::memset(block_sum.p, 0xCD, block_sum.n);
  std::memset(records.p, 0xCD, records.n);
  const bool staged = which % 2 == 1;  // as descriptors the host staged: read once, a private copy left for the others
  const BatchDesc* dev_descs = reinterpret_cast<const BatchDesc*>(staged ? priv.p : descs.p);
  const std::string what = fmt("device batch %u of %zu copies, %" PRIu64 " chunks, room for %" PRIu64 " records, wg %u max_grid %u",
                               which, n, chunks, capacity, t.wg_size, t.max_grid);

  ScanLocalArgs sl{reinterpret_cast<const BatchDesc*>(descs.p), n, reinterpret_cast<uint32_t*>(chunk_start.p),
                   reinterpret_cast<uint32_t*>(block_sum.p), staged ? reinterpret_cast<BatchDesc*>(priv.p) : nullptr};
  g_check.clear();
  g_check.allow_read(descs.p, descs.n);
  g_check.allow_write(chunk_start.p, n * 4);
  g_check.allow_write(block_sum.p, block_sum.n);
  if (staged) g_check.allow_write(priv.p, priv.n);
  g_check.seal();
  lane_emu::launch(mi355_batch_scan_local, sl, n_blocks, 1024);
  if (!machine_ok("batch prefix sum, first level", what)) return;

  ScanTopArgs st{reinterpret_cast<uint32_t*>(block_sum.p), reinterpret_cast<uint32_t*>(chunk_start.p), n, n_blocks};
  g_check.clear();
  g_check.allow_read(block_sum.p, block_sum.n);
  g_check.allow_write(block_sum.p, block_sum.n);
  g_check.allow_write(chunk_start.p + 4 * n, 4);
  g_check.seal();
  lane_emu::launch(mi355_batch_scan_top, st, 1, 1024);
  if (!machine_ok("batch prefix sum, second level", what)) return;
  uint32_t total;
  std::memcpy(&total, chunk_start.p + 4 * n, 4);
  if (total != chunks) {
    fail("batch prefix sum", what + fmt(": total %u", total));
    return;
  }

  EmitRecordsDeviceArgs er{dev_descs, reinterpret_cast<const uint32_t*>(chunk_start.p),
                           reinterpret_cast<const uint32_t*>(block_sum.p), n, reinterpret_cast<ChunkRecord*>(records.p), capacity};
  g_check.clear();
  g_check.allow_read(dev_descs, n * sizeof(BatchDesc));
  g_check.allow_read(chunk_start.p, chunk_start.n);
  g_check.allow_read(block_sum.p, block_sum.n);
  g_check.allow_write(records.p, records.n);
  g_check.seal();
  lane_emu::launch(mi355_batch_emit_records_lookup, er, static_cast<unsigned>((capacity + 255) / 256), 256);
  if (!machine_ok("batch record kernel, one lane per record", what)) return;

  // the grid is sized from a bound, as mi355_blit_copy_batch_bounded does it
  const BatchDeviceSizing sizing = batch_device_sizing(n, bytes ? bytes : 1);
  mi355_blit_plan_t p;
  const BatchLaunch l = plan_batch_records(sizing.grid_chunks, sizing.bytes, true, &t, false, &p);
  batch_lookup_kernel_t k = nullptr;
  for (const BatchLookupVariant& v : kBatchLookupVariants)
    if (v.nt_load == p.nt_load && v.store == p.store_policy) k = v.fn;
  if (!k || l.split != 4) {
    fail("batch lookup kernel", "no variant for the plan");
    return;
  }
  BatchLookupArgs a{{reinterpret_cast<const ChunkRecord*>(records.p), capacity, reinterpret_cast<const uint32_t*>(chunk_start.p) + n,
                     l.waves_per_wg, l.n_waves, make_xcd_runs(p.grid, p.xcd_run), l.prefetch_waves, 0},
                    dev_descs, reinterpret_cast<const uint32_t*>(chunk_start.p), reinterpret_cast<const uint32_t*>(block_sum.p),
                    n, reinterpret_cast<uint64_t*>(seen.p)};
  g_check.clear();
  g_check.allow_read(records.p, records.n);
  g_check.allow_read(dev_descs, n * sizeof(BatchDesc));
  g_check.allow_read(chunk_start.p, chunk_start.n);
  g_check.allow_read(block_sum.p, block_sum.n);
  g_check.allow_write(seen.p, 8);
  allow_batch_data(b);
  g_check.seal();
  lane_emu::launch(k, a, p.grid, p.wg_size);
  g_waves += static_cast<uint64_t>(p.grid) * (p.wg_size / 64);
  if (!machine_ok("batch copy with lookups", what)) return;
  check_batch_result(b, "batch copy with lookups", what);
  uint64_t left;
  std::memcpy(&left, seen.p, 8);
  if (left != (static_cast<uint64_t>(n) << 32 | chunks)) fail("batch copy with lookups", what + ": wrong numbers left for the host");
}

void batches(bool quick) {
  uint64_t index = 0;
  for (unsigned which = 0; which < (quick ? 2u : 4u); ++which) {
    for (unsigned unroll : {1u, 2u, 4u})
      for (unsigned cap : {0u, 3u, 64u}) {
        if (index++ % g_shards != g_shard) continue;
        mi355_blit_tuning_t t{};
        t.unroll = unroll;
        t.wg_size = cap == 64 ? 256 : 64;
        t.max_grid = cap;
        t.xcd_run = (which + unroll) % 2 ? 2 : 0;
        t.batch_prefetch = which % 2 ? 16 : 0;
        batch_walked(which, t, quick);
      }
    for (unsigned percent : {0u, 40u, 100u, 130u})
      for (unsigned cap : {0u, 5u}) {
        if (index++ % g_shards != g_shard) continue;
        mi355_blit_tuning_t t{};
        t.max_grid = cap;
        t.xcd_run = percent == 40 ? 2 : 0;
        batch_device(which, percent, t, quick);
      }
  }
  for (unsigned percent : {40u, 100u}) {
    if (index++ % g_shards != g_shard) continue;
    mi355_blit_tuning_t t{};
    batch_device(4, percent, t, quick);
  }
}

// ---- pitched region copies ---------------------------------------------------------

void rects(bool quick) {
  const unsigned n_cases = quick ? 300 : 2500;
  for (unsigned index = 0; index < n_cases; ++index) {
    // draw the case on every shard so that all shards see the same sequence
    const unsigned kind = static_cast<unsigned>(below(6));
    uint64_t width, rows, layers;
    switch (kind) {
      case 0: width = 1 + below(15); rows = 1 + below(40); layers = 1 + below(3); break;          // under a vector
      case 1: width = 16 + below(1100); rows = 1 + below(30); layers = 1 + below(3); break;       // narrow rows
      case 2: width = 1024 + below(2100); rows = 1 + below(12); layers = 1 + below(2); break;     // around the kernels' limit
      case 3: width = 128 * (1 + below(40)); rows = 1 + below(10); layers = 1 + below(2); break;  // whole lines
      case 4: width = 2048 + below(9000); rows = 1 + below(6); layers = 1; break;                 // several units a row
      default: width = 1 + below(300); rows = 1 + below(200); layers = 1; break;
    }
    const bool aligned = kind == 3 && below(2);
    const uint64_t sx = aligned ? 128 * below(3) : below(40), dx = aligned ? 128 * below(3) : below(300);
    uint64_t sp = sx + width + below(200), dp = dx + width + below(200);
    if (aligned) sp = (sp + 127) & ~127ull, dp = (dp + 127) & ~127ull;
    if (below(8) == 0) sp = width, dp = width;  // rows that abut on both sides merge
    const uint64_t ss = sp * rows + (aligned ? 128 * below(3) : below(100)), ds = dp * rows + (aligned ? 128 * below(3) : below(100));
    mi355_blit_tuning_t t{};
    if (below(2)) {
      t.unroll = 1u << below(3);
      t.wg_size = 64u << below(3);
      if (below(2)) t.max_grid = 1 + static_cast<uint32_t>(below(4));
      if (below(3) == 0) t.xcd_run = 2;
    }
    const unsigned s_res = aligned ? 0 : static_cast<unsigned>(below(16)), d_res = aligned ? 0 : static_cast<unsigned>(below(256));
    if (index % g_shards != g_shard) continue;
    ++g_cases;
    const bool merged = sp == width && dp == width;
    const uint64_t sx_eff = merged ? 0 : sx, dx_eff = merged ? 0 : dx;
    // surfaces that end with the last row's last byte (the source: with its last dword)
    const uint64_t s_span = (layers - 1) * ss + (rows - 1) * sp + sx_eff + width;
    const uint64_t d_span = (layers - 1) * ds + (rows - 1) * dp + dx_eff + width;
    const size_t pad = (0 - (s_res + s_span)) & 3;
    Block src(s_span, 16 + s_res, 16, pad);
    Block dst(d_span + 128, (d_res + 256 - 64) % 256, 256);
    fill_random(src.raw, 16 + s_res + s_span + pad);
    std::memset(dst.p, kGuard, d_span + 128);
    uint8_t* d = dst.p + 64;
    const mi355_pitched_ptr_t dpp{d, dp, ds}, spp{src.p, sp, ss};
    const mi355_dim3_t doff{static_cast<uint32_t>(dx_eff), 0, 0}, soff{static_cast<uint32_t>(sx_eff), 0, 0};
    const mi355_dim3_t range{static_cast<uint32_t>(width), static_cast<uint32_t>(rows), static_cast<uint32_t>(layers)};
    RectPlan rp;
    if (plan_rect(&dpp, &doff, &spp, &soff, &range, &t, &rp) != 0) {
      fail("plan_rect", "refused");
      continue;
    }
    const std::string what = fmt("region %" PRIu64 " x %" PRIu64 " x %" PRIu64 ", pitches %" PRIu64 " / %" PRIu64
                                 ", x %" PRIu64 " / %" PRIu64 ", residues %u / %u, %s, unroll %u wg %u grid %u xcd_run %u",
                                 width, rows, layers, sp, dp, sx_eff, dx_eff, s_res, d_res,
                                 rp.linear ? "linear" : rp.narrow ? "narrow" : rp.args.plain_rows ? "plain rows" : "units",
                                 rp.unroll, rp.wg_size, rp.grid, rp.xcd_run);
    g_check.clear();
    for (uint64_t z = 0; z < layers; ++z)
      for (uint64_t y = 0; y < rows; ++y) {
        allow_source(src.p + z * ss + y * sp + sx_eff, width);
        g_check.allow_write(d + z * ds + y * dp + dx_eff, width);
      }
    // Rows whose extents touch are one range to the checker; a region of one
    // merged run is a linear copy and checked as one above.
    g_check.seal();
    if (rp.empty) {
      fail("plan_rect", what + ": empty");
      continue;
    }
    if (rp.linear) {
      mi355_blit_plan_t p;
      if (plan_copy(reinterpret_cast<uint64_t>(rp.args.dst), reinterpret_cast<uint64_t>(rp.args.src), rp.args.width, 256, &t, &p) != 0) {
        fail("plan_copy", "refused");
        continue;
      }
      copy_kernel_t k = nullptr;
      for (const CopyVariant& v : kCopyVariants)
        if (v.unroll == p.unroll && v.nt_load == p.nt_load && v.store == p.store_policy && v.realign == (p.byte_shift ? 1u : 0u))
          k = v.fn;
      const CopyArgs a = make_copy_args(p, rp.args.dst, rp.args.src, rp.args.width);
      lane_emu::launch(k, a, p.grid, p.wg_size);
    } else if (rp.narrow) {
      rect_narrow_kernel_t k = nullptr;
      for (const RectNarrowVariant& v : kRectNarrowVariants)
        if (v.nt_load == rp.streaming && v.store == rp.store_policy) k = v.fn;
      if (!k) {
        fail("narrow-row kernel", what + ": no variant");
        continue;
      }
      lane_emu::launch(k, rp.nargs, rp.grid, rp.wg_size);
    } else {
      rect_kernel_t k = nullptr;
      for (const RectVariant& v : kRectVariants)
        if (v.unroll == rp.unroll && v.nt_load == rp.streaming && v.store == rp.store_policy) k = v.fn;
      if (!k) {
        fail("region kernel", what + ": no variant");
        continue;
      }
      lane_emu::launch(k, rp.args, rp.grid, rp.wg_size);
    }
    g_waves += static_cast<uint64_t>(rp.grid) * (rp.wg_size / 64);
    if (!machine_ok("region copy", what)) continue;
    // expected destination: guard bytes with the rows copied in
    std::vector<uint8_t> want(d_span + 128, kGuard);
    for (uint64_t z = 0; z < layers; ++z)
      for (uint64_t y = 0; y < rows; ++y)
        std::memcpy(want.data() + 64 + z * ds + y * dp + dx_eff, src.p + z * ss + y * sp + sx_eff, width);
    if (std::memcmp(want.data(), dst.p, want.size()) != 0) fail("region copy", what + ": destination differs");
  }
}

// ---- self test: a planted over-read must be found ------------------------------------

// Every dword load moved up by one dword (then down): the realigning copy's
// fetch of the dword behind a tile, and behind the copy's last vector, then
// leaves the last dword that holds a source byte.  Counts the cases in which
// the checker reports it.
int self_test() {
  unsigned found_up = 0, found_down = 0, clean = 0, cases = 0;
  for (unsigned so = 0; so < 16; ++so)
    for (unsigned dl = 0; dl < 16; ++dl) {
      if (((so - dl) & 3) == 0) continue;  // no dword loads outside the realigning kernel
      // no tail bytes, so that the dword behind the last vector is the source's last
      const uint64_t n = ((16 - dl) & 15) + 16 * (64 + below(200));
      const CopyCase c{n, so, dl + 16 * static_cast<unsigned>(below(16)), mi355_blit_tuning_t{}};
      ++cases;
      g_check.shift_dword_loads = 0;
      clean += run_copy(c) == 0;
      g_check.shift_dword_loads = 4;
      found_up += run_copy(c, false) != 0;
      g_check.shift_dword_loads = -4;
      found_down += run_copy(c, false) != 0;
      g_check.shift_dword_loads = 0;
    }
  std::printf("self test: %u realigning copies; clean as built: %u; dword loads moved up by 4 bytes found in %u, moved down found in %u\n",
              cases, clean, found_up, found_down);
  // moved up, the load behind the copy's last vector leaves the source in every case; moved down, the first
  // wanted dword is still inside, and what is found is the wrong bytes, not an access
  return (clean == cases && found_up == cases && g_failures == 0) ? 0 : 1;
}

}  // namespace

int main(int argc, char** argv) {
  bool quick = false, self = false;
  for (int i = 1; i < argc; ++i) {
    if (!std::strcmp(argv[i], "--quick")) quick = true;
    else if (!std::strcmp(argv[i], "--self-test")) self = true;
    else if (!std::strcmp(argv[i], "--shard") && i + 1 < argc) {
      if (std::sscanf(argv[++i], "%u/%u", &g_shard, &g_shards) != 2 || g_shards == 0 || g_shard >= g_shards) {
        std::printf("bad --shard\n");
        return 2;
      }
    }
  }
  if (self) return self_test();
  linear_copies(quick);
  const uint64_t c1 = g_cases;
  fills(quick);
  const uint64_t c2 = g_cases;
  batches(quick);
  const uint64_t c3 = g_cases;
  rects(quick);
  std::printf("shard %u/%u: %" PRIu64 " linear copies, %" PRIu64 " fills, %" PRIu64 " batches, %" PRIu64
              " region copies; %" PRIu64 " waves, %" PRIu64 " lane switches\n",
              g_shard, g_shards, c1, c2 - c1, c3 - c2, g_cases - c3, g_waves, g_m.switches);
  std::printf("%" PRIu64 " failures\n", g_failures);
  return g_failures ? 1 : 0;
}
