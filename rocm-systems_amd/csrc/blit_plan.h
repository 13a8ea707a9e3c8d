// Dispatch sizing for the gfx950 blit kernels: how a copy or fill is cut into
// head / 16-byte body / tail, and which workgroup size, grid, unroll and cache
// policy it is launched with.  Pure host arithmetic, no HIP.
//
// Takes the place of the phase arithmetic and fixed grids in ROCr's
// BlitKernel (projects/rocr-runtime/runtime/hsa-runtime/core/runtime/
// amd_blit_kernel.cpp:714-775 for copies, :796-813 for fills): there the grid
// is always 64*4*num_cus (copy) or 64*num_cus (fill) single-wave workgroups
// with one vector per lane in flight, whatever the size.
#ifndef MI355_BLIT_PLAN_H_
#define MI355_BLIT_PLAN_H_

#include <stdint.h>
#include <stdlib.h>

#include "blit_args.h"
#include "mi355_blit.h"

namespace mi355 {

// Vectors of one batched-copy chunk: one wave, four loads per lane.
constexpr uint32_t kBatchChunkVecs = 256;
// Workgroups of 256 lanes that fill one CU's wave slots (8 waves per SIMD);
// used where a kernel wants a device-filling persistent grid.
constexpr uint32_t kWgPerCu = 8;
// The grid dimension is a 32-bit count of work-items in an AQL packet.
constexpr uint64_t kMaxGridWorkItems = 0x7fffffc0ull;

struct SizeClass {
  uint64_t min_bytes;  // applies from this size up
  uint32_t wg_size;
  uint32_t unroll;
  uint32_t nt_load;
  uint32_t store_policy;
  uint32_t xcd_run_bytes;  // bytes of the runs of tiles each XCD works through; 0 = tiles in launch order
};

// Measured on MI355X (256 CUs), sweeps of 4 KiB .. 4 GiB.
// Up to a few MiB a launch is bound by its fixed cost (~3.5 us back to back)
// and the shape does not matter.  From there on transfers bypass the caches:
// loads non-temporal, stores written through L2.
//
// The hardware deals consecutive workgroups to the 8 XCDs in turn, each XCD
// with an L2 of its own.  From 50-80 MiB on it pays to permute the launch
// so that each XCD works through runs of neighbouring tiles (xcd_run
// workgroups, 576 KiB): a source line that two tiles share (tiles are anchored
// at the destination's 256-byte boundaries, so they do whenever source and
// destination differ mod 128) is then fetched into one L2 instead of two, and
// single-wave workgroups, the fastest shape for a stream, no longer pay for
// having their neighbours on another XCD.  The run is 512 KiB + 64 KiB on
// purpose: with runs of a power of two the 8 streams sit a power of two apart
// and, depending on where source and destination lie, collide in the memory
// channels (1 GiB with a byte offset, 2 KiB tiles: 315-367 us over 20
// placements with runs of 256 KiB, 320-326 us with 576 KiB, 338-344 us in
// launch order).
// Measured, 1 GiB: equally aligned 309-312 us against 314-317 us in launch
// order; source and destination differing mod 128, 311-313 us against 321-327;
// a byte offset, 310-314 us against 338-344.  At 128-256 MiB, where the
// last-level cache holds most of the transfer, 59 us against 66 us.  A byte
// offset adds one dword fetch per tile (the bytes that spill past the last
// lane); while the transfer sits in the last-level cache 2 KiB tiles amortise
// it best, beyond that 1 KiB tiles with non-temporal stores run like the
// aligned copy.  Its stores are written through while
// the 256 MiB last-level cache absorbs them and non-temporal beyond (256 MiB:
// 61 us against 79 us, 288 MiB: 93 us against 89 us).  The thresholds are where
// the shapes cross in a sweep in steps of 16-32 MiB.  Fills at one
// wave per workgroup are bound by the dispatcher's workgroup rate and want
// 4-wave workgroups.  Last match wins.
constexpr uint32_t kXcdRunBytes = 576u << 10;
// Below this size the permutation gains nothing (the transfer sits in the
// last-level cache) or loses a little.
constexpr uint64_t kXcdRunMinBytes = 64ull << 20;
// The batched copy, whose neighbouring 4 KiB chunks share source lines and cut
// destination lines: measured with 65,536 copies (2 GB), 698-701 us with runs
// of 272 chunks or more against 728-730 us in launch order.
constexpr uint32_t kBatchXcdRunChunks = 528;
constexpr SizeClass kCopyClasses[] = {      // (src - dst) % 4 == 0
    {0, 256, 1, 0, MI355_BLIT_STORE_CACHED, 0},
    {4ull << 20, 256, 1, 1, MI355_BLIT_STORE_AGENT_WT, 0},
    {80ull << 20, 64, 1, 1, MI355_BLIT_STORE_AGENT_WT, kXcdRunBytes},
};
constexpr SizeClass kCopyRealignClasses[] = {  // (src - dst) % 4 != 0
    {0, 512, 1, 0, MI355_BLIT_STORE_CACHED, 0},
    {4ull << 20, 256, 2, 1, MI355_BLIT_STORE_AGENT_WT, 0},
    {48ull << 20, 64, 2, 1, MI355_BLIT_STORE_AGENT_WT, kXcdRunBytes},
    {272ull << 20, 64, 1, 1, MI355_BLIT_STORE_NT, kXcdRunBytes},
};
constexpr SizeClass kFillClasses[] = {
    {0, 256, 1, 0, MI355_BLIT_STORE_CACHED, 0},
    {16ull << 20, 256, 1, 0, MI355_BLIT_STORE_SYSTEM_WT, 0},
};

// Copies across the host link (one side is host memory): 55-57 GB/s whatever
// the kernel does, provided it does not do too much at once.  Measured with
// pinned host memory, 256 MiB: 57.2 GB/s from the host and 57.0 GB/s to it
// with 128 workgroups of 256 striding over the tiles in address order, the
// rate of the runtime's DMA engines (57.4 / 54.9); one wave per tile, the
// shape for HBM, 55.1 / 55.6, and at 16 MiB 47 / 53 against 55 / 55.  Stores
// to the host written through at once (54.6 GB/s cached, 57.0 written
// through); below 4 MiB a copy into the device leaves its bytes in L2 for
// whoever reads them next, as a small copy within the device does.
constexpr uint32_t kHostLinkMaxGrid = 128;
constexpr SizeClass kCopyHostToDeviceClasses[] = {
    {0, 256, 1, 0, MI355_BLIT_STORE_CACHED, 0},
    {4ull << 20, 256, 1, 1, MI355_BLIT_STORE_AGENT_WT, 0},
};
constexpr SizeClass kCopyDeviceToHostClasses[] = {
    {0, 256, 1, 0, MI355_BLIT_STORE_SYSTEM_WT, 0},
    {4ull << 20, 256, 1, 1, MI355_BLIT_STORE_SYSTEM_WT, 0},
};

// The engine GpuAgent::GetBlitObject picks for an asynchronous copy within one
// GPU (amd_gpu_agent.cpp:2390-2397) and the flag behind it (core/util/flag.h:
// 206-207: atoi of HSA_FORCE_SDMA_SIZE, 1 MiB when unset or empty; atoi's int
// becomes the size_t the reference compares with).
inline uint64_t policy_force_sdma_size() {
  const char* v = getenv("HSA_FORCE_SDMA_SIZE");
  if (!v || !v[0]) return 1024 * 1024;
  return static_cast<uint64_t>(static_cast<size_t>(atoi(v)));
}

inline uint32_t policy_same_gpu_engine(uint64_t size, uint64_t force_sdma_size) {
  return size < force_sdma_size ? MI355_ENGINE_SDMA : MI355_ENGINE_BLIT_KERNEL;
}

inline bool valid_unroll(uint32_t u) { return u == 1 || u == 2 || u == 4; }

template <unsigned N>
inline const SizeClass& pick_class(const SizeClass (&tbl)[N], uint64_t bytes) {
  const SizeClass* c = &tbl[0];
  for (unsigned i = 0; i < N; ++i)
    if (bytes >= tbl[i].min_bytes) c = &tbl[i];
  return *c;
}

// Runs of workgroups per XCD: the heuristic's choice unless tuning overrides it
// (1 = launch order, which a plan states as 0).
inline uint32_t plan_xcd_run(uint32_t heuristic, const mi355_blit_tuning_t* t) {
  uint32_t run = heuristic;
  if (t && t->xcd_run) run = t->xcd_run;
  return run > 1 ? run : 0;
}

// In workgroups of waves_per_wg waves, `split` waves to a chunk.
inline uint32_t batch_xcd_run(uint64_t total_bytes, uint32_t split, uint32_t waves_per_wg,
                              const mi355_blit_tuning_t* t) {
  return plan_xcd_run(total_bytes >= kXcdRunMinBytes ? kBatchXcdRunChunks * split / waves_per_wg : 0, t);
}

// Launch shape of the batched copy over chunk records, shared by the two
// submission paths.  Measured on MI355X with 65,536 copies of 64 B..256 KiB:
// one 4 KiB chunk per 4-wave workgroup, 1 KiB per wave, is the fastest shape;
// non-temporal loads and stores are best (739 us against 824 us cached), and
// written-through stores are worst (958 us) because the copies' cut ends are
// partial lines.
struct BatchLaunch {
  uint32_t split;         // waves per chunk
  uint32_t waves_per_wg;
  uint32_t n_waves;
  uint32_t prefetch_waves;  // BatchCopyArgs::prefetch_waves
};

// total_chunks: the number of records, or a bound on it.  streaming: whether
// the batch is large enough to bypass the caches (tuning may override).  With
// shape_tunable false only the grid cap, the XCD runs and the cache policies
// follow the tuning.  Fills in *p.
inline BatchLaunch plan_batch_records(uint64_t total_chunks, uint64_t total_bytes, bool streaming,
                                      const mi355_blit_tuning_t* t, bool shape_tunable, mi355_blit_plan_t* p) {
  *p = mi355_blit_plan_t{};
  p->pieces = 1;
  p->kernel = MI355_BLIT_KERNEL_COPY_BATCH;
  p->body_vecs = total_chunks;
  if (t && t->nt_load) streaming = (t->nt_load == 2);
  p->nt_load = streaming;
  p->store_policy = streaming ? MI355_BLIT_STORE_NT : MI355_BLIT_STORE_CACHED;
  if (t && t->store_policy >= 1 && t->store_policy <= 4) p->store_policy = t->store_policy - 1;
  BatchLaunch l;
  // Single-wave workgroups, four to a chunk: a wave starts as soon as one wave
  // slot is free instead of waiting for four on one CU (65,536 copies, 4.1 GB:
  // 698 us against 700 us spread over two 8 GiB arenas, 663 against 670 packed
  // densely).
  p->wg_size = 64;
  l.split = 4;
  if (t && shape_tunable) {
    if (t->wg_size >= 64 && t->wg_size <= 1024 && t->wg_size % 64 == 0) p->wg_size = t->wg_size;
    if (valid_unroll(t->unroll)) l.split = 4 / t->unroll;
  }
  p->unroll = 4 / l.split;
  l.waves_per_wg = p->wg_size / 64;
  uint64_t wgs = (total_chunks * l.split + l.waves_per_wg - 1) / l.waves_per_wg;
  if (t && t->max_grid && wgs > t->max_grid) wgs = t->max_grid;
  if (wgs * p->wg_size > kMaxGridWorkItems) wgs = kMaxGridWorkItems / p->wg_size;
  p->grid = static_cast<uint32_t>(wgs);
  l.n_waves = static_cast<uint32_t>(wgs * l.waves_per_wg);
  p->xcd_run = batch_xcd_run(total_bytes, l.split, l.waves_per_wg, t);
  // The record a wave needs is touched one round of XCD runs earlier (in launch
  // order: 4096 workgroups earlier, a multiple of 8 and so on the same XCD).
  // Measured with 65,536 copies (4.1 GB): 700 us against 705 us without spread
  // over two 8 GiB arenas, 670 against 690 packed densely; a distance of half a
  // round or less (528 .. 2112 workgroups of 256) gains nothing, the touched
  // line then sits in another XCD's L2.
  uint32_t ahead_wgs = p->xcd_run > 1 ? 8 * p->xcd_run : 4096;
  if (t && t->batch_prefetch) ahead_wgs = t->batch_prefetch > 1 ? t->batch_prefetch : 0;
  l.prefetch_waves = ahead_wgs * l.waves_per_wg;
  return l;
}

// class_max_grid: the cap on workgroups the class asks for, 0 for none.
inline void apply_launch_shape(mi355_blit_plan_t* p, const SizeClass& cls, uint32_t num_cus,
                               const mi355_blit_tuning_t* t, uint32_t class_max_grid = 0) {
  (void)num_cus;
  p->wg_size = cls.wg_size;
  p->unroll = cls.unroll;
  p->nt_load = cls.nt_load;
  p->store_policy = cls.store_policy;
  uint64_t max_grid = class_max_grid;
  if (t) {
    if (t->wg_size >= 64 && t->wg_size <= 1024 && (t->wg_size % 64) == 0) p->wg_size = t->wg_size;
    if (valid_unroll(t->unroll)) p->unroll = t->unroll;
    if (t->nt_load) p->nt_load = (t->nt_load == 2);
    if (t->store_policy >= 1 && t->store_policy <= 4) p->store_policy = t->store_policy - 1;
    if (t->max_grid) max_grid = t->max_grid;
  }
  p->xcd_run = plan_xcd_run(cls.xcd_run_bytes / (p->wg_size / 64 * p->unroll * 1024), t);
  const uint64_t hw_max = kMaxGridWorkItems / p->wg_size;
  if (max_grid == 0 || max_grid > hw_max) max_grid = hw_max;
  // One wave per tile of 64*unroll vectors (tiles anchored at 256-byte
  // boundaries of the destination) plus one for the edges; a capped grid
  // makes the waves stride over the tiles instead.
  const uint64_t tile_vecs = 64ull * p->unroll;
  const uint64_t tiles = (p->body_vecs + p->lead_vecs + tile_vecs - 1) / tile_vecs;
  const uint64_t waves = tiles + 1;
  const uint64_t waves_per_wg = p->wg_size / 64;
  uint64_t wgs = (waves + waves_per_wg - 1) / waves_per_wg;
  if (wgs > max_grid) wgs = max_grid;
  if (wgs == 0) wgs = 1;
  p->grid = static_cast<uint32_t>(wgs);
}

inline int plan_copy(uint64_t dst, uint64_t src, uint64_t bytes, uint32_t num_cus,
                     const mi355_blit_tuning_t* t, mi355_blit_plan_t* p,
                     uint32_t route = MI355_BLIT_ROUTE_DEVICE) {
  if (!p || route > MI355_BLIT_ROUTE_DEVICE_TO_HOST) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  *p = mi355_blit_plan_t{};
  p->route = route;
  p->pieces = 1;
  uint64_t head = (16 - (dst & 15)) & 15;
  if (head > bytes) head = bytes;
  p->head_bytes = head;
  p->body_vecs = (bytes - head) / 16;
  p->tail_bytes = bytes - head - 16 * p->body_vecs;
  p->lead_vecs = static_cast<uint32_t>(((dst + head) & 255) / 16);
  p->byte_shift = static_cast<uint32_t>((src - dst) & 3);
  p->kernel = p->byte_shift ? MI355_BLIT_KERNEL_COPY_REALIGN : MI355_BLIT_KERNEL_COPY;
  if (route == MI355_BLIT_ROUTE_HOST_TO_DEVICE) {
    apply_launch_shape(p, pick_class(kCopyHostToDeviceClasses, bytes), num_cus, t, kHostLinkMaxGrid);
  } else if (route == MI355_BLIT_ROUTE_DEVICE_TO_HOST) {
    apply_launch_shape(p, pick_class(kCopyDeviceToHostClasses, bytes), num_cus, t, kHostLinkMaxGrid);
  } else {
    const SizeClass& cls = p->byte_shift ? pick_class(kCopyRealignClasses, bytes) : pick_class(kCopyClasses, bytes);
    apply_launch_shape(p, cls, num_cus, t);
  }
  return MI355_BLIT_SUCCESS;
}

// A copy of several GiB within the device is submitted as consecutive launches
// of at most 512 MiB, each a copy in its own right.  The hardware deals a
// launch's workgroups to the 8 XCDs in turn and each XCD works through its
// share at its own pace: over a long launch the 8 streams drift apart, the
// stretch of memory in use at any moment grows, and the rate sinks; a launch
// boundary brings them back together.  Measured on MI355X, us per GiB, aligned
// copy: 4 GiB in one launch 318.2-318.6, in pieces of 2 GiB 316.8, 1 GiB 314.7,
// 512 MiB 313.6-314.2, 256 MiB 316.2-316.7, 128 MiB 324.2-324.8; 8 GiB 323.4-325.5
// in one launch, 313.9-314.5 in pieces of 512 MiB; 2 GiB 315.2-316.5 against
// 313.2-314.7; 1 GiB the same either way, as are copies of the same 1 GiB over
// and over or of four different ones in turn (314.5: not a cache effect).  The
// byte-offset copy gains less (4 GiB: 320.6-321.1 -> 318.9-319.2) and must not be
// cut below 272 MiB, where its launch shape is the one for transfers the
// last-level cache holds (pieces of 256 MiB: 339); the fill, a single stream,
// loses (147.8 -> 149.6) and is not cut.  The smallest piece this makes is 384 MiB.
constexpr uint64_t kCopyPieceBytes = 512ull << 20;
constexpr uint64_t kCopySplitMinBytes = 1536ull << 20;
constexpr uint32_t kCopyMaxPieces = 32;

// The number of launches for a copy of `bytes`, at most max_pieces (what the
// submission path has room for), and the bytes of each but the last (a multiple
// of 1 MiB, so that every piece keeps the alignment of the whole).
inline uint32_t copy_pieces(uint64_t bytes, uint32_t route, uint32_t max_pieces, const mi355_blit_tuning_t* tuning,
                            uint64_t* piece_bytes) {
  *piece_bytes = bytes;
  uint64_t target = kCopyPieceBytes, from = kCopySplitMinBytes;
  if (tuning && tuning->copy_piece_mib == 1) return 1;
  if (tuning && tuning->copy_piece_mib > 1) {
    target = static_cast<uint64_t>(tuning->copy_piece_mib) << 20;
    from = target + 1;
  }
  if (route != MI355_BLIT_ROUTE_DEVICE || bytes < from) return 1;
  uint64_t n = (bytes + target - 1) / target;
  if (n > kCopyMaxPieces) n = kCopyMaxPieces;
  if (n > max_pieces) n = max_pieces;
  if (n <= 1) return 1;
  const uint64_t mib = 1ull << 20;
  const uint64_t piece = ((bytes + n - 1) / n + mib - 1) / mib * mib;
  *piece_bytes = piece;
  return static_cast<uint32_t>((bytes + piece - 1) / piece);
}

inline int plan_fill(uint64_t ptr, uint64_t num_dwords, uint32_t num_cus,
                     const mi355_blit_tuning_t* t, mi355_blit_plan_t* p) {
  if (!p) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (ptr & 3) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  *p = mi355_blit_plan_t{};
  p->pieces = 1;
  const uint64_t bytes = num_dwords * 4;
  uint64_t head = (16 - (ptr & 15)) & 15;
  if (head > bytes) head = bytes;
  p->head_bytes = head;
  p->body_vecs = (bytes - head) / 16;
  p->tail_bytes = bytes - head - 16 * p->body_vecs;
  p->lead_vecs = static_cast<uint32_t>(((ptr + head) & 255) / 16);
  p->kernel = MI355_BLIT_KERNEL_FILL;
  apply_launch_shape(p, pick_class(kFillClasses, bytes), num_cus, t);
  p->nt_load = 0;
  return MI355_BLIT_SUCCESS;
}

// Which waves of a launch take the cut tiles at both ends and the head / tail
// bytes: the two after the wave of the last full tile.
inline void plan_tail_waves(const mi355_blit_plan_t& p, uint32_t* partial_wave, uint32_t* edge_wave,
                            uint32_t* waves_per_wg, uint32_t* n_waves_out) {
  const uint64_t n_waves = static_cast<uint64_t>(p.grid) * (p.wg_size / 64);
  *waves_per_wg = p.wg_size / 64;
  *n_waves_out = static_cast<uint32_t>(n_waves);
  // full tiles, as tile_range() counts them on the device
  const uint64_t first_full = p.lead_vecs ? 1 : 0;
  const uint64_t end_full = (p.body_vecs + p.lead_vecs) / (64ull * p.unroll);
  const uint64_t n_full = end_full > first_full ? end_full - first_full : 0;
  *partial_wave = static_cast<uint32_t>(n_full % n_waves);
  *edge_wave = static_cast<uint32_t>((n_full + 1) % n_waves);
}

// The kernel argument block of a planned copy / fill: what either submission
// path hands to the kernel (p.grid workgroups of p.wg_size).
inline CopyArgs make_copy_args(const mi355_blit_plan_t& p, void* dst, const void* src, uint64_t bytes) {
  CopyArgs a{};
  a.dst = static_cast<uint8_t*>(dst);
  a.src = static_cast<const uint8_t*>(src);
  a.bytes = bytes;
  a.n_vec = p.body_vecs;
  a.head = static_cast<uint32_t>(p.head_bytes);
  a.lead = p.lead_vecs;
  plan_tail_waves(p, &a.partial_wave, &a.edge_wave, &a.waves_per_wg, &a.n_waves);
  a.xcd = make_xcd_runs(p.grid, p.xcd_run);
  return a;
}

inline FillArgs make_fill_args(const mi355_blit_plan_t& p, void* ptr, uint32_t value, uint64_t num_dwords) {
  FillArgs a{};
  a.dst = static_cast<uint32_t*>(ptr);
  a.n_dwords = num_dwords;
  a.n_vec = p.body_vecs;
  a.head = static_cast<uint32_t>(p.head_bytes / 4);
  a.lead = p.lead_vecs;
  a.value = value;
  plan_tail_waves(p, &a.partial_wave, &a.edge_wave, &a.waves_per_wg, &a.n_waves);
  a.xcd = make_xcd_runs(p.grid, p.xcd_run);
  return a;
}

}  // namespace mi355

#endif  // MI355_BLIT_PLAN_H_
