// Host arithmetic of the pitched 3-D region copy: folds the offsets into the
// base addresses, merges rows and layers that are contiguous on both sides,
// and sizes the launch of the rect kernel.  Pure host code, shared by the HIP
// and the AQL submission paths.
//
// The reference hands such copies to its SDMA engines
// (projects/rocr-runtime/runtime/hsa-runtime/core/runtime/amd_gpu_agent.cpp:
// 1255-1283) and has no shader for them.
#ifndef MI355_BLIT_RECT_H_
#define MI355_BLIT_RECT_H_

#include <stdint.h>

#include "blit_args.h"
#include "blit_plan.h"
#include "mi355_blit.h"

namespace mi355 {

// Rows that touch at most this many 16-byte destination slots go to the
// kernel that packs several rows into a wave.
constexpr uint32_t kRectNarrowSlots = 64;
// Rows that are not whole lines stay with that kernel up to this many slots:
// one lane per slot wastes nothing on a row of one unit and a bit, where the
// unit kernel runs a second, nearly empty wave (1 GiB in rows of 1100 bytes at
// odd offsets: 5.3 TB/s against 3.9, rows of 2000 bytes 4.7 against 4.1; rows of
// 3000 bytes 5.6 against 5.9, hence the limit).
constexpr uint32_t kRectNarrowRaggedSlots = 128;

struct RectPlan {
  bool empty;    // a zero in the range: nothing to move
  bool linear;   // the region is one contiguous run on both sides
  bool narrow;   // rows of a few hundred bytes: several rows per wave (nargs)
  RectArgs args; // linear: dst, src and width describe the run
  RectNarrowArgs nargs;
  uint64_t total_bytes;
  uint32_t unroll;     // vectors per lane: a wave moves a unit of 64 * unroll vectors
  uint32_t streaming;  // non-temporal loads and stores
  uint32_t store_policy;
  uint32_t wg_size;
  uint32_t grid;
  uint32_t xcd_run;    // runs of workgroups per XCD, 0 = launch order
  uint32_t route;      // MI355_BLIT_ROUTE_*
};

// Units of `unit` vectors that a row of `width` bytes is cut into when its
// destination address is `residue` modulo 256 (row_units in the kernels): the
// last unit also takes up to 15 vectors of overflow.
inline uint64_t rect_row_units(uint64_t residue, uint64_t width, uint64_t unit) {
  uint64_t head = (16 - (residue & 15)) & 15;
  if (head > width) head = width;
  const uint64_t n_virtual = (width - head) / 16 + ((residue + head) & 255) / 16;
  return n_virtual > 15 + unit ? (n_virtual - 15 + unit - 1) / unit : 1;
}

inline uint64_t rect_gcd(uint64_t a, uint64_t b) {
  while (b) {
    const uint64_t t = a % b;
    a = b;
    b = t;
  }
  return a;
}

// Whether rows of whole cache lines are better written through L2 (sc1, the
// linear copy's stores) than with non-temporal stores.  Measured on MI355X, GB/s
// of bytes moved, sc1 against nt, first over some 90 shapes (rows of 128 bytes
// to 128 KiB at pitches of 1.002 to 8 times the width), then over a grid of 84
// (rows of 2 to 256 KiB at 2, 3, 4, 6, 8, 12 and 16 times their width, each
// policy at its best walk order, the worse of three processes):
//  * rows under 1 KiB (a wave stores pieces of several rows): sc1 wins at
//    every pitch, by 1 to 18 % (512-byte rows at a 2176-byte pitch 6956 against
//    5891, 128-byte rows at 384 bytes 6812 against 5867);
//  * rows of 1 KiB and more (every wave stores one contiguous KiB): sc1 wins by
//    1 to 11 % at every pitch that is a power of two (4 KiB rows at 32 KiB 6580
//    against 5930), and by 1 to 5 % at a multiple of 128 KiB when the width is a
//    power of two as well (128 KiB rows at 384 KiB 6646 against 6324); at such a
//    pitch rows of 12, 24, 48 or 96 KiB want nt by 6 to 12 % (48 KiB rows at
//    384 KiB 5337 against 5999), and at odd multiples of 64 KiB every width does
//    (32 KiB rows at 192 KiB 5377 against 5991).  At any other pitch sc1 loses by
//    4 to 20 % (2 KiB rows at 4352 bytes 5330 against 6384, 16 KiB rows at
//    68 KiB 5493 against 6074, 128 KiB rows at 260 KiB 5775 against 6419),
//    unless the rows nearly abut (a gap of up to 3 % of the pitch: 16 KiB rows
//    at 16,640 bytes 6531 against 6382).
// The batched copy, whose chunks lie at arbitrary 256-byte boundaries, shows
// the same preference for nt.  What the pitch changes is the order in which
// the rows' lines reach the memory channels; the rule is what the measurements
// say, not a model of them.
inline bool rect_whole_lines_write_through(uint64_t width, uint64_t dst_pitch) {
  if (width < 1024) return true;
  const uint64_t pow2_divisor = dst_pitch & (~dst_pitch + 1);
  if (pow2_divisor == dst_pitch) return true;
  if (pow2_divisor >= (128u << 10) && (width & (width - 1)) == 0) return true;
  return dst_pitch >= width && (dst_pitch - width) * 32 <= dst_pitch;
}

// Whether plain rows (whole lines, tiled like a linear copy) of a large region
// are better walked in launch order than in runs of neighbouring units per XCD.
// Runs are the robust shape: over all shapes measured they are never far from
// the best.  But when both pitches are powers of two and the rows take up
// three eighths of the pitch or less, the 8 XCDs' runs lie a multiple of a
// large power of two apart and get in one another's way in the memory
// channels, and launch order -- all XCDs side by side in the same rows --
// wins: rows of 4, 8, 16, 24, 32 and 48 KiB at pitches of 2.7 to 8 times their
// width +2 to +17 % (32 KiB rows at 128 KiB 6.47 against 5.90 TB/s, at 256 KiB
// 6.48 against 5.54; 8 KiB rows at 32 KiB 6.72 against 6.13), the same in two
// processes, at any x offsets, and with one side at another power-of-two pitch
// or dense.  Outside that window launch order loses or can lose a lot (2 KiB
// rows at 16 times their width -28 %, 12 KiB rows at 64 KiB -9 %, 128 KiB rows at
// 512 KiB -25 %, either pitch off a power of two by 256 bytes -6 .. +5 %), so
// the window is kept narrow: widths of 4 KiB or a multiple of 8 KiB up to
// 48 KiB, one layer.
inline bool rect_plain_rows_in_launch_order(uint64_t width, uint64_t dst_pitch, uint64_t src_pitch,
                                            uint64_t layers) {
  const auto pow2 = [](uint64_t x) { return x && (x & (x - 1)) == 0; };
  if (layers != 1 || !pow2(dst_pitch) || !pow2(src_pitch)) return false;
  if (width > (48u << 10) || (width != (4u << 10) && width % (8u << 10) != 0)) return false;
  const auto sparse = [width](uint64_t pitch) { return pitch * 3 >= width * 8 && pitch <= width * 8; };
  const auto dense_or_sparse = [width, sparse](uint64_t pitch) { return pitch == width || sparse(pitch); };
  return (sparse(dst_pitch) || sparse(src_pitch)) && dense_or_sparse(dst_pitch) && dense_or_sparse(src_pitch);
}

// The walk order of plain rows of a large region: units per XCD run, 1 for
// launch order.  The window above first.  Beyond it, runs of 576 units, with
// three exceptions for surfaces of one power-of-two pitch on both sides, taken
// from a grid of 84 shapes (rows of 2 to 256 KiB at 2 to 16 times their width,
// each at eight combinations of store policy and run length, the worse of three
// processes) and checked on 66 other shapes in two more processes:
//  * 8 KiB rows at 16 KiB: launch order (6520 against 5884 GB/s);
//  * rows of 16 and 32 KiB at 16 times their width: launch order (6369 against
//    5984, 6196 against 5130);
//  * rows of 128 KiB and more at 512 KiB and more: runs four times as long
//    (128 KiB rows at 512 KiB 6582 against 6267; 160 KiB rows 5978 against 5786).
// With these and the store rule above the grid's shapes run 1.7 % under the best
// combination found for each on average and at most 9.6 % (2 KiB rows at
// 24 KiB), the other 66 shapes 2.2 % and 12.7 %; with runs of 576 everywhere
// outside the window and stores written through at every multiple of 64 KiB,
// 3.3 % and 20.8 %, 3.0 % and 15.9 %.  Launch order for rows with non-temporal
// stores up to a few widths apart, which the grid suggested (+2 to +5 % at
// exactly 3 times the width), lost 4 to 12 % on the other shapes (3 KiB rows at
// 10.5 KiB 5381 against 5954, 16 KiB rows at 64.25 KiB 4614 against 5112) and
// was not taken.
inline uint32_t rect_plain_rows_run_units(uint64_t width, uint64_t dst_pitch, uint64_t src_pitch, uint64_t layers) {
  const uint32_t run = kXcdRunBytes / 1024;
  if (rect_plain_rows_in_launch_order(width, dst_pitch, src_pitch, layers)) return 1;
  if (layers != 1 || dst_pitch != src_pitch || (dst_pitch & (dst_pitch - 1)) != 0) return run;
  const uint64_t k = 1024;
  if (width == 8 * k && dst_pitch == 2 * width) return 1;
  if ((width == 16 * k || width == 32 * k) && dst_pitch == 16 * width) return 1;
  if (width >= 128 * k && dst_pitch >= 512 * k) return 4 * run;
  return run;
}

inline int plan_rect(const mi355_pitched_ptr_t* dst, const mi355_dim3_t* dst_offset, const mi355_pitched_ptr_t* src,
                     const mi355_dim3_t* src_offset, const mi355_dim3_t* range, const mi355_blit_tuning_t* t,
                     RectPlan* out, uint32_t route = MI355_BLIT_ROUTE_DEVICE) {
  if (!dst || !dst_offset || !src || !src_offset || !range || !out || route > MI355_BLIT_ROUTE_DEVICE_TO_HOST)
    return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  *out = RectPlan{};
  out->route = route;
  // A region one side of which is host memory moves at the host link's rate:
  // as for a linear copy (kHostLinkMaxGrid), at most 128 workgroups of 256
  // walk the rows in address order, and stores to the host are written through
  // at once.  Measured with pinned memory, 256 MiB in rows of 64 KiB, 4 KiB and
  // 256 bytes: 57.2 GB/s from the host and 57.0 GB/s to it (the runtime's DMA
  // engines: 57.5 / 57.0, and 43.7 for the 256-byte rows) against 54-55 GB/s
  // in the shapes made for HBM.
  const bool link = route != MI355_BLIT_ROUTE_DEVICE;
  const uint64_t link_max_grid = link ? kHostLinkMaxGrid : 0;
  if (range->x == 0 || range->y == 0 || range->z == 0) {
    out->empty = true;
    return MI355_BLIT_SUCCESS;
  }
  if (!dst->base || !src->base) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  // The region must be a geometric box inside both surfaces
  // (core/runtime/amd_blit_sdma.cpp:577-585); the dword alignment that file
  // also demands (:570-575) is a limit of the SDMA packet and not kept.
  if (uint64_t(src_offset->x) + range->x > src->pitch || uint64_t(dst_offset->x) + range->x > dst->pitch)
    return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (src->slice != 0 && uint64_t(src_offset->y) + range->y > src->slice / src->pitch)
    return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (dst->slice != 0 && uint64_t(dst_offset->y) + range->y > dst->slice / dst->pitch)
    return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  if (range->z > 1 && (src->slice == 0 || dst->slice == 0)) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  uint64_t width = range->x, rows = range->y, layers = range->z;
  // x, y and z are 32-bit: rows * layers fits 64 bits, the byte total may not
  if (width > (1ull << 62) / (rows * layers)) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  uint64_t dp = dst->pitch, ds = dst->slice, sp = src->pitch, ss = src->slice;
  uint8_t* d0 = static_cast<uint8_t*>(dst->base) + dst_offset->z * ds + dst_offset->y * dp + dst_offset->x;
  const uint8_t* s0 = static_cast<const uint8_t*>(src->base) + src_offset->z * ss + src_offset->y * sp + src_offset->x;
  out->total_bytes = width * rows * layers;
  // one row per layer: the layers are the rows
  if (rows == 1) {
    rows = layers;
    layers = 1;
    dp = ds;
    sp = ss;
  }
  // rows that follow one another without a gap on both sides are one row
  while (rows > 1 && width == dp && width == sp) {
    width *= rows;
    rows = layers;
    layers = 1;
    dp = ds;
    sp = ss;
  }
  RectArgs& a = out->args;
  a.dst = d0;
  a.src = s0;
  a.width = width;
  if (rows == 1) {
    out->linear = true;
    return MI355_BLIT_SUCCESS;
  }
  if (rows * layers > 0xffffffffull) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  a.dst_pitch = dp;
  a.dst_slice = layers > 1 ? ds : 0;
  a.src_pitch = sp;
  a.src_slice = layers > 1 ? ss : 0;
  a.rows = static_cast<uint32_t>(rows);
  bool streaming = out->total_bytes >= (4ull << 20);
  if (t && t->nt_load) streaming = (t->nt_load == 2);
  out->streaming = streaming;
  out->store_policy = streaming ? MI355_BLIT_STORE_NT : MI355_BLIT_STORE_CACHED;
  const bool store_tuned = t && t->store_policy >= 1 && t->store_policy <= 4;
  if (store_tuned) out->store_policy = t->store_policy - 1;
  const bool to_host = route == MI355_BLIT_ROUTE_DEVICE_TO_HOST && !store_tuned;
  if (to_host) out->store_policy = MI355_BLIT_STORE_SYSTEM_WT;

  // every store of every row is a whole cache line
  const bool whole_lines = reinterpret_cast<uintptr_t>(d0) % 128 == 0 && dp % 128 == 0 && width % 128 == 0 &&
                           (layers == 1 || ds % 128 == 0);

  // 16-byte destination slots a row touches, at the worst alignment its rows
  // can have (they differ by multiples of g16 modulo 16)
  uint64_t g16 = rect_gcd(dp % 16, 16);
  if (layers > 1) g16 = rect_gcd(ds % 16, g16);
  uint64_t row_slots = 0;
  for (uint64_t r = reinterpret_cast<uintptr_t>(d0) % g16; r < 16; r += g16) {
    const uint64_t c = (r + width + 15) / 16;
    if (c > row_slots) row_slots = c;
  }
  if (row_slots <= kRectNarrowSlots || (!whole_lines && row_slots <= kRectNarrowRaggedSlots)) {
    out->narrow = true;
    RectNarrowArgs& n = out->nargs;
    n.dst = d0;
    n.src = s0;
    n.dst_pitch = a.dst_pitch;
    n.dst_slice = a.dst_slice;
    n.src_pitch = a.src_pitch;
    n.src_slice = a.src_slice;
    n.width = static_cast<uint32_t>(width);
    n.rows = a.rows;
    n.lines = static_cast<uint32_t>(rows * layers);
    n.lanes_per_row = static_cast<uint32_t>(row_slots);
    n.pad = 0;
    n.magic64 = magic_divisor(n.lanes_per_row);
    out->unroll = 1;
    // Measured on MI355X with 2^20 rows.  When every store is a whole cache
    // line, single-wave workgroups and, at the pitches named above
    // (rect_whole_lines_write_through), written-through stores are best (1 KiB
    // rows at 2 KiB 312 us against 349 us, 512 B rows at 1 KiB 167 against 177).  Waves that share
    // cache lines with their neighbours want to be in one workgroup, hence on
    // one CU (520 B rows at a 1 KiB pitch, 33 lanes a row: 241 us with workgroups
    // of 256, 283 us with single waves, whose neighbours run on other XCDs), and
    // non-temporal stores.
    if (whole_lines && streaming && !store_tuned && !to_host && rect_whole_lines_write_through(width, dp))
      out->store_policy = MI355_BLIT_STORE_AGENT_WT;
    // No two waves touch the same destination line when rows are whole lines,
    // or when waves hold whole rows and neighbouring rows are a line apart.
    const bool rows_apart = dp >= width + 127 && (layers == 1 || ds >= (rows - 1) * dp + width + 127);
    const bool waves_apart = whole_lines || (64 % n.lanes_per_row == 0 && rows_apart);
    out->wg_size = (t && t->wg_size >= 64 && t->wg_size <= 1024 && t->wg_size % 64 == 0) ? t->wg_size
                   : waves_apart && !link                                                  ? 64
                                                                                            : 256;
    const uint64_t waves_per_wg = out->wg_size / 64;
    const uint64_t groups = (rows * layers * n.lanes_per_row + 63) / 64;
    uint64_t wgs = (groups + waves_per_wg - 1) / waves_per_wg;
    const uint64_t max_grid = (t && t->max_grid) ? t->max_grid : link_max_grid;
    if (max_grid && wgs > max_grid) wgs = max_grid;
    if (wgs * out->wg_size > kMaxGridWorkItems) wgs = kMaxGridWorkItems / out->wg_size;
    out->grid = static_cast<uint32_t>(wgs);
    n.waves_per_wg = static_cast<uint32_t>(waves_per_wg);
    n.n_waves = static_cast<uint32_t>(wgs * waves_per_wg);
    // Waves that share lines with their neighbours want those neighbours on
    // their own XCD (runs of about kXcdRunBytes of destination span; 1000-byte
    // rows at a 2 KiB pitch 376-379 us against 407-411 us in launch order,
    // 520-byte rows at 1 KiB 455-462 against 489-501); waves that share none
    // gain nothing from it.
    uint32_t run = 0;
    if (!waves_apart && !link && out->total_bytes >= kXcdRunMinBytes) {
      const uint64_t rows_per_wave = 64 / n.lanes_per_row;  // >= 1
      const uint64_t span = waves_per_wg * (rows_per_wave * dp > 1024 ? rows_per_wave * dp : 1024);
      run = static_cast<uint32_t>(kXcdRunBytes / span);
      if (run < 32) run = 32;
    }
    out->xcd_run = plan_xcd_run(run, t);
    n.xcd = make_xcd_runs(out->grid, out->xcd_run);
    return MI355_BLIT_SUCCESS;
  }

  // Measured on MI355X, 1 GiB moved in rows of 4 KiB and of 128 KiB.  Rows whose
  // every store is a whole cache line (first row, pitches and width multiples
  // of 128 bytes): one vector per lane, workgroups of 256 (of 64 for plain
  // rows, below), stores written through L2 like the linear copy's at the
  // pitches that suit them (rect_whole_lines_write_through), 320-326 us
  // (6.6-6.7 TB/s) against 333-341 us with the shape below.  Any other rows: two vectors per lane,
  // workgroups of 128, non-temporal stores (written-through stores lose 8-15 %
  // there: the rows' cut ends are partial lines).
  uint32_t unroll = whole_lines ? 1 : 2;
  uint32_t default_wg = whole_lines ? 256 : 128;
  // Long rows that are not whole lines behave like the linear copy with a byte
  // offset: single waves with one vector per lane, in XCD runs (1 GiB moved, any
  // alignment: rows of 64 KiB 345 us against 347 us, of 128 KiB 336 against 341,
  // of 512 KiB 328 against 335, of 8 MiB 323 against 358; rows of 32 KiB equal,
  // of 16 KiB 341 against 329, hence the threshold).
  if (!whole_lines && width >= (48u << 10) && out->total_bytes >= kXcdRunMinBytes) {
    unroll = 1;
    default_wg = 64;
  }
  if (link) {
    unroll = 1;
    default_wg = 256;
  }
  if (whole_lines && streaming && !store_tuned && !to_host && rect_whole_lines_write_through(width, dp))
    out->store_policy = MI355_BLIT_STORE_AGENT_WT;
  if (t && (t->unroll == 1 || t->unroll == 2 || t->unroll == 4)) unroll = t->unroll;
  out->unroll = unroll;
  // Row destinations differ by multiples of g modulo 256: the largest unit
  // count over those residues is the number of slots every row gets.
  uint64_t g = rect_gcd(dp % 256, 256);
  if (layers > 1) g = rect_gcd(ds % 256, g);
  uint64_t slots = 0;
  for (uint64_t r = reinterpret_cast<uintptr_t>(d0) % g; r < 256; r += g) {
    const uint64_t c = rect_row_units(r, width, 64 * unroll);
    if (c > slots) slots = c;
  }
  // Rows that are tiled like a linear copy: they start at cache-line
  // boundaries of the destination, are whole lines long and lie a multiple of
  // 4 bytes from their source.  The kernel then skips everything a row's ends
  // need: a unit is a plain tile of the row from its first byte on, the last
  // one possibly a partial one (1 GiB in rows of 4224 bytes: 328 us, 368 us
  // through the general path).
  const uint64_t unit_bytes = 1024ull * unroll;
  const uintptr_t delta = reinterpret_cast<uintptr_t>(s0) - reinterpret_cast<uintptr_t>(d0);
  a.plain_rows = whole_lines && delta % 4 == 0 && sp % 4 == 0 && (layers == 1 || ss % 4 == 0);
  // A row of one unit and a few vectors is one wave's (1 GiB in rows of 1152
  // bytes: 354 us, 422 us with a second wave for the last 128 bytes); longer
  // rows end in a partial unit (rows of 4224 bytes: 328 us, 343 us with the 8
  // vectors added to the fourth unit).
  if (a.plain_rows) slots = width <= unit_bytes + 16 * 15 ? 1 : (width + unit_bytes - 1) / unit_bytes;
  const uint64_t total_slots = rows * layers * slots;
  if (total_slots > 0xffffffffull) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  a.slots = static_cast<uint32_t>(slots);
  a.total_slots = static_cast<uint32_t>(total_slots);
  a.magic_slots = magic_divisor(a.slots);
  a.magic_rows = magic_divisor(a.rows);
  // Plain rows in XCD runs want single-wave workgroups, like the linear copy.
  // Measured on 17 shapes of 1 GiB, widths 2 KiB .. 1 MiB at pitches of 1.03 to
  // 256 times the width: workgroups of 256 in launch order are up to 27 % behind
  // the best shape found for a region (3 KiB rows at a 4 KiB pitch: 414 us
  // against 324 us), single waves in launch order up to 20 %, single waves in
  // runs of 576 units at most 12 % (8 KiB rows at a 16 KiB pitch, 361 us against
  // 321 us) and within 2 % everywhere else.  Which shape wins for a given pitch
  // follows the memory channels' interleave, not the kernel.
  const bool plain_runs = a.plain_rows && !link && out->total_bytes >= kXcdRunMinBytes;
  if (plain_runs) default_wg = 64;
  out->wg_size = (t && t->wg_size >= 64 && t->wg_size <= 1024 && t->wg_size % 64 == 0) ? t->wg_size : default_wg;
  const uint64_t waves_per_wg = out->wg_size / 64;
  uint64_t wgs = (total_slots + waves_per_wg - 1) / waves_per_wg;
  const uint64_t max_grid = (t && t->max_grid) ? t->max_grid : link_max_grid;
  if (max_grid && wgs > max_grid) wgs = max_grid;
  if (wgs * out->wg_size > kMaxGridWorkItems) wgs = kMaxGridWorkItems / out->wg_size;
  out->grid = static_cast<uint32_t>(wgs);
  a.waves_per_wg = static_cast<uint32_t>(waves_per_wg);
  a.n_waves = static_cast<uint32_t>(wgs * waves_per_wg);
  // Units of rows that are not whole lines share source and destination lines
  // with their neighbours: runs of neighbouring units per XCD, as for the
  // linear copy (131,065-byte rows 344 us against 361 us in launch order).
  // Whole-line rows that are not plain go through the general path of the
  // kernel, where runs lose (347 us against 330 us).
  uint32_t run = 0;
  if ((!whole_lines || plain_runs) && !link && out->total_bytes >= kXcdRunMinBytes) {
    run = static_cast<uint32_t>(kXcdRunBytes / (waves_per_wg * 1024 * unroll));
    if (plain_runs) {
      // in units of 1 KiB, which is what a workgroup of the default shape moves
      const uint32_t units = rect_plain_rows_run_units(width, dp, sp, layers);
      run = units <= 1 ? 0 : static_cast<uint32_t>(units / (waves_per_wg * unroll));
    }
  }
  out->xcd_run = plan_xcd_run(run, t);
  a.xcd = make_xcd_runs(out->grid, out->xcd_run);
  return MI355_BLIT_SUCCESS;
}

inline void rect_launch_info(const RectPlan& rp, mi355_blit_plan_t* p) {
  *p = mi355_blit_plan_t{};
  p->kernel = MI355_BLIT_KERNEL_COPY_RECT;
  p->wg_size = rp.wg_size;
  p->grid = rp.grid;
  p->unroll = rp.unroll;
  p->nt_load = rp.streaming;
  p->store_policy = rp.store_policy;
  p->xcd_run = rp.xcd_run;
  p->route = rp.route;
  p->body_vecs = rp.narrow ? rp.nargs.lines : rp.args.total_slots;  // rows, or chunk slots
}

}  // namespace mi355

#endif  // MI355_BLIT_RECT_H_
