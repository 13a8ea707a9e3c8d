// Device kernels of the gfx950 blit engine: linear copy, dword fill, batched
// small copies, pitched 3-D region copies.  They take the place of ROCr's
// CopyAligned, CopyMisaligned and Fill shaders (projects/rocr-runtime/runtime/hsa-runtime/core/runtime/
// blit_shaders/blit_copyAligned.s:76-259, blit_copyMisaligned.s:90-182,
// blit_fill.s:91-185) but share none of their structure:
//
//  * Every global access in the body is a 16-byte global_load/store_dwordx4;
//    one wave instruction moves a contiguous 1 KiB.
//  * A wave owns a contiguous tile of 64 * U vectors and issues all U loads
//    before its first store, so U KiB per wave are in flight.  By default the
//    grid has one wave per tile: the hardware dispatcher hands tiles out in
//    address order as waves retire, which keeps the set of DRAM pages in use
//    small; measured on MI355X this beats a persistent grid-stride loop by
//    ~10 % at 1 GiB.  The grid-stride loop remains for capped grids.
//  * Where neighbouring tiles share cache lines and the transfer is large, the
//    host asks for the launch to be permuted so that each of the 8 XCDs (each
//    with its own L2) works through runs of neighbouring workgroups' tiles
//    (XcdRuns in the argument blocks, xcd_workgroup in blit_args.h):
//    the shared lines then meet in one L2.
//  * Large transfers bypass the caches: loads carry nt, stores are written
//    through L2 (sc1 / sc0 sc1), chosen per size by the host.
//  * Stores are always 16-byte aligned, and tiles are anchored at 256-byte
//    boundaries of the destination so that a wave stores whole cache lines:
//    the destination is aligned first and the source takes whatever
//    alignment is left.  When source and destination
//    differ by a multiple of 4 the loads are dword-aligned dwordx4.  Otherwise
//    each lane loads the dword-aligned 16 bytes that contain its source bytes,
//    takes the 17th..20th byte from the next lane with a DPP wave rotate, and
//    rebuilds its vector with four v_alignbyte_b32.  No sub-dword access is
//    made outside the <=15-byte head and tail of a copy.  (The region copy
//    of narrow rows is the exception: it moves a row's cut first and last
//    slot as unaligned 16-byte vectors.)
//  * The source is never read outside the aligned dwords that contain at
//    least one requested byte, so no access can touch a page the copy does
//    not own.
#ifndef MI355_BLIT_KERNELS_H_
#define MI355_BLIT_KERNELS_H_

#include <stdint.h>

// The device primitives (memory accessors, moves between lanes, ids).  A host
// build that executes these kernels lane by lane names its own header here.
#ifdef MI355_BLIT_DEVICE_HEADER
#include MI355_BLIT_DEVICE_HEADER
#else
#include "blit_device.h"
#endif

#include "blit_args.h"

namespace mi355 {

MI355_DEVICE v4u realign(v4u x, unsigned w4, unsigned r) {
  v4u o;
  o.x = shift_bytes(x.y, x.x, r);
  o.y = shift_bytes(x.z, x.y, r);
  o.z = shift_bytes(x.w, x.z, r);
  o.w = shift_bytes(w4, x.w, r);
  return o;
}

// ---------------------------------------------------------------------------
// Tiling.  The body of a transfer is n_vec 16-byte vectors starting at a
// 16-byte aligned destination address.  Tiles of 64*U vectors are anchored at
// 256-byte boundaries of the DESTINATION: with lead = (address of vector 0 &
// 255) / 16, vector v sits at virtual index v + lead and tile t covers virtual
// indices [t*64U, (t+1)*64U).  Every wave's stores then cover whole cache lines
// (the first and last tile excepted), whatever the destination's alignment;
// unanchored, each wave would share its first and last line with a neighbour
// and the memory side would see half-line writes.
// ---------------------------------------------------------------------------

struct TileRange {
  uint64_t n_virtual;   // n_vec + lead
  uint64_t first_full;  // first tile wholly inside [lead, n_virtual)
  uint64_t end_full;    // one past the last such tile
};

template <int U>
MI355_DEVICE TileRange tile_range(uint64_t n_vec, unsigned lead) {
  constexpr uint64_t kTile = kWave * U;
  TileRange t;
  t.n_virtual = n_vec + lead;
  t.first_full = lead ? 1 : 0;
  t.end_full = t.n_virtual / kTile;
  return t;
}

// Copies n_vec vectors to d (16-byte aligned).  Source vector v starts r bytes
// after s + v, where s is dword aligned; r != 0 only when SHIFT.  Called by
// whole waves: wave w of n_waves takes full tiles first_full + w, + n_waves,
// ...; wave partial_wave takes the cut tiles at either end.
template <int U, bool NTL, int NTS, bool SHIFT>
MI355_DEVICE void copy_vectors(v4u* __restrict__ d, const v4u_a4* __restrict__ s,
                                             unsigned r, uint64_t n_vec, unsigned lead,
                                             uint64_t wave, uint64_t n_waves,
                                             uint64_t partial_wave, unsigned lane) {
  constexpr uint64_t kTile = kWave * U;
  const TileRange tr = tile_range<U>(n_vec, lead);
  // virtual bases: index v + lead; never dereferenced below index lead
  v4u* dv = d - lead;
  const v4u_a4* sv = s - lead;
  for (uint64_t t = tr.first_full + wave; t < tr.end_full; t += n_waves) {
    const uint64_t base = t * kTile + lane;
    v4u x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) x[u] = ld_v4<NTL>(sv + base + u * kWave);
    if constexpr (SHIFT) {
      // Lane 0 fetches the first dword after the tile: with r != 0 it holds
      // the last r bytes the tile needs, so it is always a wanted dword.
      unsigned e = 0;
      if (lane == 0) e = ld_u32<NTL>(reinterpret_cast<const unsigned*>(sv + t * kTile + kTile));
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const unsigned nxt = (u + 1 < U) ? x[u + 1 < U ? u + 1 : u].x : e;
        const unsigned w4 = wave_rotate_down1(lane == 0 ? nxt : x[u].x);
        st_v4<NTS>(dv + base + u * kWave, realign(x[u], w4, r));
      }
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) st_v4<NTS>(dv + base + u * kWave, x[u]);
    }
  }
  if (wave == partial_wave) {
    // virtual ranges of the cut tiles: [lead, end of tile 0) and
    // [start of the last tile, n_virtual); one range when they coincide
    uint64_t lo[2], hi[2];
    int n_ranges = 0;
    if (lead) {
      lo[n_ranges] = lead;
      hi[n_ranges] = tr.n_virtual < kTile ? tr.n_virtual : kTile;
      ++n_ranges;
    }
    if (tr.n_virtual % kTile != 0 && (tr.end_full > 0 || !lead)) {
      lo[n_ranges] = tr.end_full * kTile > lead ? tr.end_full * kTile : lead;
      hi[n_ranges] = tr.n_virtual;
      ++n_ranges;
    }
    for (int i = 0; i < n_ranges; ++i) {
      for (uint64_t v = lo[i] + lane; v < hi[i]; v += kWave) {
        v4u x = ld_v4<NTL>(sv + v);
        if constexpr (SHIFT) {
          const unsigned w4 = ld_u32<NTL>(reinterpret_cast<const unsigned*>(sv + v + 1));
          x = realign(x, w4, r);
        }
        st_v4<NTS>(dv + v, x);
      }
    }
  }
}

// Head (< 16 bytes in front of the first aligned vector) and tail (< 16 bytes
// after the last one), one byte per lane: lanes 0..15 head, 16..31 tail.
MI355_DEVICE void copy_edges(uint8_t* dst, const uint8_t* src, uint64_t bytes,
                                           unsigned head, uint64_t n_vec, unsigned lane) {
  const uint64_t tail_off = head + 16 * n_vec;
  const unsigned tail = static_cast<unsigned>(bytes - tail_off);
  if (lane < head) {
    st_u8(dst + lane, ld_u8(src + lane));
  } else if (lane >= 16 && lane - 16 < tail) {
    st_u8(dst + tail_off + lane - 16, ld_u8(src + tail_off + lane - 16));
  }
}

// Index of the calling wave among all waves of the launch (wave-uniform).
MI355_DEVICE uint64_t global_wave(unsigned waves_per_wg) {
  return wave_uniform(workgroup_index() * waves_per_wg + thread_in_workgroup() / kWave);
}

// global_wave() of a launch whose workgroups take their work in runs per XCD
// (xcd_workgroup): workgroups below x.full swap places among themselves, the
// others keep theirs.  x.full == 0: launch order.
// Written without a branch on purpose: the permutation is a dozen scalar
// instructions, and with every field of x used unconditionally the compiler
// fetches the whole argument block in one go at the kernel's entry instead of
// in pieces behind each branch (three dependent scalar loads in front of a
// wave's first data load became one).
MI355_DEVICE uint64_t global_wave_xcd(unsigned waves_per_wg, const XcdRuns& x) {
  const uint32_t wg = workgroup_index();
  const uint32_t permuted = xcd_workgroup(wg, x);
  return wave_uniform((wg < x.full ? permuted : wg) * waves_per_wg + thread_in_workgroup() / kWave);
}

template <int U, bool NTL, int NTS, bool SHIFT>
MI355_DEVICE void copy_body(const CopyArgs& a) {
  const unsigned lane = thread_in_workgroup() & (kWave - 1);
  const uint64_t wave = global_wave_xcd(a.waves_per_wg, a.xcd);
  const uint64_t n_waves = a.n_waves;
  const uint8_t* sb = a.src + a.head;
  const unsigned r = SHIFT ? static_cast<unsigned>(reinterpret_cast<uintptr_t>(sb) & 3) : 0;
  copy_vectors<U, NTL, NTS, SHIFT>(reinterpret_cast<v4u*>(a.dst + a.head),
                                   reinterpret_cast<const v4u_a4*>(sb - r), r, a.n_vec, a.lead,
                                   wave, n_waves, a.partial_wave, lane);
  if (wave == a.edge_wave) copy_edges(a.dst, a.src, a.bytes, a.head, a.n_vec, lane);
}

template <int U, int NTS>
MI355_DEVICE void fill_body(const FillArgs& a) {
  const unsigned lane = thread_in_workgroup() & (kWave - 1);
  const uint64_t wave = global_wave_xcd(a.waves_per_wg, a.xcd);
  const uint64_t n_waves = a.n_waves;
  const v4u val = {a.value, a.value, a.value, a.value};
  constexpr uint64_t kTile = kWave * U;
  const TileRange tr = tile_range<U>(a.n_vec, a.lead);
  v4u* dv = reinterpret_cast<v4u*>(a.dst + a.head) - a.lead;
  for (uint64_t t = tr.first_full + wave; t < tr.end_full; t += n_waves) {
    const uint64_t base = t * kTile + lane;
#pragma unroll
    for (int u = 0; u < U; ++u) st_v4<NTS>(dv + base + u * kWave, val);
  }
  if (wave == a.partial_wave) {
    if (a.lead) {
      const uint64_t hi = tr.n_virtual < kTile ? tr.n_virtual : kTile;
      for (uint64_t v = a.lead + lane; v < hi; v += kWave) st_v4<NTS>(dv + v, val);
    }
    if (tr.n_virtual % kTile != 0 && (tr.end_full > 0 || !a.lead)) {
      const uint64_t lo = tr.end_full * kTile > a.lead ? tr.end_full * kTile : a.lead;
      for (uint64_t v = lo + lane; v < tr.n_virtual; v += kWave) st_v4<NTS>(dv + v, val);
    }
  }
  if (wave == a.edge_wave) {
    // whole dwords outside the vector body: lanes 0..3 head, 4..7 tail
    const uint64_t tail_off = a.head + 4 * a.n_vec;
    const unsigned tail = static_cast<unsigned>(a.n_dwords - tail_off);
    if (lane < a.head) st_u32(a.dst + lane, a.value);
    else if (lane >= 4 && lane - 4 < tail) st_u32(a.dst + tail_off + lane - 4, a.value);
  }
}

// ---------------------------------------------------------------------------
// Batched small copies: n descriptors {dst, src, bytes}, one submission.
// Each copy is cut into chunks of up to kChunkVecs body vectors, anchored at
// 256-byte boundaries of its destination like the tiles above (the first
// chunk also moves the head bytes, the last one the tail bytes).  A prefix sum
// over the chunk counts orders all chunks of the batch; a chunk is the unit of
// work, so a 64-byte copy and a 256 KiB copy load the device evenly.
// ---------------------------------------------------------------------------


// The head / body split of one descriptor.
struct DescShape {
  unsigned head;    // bytes in front of the first 16-byte aligned destination address
  unsigned lead;    // vector slots between the 256-byte boundary below and that address
  uint64_t n_vec;   // body vectors
};

MI355_DEVICE DescShape desc_shape(const BatchDesc& d) {
  DescShape sh;
  const unsigned a = static_cast<unsigned>(reinterpret_cast<uintptr_t>(d.dst));
  const unsigned h = (16 - (a & 15)) & 15;
  sh.head = h > d.bytes ? static_cast<unsigned>(d.bytes) : h;
  sh.lead = ((a + sh.head) & 255) / 16;
  sh.n_vec = (d.bytes - sh.head) / 16;
  return sh;
}

MI355_DEVICE unsigned desc_chunks(const BatchDesc& d) {
  if (d.bytes == 0) return 0;
  const DescShape sh = desc_shape(d);
  const uint64_t c = (sh.n_vec + sh.lead + kChunkVecs - 1) / kChunkVecs;
  return c ? static_cast<unsigned>(c) : 1u;
}

// Exclusive prefix sum over the 1024 lanes of a workgroup; *total gets the sum.
// lds holds 16 words.
MI355_DEVICE uint32_t block_scan_1024(uint32_t v, uint32_t* lds, uint32_t* total) {
  const unsigned lane = thread_in_workgroup() & (kWave - 1);
  const unsigned w = thread_in_workgroup() / kWave;
  uint32_t incl = v;
#pragma unroll
  for (unsigned off = 1; off < kWave; off <<= 1) {
    const uint32_t x = lane_read_up(incl, off);
    if (lane >= off) incl += x;
  }
  if (lane == kWave - 1) lds[w] = incl;
  workgroup_barrier();
  if (w == 0) {
    uint32_t s = lane < 16 ? lds[lane] : 0;
#pragma unroll
    for (unsigned off = 1; off < 16; off <<= 1) {
      const uint32_t x = lane_read_up(s, off);
      if (lane >= off) s += x;
    }
    if (lane < 16) lds[lane] = s;
  }
  workgroup_barrier();
  *total = lds[15];
  return (w ? lds[w - 1] : 0) + incl - v;
}

// Prefix sum of the chunk counts in two small launches (no workgroup ever
// waits for another):
//  1. mi355_batch_scan_local, one workgroup per 1024 copies: chunk_start[i] =
//     chunks of the copies before i in the same workgroup, block_sum[b] = all
//     chunks of workgroup b;
//  2. mi355_batch_scan_top, one workgroup: block_sum becomes its own exclusive
//     prefix, chunk_start[n] = all chunks.
// A copy's first chunk is block_sum[i / 1024] + chunk_start[i].  This is the
// path of device-resident descriptors; for host-resident ones the host does
// the sum (mi355_batch_emit_records).
MI355_DEVICE void scan_local_body(const ScanLocalArgs& a) {
  const BatchDesc* __restrict__ descs = a.descs;
  const uint64_t n = a.n;
  uint32_t* __restrict__ chunk_start = a.chunk_start;
  uint32_t* __restrict__ block_sum = a.block_sum;
  MI355_LDS uint32_t lds[16];
  const uint64_t i = static_cast<uint64_t>(workgroup_index()) * 1024 + thread_in_workgroup();
  BatchDesc d{nullptr, nullptr, 0};
  if (i < n) {
    if (a.private_copy) {
      const uint64_t* w = reinterpret_cast<const uint64_t*>(descs + i);
      d.dst = reinterpret_cast<uint8_t*>(ld_system_u64(w));
      d.src = reinterpret_cast<const uint8_t*>(ld_system_u64(w + 1));
      d.bytes = ld_system_u64(w + 2);
      st_obj(a.private_copy + i, d);
    } else {
      d = ld_obj(descs + i);
    }
  }
  const uint32_t c = i < n ? desc_chunks(d) : 0;
  uint32_t total;
  const uint32_t excl = block_scan_1024(c, lds, &total);
  if (i < n) st_u32(chunk_start + i, excl);
  if (thread_in_workgroup() == 0) st_u32(block_sum + workgroup_index(), total);
}

MI355_DEVICE void scan_top_body(const ScanTopArgs& a) {
  uint32_t* __restrict__ block_sum = a.block_sum;
  uint32_t* __restrict__ chunk_start = a.chunk_start;
  const uint64_t n = a.n;
  const uint32_t n_blocks = a.n_blocks;
  MI355_LDS uint32_t lds[16];
  uint32_t carry = 0;
  for (uint32_t base = 0; base < n_blocks; base += 1024) {
    const uint32_t j = base + thread_in_workgroup();
    const uint32_t v = j < n_blocks ? ld_u32<false>(block_sum + j) : 0;
    uint32_t total;
    const uint32_t excl = block_scan_1024(v, lds, &total);
    if (j < n_blocks) st_u32(block_sum + j, carry + excl);
    carry += total;
    workgroup_barrier();  // lds is reused by the next round
  }
  if (thread_in_workgroup() == 0) st_u32(chunk_start + n, carry);
}

// Chunk k of a copy.
MI355_DEVICE ChunkRecord make_record(const BatchDesc& d, uint32_t k) {
  const DescShape sh = desc_shape(d);
  const uint64_t n_virtual = sh.n_vec + sh.lead;
  uint64_t lo = static_cast<uint64_t>(k) * kChunkVecs;
  uint64_t hi = lo + kChunkVecs;
  if (lo < sh.lead) lo = sh.lead;
  if (hi > n_virtual) hi = n_virtual;
  if (hi < lo) hi = lo;  // a copy without body vectors still has one chunk
  ChunkRecord r;
  r.dst = d.dst + sh.head + 16 * (lo - sh.lead);
  r.src = d.src + sh.head + 16 * (lo - sh.lead);
  r.n_vec = static_cast<uint32_t>(hi - lo);
  r.head = k == 0 ? static_cast<uint16_t>(sh.head) : 0;
  r.tail = hi == n_virtual ? static_cast<uint16_t>(d.bytes - sh.head - 16 * sh.n_vec) : 0;
  r.lead = k == 0 ? sh.lead : 0;
  r.pad = 0;
  return r;
}

// Launched with workgroups of 256 (emit_records_grid).  A wave takes
// kEmitPiecesPerWave (pieces of) copies, one in each of its first lanes, and
// writes their records together: the chunk counts are summed across the wave,
// and lane l writes records l, l + 64, ... of the wave's combined list, finding
// each record's copy by bisecting the running sum with lane shuffles.  The
// work is balanced whatever the mix of lengths, and consecutive lanes write
// consecutive records (whole cache lines).  One lane writing all records of
// its own copy took 22 us for the benchmark's 542,613 records and 64 copies to
// a wave 11 us; but 64 copies to a wave is 64 rounds for a wave whose pieces
// are all 64 chunks long, and few waves: one copy of 2 GiB (8,192 pieces) took
// 37 us.  The descriptors and the record indices were written
// by the host, into host memory or across the bus into device memory, behind
// the GPU's caches: they are read at system scope.
// Writes the records of one wave's copies: lane l holds copy (dst, src,
// bytes) with `chunks` records (none in a lane without a copy), the wave's
// records start at out[0].
MI355_DEVICE void emit_wave_records(uint64_t dst, uint64_t src, uint64_t bytes, uint32_t chunks,
                                                  ChunkRecord* out, unsigned lane) {
  // exclusive running sum of the chunk counts over the wave's lanes
  uint32_t incl = chunks;
#pragma unroll
  for (unsigned off = 1; off < kWave; off <<= 1) {
    const uint32_t x = lane_read_up(incl, off);
    if (lane >= off) incl += x;
  }
  const uint32_t excl = incl - chunks;
  const uint32_t total = lane_read(incl, kWave - 1);
  const uint32_t dst_lo = static_cast<uint32_t>(dst), dst_hi = static_cast<uint32_t>(dst >> 32);
  const uint32_t src_lo = static_cast<uint32_t>(src), src_hi = static_cast<uint32_t>(src >> 32);
  const uint32_t len_lo = static_cast<uint32_t>(bytes), len_hi = static_cast<uint32_t>(bytes >> 32);
  // every lane runs the same number of rounds: the shuffles need all of them
  for (uint32_t base = 0; base < total; base += kWave) {
    const uint32_t j = base + lane;
    // The last lane whose running sum is <= j owns record j: lanes without
    // chunks share their sum with the next lane and lose to it, and those at
    // the wave's end have a sum of `total` and never win.
    unsigned owner = 0;
#pragma unroll
    for (unsigned step = kWave / 2; step >= 1; step >>= 1) {
      const uint32_t e = lane_read(excl, owner + step);
      if (e <= j) owner += step;
    }
    BatchDesc d;
    d.dst = reinterpret_cast<uint8_t*>(static_cast<uint64_t>(lane_read(dst_hi, owner)) << 32 |
                                       lane_read(dst_lo, owner));
    d.src = reinterpret_cast<const uint8_t*>(static_cast<uint64_t>(lane_read(src_hi, owner)) << 32 |
                                             lane_read(src_lo, owner));
    d.bytes = static_cast<uint64_t>(lane_read(len_hi, owner)) << 32 | lane_read(len_lo, owner);
    const uint32_t k = j - lane_read(excl, owner);
    if (j < total) st_obj(out + j, make_record(d, k));
  }
}

MI355_DEVICE void emit_records_body(const EmitRecordsArgs& a) {
  const unsigned lane = thread_in_workgroup() & (kWave - 1);
  const uint64_t wave = static_cast<uint64_t>(workgroup_index()) * 4 + thread_in_workgroup() / kWave;
  const uint64_t i = wave * kEmitPiecesPerWave + lane;
  const bool valid = lane < kEmitPiecesPerWave && i < a.n;
  uint64_t dst = 0, src = 0, bytes = 0;
  uint32_t first = 0;
  if (valid) {
    const uint64_t* w = reinterpret_cast<const uint64_t*>(a.descs + i);
    dst = ld_system_u64(w);
    src = ld_system_u64(w + 1);
    bytes = ld_system_u64(w + 2);
    first = ld_system_u32(a.first_record + i);
  }
  BatchDesc mine;
  mine.dst = reinterpret_cast<uint8_t*>(dst);
  mine.src = reinterpret_cast<const uint8_t*>(src);
  mine.bytes = bytes;
  const uint32_t chunks = valid ? desc_chunks(mine) : 0;
  // the wave's records are consecutive: lane 0's first record starts them
  emit_wave_records(dst, src, bytes, chunks, a.records + lane_read(first, 0), lane);
}

// Loads of one wave's share of a chunk: virtual vector indices [v0, v0 + 64 U)
// cut to [lead, lead + n_vec); up to U vectors per lane and, when the source
// is not dword aligned, the dword behind the share's last vector.
template <int U, bool NTL>
MI355_DEVICE void record_load(const ChunkRecord& rec, unsigned v0, unsigned lane,
                                            v4u (&x)[U], unsigned& e) {
  const unsigned r = static_cast<unsigned>(reinterpret_cast<uintptr_t>(rec.src)) & 3;
  const v4u_a4* sv = reinterpret_cast<const v4u_a4*>(rec.src - r) - rec.lead;
  const unsigned all = rec.lead + rec.n_vec;
  const unsigned end = all < v0 + kWave * U ? all : v0 + kWave * U;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const unsigned idx = v0 + lane + u * kWave;
    if (idx >= rec.lead && idx < end) x[u] = ld_v4<NTL>(sv + idx);
  }
  e = 0;
  if (r && end > v0 && end > rec.lead) e = ld_u32<NTL>(reinterpret_cast<const unsigned*>(sv + end));
}

// Realign and store what record_load fetched.  With a dword-aligned source
// the realignment is the identity (shift 0).
template <int U, int NTS>
MI355_DEVICE void record_store(const ChunkRecord& rec, unsigned v0, unsigned lane,
                                             const v4u (&x)[U], unsigned e) {
  const unsigned r = static_cast<unsigned>(reinterpret_cast<uintptr_t>(rec.src)) & 3;
  v4u* dv = reinterpret_cast<v4u*>(rec.dst) - rec.lead;
  const unsigned all = rec.lead + rec.n_vec;
  const unsigned end = all < v0 + kWave * U ? all : v0 + kWave * U;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const unsigned idx = v0 + lane + u * kWave;
    const unsigned nxt = x[u + 1 < U ? u + 1 : u].x;  // lane 0's copy is what lane 63 needs
    unsigned w4 = wave_rotate_down1(lane == 0 ? nxt : x[u].x);
    if (idx + 1 == end) w4 = e;
    if (idx >= rec.lead && idx < end) st_v4<NTS>(dv + idx, realign(x[u], w4, r));
  }
}

// Head bytes in front of the chunk's first vector, tail bytes behind its last.
MI355_DEVICE void record_edges(const ChunkRecord& rec, bool do_head, bool do_tail,
                                             unsigned lane) {
  if (do_head && lane < rec.head) {
    st_u8(rec.dst - rec.head + lane, ld_u8(rec.src - rec.head + lane));
  } else if (do_tail && lane >= 16 && lane - 16 < rec.tail) {
    const uint64_t off = 16ull * rec.n_vec + lane - 16;
    st_u8(rec.dst + off, ld_u8(rec.src + off));
  }
}

// A wave's record is a dependent load in front of everything else it does, and
// the records of chunks that run at the same time miss L2 together: every wave
// would wait for memory twice, once for its record and once for its data.  So
// the first wave of a chunk also reads one word of the record that the same
// XCD will need `ahead` waves later, with an ordinary vector load that returns
// before the data loads behind it: the line (four records) is then in that
// XCD's L2 when its time comes.  The value is not used; keep_alive() only keeps
// the compiler from dropping the load.
MI355_DEVICE unsigned touch_record_ahead(const ChunkRecord* records, uint64_t w, unsigned q,
                                                       unsigned ahead, unsigned split, uint64_t total_chunks,
                                                       unsigned lane) {
  unsigned v = 0;
  if (ahead && q == 0 && lane == 0) {
    const uint64_t c = (w + ahead) / split;
    if (c < total_chunks) v = ld_u32<false>(reinterpret_cast<const unsigned*>(records + c));
  }
  return v;
}

// SPLIT waves per 4 KiB chunk, chunks in global order and waves in address
// order within a chunk: the dispatcher then walks memory densely, the shape
// that streams best for a single large copy.  Each wave reads its chunk's
// record (one 32-byte scalar load) and then moves 256 / SPLIT vectors.
template <int SPLIT, bool NTL, int NTS>
MI355_DEVICE void batch_copy_records_body(const BatchCopyArgs& a) {
  constexpr int U = kChunkVecs / kWave / SPLIT;
  const ChunkRecord* __restrict__ records = a.records;
  const uint64_t total_chunks = a.total_chunks;
  const unsigned lane = thread_in_workgroup() & (kWave - 1);
  const uint64_t wave = global_wave_xcd(a.waves_per_wg, a.xcd);
  const uint64_t n_waves = a.n_waves;
  const unsigned ahead = a.prefetch_waves;
  for (uint64_t w = wave; w < total_chunks * SPLIT; w += n_waves) {
    // The record first, then the data loads it describes, and only then the
    // touch of the record ahead: nothing may stand between a wave's start and
    // its data loads that does not have to (the touch is a predicated vector
    // load, a block of its own to the compiler, and in front of the record's
    // load it delayed that load by its whole length).
    const ChunkRecord rec = ld_uniform_record(records + w / SPLIT);
    const unsigned q = static_cast<unsigned>(w % SPLIT);
    const unsigned v0 = q * (kChunkVecs / SPLIT);
    v4u x[U];
    unsigned e;
    record_load<U, NTL>(rec, v0, lane, x, e);
    const unsigned touched = touch_record_ahead(records, w, q, ahead, SPLIT, total_chunks, lane);
    record_store<U, NTS>(rec, v0, lane, x, e);
    record_edges(rec, q == 0, q == SPLIT - 1, lane);
    keep_alive(touched);
  }
}

// The copy that chunk c of a batch of device-resident descriptors belongs to,
// from the prefix sums: the group of 1024 copies it falls into, then the copy
// within the group (the last one that starts at or before c: copies without
// chunks share their start with their successor and lose to it).  c is below
// the batch's chunk total; *k is the chunk's index within its copy.
// UNIFORM: c is the same for every lane of the wave, and the prefix sums come
// in through scalar loads, as a record does.
template <bool UNIFORM>
MI355_DEVICE uint32_t ld_prefix(const uint32_t* p) {
  if constexpr (UNIFORM) return ld_uniform_u32(p);
  else return ld_u32<false>(p);
}

template <bool UNIFORM>
MI355_DEVICE uint64_t find_copy_of_chunk(const uint32_t* __restrict__ block_sum,
                                                       const uint32_t* __restrict__ chunk_start, uint64_t n,
                                                       uint32_t c, uint32_t* k) {
  uint64_t lo = 0, hi = (n + 1023) / 1024 - 1;
  while (lo < hi) {
    const uint64_t mid = lo + (hi - lo + 1) / 2;
    if (ld_prefix<UNIFORM>(block_sum + mid) <= c) lo = mid; else hi = mid - 1;
  }
  const uint32_t rem = c - ld_prefix<UNIFORM>(block_sum + lo);
  lo *= 1024;
  hi = lo + 1023 < n ? lo + 1023 : n - 1;
  while (lo < hi) {
    const uint64_t mid = lo + (hi - lo + 1) / 2;
    if (ld_prefix<UNIFORM>(chunk_start + mid) <= rem) lo = mid; else hi = mid - 1;
  }
  *k = rem - ld_prefix<UNIFORM>(chunk_start + lo);
  return lo;
}

// The record of chunk c, the same for every lane of the wave.
MI355_DEVICE ChunkRecord lookup_record(const BatchLookupArgs& a, uint32_t c) {
  uint32_t k;
  const uint64_t found = find_copy_of_chunk<true>(a.block_sum, a.chunk_start, a.n,
                                                  wave_uniform(c), &k);
  // Every lane has found the same copy: say so, and its descriptor comes in
  // through scalar loads like a record.
  const uint32_t i = wave_uniform(static_cast<uint32_t>(found));
  return make_record(ld_uniform_desc(a.descs + i), wave_uniform(k));
}

// Records for device-resident descriptors, one lane per record: the lane finds
// its copy through the prefix sums.  Launched with workgroups of 256 over the
// record buffer's capacity; lanes beyond the batch's chunk total have nothing
// to do.  Costs the same whatever the copies' lengths (a wave writing the
// records of its own 64 copies stalls on a long copy: 100 copies of 4 MiB took
// 300 us that way).
MI355_DEVICE void emit_records_lookup_body(const EmitRecordsDeviceArgs& a) {
  const uint64_t j = static_cast<uint64_t>(workgroup_index()) * 256 + thread_in_workgroup();
  const uint64_t total = ld_u32<false>(a.chunk_start + a.n);
  if (j >= total || j >= a.capacity) return;
  uint32_t k;
  const uint64_t i = find_copy_of_chunk<false>(a.block_sum, a.chunk_start, a.n, static_cast<uint32_t>(j), &k);
  st_obj(a.records + j, make_record(ld_obj(a.descs + i), k));
}

// The copy over records when only the device knows how many chunks there are:
// the grid was sized for a bound or an assumption, waves beyond the real total
// end at once, and waves stride when there are more chunks than waves.  One
// 4 KiB chunk per four waves, as above.
template <bool NTL, int NTS>
MI355_DEVICE void batch_copy_lookup_body(const BatchLookupArgs& a) {
  constexpr int SPLIT = 4;
  constexpr int U = kChunkVecs / kWave / SPLIT;
  const ChunkRecord* __restrict__ records = a.copy.records;
  const uint64_t capacity = a.copy.total_chunks;
  const uint64_t total_chunks = ld_u32<false>(a.copy.total);
  const unsigned lane = thread_in_workgroup() & (kWave - 1);
  const uint64_t wave = global_wave_xcd(a.copy.waves_per_wg, a.copy.xcd);
  const uint64_t n_waves = a.copy.n_waves;
  if (wave == 0 && lane == 0 && a.seen)
    st_system_u64(a.seen, a.n << 32 | total_chunks);
  const uint64_t have = total_chunks < capacity ? total_chunks : capacity;  // chunks with a record
  for (uint64_t w = wave; w < total_chunks * SPLIT; w += n_waves) {
    const uint64_t c = w / SPLIT;
    const unsigned q = static_cast<unsigned>(w % SPLIT);
    const ChunkRecord rec = c < capacity ? ld_uniform_record(records + c) : lookup_record(a, static_cast<uint32_t>(c));
    const unsigned v0 = q * (kChunkVecs / SPLIT);
    v4u x[U];
    unsigned e;
    record_load<U, NTL>(rec, v0, lane, x, e);
    const unsigned touched = touch_record_ahead(records, w, q, a.copy.prefetch_waves, SPLIT, have, lane);
    record_store<U, NTS>(rec, v0, lane, x, e);
    record_edges(rec, q == 0, q == SPLIT - 1, lane);
    keep_alive(touched);
  }
}

// Pitched 3-D region copy.  Every row is a copy of `width` bytes, cut into
// units of 64 * U vectors anchored at 256-byte boundaries of its destination
// like the tiles of a linear copy; one wave moves one unit.  A row's last unit
// also takes up to kRowOverflowVecs vectors beyond its end (one more vector
// for a few lanes), so that a row whose destination sits a little above a
// 256-byte boundary does not need a wave for the spill alone.  Everything
// follows from the unit's index by arithmetic: unit s is unit s % slots of row
// s / slots, `slots` being the largest unit count any row has; rows that need
// fewer skip the rest.  No memory beyond the two regions, one launch.
constexpr unsigned kRowOverflowVecs = 15;

MI355_DEVICE uint64_t row_units(uint64_t n_virtual, unsigned unit) {
  return n_virtual > kRowOverflowVecs + unit ? (n_virtual - kRowOverflowVecs + unit - 1) / unit : 1;
}

// One unit slot of a region whose rows are tiled like a linear copy
// (RectArgs::plain_rows): U loads and U stores per lane and nothing else.  A
// row's last unit may be a partial one, whose lanes beyond the row's end have
// nothing to do, or have up to kRowOverflowVecs vectors more than a unit, which
// its first lanes take.
template <int U, bool NTL, int NTS>
MI355_DEVICE void rect_plain_unit(const RectArgs& a, uint32_t slot, unsigned lane) {
  constexpr unsigned kUnit = kWave * U;
  const uint32_t line = div_magic(slot, a.magic_slots);
  const uint32_t kq = slot - line * a.slots;
  const uint32_t layer = div_magic(line, a.magic_rows);
  const uint32_t y = line - layer * a.rows;
  const uint64_t in_row = static_cast<uint64_t>(kq) * (kUnit * 16) + lane * 16;
  const v4u_a4* sv = reinterpret_cast<const v4u_a4*>(a.src + layer * a.src_slice + y * a.src_pitch + in_row);
  v4u* dv = reinterpret_cast<v4u*>(a.dst + layer * a.dst_slice + y * a.dst_pitch + in_row);
  const bool over = kq + 1 == a.slots && in_row + U * (kWave * 16) < a.width;
  v4u x[U + 1];
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (in_row + u * (kWave * 16) < a.width) x[u] = ld_v4<NTL>(sv + u * kWave);
  if (over) x[U] = ld_v4<NTL>(sv + U * kWave);
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (in_row + u * (kWave * 16) < a.width) st_v4<NTS>(dv + u * kWave, x[u]);
  if (over) st_v4<NTS>(dv + U * kWave, x[U]);
}

// One unit slot of a region with rows of any alignment.  Most units of a wide
// row lie inside it (neither its first nor its last): those are found with as
// little arithmetic as possible and moved like a tile of the linear copy, the
// others take the general path behind.  (Every instruction in front of a
// wave's first load counts: with 32 waves on a CU sharing its issue slots, a
// hundred scalar instructions are a fifth of a wave's life.)
template <int U, bool NTL, int NTS>
MI355_DEVICE void rect_unit(const RectArgs& a, uint32_t slot, unsigned lane) {
  constexpr unsigned kUnit = kWave * U;
  const uint32_t line = div_magic(slot, a.magic_slots);  // row index through all layers
  const uint32_t kq = slot - line * a.slots;
  uint8_t* drow = a.dst + line * a.dst_pitch;
  const uint8_t* srow = a.src + line * a.src_pitch;
  if (a.total_slots > a.slots * a.rows) {  // more than one layer
    const uint32_t layer = div_magic(line, a.magic_rows);
    const uint32_t y = line - layer * a.rows;
    drow = a.dst + layer * a.dst_slice + y * a.dst_pitch;
    srow = a.src + layer * a.src_slice + y * a.src_pitch;
  }
  // Rows of this kernel are wider than 64 slots, so a row's head (the bytes in
  // front of its first 16-byte aligned destination address) is never cut.
  const unsigned head = (0u - static_cast<unsigned>(reinterpret_cast<uintptr_t>(drow))) & 15;
  const unsigned lead = (static_cast<unsigned>(reinterpret_cast<uintptr_t>(drow)) + head) & 255;  // bytes below the body in its first unit
  // merged rows can be longer than 2^32 vectors: 64-bit counts
  const uint64_t n_virtual = (lead + (a.width - head)) >> 4;
  const uint64_t units = row_units(n_virtual, kUnit);
  if (kq != 0 && kq + 1 < units) {
    // destination of the unit's lane 0: 256-byte aligned, kq units above the row's anchor
    uint8_t* const d = drow + head - lead + static_cast<uint64_t>(kq) * (kUnit * 16);
    const uint8_t* const sb = srow + (d - drow);
    const unsigned r = static_cast<unsigned>(reinterpret_cast<uintptr_t>(sb)) & 3;
    const v4u_a4* sv = reinterpret_cast<const v4u_a4*>(sb - r) + lane;
    v4u* dv = reinterpret_cast<v4u*>(d) + lane;
    v4u x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) x[u] = ld_v4<NTL>(sv + u * kWave);
    // lane 0 fetches the dword behind the unit: with r != 0 it holds the
    // last r bytes the unit needs, and the row goes on behind it
    unsigned e = 0;
    if (r && lane == 0) e = ld_u32<NTL>(reinterpret_cast<const unsigned*>(sv + kUnit));
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const unsigned nxt = (u + 1 < U) ? x[u + 1 < U ? u + 1 : u].x : e;
      const unsigned w4 = wave_rotate_down1(lane == 0 ? nxt : x[u].x);
      st_v4<NTS>(dv + u * kWave, realign(x[u], w4, r));
    }
    return;
  }
  if (kq >= units) return;  // the row has fewer units than the widest one
  // The row's first or last unit (or its only one): a cut range of vectors,
  // the head and tail bytes, one more predicated vector per lane for the
  // overflow of a last unit.
  const bool last = kq + 1 == units;
  const unsigned lead_vecs = lead >> 4;
  const uint64_t v0 = static_cast<uint64_t>(kq) * kUnit;
  const uint64_t lo = v0 > lead_vecs ? v0 : lead_vecs;
  const uint64_t end = last ? n_virtual : v0 + kUnit;
  const uint8_t* sb = srow + head;
  const unsigned r = static_cast<unsigned>(reinterpret_cast<uintptr_t>(sb)) & 3;
  const v4u_a4* sv = reinterpret_cast<const v4u_a4*>(sb - r) - lead_vecs;
  v4u* dv = reinterpret_cast<v4u*>(drow + head) - lead_vecs;
  v4u x[U + 1];
#pragma unroll
  for (int u = 0; u <= U; ++u) {
    const uint64_t idx = v0 + lane + u * kWave;
    if (idx >= lo && idx < end) x[u] = ld_v4<NTL>(sv + idx);
  }
  // the dword behind the unit's last vector: with r != 0 it holds that
  // vector's last r bytes
  unsigned e = 0;
  if (r && end > lo) e = ld_u32<NTL>(reinterpret_cast<const unsigned*>(sv + end));
#pragma unroll
  for (int u = 0; u <= U; ++u) {
    const uint64_t idx = v0 + lane + u * kWave;
    const unsigned nxt = x[u < U ? u + 1 : u].x;  // lane 0's copy is what lane 63 needs
    unsigned w4 = wave_rotate_down1(lane == 0 ? nxt : x[u].x);
    if (idx + 1 == end) w4 = e;
    if (idx >= lo && idx < end) st_v4<NTS>(dv + idx, realign(x[u], w4, r));
  }
  // bytes in front of the first vector and behind the last
  const uint64_t body_end = head + 16 * (n_virtual - lead_vecs);
  const unsigned tail = static_cast<unsigned>(a.width - body_end);
  if (kq == 0 && lane < head) {
    st_u8(drow + lane, ld_u8(srow + lane));
  } else if (last && lane >= 16 && lane - 16 < tail) {
    const uint64_t off = body_end + lane - 16;
    st_u8(drow + off, ld_u8(srow + off));
  }
}

template <int U, bool NTL, int NTS>
MI355_DEVICE void rect_copy_body(const RectArgs& a) {
  const unsigned lane = thread_in_workgroup() & (kWave - 1);
  uint64_t w = global_wave_xcd(a.waves_per_wg, a.xcd);
  if (w >= a.total_slots) return;
  // A grid with a wave for every unit slot (the usual case) goes through the
  // body once; waves of a capped grid stride over the slots.
  if (a.plain_rows) {
    do {
      rect_plain_unit<U, NTL, NTS>(a, static_cast<uint32_t>(w), lane);
      w += a.n_waves;
    } while (w < a.total_slots);
    return;
  }
  do {
    rect_unit<U, NTL, NTS>(a, static_cast<uint32_t>(w), lane);
    w += a.n_waves;
  } while (w < a.total_slots);
}

// Moves bytes [off, end) of the 16-byte aligned destination slot `slot`, not
// all 16 of them; sa is the source of byte off.  Whole dwords where the range
// has them, single bytes at its ragged ends; the source is read in the aligned
// dwords that hold at least one wanted byte, all loads before the first store.
template <bool NTL>
MI355_DEVICE void copy_partial_slot(uintptr_t slot, unsigned off, unsigned end,
                                                  const uint8_t* sa) {
  const uintptr_t ss = reinterpret_cast<uintptr_t>(sa) - off;  // source of the slot's byte 0
  const unsigned r = static_cast<unsigned>(ss) & 3;
  const unsigned* base = reinterpret_cast<const unsigned*>(ss - r);
  unsigned wd[5];
#pragma unroll
  for (int k = 0; k < 5; ++k) {
    const int b0 = 4 * k - static_cast<int>(r);  // slot byte the dword starts at
    const bool wanted = b0 < static_cast<int>(end) && b0 + 4 > static_cast<int>(off);
    wd[k] = wanted ? ld_u32<NTL>(base + k) : 0u;
  }
  const v4u x = {wd[0], wd[1], wd[2], wd[3]};
  const v4u img = realign(x, wd[4], r);
  const unsigned o[4] = {img.x, img.y, img.z, img.w};
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const unsigned b_lo = 4u * q > off ? 4u * q : off;
    const unsigned b_hi = 4u * q + 4 < end ? 4u * q + 4 : end;
    if (b_hi <= b_lo) continue;
    if (b_hi - b_lo == 4) {
      st_u32(reinterpret_cast<unsigned*>(slot + 4 * q), o[q]);
    } else {
#pragma unroll
      for (unsigned b = 0; b < 4; ++b)
        if (4u * q + b >= b_lo && 4u * q + b < b_hi)
          st_u8(reinterpret_cast<uint8_t*>(slot + 4 * q + b), static_cast<uint8_t>(o[q] >> (8 * b)));
    }
  }
}

// Region copy of narrow rows.  With one wave per row a 256-byte row would use
// a quarter of the wave and the launch would be bound by the rate at which
// waves start.  Here every 16-byte slot of a row's destination gets a lane:
// the (row, slot) pairs of the whole region are numbered row by row and wave w
// takes numbers [64 w, 64 w + 64), whatever rows they belong to, so all lanes
// work and a wave's loads and stores cover several whole rows.  A slot the row
// covers completely is one aligned 16-byte store.  A slot cut by the row's
// first or last byte is moved as the 16 bytes at the row's start or end
// instead, an unaligned vector that overlaps its neighbour's slot with the
// same values: no byte loop and no divergence.  Only rows under 16 bytes go
// through copy_partial_slot.
template <bool NTL, int NTS>
MI355_DEVICE void rect_narrow_body(const RectNarrowArgs& a) {
  const unsigned lane = thread_in_workgroup() & (kWave - 1);
  const uint64_t wave = global_wave_xcd(a.waves_per_wg, a.xcd);
  const uint32_t lpr = a.lanes_per_row;
  const uint64_t total = static_cast<uint64_t>(a.lines) * lpr;
  const uint64_t n_groups = (total + kWave - 1) / kWave;
  for (uint64_t w = wave; w < n_groups; w += a.n_waves) {
    // row and slot of this lane's number 64 w + lane
    const uint64_t first = w * kWave;
    const uint64_t line0 = lpr == 1 ? first : mul_hi_u64(first, a.magic64);  // first / lpr
    const unsigned t = static_cast<unsigned>(first - line0 * lpr) + lane;    // < lpr + 64
    const unsigned g = div_magic(t, a.magic64);                              // t / lpr
    const unsigned j = t - g * lpr;
    const uint64_t line = line0 + g;
    if (line >= a.lines) continue;
    uint32_t layer = 0, y = static_cast<uint32_t>(line);
    if (a.lines > a.rows) {
      layer = static_cast<uint32_t>(line) / a.rows;
      y = static_cast<uint32_t>(line) - layer * a.rows;
    }
    uint8_t* d = a.dst + layer * a.dst_slice + y * a.dst_pitch;
    const uint8_t* s = a.src + layer * a.src_slice + y * a.src_pitch;
    const uintptr_t row_lo = reinterpret_cast<uintptr_t>(d);
    const uintptr_t row_hi = row_lo + a.width;
    const uintptr_t slot = (row_lo & ~static_cast<uintptr_t>(15)) + 16 * j;
    if (slot >= row_hi) continue;  // rows that start higher in their first slot need one slot less
    if (a.width >= 16) {
      uintptr_t p = slot > row_lo ? slot : row_lo;
      if (p + 16 > row_hi) p = row_hi - 16;
      st_v4_any<NTS>(p, ld_v4_any<NTL>(s + (p - row_lo)));
    } else {
      const uintptr_t lo = slot > row_lo ? slot : row_lo;
      const uintptr_t hi = slot + 16 < row_hi ? slot + 16 : row_hi;
      copy_partial_slot<NTL>(slot, static_cast<unsigned>(lo - slot), static_cast<unsigned>(hi - slot),
                             s + (lo - row_lo));
    }
  }
}

// ---------------------------------------------------------------------------
// Completion of an HSA signal from the device, queued behind a command.  In
// the reference the packet processor does this with the dispatch packet's
// completion_signal field (core/runtime/amd_blit_kernel.cpp:884); an agent
// other than the packet processor follows the protocol ROCr's SDMA engine
// uses (core/runtime/amd_blit_sdma.cpp:478-514): atomically decrement the
// value and, when the signal has an event mailbox, post the event id there
// and raise the interrupt that wakes waiters sleeping in the kernel driver.
// ---------------------------------------------------------------------------

MI355_DEVICE void signal_complete_body(const SignalArgs& a) {
  HsaSignalAbi* sig = a.sig;
  if (thread_in_workgroup() != 0) return;
  if (a.mode == kSignalStampStart) {
    st_system_release_u64(&sig->start_ts, realtime_ticks());
    return;
  }
  if (a.mode == kSignalStampEndAndComplete || a.mode == kSignalStampEnd) {
    st_system_release_u64(&sig->end_ts, realtime_ticks());
    if (a.mode == kSignalStampEnd) return;
  }
  signal_decrement_system(&sig->value);
  uint64_t* mailbox = reinterpret_cast<uint64_t*>(sig->event_mailbox_ptr);
  if (mailbox) {
    const uint32_t id = sig->event_id;
    st_system_release_u64(mailbox, static_cast<uint64_t>(id));
    send_interrupt(id);
  }
}

}  // namespace mi355

// ---------------------------------------------------------------------------
// Kernel entry points.  C linkage and systematic names, so that the same
// kernels can be launched through HIP (by address) and looked up by name in
// the stand-alone code object that the AQL path loads.  Each takes one
// plain struct: its bytes are the kernarg segment.
//   mi355_copy_u<unroll>_l<nt loads>_s<store policy>_r<realign>
//   mi355_fill_u<unroll>_s<store policy>
//   mi355_batch_records_p<waves per chunk>_l<nt loads>_s<store policy>
//   mi355_batch_lookup_l<nt loads>_s<store policy>
//   mi355_rect_u<unroll>_l<nt loads>_s<store policy>
//   mi355_rect_narrow_l<nt loads>_s<store policy>
// ---------------------------------------------------------------------------
#include "blit_kernel_list.h"

#define MI355_DEFINE_COPY(U, L, S, R)                                                  \
  MI355_KERNEL(1024) void                                   \
      mi355_copy_u##U##_l##L##_s##S##_r##R(mi355::CopyArgs a) {                        \
    mi355::copy_body<U, L != 0, S, R != 0>(a);                                         \
  }
MI355_FOR_EACH_COPY_KERNEL(MI355_DEFINE_COPY)

#define MI355_DEFINE_FILL(U, S)                                                        \
  MI355_KERNEL(1024) void mi355_fill_u##U##_s##S(mi355::FillArgs a) { \
    mi355::fill_body<U, S>(a);                                                         \
  }
MI355_FOR_EACH_FILL_KERNEL(MI355_DEFINE_FILL)

#define MI355_DEFINE_BATCH_RECORDS(P, L, S)                                            \
  MI355_KERNEL(1024) void                                   \
      mi355_batch_records_p##P##_l##L##_s##S(mi355::BatchCopyArgs a) {                 \
    mi355::batch_copy_records_body<P, L != 0, S>(a);                                   \
  }
MI355_FOR_EACH_BATCH_RECORDS_KERNEL(MI355_DEFINE_BATCH_RECORDS)

#define MI355_DEFINE_RECT(U, L, S)                                                     \
  MI355_KERNEL(1024) void                                   \
      mi355_rect_u##U##_l##L##_s##S(mi355::RectArgs a) {                               \
    mi355::rect_copy_body<U, L != 0, S>(a);                                            \
  }
MI355_FOR_EACH_RECT_KERNEL(MI355_DEFINE_RECT)

#define MI355_DEFINE_RECT_NARROW(L, S)                                                 \
  MI355_KERNEL(1024) void                                   \
      mi355_rect_narrow_l##L##_s##S(mi355::RectNarrowArgs a) {                         \
    mi355::rect_narrow_body<L != 0, S>(a);                                             \
  }
MI355_FOR_EACH_RECT_NARROW_KERNEL(MI355_DEFINE_RECT_NARROW)

#define MI355_DEFINE_BATCH_LOOKUP(L, S)                                                \
  MI355_KERNEL(1024) void                                   \
      mi355_batch_lookup_l##L##_s##S(mi355::BatchLookupArgs a) {                       \
    mi355::batch_copy_lookup_body<L != 0, S>(a);                                       \
  }
MI355_FOR_EACH_BATCH_LOOKUP_KERNEL(MI355_DEFINE_BATCH_LOOKUP)

MI355_KERNEL(1024) void mi355_batch_scan_local(mi355::ScanLocalArgs a) {
  mi355::scan_local_body(a);
}
MI355_KERNEL(1024) void mi355_batch_scan_top(mi355::ScanTopArgs a) {
  mi355::scan_top_body(a);
}
MI355_KERNEL(256) void mi355_batch_emit_records(mi355::EmitRecordsArgs a) {
  mi355::emit_records_body(a);
}
MI355_KERNEL(256) void mi355_batch_emit_records_lookup(mi355::EmitRecordsDeviceArgs a) {
  mi355::emit_records_lookup_body(a);
}
MI355_KERNEL(64) void mi355_signal_complete(mi355::SignalArgs a) {
  mi355::signal_complete_body(a);
}

#endif  // MI355_BLIT_KERNELS_H_
