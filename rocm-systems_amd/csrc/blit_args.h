// Kernel argument blocks of the gfx950 blit kernels, shared by device code and
// by the two host sides that launch it (HIP launch and hand-built AQL packets).
// Each kernel takes exactly one of these structs by value: its bytes are the
// kernel's kernarg segment.  They take the place of BlitKernel::KernelArgs
// (projects/rocr-runtime/runtime/hsa-runtime/core/inc/amd_blit_kernel.h:122-154).
// Plain C++; the one function here is also compiled for the device.
#ifndef MI355_BLIT_ARGS_H_
#define MI355_BLIT_ARGS_H_

#include <stdint.h>

#ifdef __HIPCC__
#define MI355_HOST_DEVICE __host__ __device__
#else
#define MI355_HOST_DEVICE
#endif

namespace mi355 {

constexpr unsigned kWave = 64;

// Division of a 32-bit n by an invariant d without a divide: with m =
// magic_divisor(d) = ceil(2^64 / d), n / d == (n * m) >> 64 for all n < 2^32
// (the error n * (m * d - 2^64) stays below 2^64).  d == 1 has no such m in 64
// bits and is encoded as 0.
inline uint64_t magic_divisor(uint32_t d) { return d > 1 ? ~0ull / d + 1 : 0; }

MI355_HOST_DEVICE inline uint32_t div_magic(uint32_t n, uint64_t magic) {
#ifdef __HIP_DEVICE_COMPILE__
  // a select, not a branch: the multiplication is cheaper than the jump
  const uint32_t q = static_cast<uint32_t>(__umul64hi(n, magic));
  return magic ? q : n;
#else
  return magic ? static_cast<uint32_t>((static_cast<unsigned __int128>(n) * magic) >> 64) : n;
#endif
}

// XCD-aware launch order.  The hardware deals consecutive workgroups to the 8
// XCDs in turn (workgroup b runs on XCD b % 8).  With run != 0, workgroup
// b < full does the work of workgroup xcd_workgroup(b) instead, which gives
// every XCD runs of `run` neighbouring workgroups: XCD x takes workgroups
// [x * run, (x + 1) * run) of every round of 8 * run.  A permutation of
// [0, full); full is a multiple of 8 * run and the workgroups from there on
// keep their place.
struct XcdRuns {
  uint32_t run;    // workgroups per run; 0 = launch order
  uint32_t full;   // workgroups that take part; 0 when run == 0
  uint64_t magic;  // magic_divisor(run)
};

MI355_HOST_DEVICE inline uint32_t xcd_workgroup(uint32_t b, const XcdRuns& x) {
  const uint32_t xcd = b & 7, j = b >> 3;
  const uint32_t q = div_magic(j, x.magic);
  return (q * 8 + xcd) * x.run + (j - q * x.run);
}

// The permutation of a launch of `grid` workgroups in runs of `run` (0 or 1:
// launch order): whole rounds of 8 runs take part.
inline XcdRuns make_xcd_runs(uint32_t grid, uint32_t run) {
  XcdRuns x{0, 0, 0};
  if (run > 1) {
    const uint64_t round = 8ull * run;
    x.run = run;
    x.full = static_cast<uint32_t>(grid / round * round);
    x.magic = magic_divisor(run);
  }
  return x;
}

constexpr unsigned kChunkVecs = 256;  // vectors of one batched-copy chunk: 4 KiB

struct CopyArgs {
  uint8_t* dst;
  const uint8_t* src;
  uint64_t bytes;
  uint64_t n_vec;  // 16-byte vectors in the body
  uint32_t head;   // bytes in front of the body, <= 15
  uint32_t lead;   // ((dst + head) & 255) / 16: vector slots below the body in its first tile
  // Waves that take the cut tiles at both ends and the head/tail bytes: the
  // two after the wave of the last full tile, worked out on the host.
  uint32_t partial_wave;
  uint32_t edge_wave;
  // Launch shape, passed explicitly so that the kernels need no implicit
  // kernel arguments and can be dispatched from a hand-built AQL packet.
  uint32_t waves_per_wg;
  uint32_t n_waves;  // grid * waves_per_wg
  XcdRuns xcd;
};

struct FillArgs {
  uint32_t* dst;
  uint64_t n_dwords;
  uint64_t n_vec;  // 16-byte vectors in the body
  uint32_t head;   // dwords in front of the body, <= 3
  uint32_t lead;   // as in CopyArgs
  uint32_t value;
  uint32_t partial_wave;  // as in CopyArgs
  uint32_t edge_wave;
  uint32_t waves_per_wg;
  uint32_t n_waves;
  XcdRuns xcd;
};

struct BatchDesc {
  uint8_t* dst;
  const uint8_t* src;
  uint64_t bytes;
};

// Everything a wave needs to move one chunk, so that it reads one record
// instead of a map entry, a descriptor and two prefix sums in sequence.
struct __attribute__((aligned(32))) ChunkRecord {
  uint8_t* dst;        // first 16-byte vector of the chunk (16-byte aligned)
  const uint8_t* src;  // source byte that lands on dst[0]
  uint32_t n_vec;      // vectors in the chunk, <= kChunkVecs - lead
  uint16_t head;       // bytes in front of dst, first chunk of a copy only
  uint16_t tail;       // bytes behind the last vector, last chunk only
  uint32_t lead;       // (dst & 255) / 16: non-zero on a copy's first chunk only
  uint32_t pad;
};
static_assert(sizeof(ChunkRecord) == 32, "one s_load_dwordx8");

struct ScanLocalArgs {
  const BatchDesc* descs;
  uint64_t n;
  uint32_t* chunk_start;
  uint32_t* block_sum;
  // Not null: descs were staged by the host (into host memory, or across the
  // bus into device memory, behind the GPU's caches); they are read at system
  // scope and copied here for the kernels that follow.
  BatchDesc* private_copy;
};

struct ScanTopArgs {
  uint32_t* block_sum;
  uint32_t* chunk_start;
  uint64_t n;
  uint32_t n_blocks;
};

// Host-resident descriptors: the host has cut them into pieces and summed
// their chunk counts.  A wave of the record kernel takes kEmitPiecesPerWave
// pieces, one in each of its first lanes, and all of its 64 lanes write their
// records; emit_records_grid is the number of 256-lane workgroups n pieces need.
constexpr unsigned kEmitPiecesPerWave = 8;
inline uint32_t emit_records_grid(uint64_t n) {
  const uint64_t per_wg = 4 * kEmitPiecesPerWave;
  return static_cast<uint32_t>((n + per_wg - 1) / per_wg);
}

struct EmitRecordsArgs {
  const BatchDesc* descs;       // staged by the host
  const uint32_t* first_record; // index of each piece's first record
  uint64_t n;
  ChunkRecord* records;
};

// Device-resident descriptors: the prefix sum was done on the device
// (chunk_start within each group of 1024 copies, block_sum across groups); one
// lane per record, records beyond `capacity` are not written.
struct EmitRecordsDeviceArgs {
  const BatchDesc* descs;
  const uint32_t* chunk_start;
  const uint32_t* block_sum;
  uint64_t n;
  ChunkRecord* records;
  uint64_t capacity;
};

struct BatchCopyArgs {
  const ChunkRecord* records;
  uint64_t total_chunks;  // the number of records
  // Device-resident descriptors only (BatchLookupArgs): where the device has
  // put the number of chunks.  Null when the host knows it.
  const uint32_t* total;
  uint32_t waves_per_wg;
  uint32_t n_waves;
  XcdRuns xcd;
  // Not 0: the first wave of a chunk also touches the record of the chunk this
  // many waves ahead of it, which the same XCD gets to a few microseconds later
  // (one round of XCD runs on; in launch order a multiple of 8 workgroups), so
  // that the record is in that XCD's L2 when its own waves ask for it.
  uint32_t prefetch_waves;
  uint32_t pad;
};

// The copy over records for device-resident descriptors, whose number of
// chunks only the device knows: copy.total points at it, copy.total_chunks is
// the number of records there was room for, and a chunk beyond that is looked
// up in the prefix sums instead (a batch larger than the caller's bound, or
// than the library assumed, is slower, not wrong).
struct BatchLookupArgs {
  BatchCopyArgs copy;
  const BatchDesc* descs;
  const uint32_t* chunk_start;  // within each group of 1024 copies
  const uint32_t* block_sum;    // chunks in front of each group
  uint64_t n;
  // Host memory where one lane leaves n << 32 | chunks for the host to size
  // the next such batch by; may be null.
  uint64_t* seen;
};

// A pitched 3-D region copy: `layers` slices of `rows` rows of `width` bytes.
// dst and src address the first byte of row 0 in layer 0 (offsets folded in by
// the host).  Each row is cut into units of 64 * unroll vectors, one per wave;
// `slots` is the largest unit count any row has, so that unit slot s belongs
// to row s / slots: no prefix sum and no memory beyond the two regions.
struct RectArgs {
  uint8_t* dst;
  const uint8_t* src;
  uint64_t dst_pitch;
  uint64_t dst_slice;
  uint64_t src_pitch;
  uint64_t src_slice;
  uint64_t width;
  uint32_t rows;
  uint32_t slots;
  uint32_t total_slots;  // rows * layers * slots
  uint32_t waves_per_wg;
  uint32_t n_waves;
  XcdRuns xcd;
  // n / slots == div_magic(n, magic_slots) and n / rows == div_magic(n,
  // magic_rows) for every 32-bit n (magic_divisor below).
  uint64_t magic_slots;
  uint64_t magic_rows;
  // Not 0: every row starts at a cache-line boundary of the destination, is a
  // whole number of lines long and lies a multiple of 4 bytes from its source,
  // so that no unit has a head, a tail or bytes to realign: unit k of a row is
  // the row's bytes [k, k + 1) * 1024 * U, cut at the row's end.
  uint32_t plain_rows;
  uint32_t pad;
};

// The same region copy for rows of up to about 1 KiB: every 16-byte slot of a
// row's destination takes a lane, lanes_per_row of them per row, and the
// (row, slot) pairs of the whole region are dealt out to waves 64 at a time.
struct RectNarrowArgs {
  uint8_t* dst;
  const uint8_t* src;
  uint64_t dst_pitch;
  uint64_t dst_slice;
  uint64_t src_pitch;
  uint64_t src_slice;
  uint64_t magic64;  // ceil(2^64 / lanes_per_row): n / lanes_per_row == mulhi(n, magic64), n < 2^38
  uint32_t width;
  uint32_t rows;     // rows per layer
  uint32_t lines;    // rows * layers
  uint32_t lanes_per_row;
  uint32_t pad;
  uint32_t waves_per_wg;
  uint32_t n_waves;
  XcdRuns xcd;
};

// Layout of amd_signal_t (inc/amd_hsa_signal.h, struct amd_signal_s).
struct HsaSignalAbi {
  int64_t kind;
  int64_t value;
  uint64_t event_mailbox_ptr;
  uint32_t event_id;
  uint32_t reserved1;
  uint64_t start_ts;
  uint64_t end_ts;
  uint64_t queue_ptr;
  uint32_t reserved3[2];
};
static_assert(sizeof(HsaSignalAbi) == 64, "amd_signal_t is 64 bytes");

// What mi355_signal_complete does to the signal.  The stamps are the signal's
// start_ts / end_ts, which the packet processor writes for a dispatch on a
// queue with the profiling bit set (amd_blit_kernel.cpp:839-842) and
// hsa_amd_profiling_get_async_copy_time reads (hsa_ext_amd.cpp:474-502); on a
// HIP stream there is no such bit and one-lane kernels in front of and behind
// the command write them.
constexpr uint32_t kSignalComplete = 0;             // decrement, wake waiters
constexpr uint32_t kSignalStampStart = 1;           // start_ts = now, nothing else
constexpr uint32_t kSignalStampEndAndComplete = 2;  // end_ts = now, then complete
constexpr uint32_t kSignalStampEnd = 3;             // end_ts = now, nothing else

struct SignalArgs {
  HsaSignalAbi* sig;
  uint32_t mode;
  uint32_t pad;
};

}  // namespace mi355

#endif  // MI355_BLIT_ARGS_H_
