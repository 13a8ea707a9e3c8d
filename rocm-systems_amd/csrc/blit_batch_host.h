// Host half of the batched copy with host-resident descriptors, shared by the
// HIP and the AQL submission paths: validation, the chunk count of every
// copy, and the staging image the GPU reads.  Pure host code.
//
// The host walks the descriptors anyway to validate them, so it also does the
// prefix sum over their chunk counts: the GPU then needs one small kernel (a
// wave writes the chunk records of its 8 copies) before the copy kernel.
// Copies of more than 64 chunks are cut into pieces of 64 chunks that are
// copies in their own right, so that no wave has more than 64 rounds of
// records to write.  No counterpart in the reference.
#ifndef MI355_BLIT_BATCH_HOST_H_
#define MI355_BLIT_BATCH_HOST_H_

#include <stdint.h>
#include <string.h>

#include <vector>

#include "blit_args.h"
#include "blit_plan.h"
#include "mi355_blit.h"

namespace mi355 {

// A long copy is handed to the GPU as pieces of 64 chunks, copies in their
// own right: the record kernel gives a wave 8 pieces (kEmitPiecesPerWave),
// whose records it writes 64 at a time, so a wave has at most 8 rounds to go
// through however long the copies are (100 copies of 4 MiB: 138 us; 161 us with
// 64 pieces to a wave, 228 us with pieces of 1 MiB on top of that).  Pieces end
// where the copy's own chunks end, so cutting adds no chunk.
constexpr uint64_t kBatchPieceChunks = 64;
constexpr uint64_t kBatchPieceBytes = kBatchPieceChunks * 16 * kBatchChunkVecs;  // plus up to 15 bytes at either end

struct BatchShape {
  uint64_t pieces = 0;        // descriptors after cutting
  uint64_t total_chunks = 0;  // 4 KiB chunks of all pieces
  uint64_t total_bytes = 0;
};

// Chunks of one copy (desc_chunks in the kernels).
inline uint64_t batch_desc_chunks(uint64_t dst, uint64_t bytes) {
  if (bytes == 0) return 0;
  uint64_t head = (16 - (dst & 15)) & 15;
  if (head > bytes) head = bytes;
  const uint64_t n_vec = (bytes - head) / 16;
  const uint64_t lead = ((dst + head) & 255) / 16;
  const uint64_t c = (n_vec + lead + kBatchChunkVecs - 1) / kBatchChunkVecs;
  return c ? c : 1;
}

// The most chunks n copies of at most max_total_bytes together can have: a
// copy of b bytes has at most ceil((b / 16 + 15) / 256) <= b / 4096 + 2 of
// them (15 = the vectors between the 256-byte line and the copy's first aligned
// byte).  0 when the record indices would not fit their 32 bits.
inline uint64_t batch_bound_chunks(uint64_t n, uint64_t max_total_bytes) {
  const uint64_t c = max_total_bytes / (16 * kBatchChunkVecs) + 2 * n;
  return c < 0xffffffffull ? c : 0;
}

// Device-resident descriptors: the host sizes the record buffer and the grid
// without knowing the lengths.  With a bound from the caller both follow the
// bound.  Without one the library goes by the last such batch on the engine,
// whose copy kernel left its numbers of copies and chunks in host memory
// (`seen`, copies << 32 | chunks; 0 = none yet): the same chunks per copy less
// 1.5 %, and before any batch has reported, 8 chunks (32 KiB) a copy.  The grid
// has one 4-wave workgroup per chunk; waves beyond the real total end at once
// (0.2 ns of dispatch each: 65,536 copies of 256 bytes take 64 us on a grid of
// 65,536 workgroups and 160 us on one of 524,288), waves stride when there are
// more chunks than workgroups (65,536 copies of 2 GB: 698 us, 766 us on a
// quarter of the workgroups), and there is room for twice as many records.
// Either way a chunk beyond the records is found through the prefix sums by
// the copy kernel itself: a wrong guess or a bound that is exceeded costs
// speed, not correctness.  Records are capped at 512 MiB.
constexpr uint64_t kBatchMaxDeviceRecords = 1ull << 24;
constexpr uint64_t kBatchMinDeviceRecords = 1ull << 16;
constexpr uint64_t kBatchAssumedChunksPerCopy = 8;

struct BatchDeviceSizing {
  uint64_t records;      // capacity of the record buffer
  uint64_t grid_chunks;  // chunks the grid has a workgroup for
  uint64_t bytes;        // what the launch heuristics take the batch's size to be
};

// likely_chunks: the host's own estimate of the chunk count (batch_stage_raw),
// 0 for none; the grid then follows it instead of the bytes.
inline BatchDeviceSizing batch_device_sizing(uint64_t n, uint64_t max_total_bytes, uint64_t seen = 0,
                                             uint64_t likely_chunks = 0) {
  BatchDeviceSizing z;
  if (max_total_bytes) {
    // 0: a bound beyond what 32-bit record indices can count, which no batch
    // can need (the caller answers INVALID_ARGUMENT)
    uint64_t c = batch_bound_chunks(n, max_total_bytes);
    if (c > kBatchMaxDeviceRecords) c = kBatchMaxDeviceRecords;
    z.records = c;
    // Room for the most chunks the bound allows (two more than bytes / 4096
    // per copy), a grid for a little less than is likely (half a chunk more
    // per copy than bytes / 4096).  A wave without a chunk is not free -- it
    // takes a slot until it has read the chunk count -- while waves that stride
    // to a second chunk cost next to nothing: 65,536 copies of 2 GB
    // (542,613 chunks) take 712 us on a grid for 559,585 chunks, 700 us on one
    // for 542,613, 535,000 or 524,288, 705 us on one for 500,000.
    z.grid_chunks = max_total_bytes / (16 * kBatchChunkVecs) + n / 2 + 1;
    if (z.grid_chunks < n) z.grid_chunks = n;  // short copies: a chunk each
    if (likely_chunks) z.grid_chunks = likely_chunks - likely_chunks / 64 + 1;
    if (z.grid_chunks > c) z.grid_chunks = c;
    z.bytes = max_total_bytes;
  } else {
    const uint64_t seen_copies = seen >> 32, seen_chunks = seen & 0xffffffffull;
    if (seen_copies && seen_chunks) {
      // both below 2^32: the product fits
      const uint64_t likely = (seen_chunks * n + seen_copies - 1) / seen_copies;
      z.grid_chunks = likely - likely / 64 + 1;
    } else {
      z.grid_chunks = kBatchAssumedChunksPerCopy * n;
    }
    z.records = 2 * z.grid_chunks + 32;
    if (z.records < kBatchMinDeviceRecords) z.records = kBatchMinDeviceRecords;
    if (z.records > kBatchMaxDeviceRecords) z.records = kBatchMaxDeviceRecords;
    if (z.grid_chunks > z.records) z.grid_chunks = z.records;
    z.bytes = z.grid_chunks * (16 * kBatchChunkVecs);
  }
  return z;
}

// Calls f(dst, src, bytes) for every piece of one copy.
template <typename F>
inline void batch_for_each_piece(const mi355_blit_desc_t& d, F f) {
  const uint64_t dst = reinterpret_cast<uintptr_t>(d.dst), src = reinterpret_cast<uintptr_t>(d.src);
  // the copy's chunks are 4 KiB steps from the 256-byte boundary at or below
  // its first 16-byte aligned destination byte
  uint64_t head = (16 - (dst & 15)) & 15;
  if (head > d.bytes) head = d.bytes;
  const uint64_t anchor = (dst + head) & ~255ull;
  uint64_t at = 0;
  for (uint64_t piece = 1; at < d.bytes; ++piece) {
    uint64_t end = anchor + piece * kBatchPieceBytes - dst;
    // fewer than 16 bytes left over are the tail of this piece's last chunk
    if (end > d.bytes || d.bytes - end < 16) end = d.bytes;
    f(dst + at, src + at, end - at);
    at = end;
  }
}

// The staging image of a batch, built in ordinary host memory: the pieces and,
// for each, the index of its first chunk record.  The vectors are storage that
// is kept between calls; the image is their first `count` entries.
struct BatchImage {
  std::vector<BatchDesc> pieces;
  std::vector<uint32_t> first_record;
  size_t count = 0;
};

// Validates the descriptors, cuts them into pieces, sums the chunk counts: one
// pass.  With the copy into the staging buffer a submission costs the host
// 3.6 ns per descriptor (236 us for 65,536), which is what bounds a batch of
// many tiny copies: the GPU finishes 65,536 copies of 256 bytes in 67 us.
inline int batch_build(const mi355_blit_desc_t* descs, size_t n, BatchImage* image, BatchShape* out) {
  BatchShape s;
  image->count = 0;
  size_t cap = image->pieces.size();
  if (cap < n + 16) {
    cap = n + n / 8 + 16;
    image->pieces.resize(cap);
    image->first_record.resize(cap);
  }
  BatchDesc* pieces = image->pieces.data();
  uint32_t* first = image->first_record.data();
  size_t k = 0;
  uint64_t chunks = 0, bytes = 0;
  auto add = [&](uint64_t dst, uint64_t src, uint64_t len) {
    if (k == cap) {
      cap *= 2;
      image->pieces.resize(cap);
      image->first_record.resize(cap);
      pieces = image->pieces.data();
      first = image->first_record.data();
    }
    pieces[k].dst = reinterpret_cast<uint8_t*>(dst);
    pieces[k].src = reinterpret_cast<const uint8_t*>(src);
    pieces[k].bytes = len;
    first[k] = static_cast<uint32_t>(chunks);
    chunks += batch_desc_chunks(dst, len);
    ++k;
  };
  for (size_t i = 0; i < n; ++i) {
    const mi355_blit_desc_t& d = descs[i];
    if (d.bytes == 0) continue;
    if (!d.dst || !d.src) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
    bytes += d.bytes;
    const uint64_t dst = reinterpret_cast<uintptr_t>(d.dst);
    if (d.bytes <= kBatchPieceBytes - 256)
      add(dst, reinterpret_cast<uintptr_t>(d.src), d.bytes);  // the usual case: one piece wherever it starts
    else
      batch_for_each_piece(d, add);
    if (chunks > 0xffffffffull) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  }
  if (k > 0xffffffffull) return MI355_BLIT_ERROR_INVALID_ARGUMENT;
  image->count = k;
  s.pieces = k;
  s.total_chunks = chunks;
  s.total_bytes = bytes;
  *out = s;
  return MI355_BLIT_SUCCESS;
}

// Whether a batch of host-resident descriptors is better handed to the GPU as
// it is: the host's walk costs 2.2 ns per descriptor (3.6 ns with the copy
// into the staging buffer), the GPU needs 0.33 ns per KiB moved, so from
// thousands of copies of a few KiB on the host is the slower of the two
// (65,536 copies of 4000 bytes: 237 us through the walk, 107 us as
// device-resident descriptors).  Judged from 64 descriptors spread over the
// batch; a wrong guess costs time on one side or the other, nothing else.
constexpr size_t kBatchRawMinCopies = 4096;
constexpr uint64_t kBatchRawMaxMeanBytes = 8192;

// engine_idle: nothing of this engine is still running (no batch, no other
// command), so nothing hides the walk: a batch submitted to an idle engine starts as late as the host
// finishes with it.  Staged as they are the descriptors cost the host 1 ns
// each instead of 3.6 and the GPU two small launches more: 65,536 copies of
// 64 B .. 256 KiB, one batch at a time, take 927 us from submission to
// completion through the walk and 720 us as device-resident descriptors;
// submitted back to back the walk is hidden behind the batch before and wins
// (693 against 705 us a batch).  t->batch_staging overrides the choice.
// engine_idle is only asked when the answer depends on it.
template <typename IdleFn>
inline bool batch_prefers_raw_staging(const mi355_blit_desc_t* descs, size_t n, IdleFn engine_idle,
                                      const mi355_blit_tuning_t* t) {
  if (t && t->batch_staging) return t->batch_staging == 2;
  if (n < kBatchRawMinCopies) return false;
  uint64_t sum = 0;
  const size_t step = n / 64;
  for (size_t k = 0; k < 64; ++k) sum += descs[k * step].bytes;
  return sum <= 64 * kBatchRawMaxMeanBytes || engine_idle();
}

// Copies the descriptors as they are to where the GPU reads them, checking
// them on the way (a copy of bytes needs both pointers) and adding up their
// bytes.  *likely_chunks gets an estimate of the batch's chunk count for the
// grid: the bytes' share is exact, bytes / 4096, and what the copies' ends add
// to it -- between nothing and a chunk a copy, depending on where the copies
// start and end within their chunks -- is taken from about a thousand
// descriptors spread over the batch (65,536 copies of 4000 bytes have 65,536
// chunks, not the 96,769 that half a chunk a copy would make of them:
// 123 against 142 us).
inline int batch_stage_raw(const mi355_blit_desc_t* descs, size_t n, void* stage, uint64_t* total_bytes,
                           uint64_t* likely_chunks) {
  BatchDesc* out = static_cast<BatchDesc*>(stage);
  uint64_t bytes = 0;
  bool bad = false;
  for (size_t i = 0; i < n; ++i) {
    const mi355_blit_desc_t& d = descs[i];
    bad |= d.bytes != 0 && (!d.dst || !d.src);
    bytes += d.bytes;
    out[i].dst = static_cast<uint8_t*>(d.dst);
    out[i].src = static_cast<const uint8_t*>(d.src);
    out[i].bytes = d.bytes;
  }
  *total_bytes = bytes;
  // every descriptor of a small batch; of a large one 1024 at golden-ratio
  // steps, which no period in the batch's make-up can fall in with
  const uint64_t samples = n > 1024 ? 1024 : n;
  uint64_t sample_chunks = 0, sample_bytes = 0;
  for (uint64_t k = 0; k < samples; ++k) {
    const size_t i = n > 1024 ? static_cast<size_t>(k * 0x9e3779b97f4a7c15ull % n) : static_cast<size_t>(k);
    sample_chunks += batch_desc_chunks(reinterpret_cast<uintptr_t>(descs[i].dst), descs[i].bytes);
    sample_bytes += descs[i].bytes;
  }
  const uint64_t chunk_bytes = 16 * kBatchChunkVecs;
  const uint64_t ends = sample_chunks * chunk_bytes > sample_bytes ? sample_chunks * chunk_bytes - sample_bytes : 0;
  *likely_chunks = bytes / chunk_bytes +
                   static_cast<uint64_t>(static_cast<double>(ends) / static_cast<double>(chunk_bytes * samples) *
                                         static_cast<double>(n));
  return bad ? MI355_BLIT_ERROR_INVALID_ARGUMENT : MI355_BLIT_SUCCESS;
}

// Bytes of the staging buffer for `pieces` descriptors: the descriptors, then,
// right behind them, each one's first record index.
inline size_t batch_stage_bytes(uint64_t pieces) {
  return static_cast<size_t>(pieces) * (sizeof(BatchDesc) + sizeof(uint32_t));
}

// Copies the image to where the GPU reads it.
inline void batch_stage(const BatchImage& image, void* stage) {
  const size_t n = image.count;
  memcpy(stage, image.pieces.data(), n * sizeof(BatchDesc));
  memcpy(static_cast<uint8_t*>(stage) + n * sizeof(BatchDesc), image.first_record.data(), n * sizeof(uint32_t));
}

}  // namespace mi355

#endif  // MI355_BLIT_BATCH_HOST_H_
