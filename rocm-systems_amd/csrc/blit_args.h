// Kernel argument blocks of the gfx950 blit kernels, shared by device code and
// by the two host sides that launch it (HIP launch and hand-built AQL packets).
// Each kernel takes exactly one of these structs by value: its bytes are the
// kernel's kernarg segment.  They take the place of BlitKernel::KernelArgs
// (projects/rocr-runtime/runtime/hsa-runtime/core/inc/amd_blit_kernel.h:122-154).
// Plain C++ without any HIP construct.
#ifndef MI355_BLIT_ARGS_H_
#define MI355_BLIT_ARGS_H_

#include <stdint.h>

namespace mi355 {

constexpr unsigned kWave = 64;
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
};

struct ScanTopArgs {
  uint32_t* block_sum;
  uint32_t* chunk_start;
  uint64_t n;
  uint32_t n_blocks;
};

struct FinalizeArgs {
  uint64_t n;
  uint32_t* chunk_start;
  const uint32_t* block_sum;
};

struct MakeRecordsArgs {
  const BatchDesc* descs;
  uint64_t n;
  const uint32_t* chunk_start;
  const uint32_t* block_sum;
  uint64_t total_chunks;
  ChunkRecord* records;
  uint32_t n_blocks;
};

struct BatchCopyArgs {
  const ChunkRecord* records;
  uint64_t total_chunks;
  uint32_t waves_per_wg;
  uint32_t n_waves;
};

struct BatchStridedArgs {
  const BatchDesc* descs;
  uint64_t n;
  const uint32_t* chunk_start;
  uint32_t waves_per_wg;
  uint32_t n_waves;
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

struct SignalArgs {
  HsaSignalAbi* sig;
};

}  // namespace mi355

#endif  // MI355_BLIT_ARGS_H_
