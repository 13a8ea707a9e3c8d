// Where the 8 XCDs of an MI355X are in one long copy launch, over time.
//
// The launch permutation of the blit kernels (xcd_workgroup, csrc/blit_args.h)
// rests on one assumption about the hardware: workgroup b of a launch runs on
// XCD b % 8.  This program checks it and measures what follows from it.  It
// runs a copy kernel of the product's shape (single-wave workgroups, one
// 16-byte vector per lane, non-temporal loads, stores written through, the
// product's permutation) in which one workgroup in 64 of every XCD notes the
// XCD it runs on (HW_REG_XCC_ID) and the time (s_memrealtime, 100 MHz) at its
// start and when its store has completed.  From the notes: the XCD of every
// residue b % 8; how many of its own workgroups each XCD has started at 16
// points in time; and when each XCD finished.  The XCDs run at slightly
// different rates, each works through a share fixed by b % 8, and the launch
// ends when the slowest has finished: the others' idle time at the end grows
// with the length of the launch, which is why the library cuts long copies
// into pieces (copy_pieces, csrc/blit_plan.h).
//
// usage: xcd_progress [GiB = 4] [workgroups per XCD run = 576; 1 = launch order]
// Prints a table and, last, one line of JSON.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <algorithm>
#include <vector>

#include "blit_args.h"

using mi355::XcdRuns;

typedef unsigned v4u __attribute__((ext_vector_type(4)));

struct Note {
  uint32_t wg, tile, xcc, written;
  uint64_t t0, t1;
};

#define CHECK(x)                                                                  \
  do {                                                                            \
    hipError_t e_ = (x);                                                          \
    if (e_ != hipSuccess) {                                                       \
      fprintf(stderr, "HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
      return 2;                                                                   \
    }                                                                             \
  } while (0)

constexpr uint32_t kNoteEvery = 512;  // of every 512 consecutive workgroups the first 8 take notes: one per XCD

__global__ __launch_bounds__(64) void copy_and_note(const v4u* __restrict__ src, v4u* __restrict__ dst,
                                                     uint32_t n_tiles, XcdRuns x, Note* notes) {
  const uint32_t wg = blockIdx.x;
  const uint32_t tile = wg < x.full ? mi355::xcd_workgroup(wg, x) : wg;
  if (tile >= n_tiles) return;
  const bool noting = ((wg >> 3) % (kNoteEvery / 8)) == 0;
  uint64_t t0 = 0;
  if (noting) t0 = __builtin_amdgcn_s_memrealtime();
  const uint64_t i = static_cast<uint64_t>(tile) * 64 + threadIdx.x;
  const v4u v = __builtin_nontemporal_load(src + i);
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(dst + i), "v"(v) : "memory");
  if (noting && threadIdx.x == 0) {
    uint32_t xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    notes[(wg / kNoteEvery) * 8 + (wg & 7)] = Note{wg, tile, xcc & 15, 1, t0, __builtin_amdgcn_s_memrealtime()};
  }
}

int main(int argc, char** argv) {
  const uint64_t gib = argc > 1 ? strtoull(argv[1], nullptr, 10) : 4;
  const uint32_t run = argc > 2 ? static_cast<uint32_t>(atoi(argv[2])) : 576;
  if (gib < 1 || gib > 32) {
    fprintf(stderr, "size out of range: 1..32 GiB\n");
    return 2;
  }
  const uint64_t bytes = gib << 30;
  const uint32_t n_tiles = static_cast<uint32_t>(bytes / 1024);
  v4u *src = nullptr, *dst = nullptr;
  Note* notes = nullptr;
  CHECK(hipMalloc(&src, bytes));
  CHECK(hipMalloc(&dst, bytes));
  CHECK(hipMemset(src, 0x5a, bytes));
  CHECK(hipMemset(dst, 0, bytes));
  const uint32_t n_notes = (n_tiles / kNoteEvery + 1) * 8;
  CHECK(hipMalloc(&notes, n_notes * sizeof(Note)));
  CHECK(hipMemset(notes, 0, n_notes * sizeof(Note)));
  const XcdRuns x = mi355::make_xcd_runs(n_tiles, run);
  hipStream_t s;
  CHECK(hipStreamCreate(&s));
  // the launches before the one that is read bring the device to its sustained state
  const int settle = static_cast<int>(16 / gib) + 2;
  for (int i = 0; i < settle; ++i)
    hipLaunchKernelGGL(copy_and_note, dim3(n_tiles), dim3(64), 0, s, src, dst, n_tiles, x, notes);
  CHECK(hipStreamSynchronize(s));
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  CHECK(hipEventRecord(e0, s));
  hipLaunchKernelGGL(copy_and_note, dim3(n_tiles), dim3(64), 0, s, src, dst, n_tiles, x, notes);
  CHECK(hipEventRecord(e1, s));
  CHECK(hipStreamSynchronize(s));
  float ms = 0;
  CHECK(hipEventElapsedTime(&ms, e0, e1));
  std::vector<Note> h(n_notes);
  CHECK(hipMemcpy(h.data(), notes, n_notes * sizeof(Note), hipMemcpyDeviceToHost));
  // the copy itself
  std::vector<uint32_t> probe(256);
  CHECK(hipMemcpy(probe.data(), reinterpret_cast<uint8_t*>(dst) + bytes - 1024, 1024, hipMemcpyDeviceToHost));
  for (uint32_t w : probe)
    if (w != 0x5a5a5a5au) {
      fprintf(stderr, "the copy did not copy\n");
      return 1;
    }

  uint64_t tmin = ~0ull, tmax = 0;
  uint32_t logged = 0;
  for (const Note& n : h)
    if (n.written) {
      tmin = std::min(tmin, n.t0);
      tmax = std::max(tmax, n.t1);
      ++logged;
    }
  int xcc_of[8];
  for (int& v : xcc_of) v = -1;
  uint32_t agree = 0;
  for (const Note& n : h)
    if (n.written) {
      if (xcc_of[n.wg & 7] < 0) xcc_of[n.wg & 7] = static_cast<int>(n.xcc);
      if (xcc_of[n.wg & 7] == static_cast<int>(n.xcc)) ++agree;
    }
  printf("copy of %llu GiB in one launch, %s: %.1f us per GiB (HIP events), %.1f us from the first noted start to the last noted end\n",
         static_cast<unsigned long long>(gib), run > 1 ? "permuted in XCD runs" : "launch order", ms * 1e3 / gib,
         (tmax - tmin) / 100.0);
  printf("XCD of the workgroups with b %% 8 = 0..7:");
  for (int v : xcc_of) printf(" %d", v);
  printf("   (%u of %u noting workgroups agree)\n", agree, logged);

  std::vector<std::vector<uint64_t>> starts(16);
  uint64_t finished[16] = {0};
  for (const Note& n : h)
    if (n.written) {
      starts[n.xcc].push_back(n.t0 - tmin);
      finished[n.xcc] = std::max(finished[n.xcc], n.t1 - tmin);
    }
  for (auto& v : starts) std::sort(v.begin(), v.end());
  constexpr int kSlices = 16;
  double spread_k[kSlices];
  printf("   time | own workgroups started, in thousands, XCD 0..7 | most - fewest\n");
  for (int sl = 1; sl <= kSlices; ++sl) {
    const uint64_t t = (tmax - tmin) * sl / kSlices;
    printf("%5.0f us |", t / 100.0);
    uint64_t lo = ~0ull, hi = 0;
    for (int xcc = 0; xcc < 8; ++xcc) {
      const uint64_t c = std::upper_bound(starts[xcc].begin(), starts[xcc].end(), t) - starts[xcc].begin();
      const uint64_t wgs = c * (kNoteEvery / 8);
      printf(" %7.1f", wgs / 1e3);
      lo = std::min(lo, wgs);
      hi = std::max(hi, wgs);
    }
    spread_k[sl - 1] = (hi - lo) / 1e3;
    printf(" | %5.1f\n", spread_k[sl - 1]);
  }
  uint64_t first_done = ~0ull, last_done = 0;
  printf("last noted end per XCD, us:");
  for (int xcc = 0; xcc < 8; ++xcc) {
    printf(" %.1f", finished[xcc] / 100.0);
    first_done = std::min(first_done, finished[xcc]);
    last_done = std::max(last_done, finished[xcc]);
  }
  printf("\nthe first XCD to finish waits %.1f us for the last (%.2f %% of the launch)\n", (last_done - first_done) / 100.0,
         100.0 * (last_done - first_done) / (tmax - tmin));

  printf("{\"gib\": %llu, \"xcd_run\": %u, \"us_per_gib\": %.2f, \"noting_workgroups\": %u, \"agree\": %u, \"xcc_of_residue\": [",
         static_cast<unsigned long long>(gib), run, ms * 1e3 / gib, logged, agree);
  for (int i = 0; i < 8; ++i) printf("%d%s", xcc_of[i], i < 7 ? ", " : "");
  printf("], \"spread_thousand_workgroups\": [");
  for (int i = 0; i < kSlices; ++i) printf("%.1f%s", spread_k[i], i < kSlices - 1 ? ", " : "");
  printf("], \"finish_spread_us\": %.1f, \"launch_us\": %.1f}\n", (last_done - first_done) / 100.0, (tmax - tmin) / 100.0);
  hipFree(src);
  hipFree(dst);
  hipFree(notes);
  return 0;
}
