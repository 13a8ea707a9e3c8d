// Waiting for an HSA signal without waiting forever.  ROCr's BlitKernel waits
// for its completion signal with an unbounded hsa_signal_wait_scacquire and
// answers HSA_STATUS_ERROR when the wait returns a value other than 0
// (projects/rocr-runtime/runtime/hsa-runtime/core/runtime/amd_blit_kernel.cpp:
// 632-636, 830-834); a queue that has stopped on an asynchronous error never
// decrements the signal, and what ends the wait there is the runtime's queue
// error handler (core/runtime/queue.cpp:52-59, which aborts the process).
// Here the wait is cut into bounded slices, and between slices it looks at the
// flag the queue's error callback sets: the caller gets HSA_STATUS_ERROR
// instead of a hang.  Pure C++, no HSA types: the slice itself is a callable,
// so that the loop can be tested without a GPU.
#ifndef MI355_AQL_WAIT_H_
#define MI355_AQL_WAIT_H_

#include <stdint.h>

#include <atomic>

namespace mi355 {

constexpr int kWaitSuccess = 0x0;   // HSA_STATUS_SUCCESS
constexpr int kWaitError = 0x1000;  // HSA_STATUS_ERROR

// wait_slice(ticks) waits at most `ticks` for the signal to drop below 1 and
// returns the value it saw last (hsa_signal_wait_scacquire with condition LT 1).
// Returns success when the signal reached 0; an error when it went negative
// (how a failed command is reported, inc/hsa_ext_amd.h:1735-1739) or when
// `queue_error` was found set after a slice that did not see it below 1.
template <class WaitSlice>
inline int wait_below_one(WaitSlice wait_slice, const std::atomic<bool>& queue_error, uint64_t slice_ticks) {
  for (;;) {
    const int64_t v = wait_slice(slice_ticks);
    if (v < 1) return v == 0 ? kWaitSuccess : kWaitError;
    if (queue_error.load(std::memory_order_acquire)) return kWaitError;
  }
}

}  // namespace mi355

#endif  // MI355_AQL_WAIT_H_
