// Work-queue protocol of the resident-workgroup launches (fna_fwd_queue_kernel and its 8-bit form).
//
// A launch has `nq * per_queue` positions (the workgroup ids a one-workgroup-per-Q-tile launch
// would use); position `ticket * nq + x` belongs to queue x, whose counter lives at word
// `x * kQueueStride` of a small block of device memory that is all zero when the launch starts.
// A resident workgroup increments the counter of its home queue, takes the old value as its
// ticket, and works on that position; a ticket at or beyond `per_queue` means the queue is empty
// for good (counters only grow during a launch), and the workgroup moves on to the next queue,
// never to return.  A workgroup that has found every queue empty increments the done word; the
// one that reads `workgroups - 1` there is the last to leave and stores zeros back.
//
// This file holds the decisions of that protocol as plain functions, free of device code, so that
// the kernels and the host-side model that walks through every interleaving of a small launch
// (tests/test_queue_protocol.py) run the same code.  It has no counterpart in SHI-Labs/NATTEN,
// whose persistent tile scheduler is static (csrc/include/natten/cuda/fmha_blackwell/kernel/
// fmha_tile_scheduler.hpp:146-149 strides blockIdx over the tiles).
#pragma once

#include <stdint.h>

#if defined(__HIPCC__) || defined(__CUDACC__)
#define NA_QUEUE_FN __host__ __device__ inline
#else
#define NA_QUEUE_FN inline
#endif

namespace natten_amd {

constexpr int kNumXcd = 8;
constexpr int kQueueStride = 16;  // uint32 counters per 64-byte line
constexpr int kQueueWords = kNumXcd * kQueueStride;
constexpr int kQueueDoneWord = 1;  // workgroups that have left the loop (in the first queue's line)

// Word of the counter a workgroup tries after it has found `victim` queues empty: its home queue
// first, then the others in turn.
NA_QUEUE_FN int queue_counter_word(int home, int victim, int nq = kNumXcd) { return ((home + victim) % nq) * kQueueStride; }

// What the old value `ticket` of that counter means.  Returns the launch position to work on, or
// -1 when the queue was empty; `victim` then counts one more empty queue, and the caller tries
// the next one unless `victim == nq` (nothing is left anywhere).
NA_QUEUE_FN int queue_position(int home, int& victim, uint32_t ticket, int per_queue, int nq = kNumXcd) {
  if (ticket < uint32_t(per_queue)) return int(ticket) * nq + (home + victim) % nq;
  ++victim;
  return -1;
}

// Whether the workgroup that read `left` from the done word is the last one out.
NA_QUEUE_FN bool queue_last_one_out(uint32_t left, uint32_t workgroups) { return left == workgroups - 1; }

// Upper bound on the counter increments one workgroup makes in a launch, whatever the others do:
// every increment either yields one of the nq * per_queue positions or retires one of nq queues.
NA_QUEUE_FN long long queue_max_increments(int per_queue, int nq = kNumXcd) { return (long long)nq * per_queue + nq; }

}  // namespace natten_amd
