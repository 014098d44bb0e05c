// Host build of the work-queue decisions the kernels run (natten_amd/csrc/work_queue.hpp), for
// tests/test_queue_protocol.py: compiled with g++ at test time, no device code.
#include "../natten_amd/csrc/work_queue.hpp"

extern "C" {

int wq_num_xcd(void) { return natten_amd::kNumXcd; }
int wq_stride(void) { return natten_amd::kQueueStride; }
int wq_words(void) { return natten_amd::kQueueWords; }
int wq_done_word(void) { return natten_amd::kQueueDoneWord; }

int wq_counter_word(int home, int victim, int nq) { return natten_amd::queue_counter_word(home, victim, nq); }

// returns the position (or -1) and writes the advanced victim count back
int wq_position(int home, int* victim, uint32_t ticket, int per_queue, int nq) {
  return natten_amd::queue_position(home, *victim, ticket, per_queue, nq);
}

int wq_last_one_out(uint32_t left, uint32_t workgroups) { return natten_amd::queue_last_one_out(left, workgroups) ? 1 : 0; }

long long wq_max_increments(int per_queue, int nq) { return natten_amd::queue_max_increments(per_queue, nq); }
}
