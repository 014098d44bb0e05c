// Two-way attention merge as one elementwise kernel (float32 arithmetic):
//   out = o0 - sigmoid(lse1 - lse0) * (o0 - o1),   lse = lse0 - logsigmoid(lse0 - lse1)
// Formula: SHI-Labs/NATTEN src/natten/attn_merge.py:83-95.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace natten_amd {

template <typename T>
__device__ __forceinline__ float merge_load(const T* p) { return static_cast<float>(*p); }

// One wave-row mapping: each thread handles one (row, 8-element slice) pair; the row's scalars
// are recomputed per thread (cheap) so no cross-lane traffic is needed.
template <typename T>
__global__ void __launch_bounds__(256) merge_kernel(const T* __restrict__ o0, const float* __restrict__ l0,
                                                    const T* __restrict__ o1, const float* __restrict__ l1,
                                                    T* out, float* lse_out, int64_t rows, int head_dim) {
  const int64_t total = rows * head_dim;
  for (int64_t idx = int64_t(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += int64_t(gridDim.x) * 256) {
    const int64_t row = idx / head_dim;
    const int col = int(idx - row * head_dim);
    const float a = l0[row], b = l1[row];
    // sigmoid(b - a) and logsigmoid(a - b) = -log(1 + exp(b - a)), written to stay finite
    const float d = b - a;
    float sig, lse;
    if (d <= 0.f) {
      const float e = __expf(d);
      sig = e / (1.f + e);
      lse = a + log1pf(e);
    } else {
      const float e = __expf(-d);
      sig = 1.f / (1.f + e);
      lse = b + log1pf(e);
    }
    if (a == -INFINITY && b == -INFINITY) {
      sig = 0.f;
      lse = -INFINITY;
    }
    const float x0 = static_cast<float>(o0[idx]), x1 = static_cast<float>(o1[idx]);
    out[idx] = static_cast<T>(x0 - sig * (x0 - x1));
    if (col == 0) lse_out[row] = lse;
  }
}

}  // namespace natten_amd
