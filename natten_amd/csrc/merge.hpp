// Two-way attention merge as one elementwise kernel (float32 arithmetic):
//   out = o0 - sigmoid(lse1 - lse0) * (o0 - o1),   lse = lse0 - logsigmoid(lse0 - lse1)
// Formula: SHI-Labs/NATTEN src/natten/attn_merge.py:83-95.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace natten_amd {

// sigmoid(l1 - l0) and the merged LSE of one row, written to stay finite for any pair
__device__ __forceinline__ void merge_row_scalars(float a, float b, float& sig, float& lse) {
  const float d = b - a;
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
}

// VEC elements per thread (16 bytes of a 16-bit payload, 16 or 32 of a float one): a thread owns
// one (row, VEC-element slice) pair, reads the row's two LSEs once and moves its slice with one
// access per operand; the thread of a row's first slice writes the merged LSE.  VEC == 1 is the
// form for head dims or pointers that do not allow the wide accesses.
template <typename T, int VEC>
__global__ void __launch_bounds__(256) merge_kernel(const T* __restrict__ o0, const float* __restrict__ l0,
                                                    const T* __restrict__ o1, const float* __restrict__ l1,
                                                    T* out, float* lse_out, int64_t rows, int head_dim) {
  typedef T tvec __attribute__((ext_vector_type(VEC)));
  const int slices = head_dim / VEC;
  const int64_t total = rows * slices;
  for (int64_t idx = int64_t(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += int64_t(gridDim.x) * 256) {
    const int64_t row = idx / slices;
    const int slice = int(idx - row * slices);
    float sig, lse;
    merge_row_scalars(l0[row], l1[row], sig, lse);
    const int64_t at = row * head_dim + int64_t(slice) * VEC;
    if constexpr (VEC == 1) {
      const float x0 = static_cast<float>(o0[at]), x1 = static_cast<float>(o1[at]);
      out[at] = static_cast<T>(x0 - sig * (x0 - x1));
    } else {
      const tvec a = *reinterpret_cast<const tvec*>(o0 + at);
      const tvec b = *reinterpret_cast<const tvec*>(o1 + at);
      tvec r;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float x0 = static_cast<float>(a[i]), x1 = static_cast<float>(b[i]);
        r[i] = static_cast<T>(x0 - sig * (x0 - x1));
      }
      *reinterpret_cast<tvec*>(out + at) = r;
    }
    if (slice == 0) lse_out[row] = lse;
  }
}

// N-way merge of partial attentions that lie one after the other (`parts[i]` = part 0 + i *
// part_stride elements, `lses[i]` = lse 0 + i * rows): out = sum_i w_i o_i with
// w_i = exp(lse_i - lse), lse = log sum_i exp(lse_i), in float32, rounded once.  The same value as
// the two-way merge applied n - 1 times, without the roundings of its intermediate results.
// A row whose parts all hold no key (every lse -inf) gives zeros and -inf.
template <typename T, int VEC>
__global__ void __launch_bounds__(256) merge_parts_kernel(const T* __restrict__ parts, const float* __restrict__ lses,
                                                          int num_parts, int64_t part_stride, T* out, float* lse_out,
                                                          int64_t rows, int head_dim) {
  typedef T tvec __attribute__((ext_vector_type(VEC)));
  const int slices = head_dim / VEC;
  const int64_t total = rows * slices;
  for (int64_t idx = int64_t(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += int64_t(gridDim.x) * 256) {
    const int64_t row = idx / slices;
    const int slice = int(idx - row * slices);
    float mx = -INFINITY;
    for (int i = 0; i < num_parts; ++i) mx = fmaxf(mx, lses[i * rows + row]);
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
    float sum = 0.f;
    const int64_t at = row * head_dim + int64_t(slice) * VEC;
    if (mx != -INFINITY) {
      for (int i = 0; i < num_parts; ++i) {
        const float w = __expf(lses[i * rows + row] - mx);  // 0 for a part without keys
        sum += w;
        if constexpr (VEC == 1) {
          acc[0] += w * static_cast<float>(parts[i * part_stride + at]);
        } else {
          const tvec a = *reinterpret_cast<const tvec*>(parts + i * part_stride + at);
#pragma unroll
          for (int e = 0; e < VEC; ++e) acc[e] += w * static_cast<float>(a[e]);
        }
      }
    }
    const float inv = sum > 0.f ? 1.f / sum : 0.f;
    if constexpr (VEC == 1) {
      out[at] = static_cast<T>(acc[0] * inv);
    } else {
      tvec r;
#pragma unroll
      for (int e = 0; e < VEC; ++e) r[e] = static_cast<T>(acc[e] * inv);
      *reinterpret_cast<tvec*>(out + at) = r;
    }
    if (slice == 0) lse_out[row] = sum > 0.f ? mx + __logf(sum) : -INFINITY;
  }
}

}  // namespace natten_amd
