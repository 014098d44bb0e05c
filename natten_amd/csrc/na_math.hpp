// Integer window / tile arithmetic of neighborhood attention, shared by host and device code.
//
// Semantics follow SHI-Labs/NATTEN:
//   window start / end ........ csrc/include/natten/cuda/fna_blackwell/collective/fna_fusion.hpp:88-123
//   dilation-group extent ..... csrc/include/natten/cuda/fna_blackwell/collective/fna_fusion.hpp:250-256
//   KV tile box of a Q tile ... csrc/include/natten/cuda/fna_blackwell/collective/fna_fusion.hpp:315-347
// All quantities are non-negative ints, division truncates.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace natten_amd {

#define NA_HD __host__ __device__ __forceinline__

NA_HD int na_min(int a, int b) { return a < b ? a : b; }
NA_HD int na_max(int a, int b) { return a > b ? a : b; }
NA_HD int na_ceil_div(int a, int b) { return (a + b - 1) / b; }

// First key coordinate attended by query coordinate i (both inside one dilation group of
// extent L); queries of one stride group share the window of the group's leader.
NA_HD int na_window_start(int i, int k, int s, int L, bool causal) {
  const int wl = k / 2;
  const int wr = k / 2 + (k % 2 - 1);
  if (causal) {
    const int leader = na_min((i / s) * s + s - 1, L - 1);
    return na_max(leader - wl - wr, 0);
  }
  const int leader = na_min((i / s) * s + s / 2, L - 1);
  return na_max(leader - wl, 0) + ((leader + wr >= L) ? (L - wr - leader - 1) : 0);
}

NA_HD int na_window_end(int i, int start, int k, int L, bool causal) {
  return causal ? na_min(i + 1, L) : start + k;
}

// Number of tokens of dilation group g along a dimension of extent X.
NA_HD int na_group_extent(int X, int d, int g) { return X / d + 1 - ((g + (d - X % d)) / d); }

}  // namespace natten_amd
