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

// Division by a launch constant without a divide: floor(n / d) = (mul * n) >> shift (64-bit product)
// for every 0 <= n < 2^31 and 1 <= d < 2^31, with shift = 31 + ceil(log2 d) and
// mul = floor(2^shift / d) + 1 < 2^32 + 1 (the error mul * d - 2^shift lies in (0, d], which is at most
// 2^(shift - 31): small enough not to carry into the quotient for dividends below 2^31).
// The kernels' per-workgroup set-up divides by strides, dilations and tile counts dozens of
// times; a hardware integer division costs about thirty instructions, this three.
struct NaDiv {
  uint32_t mul;
  uint32_t shift;
};

inline NaDiv na_make_div(int d) {
  int lg = 0;
  while ((int64_t(1) << lg) < d) ++lg;
  NaDiv f;
  f.shift = uint32_t(31 + lg);
  f.mul = uint32_t(((uint64_t(1) << f.shift) / uint64_t(d)) + 1);  // d == 2^lg gives 2^31 + 1, the largest value
  return f;
}

NA_HD int na_div(int n, NaDiv f) { return int((uint64_t(f.mul) * uint64_t(uint32_t(n))) >> f.shift); }

// na_window_start with the stride's division precomputed (s_div = na_make_div(s))
NA_HD int na_window_start(int i, int k, int s, NaDiv s_div, int L, bool causal) {
  const int wl = int(uint32_t(k) >> 1);
  const int wr = wl + int(uint32_t(k) & 1u) - 1;
  const int group_first = na_div(i, s_div) * s;
  if (causal) {
    const int leader = na_min(group_first + s - 1, L - 1);
    return na_max(leader - wl - wr, 0);
  }
  const int leader = na_min(group_first + int(uint32_t(s) >> 1), L - 1);
  return na_max(leader - wl, 0) + ((leader + wr >= L) ? (L - wr - leader - 1) : 0);
}

// Keys of a 64-key KV tile are numbered with dimension 0 fastest and all tile extents are powers of
// two, so a key's coordinate along one dimension is a bit field of its number: (i >> lg_stride) &
// (2^lg_extent - 1).  Bit i of the result is set when that coordinate of key i is >= x
// (0 <= x <= 2^lg_extent).  The keys with coordinate in [lo, hi) are then
// na_keys_at_or_after(lo) & ~na_keys_at_or_after(hi), and a multi-dimensional window inside the
// tile is the AND of its per-dimension masks: what the kernels' element mask tests.
NA_HD uint64_t na_ones64(int n) { return n >= 64 ? ~uint64_t(0) : ((uint64_t(1) << n) - 1); }
NA_HD uint64_t na_keys_at_or_after(int x, int lg_stride, int lg_extent) {
  const int lg_period = lg_stride + lg_extent;  // the pattern repeats every 2^lg_period keys
  uint64_t m = na_ones64(1 << lg_period) & ~na_ones64(x << lg_stride);
  for (int s = lg_period; s < 6; ++s) m |= m << (1 << s);
  return m;
}

// A lane of the forward kernels holds 32 of a tile's 64 logits: logit r (0..15) of sub-block sb
// (0..1) belongs to key 32 sb + 8 (r / 4) + 4 g + r % 4, where g is the lane's half of the wave.
// The bits of a key set that a lane of half g needs, bit 16 sb + r for its logit (sb, r): of every
// byte of the set the nibble at 4 g, the eight nibbles packed into one word.
NA_HD uint32_t na_lane_half_bits(uint64_t keys, int g) {
  uint32_t out = 0;
  for (int sb = 0; sb < 2; ++sb) {
    uint32_t w = uint32_t(keys >> (32 * sb + 4 * g)) & 0x0f0f0f0fu;  // nibbles of keys 8 m + 4 g .. + 3 at bits 8 m
    w = (w | (w >> 4)) & 0x00ff00ffu;
    w = (w | (w >> 8)) & 0x0000ffffu;
    out |= w << (16 * sb);
  }
  return out;
}
// ... and back: the key set whose bits for both halves are `half0` and `half1` (host-side checks).
NA_HD uint64_t na_keys_of_lane_halves(uint32_t half0, uint32_t half1) {
  uint64_t keys = 0;
  for (int g = 0; g < 2; ++g)
    for (int b = 0; b < 32; ++b) {
      const int sb = b >> 4, r = b & 15;
      if (((g ? half1 : half0) >> b) & 1u) keys |= uint64_t(1) << (32 * sb + 8 * (r / 4) + 4 * g + r % 4);
    }
  return keys;
}

// Number of tokens of dilation group g along a dimension of extent X.
NA_HD int na_group_extent(int X, int d, int g) { return X / d + 1 - ((g + (d - X % d)) / d); }

// The queries that attend key coordinates j0 .. j1 of a dimension form an interval, because
// window start and end are non-decreasing in the query coordinate: its first element is the
// first query whose window ends past j0, its last the last query whose window starts at or
// before j1 (queries 0 .. Lq-1, keys of extent L).  Both by bisection.  An empty interval comes
// back as first > last.
NA_HD int na_first_query_attending(int j0, int k, int s, int L, int Lq, bool causal) {
  int lo = 0, hi = Lq;  // answer in [lo, hi]; hi == Lq: none
  while (lo < hi) {
    const int mid = (lo + hi) / 2;
    const int st = na_window_start(mid, k, s, L, causal);
    if (na_window_end(mid, st, k, L, causal) > j0) hi = mid;
    else lo = mid + 1;
  }
  return lo;
}

NA_HD int na_last_query_attending(int j1, int k, int s, int L, int Lq, bool causal) {
  int lo = -1, hi = Lq - 1;  // answer in [lo, hi]; lo == -1: none
  while (lo < hi) {
    const int mid = (lo + hi + 1) / 2;
    if (na_window_start(mid, k, s, L, causal) <= j1) lo = mid;
    else hi = mid - 1;
  }
  return lo;
}

}  // namespace natten_amd
