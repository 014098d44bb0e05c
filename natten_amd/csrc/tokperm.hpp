// Token permute / unpermute for gfx950: a coalesced row gather / scatter.
//
// Index map restated from SHI-Labs/NATTEN
//   src/natten/token_permute/torch_impl.py:99-187 (view [B, (R, t, d) per dim, H, Dh], permute to
//       [B, d..., R..., t..., H, Dh], dimension order reversed inside each kind when flipping)
//   csrc/include/natten/cuda/tokperm/token_permute_kernel.cuh:40-163 (coordinate maps),
//   :338-340 (padding is written as zero)
// One kernel serves both directions: it walks the permuted index space, decodes the original
// coordinate, and copies one token row (heads * head_dim elements, contiguous on both sides).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace natten_amd {

struct TokPermParams {
  const char* src;
  char* dst;
  int na_dim;
  int batch;            // original batch
  int num_groups;       // prod(dilation)
  int64_t perm_len;     // tokens per (batch, group) in the permuted layout
  int64_t orig_len;     // tokens per batch in the original layout
  int64_t row_bytes;    // heads * head_dim * elem_bytes
  // decode order, fastest first: the `na_dim` tile offsets, then the `na_dim` tile indices
  int t_size[3], r_size[3], t_dim[3];  // t_dim[i]: which original dimension slot i refers to
  int g_size[3];                       // dilation, fastest first, same slot -> dim mapping
  int layout[3], tile[3], dil[3];      // by original dimension
};

// Decodes permuted token `tok` (index over [batch * groups, perm_len]): returns whether it maps to
// a real token and, if so, that token's index over [batch, orig_len].
__device__ __forceinline__ bool tokperm_decode(const TokPermParams& p, int64_t tok, int64_t& orig_tok) {
  const int64_t bgi = tok / p.perm_len;
  int64_t pos = tok - bgi * p.perm_len;
  const int b = int(bgi / p.num_groups);
  int gl = int(bgi - int64_t(b) * p.num_groups);
  int tau[3] = {0, 0, 0}, rr[3] = {0, 0, 0}, dl[3] = {0, 0, 0};
#pragma unroll
  for (int i = 0; i < 3; ++i)
    if (i < p.na_dim) {
      tau[p.t_dim[i]] = int(pos % p.t_size[i]);
      pos /= p.t_size[i];
    }
#pragma unroll
  for (int i = 0; i < 3; ++i)
    if (i < p.na_dim) {
      rr[p.t_dim[i]] = int(pos % p.r_size[i]);
      pos /= p.r_size[i];
      dl[p.t_dim[i]] = gl % p.g_size[i];
      gl /= p.g_size[i];
    }
  bool inside = true;
  int64_t lin = 0;
#pragma unroll
  for (int a = 0; a < 3; ++a)
    if (a < p.na_dim) {
      const int x = rr[a] * (p.tile[a] * p.dil[a]) + tau[a] * p.dil[a] + dl[a];
      inside = inside && (x < p.layout[a]);
      lin = lin * p.layout[a] + x;
    }
  orig_tok = int64_t(b) * p.orig_len + lin;
  return inside;
}

// VEC = bytes moved per thread per step (16, 4, 2 or 1)
template <int VEC, bool UNPERMUTE>
__global__ void __launch_bounds__(256) tokperm_kernel(const TokPermParams p) {
  const int64_t chunks_per_row = p.row_bytes / VEC;
  const int64_t total = int64_t(p.batch) * p.num_groups * p.perm_len * chunks_per_row;
  for (int64_t idx = int64_t(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += int64_t(gridDim.x) * 256) {
    const int64_t tok = idx / chunks_per_row;
    const int64_t chunk = idx - tok * chunks_per_row;
    int64_t orig_tok;
    const bool inside = tokperm_decode(p, tok, orig_tok);
    const int64_t perm_off = tok * p.row_bytes + chunk * VEC;
    const int64_t orig_off = orig_tok * p.row_bytes + chunk * VEC;
    if constexpr (VEC == 16) {
      typedef uint32_t u4 __attribute__((ext_vector_type(4)));
      if constexpr (UNPERMUTE) {
        if (inside) *reinterpret_cast<u4*>(p.dst + orig_off) = *reinterpret_cast<const u4*>(p.src + perm_off);
      } else {
        u4 val = {0, 0, 0, 0};
        if (inside) val = *reinterpret_cast<const u4*>(p.src + orig_off);
        *reinterpret_cast<u4*>(p.dst + perm_off) = val;
      }
    } else {
      using E = typename std::conditional<VEC == 4, uint32_t, typename std::conditional<VEC == 2, uint16_t, uint8_t>::type>::type;
      if constexpr (UNPERMUTE) {
        if (inside) *reinterpret_cast<E*>(p.dst + orig_off) = *reinterpret_cast<const E*>(p.src + perm_off);
      } else {
        E val = 0;
        if (inside) val = *reinterpret_cast<const E*>(p.src + orig_off);
        *reinterpret_cast<E*>(p.dst + perm_off) = val;
      }
    }
  }
}

// The same copy for rows of at least 256 bytes in 16-byte chunks: a wave takes one token row at
// a time, so the row's index arithmetic (a dozen 64-bit divisions) runs once per row on the
// scalar unit instead of once per 16 bytes on every lane, and its lanes move up to four chunks
// each per step (loads first, then stores).  Permuted rows are written / read exactly once and
// never needed again soon: their stores bypass the cache hierarchy's reuse tracking (non-temporal).
template <bool UNPERMUTE>
__global__ void __launch_bounds__(256) tokperm_rows_kernel(const TokPermParams p) {
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  const int chunks = int(p.row_bytes / 16);
  const int64_t rows = int64_t(p.batch) * p.num_groups * p.perm_len;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(int(threadIdx.x >> 6));
  const int64_t n_waves = int64_t(gridDim.x) * 4;
  for (int64_t tok = int64_t(blockIdx.x) * 4 + wave; tok < rows; tok += n_waves) {
    int64_t orig_tok;
    const bool inside = tokperm_decode(p, tok, orig_tok);  // wave-uniform
    if (UNPERMUTE && !inside) continue;
    const u4* src = reinterpret_cast<const u4*>(p.src + (UNPERMUTE ? tok : orig_tok) * p.row_bytes);
    u4* dst = reinterpret_cast<u4*>(p.dst + (UNPERMUTE ? orig_tok : tok) * p.row_bytes);
    for (int c0 = 0; c0 < chunks; c0 += 256) {
      u4 val[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = c0 + u * 64 + lane;
        val[u] = u4{0, 0, 0, 0};
        if (c < chunks && (UNPERMUTE || inside)) val[u] = __builtin_nontemporal_load(src + c);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = c0 + u * 64 + lane;
        if (c < chunks) __builtin_nontemporal_store(val[u], dst + c);
      }
    }
  }
}

// Token permute that also widens 8-bit floating point to bf16 (exact: every e4m3 / e5m2 value is
// a bf16 value).  row_bytes counts SOURCE bytes (one per element, a multiple of 8); the
// destination row holds twice as many.  Each thread converts 8 elements: 8 bytes in, 16 out.
// E5M2 = false: OCP e4m3fn, true: OCP e5m2.
template <bool E5M2>
__global__ void __launch_bounds__(256) tokperm_widen_kernel(const TokPermParams p) {
  typedef uint32_t u2 __attribute__((ext_vector_type(2)));
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  const int64_t chunks_per_row = p.row_bytes / 8;
  const int64_t total = int64_t(p.batch) * p.num_groups * p.perm_len * chunks_per_row;
  for (int64_t idx = int64_t(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += int64_t(gridDim.x) * 256) {
    const int64_t tok = idx / chunks_per_row;
    const int64_t chunk = idx - tok * chunks_per_row;
    int64_t orig_tok;
    const bool inside = tokperm_decode(p, tok, orig_tok);
    u4 val = {0, 0, 0, 0};
    if (inside) {
      const u2 raw = *reinterpret_cast<const u2*>(p.src + orig_tok * p.row_bytes + chunk * 8);
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        f2 lo, hi;
        if constexpr (E5M2) {
          lo = __builtin_amdgcn_cvt_pk_f32_bf8(raw[w], false);
          hi = __builtin_amdgcn_cvt_pk_f32_bf8(raw[w], true);
        } else {
          lo = __builtin_amdgcn_cvt_pk_f32_fp8(raw[w], false);
          hi = __builtin_amdgcn_cvt_pk_f32_fp8(raw[w], true);
        }
        // the values are exactly representable: the low 16 bits of each float are zero
        val[2 * w] = (__float_as_uint(lo[0]) >> 16) | (__float_as_uint(lo[1]) & 0xffff0000u);
        val[2 * w + 1] = (__float_as_uint(hi[0]) >> 16) | (__float_as_uint(hi[1]) & 0xffff0000u);
      }
    }
    *reinterpret_cast<u4*>(p.dst + (tok * p.row_bytes + chunk * 8) * 2) = val;
  }
}

}  // namespace natten_amd
