// Fused neighborhood attention forward for gfx950 (MI355X): one workgroup per Q tile of one
// (batch*dilation-group, head); K/V tiles staged in LDS; S^T = K Q^T and O^T = V^T P^T on
// 32x32x16 MFMA so that every lane owns exactly one query row (row max / row sum are per-lane
// scalars plus one exchange between the two half-waves).
//
// The structure it restates (not the code): SHI-Labs/NATTEN
//   csrc/include/natten/cuda/fna_blackwell/collective/fna_fusion.hpp:315-347 (KV tile box per Q tile)
//   csrc/include/natten/cuda/fna_blackwell/collective/fna_fusion.hpp:384-436 (element mask)
//   csrc/include/natten/cuda/fna_blackwell/collective/sm100_fna_fwd_mainloop_tma_warpspecialized.hpp:618-861,
//   :1314-1327 (online softmax in the exp2 domain, O / rowsum, LSE = ln(rowsum) + scale * rowmax)
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "na_math.hpp"

namespace natten_amd {

struct FnaParams {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  float* lse;
  int batch, heads_q, heads_kv;
  int seqlen_q, seqlen_kv;  // rows of the (permuted) sequences
  int num_groups;           // prod(dilation)
  int qkv_shape[3];         // original token layout
  int ksize[3], stride[3], dil[3], causal[3];
  int q_tile[3], kv_tile[3];
  int q_tiled[3], kv_tiled[3];  // tiles per dimension of the padded per-group layouts
  float scale;                  // softmax scale (dequantisation scales of q and k folded in)
  float out_scale;              // dequantisation scale of v
};

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

#define NA_LDS __attribute__((address_space(3)))

template <typename T>
struct Mma;

template <>
struct Mma<__bf16> {
  using vec8 = bf16x8_t;
  static __device__ __forceinline__ f32x16_t run(vec8 a, vec8 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

template <>
struct Mma<_Float16> {
  using vec8 = f16x8_t;
  static __device__ __forceinline__ f32x16_t run(vec8 a, vec8 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// LDS transpose read: the 16 lanes of a group each point at 4 consecutive 16-bit elements of
// a row (lane 4e+j -> row e, columns 4j..4j+3 of a 4x16 block); lane c of the group receives
// column c of the block (rows 0..3).
static __device__ __forceinline__ s16x4_t lds_read_tr16(const char* p) {
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wold-style-cast"
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((NA_LDS s16x4_t*)(p));
#pragma clang diagnostic pop
}

static __device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

constexpr uint32_t kGuardBits = (1u << 9) | (1u << 19) | (1u << 29);

template <int D, int KVT>
struct FnaSmem {
  static constexpr int KROW = D * 2 + 16;  // bytes per K row (padding breaks bank conflicts of b128 reads)
  static constexpr int VROW = D * 2 + 32;  // bytes per V row (padding for the transpose reads)
  static constexpr int BYTES = KVT * (KROW + VROW) + KVT * 4;
};

template <typename T, int D, int NWAVES, int MQ, int KVT>
__global__ void __launch_bounds__(NWAVES * 64) fna_fwd_kernel(const FnaParams p) {
  constexpr int NT = NWAVES * 64;
  constexpr int QT = NWAVES * MQ * 32;
  constexpr int KSTEPS = D / 16;
  constexpr int DB = D / 32;
  constexpr int NSB = KVT / 32;
  constexpr int KROW = FnaSmem<D, KVT>::KROW;
  constexpr int VROW = FnaSmem<D, KVT>::VROW;
  using M = Mma<T>;
  using vec8 = typename M::vec8;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* sK = smem;
  char* sV = smem + KVT * KROW;
  uint32_t* sTab = reinterpret_cast<uint32_t*>(smem + KVT * (KROW + VROW));

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int g = lane >> 5;
  const int qtile_idx = blockIdx.x;
  const int head = blockIdx.y;
  const int bg = blockIdx.z;
  const int head_kv = head / (p.heads_q / p.heads_kv);

  // ---- workgroup-uniform setup: dilation group, Q tile origin, KV tile box -------------------
  int extent[3], q_first[3], box_tile0[3], box_n[3], full_lo[3], full_hi[3];
  {
    int gl = bg % p.num_groups;
    int t = qtile_idx;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int gi = gl % p.dil[a];
      gl /= p.dil[a];
      extent[a] = na_group_extent(p.qkv_shape[a], p.dil[a], gi);
      const int tc = t % p.q_tiled[a];
      t /= p.q_tiled[a];
      q_first[a] = tc * p.q_tile[a];
      const int qf = q_first[a], ql = qf + p.q_tile[a] - 1;
      const bool c = p.causal[a] != 0;
      const int st_f = na_window_start(qf, p.ksize[a], p.stride[a], extent[a], c);
      const int en_f = na_window_end(qf, st_f, p.ksize[a], extent[a], c);
      const int st_l = na_window_start(ql, p.ksize[a], p.stride[a], extent[a], c);
      const int en_l = na_window_end(ql, st_l, p.ksize[a], extent[a], c);
      box_tile0[a] = st_f / p.kv_tile[a];
      box_n[a] = na_ceil_div(en_l, p.kv_tile[a]) - box_tile0[a];
      full_lo[a] = st_l;  // intersection of the tile's windows: [start(last), end(first))
      full_hi[a] = en_f;
    }
  }
  const int total_tiles = box_n[0] * box_n[1] * box_n[2];

  // in-tile coordinates of every KV position, packed in 10-bit fields
  for (int i = tid; i < KVT; i += NT) {
    int r = i;
    const int t0 = r % p.kv_tile[0];
    r /= p.kv_tile[0];
    const int t1 = r % p.kv_tile[1];
    r /= p.kv_tile[1];
    sTab[i] = uint32_t(t0) | (uint32_t(t1) << 10) | (uint32_t(r) << 20);
  }

  // ---- per-lane setup: this lane's query rows, their windows, Q fragments ---------------------
  int wst[MQ][3], wen[MQ][3];
  vec8 qf[MQ][KSTEPS];
  const int64_t q_row_stride = int64_t(p.heads_q) * D;
  const int64_t kv_row_stride = int64_t(p.heads_kv) * D;
  const T* qbase = reinterpret_cast<const T*>(p.q) + int64_t(bg) * p.seqlen_q * q_row_stride + int64_t(head) * D;
  const T* kbase = reinterpret_cast<const T*>(p.k) + int64_t(bg) * p.seqlen_kv * kv_row_stride + int64_t(head_kv) * D;
  const T* vbase = reinterpret_cast<const T*>(p.v) + int64_t(bg) * p.seqlen_kv * kv_row_stride + int64_t(head_kv) * D;
#pragma unroll
  for (int mb = 0; mb < MQ; ++mb) {
    int r = (wave * MQ + mb) * 32 + l32;
    const int row = qtile_idx * QT + r;
    int off[3];
    off[0] = r % p.q_tile[0];
    r /= p.q_tile[0];
    off[1] = r % p.q_tile[1];
    off[2] = r / p.q_tile[1];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int c = q_first[a] + off[a];
      wst[mb][a] = na_window_start(c, p.ksize[a], p.stride[a], extent[a], p.causal[a] != 0);
      wen[mb][a] = na_window_end(c, wst[mb][a], p.ksize[a], extent[a], p.causal[a] != 0);
    }
    const int row_c = na_min(row, p.seqlen_q - 1);
    const T* qrow = qbase + int64_t(row_c) * q_row_stride + g * 8;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) qf[mb][ks] = *reinterpret_cast<const vec8*>(qrow + ks * 16);
  }

  f32x16_t acc[MQ][DB];
  float m_run[MQ], l_run[MQ];
#pragma unroll
  for (int mb = 0; mb < MQ; ++mb) {
    m_run[mb] = -INFINITY;
    l_run[mb] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mb][db][r] = 0.f;
  }
  const float c_log2 = p.scale * 1.4426950408889634f;

  // ---- main loop over the KV tile box (dimension 0 fastest) ----------------------------------
  int itc[3] = {0, 0, 0};
  for (int it = 0; it < total_tiles; ++it) {
    int origin[3];
    bool full = true;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      origin[a] = (box_tile0[a] + itc[a]) * p.kv_tile[a];
      full = full && (origin[a] >= full_lo[a]) && (origin[a] + p.kv_tile[a] <= full_hi[a]);
    }
    const int kv_lin = (box_tile0[0] + itc[0]) +
                       p.kv_tiled[0] * ((box_tile0[1] + itc[1]) + p.kv_tiled[1] * (box_tile0[2] + itc[2]));
    const int kv_row0 = kv_lin * KVT;

    __syncthreads();  // everyone is done reading the previous tile (and sTab is written)
    {
      constexpr int CPR = D / 8;  // 16-byte chunks per row
      constexpr int PER = (KVT * CPR) / NT;
      static_assert((KVT * CPR) % NT == 0, "tile does not split evenly over the workgroup");
      u32x4_t kreg[PER], vreg[PER];
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int c = i * NT + tid;
        const int row = c / CPR, col = c % CPR;
        const int grow = kv_row0 + row;
        if (grow < p.seqlen_kv) {
          kreg[i] = *reinterpret_cast<const u32x4_t*>(kbase + int64_t(grow) * kv_row_stride + col * 8);
          vreg[i] = *reinterpret_cast<const u32x4_t*>(vbase + int64_t(grow) * kv_row_stride + col * 8);
        } else {
          kreg[i] = u32x4_t{0, 0, 0, 0};
          vreg[i] = u32x4_t{0, 0, 0, 0};
        }
      }
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int c = i * NT + tid;
        const int row = c / CPR, col = c % CPR;
        *reinterpret_cast<u32x4_t*>(sK + row * KROW + col * 16) = kreg[i];
        *reinterpret_cast<u32x4_t*>(sV + row * VROW + col * 16) = vreg[i];
      }
    }
    __syncthreads();

    // S^T = K Q^T : lane owns query row l32 (per q block) and 16 key rows per 32-key sub-block
    f32x16_t S[MQ][NSB];
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb) {
#pragma unroll
      for (int mb = 0; mb < MQ; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) S[mb][sb][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        const vec8 kf = *reinterpret_cast<const vec8*>(sK + (sb * 32 + l32) * KROW + (ks * 2 + g) * 16);
#pragma unroll
        for (int mb = 0; mb < MQ; ++mb) S[mb][sb] = M::run(kf, qf[mb][ks], S[mb][sb]);
      }
    }

    vec8 pf[MQ][NSB][2];
#pragma unroll
    for (int mb = 0; mb < MQ; ++mb) {
      if (!full) {
        // window of this lane's query relative to the tile origin, clamped to the tile
        uint32_t addc = 0, subc = 0;
#pragma unroll
        for (int a = 0; a < 3; ++a) {
          const int lo = na_min(na_max(wst[mb][a] - origin[a], 0), p.kv_tile[a]);
          const int hi = na_min(na_max(wen[mb][a] - origin[a], 0), p.kv_tile[a]);
          addc |= uint32_t(512 - lo) << (10 * a);
          subc |= uint32_t(511 + hi) << (10 * a);
        }
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const u32x4_t tc4 = *reinterpret_cast<const u32x4_t*>(&sTab[sb * 32 + 8 * j + 4 * g]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const uint32_t tp = tc4[i];
              const uint32_t ok = (tp + addc) & (subc - tp) & kGuardBits;
              S[mb][sb][4 * j + i] = (ok == kGuardBits) ? S[mb][sb][4 * j + i] : -INFINITY;
            }
          }
      }
      float mx = -INFINITY;
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, S[mb][sb][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float m_new = fmaxf(m_run[mb], mx);
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = fast_exp2((m_run[mb] - m_use) * c_log2);
      const float msc = m_use * c_log2;
      m_run[mb] = m_new;
      float psum = 0.f;
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          vec8 pv;
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const float pe = fast_exp2(S[mb][sb][8 * h + i] * c_log2 - msc);
            psum += pe;
            pv[i] = static_cast<T>(pe);
          }
          pf[mb][sb][h] = pv;
        }
      l_run[mb] = l_run[mb] * alpha + psum;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mb][db][r] *= alpha;
    }

    // O^T += V^T P^T : the k-slot order of the P fragment (rows 4g..4g+3 and 8+4g..8+4g+3 of
    // each 16-key half) is matched by two transpose reads of V.
    {
      const int l16 = lane & 15;
      const int e = l16 >> 2, j4 = l16 & 3;
      const int colb = ((l32 >> 4) * 16 + 4 * j4) * 2;
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const char* vrow = sV + (sb * 32 + h * 16 + 4 * g + e) * VROW + colb;
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            const s16x4_t lo = lds_read_tr16(vrow + db * 64);
            const s16x4_t hi = lds_read_tr16(vrow + db * 64 + 8 * VROW);
            const s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            const vec8 vf = __builtin_bit_cast(vec8, both);
#pragma unroll
            for (int mb = 0; mb < MQ; ++mb) acc[mb][db] = M::run(vf, pf[mb][sb][h], acc[mb][db]);
          }
        }
    }

    if (++itc[0] == box_n[0]) {
      itc[0] = 0;
      if (++itc[1] == box_n[1]) {
        itc[1] = 0;
        ++itc[2];
      }
    }
  }

  // ---- epilogue: O = acc / rowsum, LSE = ln(rowsum) + scale * rowmax -------------------------
  T* obase = reinterpret_cast<T*>(p.o) + int64_t(bg) * p.seqlen_q * q_row_stride + int64_t(head) * D;
#pragma unroll
  for (int mb = 0; mb < MQ; ++mb) {
    const float l = l_run[mb] + __shfl_xor(l_run[mb], 32);
    const float inv = (l > 0.f) ? p.out_scale / l : 0.f;
    const int row = qtile_idx * QT + (wave * MQ + mb) * 32 + l32;
    if (row < p.seqlen_q) {
      T* orow = obase + int64_t(row) * q_row_stride;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          typedef T tx4 __attribute__((ext_vector_type(4)));
          tx4 o4;
#pragma unroll
          for (int i = 0; i < 4; ++i) o4[i] = static_cast<T>(acc[mb][db][4 * j + i] * inv);
          *reinterpret_cast<tx4*>(orow + db * 32 + 8 * j + 4 * g) = o4;
        }
      if (g == 0) {
        const float lse = (l > 0.f) ? (m_run[mb] * p.scale + __logf(l)) : -INFINITY;
        p.lse[(int64_t(bg) * p.seqlen_q + row) * p.heads_q + head] = lse;
      }
    }
  }
}

}  // namespace natten_amd
