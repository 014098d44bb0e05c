// Fused neighborhood attention forward for float32 operands on gfx950, on token-permuted sequences.
// The reference runs float32 through its CUTLASS 2.x kernels and, on CPU, through flex attention
// (SHI-Labs/NATTEN tests/test_fna.py:107-131 states the tolerance: 1e-4 on the output); here it is a
// plain kernel of its own: S^T = K Q^T and O^T += V^T P^T on v_mfma_f32_32x32x2_f32 (IEEE float32
// products and sums), exact online softmax in float32 (no lazy rescale, P not rounded), every logit
// tested against its query's window (no whole-tile classification).  One workgroup per Q tile of
// 128 rows, 64-key tiles staged through LDS with ordinary loads; built for correctness at the
// stated dtype, not tuned like fna_fwd_kernel.
#pragma once

#include "fna_fwd.hpp"

namespace natten_amd {

// Same matrix layouts as the 16-bit kernel: the lane (l32 = lane % 32, g = lane / 32) owns query
// column l32 of the wave's 32-row block; of a 32 x 32 result block it holds rows
// 8 * (r / 4) + 4 * g + r % 4, r = 0..15.  A 32x32x2 instruction multiplies two k-indices, one per
// g; which head-dim element (QK) or key (PV) a k-index stands for is free as long as both operands
// agree: QK uses element g * D/2 + step, PV key 8 * (r / 4) + 4 * g + r % 4 (so a P register is the
// B operand as it stands).
template <int D>
__global__ void __launch_bounds__(256) fna_fwd_f32_kernel(const FnaParams p) {
  constexpr int KVT = 64, QT = 128, NT = 256;
  constexpr int LDW = D + 4;   // floats per LDS row: 16-byte aligned rows, 4 banks apart
  constexpr int HALF = D / 2;  // head-dim elements per k-index half
  constexpr int DB = D / 32;
  __shared__ __attribute__((aligned(16))) float sK[KVT * LDW];
  __shared__ __attribute__((aligned(16))) float sV[KVT * LDW];
  __shared__ int sCrd[KVT][4];  // in-tile coordinates of every KV position (dimension 0 fastest)

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int g = lane >> 5;

  // ---- workgroup -> (batch * dilation group, head, Q tile) ---------------------------------------
  const int pid = blockIdx.x;
  const int qtile = pid % p.num_q_tiles;
  const int bh = pid / p.num_q_tiles;
  const int head = bh % p.heads_q;
  const int bg = bh / p.heads_q;
  const int head_kv = head / (p.heads_q / p.heads_kv);

  int extent[3], q_first[3], t_lo[3], t_hi[3];
  {
    int gl = bg % p.num_groups;
    int tq = qtile;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int gi = gl % p.dil[a];
      gl /= p.dil[a];
      extent[a] = na_group_extent(p.qkv_shape[a], p.dil[a], gi);
      const int tc = tq % p.q_tiled[a];  // Q tiles are enumerated with dimension 0 fastest
      tq /= p.q_tiled[a];
      q_first[a] = tc * p.q_tile[a];
      // KV tiles that the windows of the tile's queries reach (padding queries act as the last real one)
      const bool c = p.causal[a] != 0;
      const int qf = na_min(q_first[a], extent[a] - 1);
      const int ql = na_min(q_first[a] + p.q_tile[a] - 1, extent[a] - 1);
      const int st_f = na_window_start(qf, p.ksize[a], p.stride[a], extent[a], c);
      const int st_l = na_window_start(ql, p.ksize[a], p.stride[a], extent[a], c);
      const int en_l = na_window_end(ql, st_l, p.ksize[a], extent[a], c);
      t_lo[a] = st_f / p.kv_tile[a];
      t_hi[a] = (en_l - 1) / p.kv_tile[a];
    }
  }
  if (tid < KVT) {
    int i = tid;
    sCrd[tid][0] = i % p.kv_tile[0];
    i /= p.kv_tile[0];
    sCrd[tid][1] = i % p.kv_tile[1];
    sCrd[tid][2] = i / p.kv_tile[1];
    sCrd[tid][3] = 0;
  }

  // ---- this lane's query: row of the tile (dimension 0 fastest), window, fragment ----------------
  const int row = wave * 32 + l32;
  int ws[3], we[3];
  {
    int r = row;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int off = r % p.q_tile[a];
      r /= p.q_tile[a];
      const int c = na_min(q_first[a] + off, extent[a] - 1);
      const bool cz = p.causal[a] != 0;
      ws[a] = na_window_start(c, p.ksize[a], p.stride[a], extent[a], cz);
      we[a] = na_window_end(c, ws[a], p.ksize[a], extent[a], cz);
    }
  }
  const int64_t q_row = int64_t(bg) * p.seqlen_q + int64_t(qtile) * QT + row;
  const float c_log2 = p.scale * 1.4426950408889634f;
  float qf[HALF];
  {
    const float* qrow = static_cast<const float*>(p.q) + (q_row * p.heads_q + head) * D + g * HALF;
#pragma unroll
    for (int i = 0; i < HALF; i += 4) {
      const f32x4_t x = *reinterpret_cast<const f32x4_t*>(qrow + i);
#pragma unroll
      for (int e = 0; e < 4; ++e) qf[i + e] = x[e] * c_log2;
    }
  }

  f32x16_t acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  const int64_t kv_row_stride = int64_t(p.heads_kv) * D;
  const float* kbase = static_cast<const float*>(p.k) + (int64_t(bg) * p.seqlen_kv * p.heads_kv + head_kv) * D;
  const float* vbase = static_cast<const float*>(p.v) + (int64_t(bg) * p.seqlen_kv * p.heads_kv + head_kv) * D;

  for (int t2 = t_lo[2]; t2 <= t_hi[2]; ++t2)
    for (int t1 = t_lo[1]; t1 <= t_hi[1]; ++t1)
      for (int t0 = t_lo[0]; t0 <= t_hi[0]; ++t0) {
        const int64_t row0 = int64_t(t0 + p.kv_tiled[0] * (t1 + p.kv_tiled[1] * t2)) * KVT;
        const int org[3] = {t0 * p.kv_tile[0], t1 * p.kv_tile[1], t2 * p.kv_tile[2]};
        workgroup_sync();  // everyone is done with the previous tile (and sCrd is written)
#pragma unroll
        for (int c = tid; c < KVT * (D / 4); c += NT) {
          const int r = c / (D / 4), c4 = c % (D / 4);
          const int64_t off = (row0 + r) * kv_row_stride + c4 * 4;
          *reinterpret_cast<f32x4_t*>(&sK[r * LDW + c4 * 4]) = *reinterpret_cast<const f32x4_t*>(kbase + off);
          *reinterpret_cast<f32x4_t*>(&sV[r * LDW + c4 * 4]) = *reinterpret_cast<const f32x4_t*>(vbase + off);
        }
        workgroup_sync();

        // S^T = K Q^T (already in the exp2 domain), two blocks of 32 keys
        f32x16_t S[2];
#pragma unroll
        for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
          for (int r = 0; r < 16; ++r) S[sb][r] = 0.f;
          const float* krow = &sK[(sb * 32 + l32) * LDW + g * HALF];
#pragma unroll
          for (int i = 0; i < HALF; i += 4) {
            const f32x4_t k4 = *reinterpret_cast<const f32x4_t*>(krow + i);
#pragma unroll
            for (int e = 0; e < 4; ++e) S[sb] = __builtin_amdgcn_mfma_f32_32x32x2f32(k4[e], qf[i + e], S[sb], 0, 0, 0);
          }
        }
        // window test of every (key, query) pair, row maximum
        float mx = -INFINITY;
#pragma unroll
        for (int sb = 0; sb < 2; ++sb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = sb * 32 + 8 * (r / 4) + 4 * g + (r % 4);
            bool in = true;
#pragma unroll
            for (int a = 0; a < 3; ++a) {
              const int kc = org[a] + sCrd[key][a];
              in = in && (kc >= ws[a]) && (kc < we[a]);
            }
            S[sb][r] = in ? S[sb][r] : -INFINITY;
            mx = fmaxf(mx, S[sb][r]);
          }
        mx = fmaxf(mx, __shfl_xor(mx, 32));  // the two halves of a query's keys
        const float m_new = fmaxf(m_run, mx);
        // (a query none of whose keys lie in this tile keeps m_new = m_run, possibly -inf: all p are 0)
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = exp2f(m_run - m_use);  // 0 while m_run is -inf
        float psum = 0.f;
#pragma unroll
        for (int sb = 0; sb < 2; ++sb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            S[sb][r] = exp2f(S[sb][r] - m_use);
            psum += S[sb][r];
          }
        l_run = l_run * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[db][r] *= alpha;
        // O^T += V^T P^T: k-index g of step (sb, r) is key sb * 32 + 8 * (r / 4) + 4 * g + r % 4
#pragma unroll
        for (int sb = 0; sb < 2; ++sb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = sb * 32 + 8 * (r / 4) + 4 * g + (r % 4);
#pragma unroll
            for (int db = 0; db < DB; ++db)
              acc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(sV[key * LDW + db * 32 + l32], S[sb][r], acc[db], 0, 0, 0);
          }
      }

  // ---- epilogue: O = acc / rowsum, LSE = ln(rowsum) + ln2 * rowmax --------------------------------
  const float l = l_run + __shfl_xor(l_run, 32);
  const float inv = (l > 0.f) ? 1.f / l : 0.f;
  float* orow = static_cast<float*>(p.o) + (q_row * p.heads_q + head) * D;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f32x4_t o4;
#pragma unroll
      for (int i = 0; i < 4; ++i) o4[i] = acc[db][4 * j + i] * inv;
      *reinterpret_cast<f32x4_t*>(orow + db * 32 + 8 * j + 4 * g) = o4;
    }
  if (g == 0) p.lse[q_row * p.heads_q + head] = (l > 0.f) ? (m_run * 0.6931471805599453f + logf(l)) : -INFINITY;
}

}  // namespace natten_amd
