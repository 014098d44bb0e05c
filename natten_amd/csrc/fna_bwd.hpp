// Fused neighborhood attention backward for gfx950 (MI355X).
//
// One kernel template, two roles.  A workgroup owns a "stationary" tile of 128 rows (one row
// per lane and 32-row block, four waves) and streams 64-row tiles of the other side through
// LDS:
//   dQ role  : stationary = queries (operands Q, dO; result dQ), streamed = keys (K, V)
//   dKV role : stationary = keys    (operands K, V; results dK, dV), streamed = queries (Q, dO)
// Per streamed tile, with Y1/Y2 the streamed and X1/X2 the stationary operands:
//   S^T  = Y1 X1^T,  dP^T = Y2 X2^T                     (32x32x16 MFMA, the lane owns a stationary row)
//   P    = exp2(c S - log2e LSE) on unmasked pairs, 0 elsewhere;  dS = P (dP - delta)
//   acc1^T += Y1^T dS^T   (dQ = scale * sum_k dS k  /  dK = scale * sum_q dS q)
//   acc2^T += Y2^T P^T    (dKV role only: dV = sum_q P dO)
// LSE and delta = rowsum(dO * O) belong to the query: per-lane scalars in the dQ role, a small
// per-tile LDS table in the dKV role.  Nothing is accumulated through memory, so both results
// are deterministic.
//
// What it restates (not the code): SHI-Labs/NATTEN
//   csrc/include/natten/cuda/reference/fna_reference_backward.hpp:60-150, :165-265, :282-380
//     (P = exp(scale q.k - LSE), dS = P scale (dO.v - dO.o), dQ / dK / dV as sums over the mask)
//   csrc/include/natten/cuda/fna_blackwell/collective/fna_fusion_bwd.hpp:256-318 (the Q tiles a KV tile meets;
//     here the query interval is found by bisection on the forward window functions instead)
// Operands are token-permuted sequences whose tiles hold 128 tokens; such a tile splits, along
// its slowest dimension, into two contiguous 64-token tiles, which is what the other role streams.
#pragma once

#include "fna_fwd.hpp"

namespace natten_amd {

struct FnaBwdParams {
  const void* q;      // [batch, seqlen_q, heads_q, D]   (batch counts dilation groups)
  const void* k;      // [batch, seqlen_kv, heads_kv, D]
  const void* v;
  const void* d_out;  // like q
  const float* lse;   // [batch, seqlen_q, heads_q], natural log
  const float* delta; // [batch, seqlen_q, heads_q], rowsum(d_out * out)
  void* dq;
  void* dk;
  void* dv;
  int batch, heads_q, heads_kv;
  int seqlen_q, seqlen_kv;
  int num_groups;
  int qkv_shape[3];
  int q_extent0;  // > 0: queries along dimension 0 (dense attention with its own query count); 0: as the keys
  int ksize[3], stride[3], dil[3], causal[3];
  int q_tile[3], kv_tile[3];    // 128-token tiles of the two permuted layouts
  int q_tiled[3], kv_tiled[3];  // tiles per dimension
  int q_split, kv_split;        // the dimension along which a 128-token tile of either side halves
                                // (its last dimension of extent > 1, so that the halves are contiguous)
  float scale;
};

template <typename T, int D, bool KV_STATIONARY>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
fna_bwd_kernel(const FnaBwdParams p) {
  constexpr int NT = 256;
  constexpr int AT = 128;  // stationary rows
  constexpr int BT = 64;   // streamed rows per tile
  constexpr int KSTEPS = D / 16;
  constexpr int DB = D / 32;
  constexpr int NSB = BT / 32;
  using L = FnaSmem<D, BT>;
  constexpr int ROWB = L::ROWB;
  constexpr int CPR = L::CPR;
  constexpr int TILE_BYTES = L::TILE_BYTES;
  constexpr int CHUNKS = BT * CPR;
  constexpr int PER = CHUNKS / NT;
  static_assert(CHUNKS % NT == 0 && PER >= 1, "a streamed tile must be a whole number of workgroup-wide copies");
  using M = Mma<T>;
  using vec8 = typename M::vec8;

  // two stages of: Y1 in the layout of b128 row reads, Y1 in the layout of transpose reads, Y2 likewise
  __shared__ __attribute__((aligned(1024))) char sY1k[2 * TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sY1t[2 * TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sY2k[2 * TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sY2t[KV_STATIONARY ? 2 * TILE_BYTES : 1024];
  __shared__ __attribute__((aligned(16))) uint32_t sTabA[2 * BT];
  __shared__ __attribute__((aligned(16))) uint32_t sTabB[2 * BT];
  __shared__ __attribute__((aligned(16))) float sLse[2 * BT];
  __shared__ __attribute__((aligned(16))) float sDelta[2 * BT];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int g = lane >> 5;

  const int* a_tile = KV_STATIONARY ? p.kv_tile : p.q_tile;
  const int* a_tiled = KV_STATIONARY ? p.kv_tiled : p.q_tiled;
  const int* b_tile = KV_STATIONARY ? p.q_tile : p.kv_tile;
  const int* b_tiled = KV_STATIONARY ? p.q_tiled : p.kv_tiled;
  const int heads_a = KV_STATIONARY ? p.heads_kv : p.heads_q;
  const int heads_b = KV_STATIONARY ? p.heads_q : p.heads_kv;
  const int seq_a = KV_STATIONARY ? p.seqlen_kv : p.seqlen_q;
  const int seq_b = KV_STATIONARY ? p.seqlen_q : p.seqlen_kv;
  const int rep = p.heads_q / p.heads_kv;
  const int split_dim = KV_STATIONARY ? p.q_split : p.kv_split;  // of the streamed side

  // ---- workgroup -> (batch * group, head, stationary tile) --------------------------------------
  const int num_a = a_tiled[0] * a_tiled[1] * a_tiled[2];
  const int at = int(blockIdx.x) % num_a;
  const int head_a = (int(blockIdx.x) / num_a) % heads_a;
  const int bg = int(blockIdx.x) / (num_a * heads_a);

  int extent[3], q_extent[3], a_first[3], b_sub[3], box_tile0[3], box_n[3];
  bool empty = false;
  {
    int gl = bg % p.num_groups;
    int tc[3];
    tc[0] = at % a_tiled[0];
    tc[1] = (at / a_tiled[0]) % a_tiled[1];
    tc[2] = at / (a_tiled[0] * a_tiled[1]);
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int gi = gl % p.dil[a];
      gl /= p.dil[a];
      extent[a] = na_group_extent(p.qkv_shape[a], p.dil[a], gi);
      q_extent[a] = (a == 0 && p.q_extent0 > 0) ? p.q_extent0 : extent[a];
      a_first[a] = tc[a] * a_tile[a];
      b_sub[a] = (a == split_dim) ? b_tile[a] / 2 : b_tile[a];
      const bool c = p.causal[a] != 0;
      int lo, hi;  // first and last streamed coordinate this tile meets
      if constexpr (!KV_STATIONARY) {
        const int qf = a_first[a], ql = na_min(qf + a_tile[a], q_extent[a]) - 1;
        if (qf >= q_extent[a]) empty = true;
        lo = na_window_start(qf, p.ksize[a], p.stride[a], extent[a], c);
        const int st_l = na_window_start(na_max(ql, 0), p.ksize[a], p.stride[a], extent[a], c);
        hi = na_window_end(na_max(ql, 0), st_l, p.ksize[a], extent[a], c) - 1;
      } else {
        const int j0 = a_first[a], j1 = na_min(j0 + a_tile[a], extent[a]) - 1;
        if (j0 >= extent[a]) empty = true;
        lo = na_first_query_attending(j0, p.ksize[a], p.stride[a], extent[a], q_extent[a], c);
        hi = na_last_query_attending(na_max(j1, 0), p.ksize[a], p.stride[a], extent[a], q_extent[a], c);
        if (lo > hi) empty = true;
      }
      lo = na_max(lo, 0);
      hi = na_max(hi, lo);
      box_tile0[a] = lo / b_sub[a];
      box_n[a] = hi / b_sub[a] + 1 - box_tile0[a];
    }
  }

  // ---- this lane's stationary row -----------------------------------------------------------------
  const int r_in = wave * 32 + l32;  // row inside the tile: dimension 0 fastest
  int a_off[3];
  a_off[0] = r_in % a_tile[0];
  a_off[1] = (r_in / a_tile[0]) % a_tile[1];
  a_off[2] = r_in / (a_tile[0] * a_tile[1]);
  const int64_t a_row = (int64_t(bg) * seq_a + int64_t(at) * AT + r_in);
  const int64_t a_stride = int64_t(heads_a) * D;
  const int64_t b_stride = int64_t(heads_b) * D;
  const float kLog2e = 1.4426950408889634f;

  typedef T tx4 __attribute__((ext_vector_type(4)));
  auto store_rows = [&](void* dst, const f32x16_t (&acc)[DB], float mul) {
    T* orow = reinterpret_cast<T*>(dst) + a_row * a_stride + int64_t(head_a) * D;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        tx4 o4;
#pragma unroll
        for (int i = 0; i < 4; ++i) o4[i] = static_cast<T>(acc[db][4 * j + i] * mul);
        *reinterpret_cast<tx4*>(orow + db * 32 + 8 * j + 4 * g) = o4;
      }
  };

  f32x16_t acc1[DB], acc2[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc1[db][r] = acc2[db][r] = 0.f;

  if (empty) {
    // padding rows, or rows nothing attends: their gradients are zero
    if constexpr (KV_STATIONARY) {
      store_rows(p.dk, acc1, 0.f);
      store_rows(p.dv, acc2, 0.f);
    } else {
      store_rows(p.dq, acc1, 0.f);
    }
    return;
  }

  // stationary operand fragments: row r_in, elements 16*ks + 8*g .. +7
  const T* x1 = reinterpret_cast<const T*>(KV_STATIONARY ? p.k : p.q) + a_row * a_stride + int64_t(head_a) * D + g * 8;
  const T* x2 = reinterpret_cast<const T*>(KV_STATIONARY ? p.v : p.d_out) + a_row * a_stride + int64_t(head_a) * D + g * 8;
  vec8 x1f[KSTEPS], x2f[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) {
    x1f[ks] = *reinterpret_cast<const vec8*>(x1 + ks * 16);
    x2f[ks] = *reinterpret_cast<const vec8*>(x2 + ks * 16);
  }

  // mask state of the lane
  int wst[3] = {0, 0, 0}, wen[3] = {0, 0, 0};  // dQ role: window of the lane's query
  uint32_t key_packed = 0;                     // dKV role: in-tile coordinates of the lane's key
  float lse_l = 0.f, delta_l = 0.f;
  if constexpr (!KV_STATIONARY) {
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int c = a_first[a] + a_off[a];
      wst[a] = na_window_start(c, p.ksize[a], p.stride[a], extent[a], p.causal[a] != 0);
      wen[a] = na_window_end(c, wst[a], p.ksize[a], extent[a], p.causal[a] != 0);
    }
    lse_l = p.lse[a_row * p.heads_q + head_a] * kLog2e;
    delta_l = p.delta[a_row * p.heads_q + head_a];
    // in-tile coordinates of every streamed position, packed in 10-bit fields
    for (int i = tid; i < BT; i += NT) {
      const int t0 = i % b_sub[0];
      const int t1 = (i / b_sub[0]) % b_sub[1];
      const int t2 = i / (b_sub[0] * b_sub[1]);
      sTabA[i] = uint32_t(t0) | (uint32_t(t1) << 10) | (uint32_t(t2) << 20);
    }
  } else {
    key_packed = uint32_t(a_off[0]) | (uint32_t(a_off[1]) << 10) | (uint32_t(a_off[2]) << 20);
  }

  // ---- streamed tiles ---------------------------------------------------------------------------
  const int total = box_n[0] * box_n[1] * box_n[2];
  const int n_iter = KV_STATIONARY ? total * rep : total;
  const T* y1_all = reinterpret_cast<const T*>(KV_STATIONARY ? p.q : p.k);
  const T* y2_all = reinterpret_cast<const T*>(KV_STATIONARY ? p.d_out : p.v);

  // copy i of a thread moves chunk P = i * NT + tid of the tile (row P / CPR, LDS slot P % CPR)
  uint32_t off_k[PER], off_t[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int P = i * NT + tid;
    const int row = P / CPR, slot = P % CPR;
    off_k[i] = uint32_t(row) * uint32_t(b_stride * 2) + uint32_t(L::k_slot(row, slot) * 16);
    off_t[i] = uint32_t(row) * uint32_t(b_stride * 2) + uint32_t(L::v_slot(row, slot) * 16);
  }

  struct Tile {
    int origin[3];  // coordinate of the tile's first token
    int row0;       // its first row in the streamed side's permuted sequence
    int head_b;
  };
  auto tile_of = [&](int it) {
    Tile t;
    const int j = it % total;
    int c[3];
    c[2] = j % box_n[2];
    c[1] = (j / box_n[2]) % box_n[1];
    c[0] = j / (box_n[2] * box_n[1]);
    int cc[3], half = 0;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      c[a] += box_tile0[a];
      t.origin[a] = c[a] * b_sub[a];
      const bool split = (a == split_dim);
      half |= split ? (c[a] & 1) : 0;
      cc[a] = split ? (c[a] >> 1) : c[a];
    }
    t.row0 = (cc[0] + b_tiled[0] * (cc[1] + b_tiled[1] * cc[2])) * AT + half * BT;
    t.head_b = KV_STATIONARY ? head_a * rep + it / total : head_a / rep;
    return t;
  };

  auto issue = [&](int it, int stage) {
    const Tile t = tile_of(it);
    const int64_t row = int64_t(bg) * seq_b + t.row0;
    if constexpr (KV_STATIONARY) {
      // Per streamed query: its window relative to this workgroup's key tile, and its LSE / delta.
      // Done ahead of the tile copies, so that waiting for these loads does not wait for the copies.
      if (wave == 0) {
        const int e = lane;
        int qo[3];
        qo[0] = e % b_sub[0];
        qo[1] = (e / b_sub[0]) % b_sub[1];
        qo[2] = e / (b_sub[0] * b_sub[1]);
        uint32_t addc = 0, subc = 0;
        bool valid = true;
#pragma unroll
        for (int a = 0; a < 3; ++a) {
          const int qc = t.origin[a] + qo[a];
          valid = valid && (qc < q_extent[a]);
          const int st = na_window_start(qc, p.ksize[a], p.stride[a], extent[a], p.causal[a] != 0);
          const int en = na_window_end(qc, st, p.ksize[a], extent[a], p.causal[a] != 0);
          const int lo = na_min(na_max(st - a_first[a], 0), a_tile[a]);
          const int hi = na_min(na_max(en - a_first[a], 0), a_tile[a]);
          addc |= uint32_t(512 - lo) << (10 * a);
          subc |= uint32_t(511 + hi) << (10 * a);
        }
        sTabA[stage * BT + e] = valid ? addc : 0u;  // no guard bit survives a zero addend
        sTabB[stage * BT + e] = valid ? subc : 0u;
      } else if (wave == 1) {
        sLse[stage * BT + lane] = p.lse[(row + lane) * p.heads_q + t.head_b] * kLog2e;
      } else if (wave == 2) {
        sDelta[stage * BT + lane] = p.delta[(row + lane) * p.heads_q + t.head_b];
      }
    }
    const T* y1 = y1_all + row * b_stride + int64_t(t.head_b) * D;
    const T* y2 = y2_all + row * b_stride + int64_t(t.head_b) * D;
    const uint32_t dst = uint32_t(stage * TILE_BYTES + wave * 1024);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const uint32_t d = dst + uint32_t(i * NT * 16);
      async_copy16_asm<0>(y1, off_k[i], lds_address(sY1k) + d);
      async_copy16_asm<0>(y1, off_t[i], lds_address(sY1t) + d);
      async_copy16_asm<0>(y2, off_k[i], lds_address(sY2k) + d);
      if constexpr (KV_STATIONARY) async_copy16_asm<0>(y2, off_t[i], lds_address(sY2t) + d);
    }
  };

  // lane-constant LDS read offsets (same fragment layouts as the forward kernel)
  int k_off[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) k_off[ks] = l32 * ROWB + L::k_slot(l32, ks * 2 + g) * 16;
  const int l16 = lane & 15;
  const int v_e = l16 >> 2, v_j4 = l16 & 3;
  const int v_row = 4 * g + v_e;
  const int v_chunk = (l32 >> 4) * 2 + (v_j4 >> 1);
  const int v_sub = (v_j4 & 1) * 8;
  auto row_frag = [&](const char* s, int sb, int ks) {
    return *reinterpret_cast<const vec8*>(s + sb * 32 * ROWB + k_off[ks]);
  };
  // transposed fragment: sub-block sb, 16-row half h, 32-column block db
  auto tr_frag = [&](const char* s, int sb, int h, int db) {
    const int r0 = sb * 32 + h * 16 + v_row;
    const int c = db * 4 + v_chunk;
    const s16x4_t lo = lds_read_tr16(s + r0 * ROWB + v_sub + L::v_slot(r0, c) * 16);
    const s16x4_t hi = lds_read_tr16(s + (r0 + 8) * ROWB + v_sub + L::v_slot(r0 + 8, c) * 16);
    return __builtin_bit_cast(vec8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  const float c_log2 = p.scale * kLog2e;

  issue(0, 0);
  for (int it = 0; it < n_iter; ++it) {
    const int stage = it & 1;
    wait_vmcnt<0>();
    __syncthreads();  // tile `it` and its tables are in LDS; everyone is done with the other stage
    if (it + 1 < n_iter) issue(it + 1, stage ^ 1);

    const char* y1k = sY1k + stage * TILE_BYTES;
    const char* y1t = sY1t + stage * TILE_BYTES;
    const char* y2k = sY2k + stage * TILE_BYTES;
    const char* y2t = sY2t + (KV_STATIONARY ? stage * TILE_BYTES : 0);

    f32x16_t S[NSB], dP[NSB];
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) S[sb][r] = dP[sb][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        S[sb] = M::run(row_frag(y1k, sb, ks), x1f[ks], S[sb]);
        dP[sb] = M::run(row_frag(y2k, sb, ks), x2f[ks], dP[sb]);
      }
    }

    // mask constants of the lane for this tile
    uint32_t addc = 0, subc = 0;
    if constexpr (!KV_STATIONARY) {
      const Tile t = tile_of(it);
#pragma unroll
      for (int a = 0; a < 3; ++a) {
        const int lo = na_min(na_max(wst[a] - t.origin[a], 0), b_sub[a]);
        const int hi = na_min(na_max(wen[a] - t.origin[a], 0), b_sub[a]);
        addc |= uint32_t(512 - lo) << (10 * a);
        subc |= uint32_t(511 + hi) << (10 * a);
      }
    }

    vec8 pf[NSB][2], dsf[NSB][2];
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const int e0 = sb * 32 + 8 * jj + 4 * g;  // the lane's registers 4*jj .. 4*jj+3 are streamed rows e0 .. e0+3
        u32x4_t ta, tb;
        float ls[4], dl[4];
        if constexpr (KV_STATIONARY) {
          ta = *reinterpret_cast<const u32x4_t*>(&sTabA[stage * BT + e0]);
          tb = *reinterpret_cast<const u32x4_t*>(&sTabB[stage * BT + e0]);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            ls[i] = sLse[stage * BT + e0 + i];
            dl[i] = sDelta[stage * BT + e0 + i];
          }
        } else {
          ta = *reinterpret_cast<const u32x4_t*>(&sTabA[e0]);
          tb = ta;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            ls[i] = lse_l;
            dl[i] = delta_l;
          }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = 4 * jj + i;
          uint32_t ok;
          if constexpr (KV_STATIONARY) ok = (key_packed + ta[i]) & (tb[i] - key_packed) & kGuardBits;
          else ok = (ta[i] + addc) & (subc - ta[i]) & kGuardBits;
          const float x = fast_exp2(S[sb][r] * c_log2 - ls[i]);
          const float pv = (ok == kGuardBits) ? x : 0.f;
          const float ds = pv * (dP[sb][r] - dl[i]);
          pf[sb][r / 8][r % 8] = static_cast<T>(pv);
          dsf[sb][r / 8][r % 8] = static_cast<T>(ds);
        }
      }

#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          acc1[db] = M::run(tr_frag(y1t, sb, h, db), dsf[sb][h], acc1[db]);
          if constexpr (KV_STATIONARY) acc2[db] = M::run(tr_frag(y2t, sb, h, db), pf[sb][h], acc2[db]);
        }
  }
  wait_vmcnt<0>();

  if constexpr (KV_STATIONARY) {
    store_rows(p.dk, acc1, p.scale);
    store_rows(p.dv, acc2, 1.f);
  } else {
    store_rows(p.dq, acc1, p.scale);
  }
}

// delta[item] = sum_d out[item, d] * d_out[item, d] over `items` rows of D contiguous elements
// (the reference's compute_delta, csrc/include/natten/compute_delta.h:33-36,
// csrc/include/natten/cuda/reduction/compute_delta.cuh).  D / 8 lanes
// share a row, 16 bytes each.
template <typename T, int D>
__global__ void __launch_bounds__(256) delta_kernel(const T* out, const T* d_out, float* delta, int64_t items) {
  constexpr int LPI = D / 8;  // lanes per item
  typedef T tx8 __attribute__((ext_vector_type(8)));
  const int64_t gtid = int64_t(blockIdx.x) * 256 + threadIdx.x;
  const int64_t item = gtid / LPI;
  const int part = int(gtid % LPI);
  float s = 0.f;
  if (item < items) {
    const tx8 a = *reinterpret_cast<const tx8*>(out + item * D + part * 8);
    const tx8 b = *reinterpret_cast<const tx8*>(d_out + item * D + part * 8);
#pragma unroll
    for (int i = 0; i < 8; ++i) s += float(a[i]) * float(b[i]);
  }
#pragma unroll
  for (int o = LPI / 2; o > 0; o >>= 1) s += __shfl_xor(s, o);
  if (item < items && part == 0) delta[item] = s;
}

}  // namespace natten_amd
