// Fused neighborhood attention backward for gfx950 (MI355X).
//
// One kernel template, several roles.  A workgroup owns a "stationary" tile of 128 rows (one
// row per lane and 32-row block, four waves) and streams 64-row tiles of the other side
// through LDS:
//   dQ role          : stationary = queries (operands Q, dO; result dQ), streamed = keys (K, V)
//   dKV, paired role : stationary = keys    (operands K, V; results dK and dV), streamed = queries (Q, dO)
// Per streamed tile, with Y1/Y2 the streamed and X1/X2 the stationary operands:
//   S^T  = Y1 X1^T,  dP^T = Y2 X2^T                     (32x32x16 MFMA, the lane owns a stationary row)
//   P    = exp2(S - log2e LSE) on unmasked pairs, 0 elsewhere;  dS = P (dP - delta)
//   acc1^T += Y1^T dS^T   (dQ = scale * sum_k dS k  /  dK = ln 2 * sum_q dS q')
// The logits are formed from the same operand as in the forward kernel, q' = round(q * scale *
// log2(e)) in the operand type, so that S is the forward's logit to the last bit of its operands
// and P the probability its LSE normalises (the rows of P sum to one); with the unscaled queries
// the two passes' logits differ by the rounding of q', and a probability of a one-key window
// comes out as 1 +- 0.5 % instead of 1.  The dQ role scales its stationary query fragments as it
// loads them; the key-stationary roles stream q' from a copy (qs) that a pass over q writes first.
//   acc2^T += Y2^T P^T    (dV = sum_q P dO)
// In the dKV role one wave forms all of this for its 32 key rows.  At head dim 128 the
// accumulators, stationary fragments and both products of that no longer fit the 256 vector
// registers a matrix instruction can address directly; the paired role then splits the work
// over two waves without recomputing anything: eight waves per workgroup, waves w and w + 4
// share the 32 key rows of block w; wave w ("P wave") forms S^T, the probabilities and dV,
// wave w + 4 ("dS wave") forms dP^T, takes the probabilities from LDS (fp16, one tile later),
// and forms dS and dK.  LSE and delta = rowsum(dO * O) belong to the
// query: per-lane scalars in the dQ role, a small per-tile LDS table in the others.  Nothing
// is accumulated through memory, so the results are deterministic.
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
  const void* qs;     // like q: round(q * scale * log2(e)), the forward kernel's logit operand (key-stationary roles)
  const void* k;      // [batch, seqlen_kv, heads_kv, D]
  const void* v;
  const void* d_out;  // like q
  const float* lse;   // [batch, heads_q, seqlen_q] (head-major: a tile's values are contiguous), natural log
  const float* delta; // [batch, heads_q, seqlen_q], rowsum(d_out * out)
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
  // Operand layout.  fused == 0: token-permuted sequences as described above.  fused == 1: the
  // original tensors [batch, X0, X1, X2, heads, D] (lse / delta [batch, heads, X0 * X1 * X2]);
  // the kernel gathers and scatters the rows of a tile itself.
  int fused;
  // fused == 1 only: some extent is not a multiple of dilation x tile, so tiles may reach past a
  // dilation group (every group is at least a tile wide in every dimension).  Rows of the stationary
  // tile past the group's end are computed on a clamped copy and not stored; a streamed tile that
  // would reach past it is gathered from one tile extent before the end, and its leading rows,
  // which the tile before it delivered, take no part (as in the forward kernel).
  int edge;
  int tok_stride[3];  // tokens per unit step of an original coordinate: X1*X2, X2, 1
  int tokens;         // X0 * X1 * X2
  // Sequence-packed dense attention (VARLEN instances only; null otherwise).  `batch` sequences
  // lie back to back in one row range (the tensors have batch 1; seqlen_q / seqlen_kv count all
  // their rows), each padded to a multiple of 128 rows: sequence b owns query rows
  // pcu_q[b] .. pcu_q[b+1]-1 of which the first cu_q[b+1] - cu_q[b] are real, keys likewise;
  // q_tiled[0] / kv_tiled[0] count the tiles of the longest sequence.
  const int32_t* cu_q;    // [batch + 1] cumulative real lengths
  const int32_t* cu_kv;
  const int32_t* pcu_q;   // [batch + 1] cumulative padded lengths (row offsets into the tensors)
  const int32_t* pcu_kv;
  // Workgroup order of the key-stationary launch.  0: every XCD takes one contiguous eighth of
  // the (batch, head, tile) space.  > 0: runs of this many consecutive tiles are dealt round-robin
  // to the XCDs (the grid is then a whole number of rounds of 8 runs).
  int kv_wg_run;
  // Host side only: which launches a call makes (bit 0: the dQ role, bit 1: the dK / dV role; 0 = both).
  int roles;
};

enum BwdRole : int { kBwdDQ = 0, kBwdDKV = 1, kBwdPair = 2 };

template <typename T, int D, int ROLE, bool VARLEN = false>
__global__ void __launch_bounds__(ROLE == kBwdPair ? 512 : 256) __attribute__((amdgpu_waves_per_eu(2, 2)))
fna_bwd_kernel(const FnaBwdParams p) {
  constexpr bool KV_STATIONARY = ROLE != kBwdDQ;
  constexpr bool PAIR = ROLE == kBwdPair;
  // what one wave's tile body forms (a P wave of the paired role is a dV wave that also hands on
  // its probabilities; the dS waves have a body of their own)
  constexpr bool HAS_DS = !PAIR;                      // dP, dS and acc1 (dQ or dK)
  constexpr bool HAS_PV = ROLE == kBwdDKV || PAIR;  // acc2 (dV; dK in a dS wave)
  constexpr int NT = PAIR ? 512 : 256;
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
  static_assert(NSB == 2, "the slot schedule is written for two 32-row sub-blocks");
  using M = Mma<T>;
  using vec8 = typename M::vec8;
  using vec2 = typename M::vec2;
  typedef _Float16 h16x2_t __attribute__((ext_vector_type(2)));

  // One copy of Y1 and one of Y2 per stage, in the layout that serves row reads (S, dP) and
  // transpose reads (the accumulations) alike.
  // Stages: tiles are copied NS - 1 ahead.  Two stages at head dim 128 keep a workgroup under
  // half of the CU's LDS, so that two workgroups (two waves per SIMD) share a CU.
  // The paired role copies two tiles ahead, at any point of a step: Y2 (dO) is read in its own
  // step only and has three stages; Y1 (Q) and the tables are read for two steps (the dS waves
  // run one tile behind) and have four.
  constexpr int NS = (D == 128 && !PAIR) ? 2 : 3;
  constexpr int NS1 = PAIR ? 4 : NS;  // stages of Y1 and of the tables
  static_assert(!PAIR || D == 128, "the paired role is for head dim 128 (smaller ones fit the combined role)");
  __shared__ __attribute__((aligned(1024))) char sY1[NS1 * TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sY2[NS * TILE_BYTES];
  __shared__ __attribute__((aligned(16))) uint32_t sTabA[NS1 * BT];
  __shared__ __attribute__((aligned(16))) uint32_t sTabB[NS1 * BT];
  __shared__ __attribute__((aligned(16))) float sLse[NS1 * BT];
  __shared__ __attribute__((aligned(16))) float sDelta[NS1 * BT];
  __shared__ __attribute__((aligned(16))) float sSpare[BT];
  // paired role: probabilities from the P waves to the dS waves, fp16, [tile parity][row block]
  // [sub-block][half of the 16 values][lane] x 16 bytes
  __shared__ __attribute__((aligned(16))) char sX[PAIR ? 2 * 4 * NSB * 2 * 64 * 16 : 16];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rw = PAIR ? (wave & 3) : wave;  // 32-row block of the stationary tile
  const int part = PAIR ? (wave >> 2) : 0;  // paired role: 0 = P wave, 1 = dS wave
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
  // Workgroup ids go round-robin to the 8 XCDs; each XCD takes one contiguous eighth of the
  // (batch, head, tile) space, so that the workgroups resident on an XCD are neighbouring tiles
  // of one head and find each other's streamed tiles in that XCD's L2.  The paired role, with
  // half as many workgroups resident, does better with short runs dealt round-robin: the XCDs
  // then work on neighbouring runs of one head at a time and meet in the memory-side cache.
  const int num_a = a_tiled[0] * a_tiled[1] * a_tiled[2];
  const int total_wg = p.batch * heads_a * num_a;
  const int wg_run = KV_STATIONARY ? p.kv_wg_run : 0;
  int lin;
  if (wg_run > 0) {
    const int local = int(blockIdx.x) / kNumXcd;
    lin = ((local / wg_run) * kNumXcd + int(blockIdx.x) % kNumXcd) * wg_run + local % wg_run;
  } else {
    const int chunk = (total_wg + kNumXcd - 1) / kNumXcd;
    lin = (int(blockIdx.x) % kNumXcd) * chunk + int(blockIdx.x) / kNumXcd;
  }
  if (lin >= total_wg) return;
  // Within a head the tiles are taken with dimension 0 slowest: the workgroups running side by
  // side are then neighbours in the faster dimensions at the same dimension-0 position and
  // walk the same streamed tiles at about the same time.
  int tc[3];
  {
    const int rm = lin % num_a;
    tc[2] = rm % a_tiled[2];
    tc[1] = (rm / a_tiled[2]) % a_tiled[1];
    tc[0] = rm / (a_tiled[2] * a_tiled[1]);
    // a causal dimension 0: the query tiles with the longest key ranges are the last ones;
    // they start first (key tiles are already in that order)
    if (!KV_STATIONARY && p.causal[0]) tc[0] = a_tiled[0] - 1 - tc[0];
  }
  const int at = tc[0] + a_tiled[0] * (tc[1] + a_tiled[1] * tc[2]);  // position in the permuted sequence
  const int head_a = (lin / num_a) % heads_a;
  const int bg = lin / (num_a * heads_a);

  // first rows of this batch entry's sequences, its lse / delta values of head 0, and the
  // parameters a packed sequence overrides
  int64_t seq_row_a = int64_t(bg) * seq_a, seq_row_b = int64_t(bg) * seq_b;
  int64_t stat_row_q = int64_t(bg) * p.heads_q * p.seqlen_q;
  int64_t stat_head_stride = p.seqlen_q;
  int ksz[3] = {p.ksize[0], p.ksize[1], p.ksize[2]};
  int keys0 = p.qkv_shape[0], queries0 = p.q_extent0;
  bool empty = false;
  if constexpr (VARLEN) {
    const int q0 = p.cu_q[bg], kv0 = p.cu_kv[bg], pq0 = p.pcu_q[bg], pkv0 = p.pcu_kv[bg];
    const int len_q = p.cu_q[bg + 1] - q0, len_kv = p.cu_kv[bg + 1] - kv0;
    const int pad_q = p.pcu_q[bg + 1] - pq0, pad_kv = p.pcu_kv[bg + 1] - pkv0;
    // offsets the tensors cannot hold are not followed
    if (len_q < 0 || len_kv < 0 || pq0 < 0 || pkv0 < 0 || pad_q < len_q || pad_kv < len_kv ||
        ((pq0 | pkv0 | pad_q | pad_kv) & 127) != 0 || pq0 + pad_q > p.seqlen_q || pkv0 + pad_kv > p.seqlen_kv)
      return;
    if (tc[0] * AT >= (KV_STATIONARY ? pad_kv : pad_q)) return;  // the longest sequence has more tiles than this one
    seq_row_a = KV_STATIONARY ? pkv0 : pq0;
    seq_row_b = KV_STATIONARY ? pq0 : pkv0;
    stat_row_q = pq0;
    keys0 = ksz[0] = na_max(len_kv, 1);
    queries0 = na_max(len_q, 1);
    empty = len_q == 0 || len_kv == 0;  // nothing attends, or attends to nothing: zero gradients
  }

  int extent[3], q_extent[3], a_first[3], b_sub[3], box_tile0[3], box_n[3], full_t0[3], full_t1[3];
  int tok_step[3];    // original layout: tokens per unit step of a coordinate inside a dilation group
  int group_tok = 0;  // original layout: token of the dilation group's first element
  {
    int gl = bg % p.num_groups;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int gi = gl % p.dil[a];
      gl /= p.dil[a];
      tok_step[a] = p.dil[a] * p.tok_stride[a];
      group_tok += gi * p.tok_stride[a];
      extent[a] = na_group_extent(a == 0 ? keys0 : p.qkv_shape[a], p.dil[a], gi);
      q_extent[a] = (a == 0 && queries0 > 0) ? queries0 : extent[a];
      a_first[a] = tc[a] * a_tile[a];
      b_sub[a] = (a == split_dim) ? b_tile[a] / 2 : b_tile[a];
      const bool c = p.causal[a] != 0;
      int lo, hi;  // first and last streamed coordinate this tile meets
      if constexpr (!KV_STATIONARY) {
        const int qf = a_first[a], ql = na_min(qf + a_tile[a], q_extent[a]) - 1;
        if (qf >= q_extent[a]) empty = true;
        lo = na_window_start(qf, ksz[a], p.stride[a], extent[a], c);
        const int st_l = na_window_start(na_max(ql, 0), ksz[a], p.stride[a], extent[a], c);
        hi = na_window_end(na_max(ql, 0), st_l, ksz[a], extent[a], c) - 1;
      } else {
        const int j0 = a_first[a], j1 = na_min(j0 + a_tile[a], extent[a]) - 1;
        if (j0 >= extent[a]) empty = true;
        lo = na_first_query_attending(j0, ksz[a], p.stride[a], extent[a], q_extent[a], c);
        hi = na_last_query_attending(na_max(j1, 0), ksz[a], p.stride[a], extent[a], q_extent[a], c);
        if (lo > hi) empty = true;
      }
      lo = na_max(lo, 0);
      hi = na_max(hi, lo);
      box_tile0[a] = lo / b_sub[a];
      box_n[a] = hi / b_sub[a] + 1 - box_tile0[a];
      // Streamed tiles every row of which pairs with every row of the stationary tile (no mask
      // needed) form an interval of tile coordinates per dimension, again by monotonicity:
      // streamed coordinates flo .. fhi pair with all stationary ones.
      int flo, fhi;
      if constexpr (!KV_STATIONARY) {
        const int qf = a_first[a], ql = qf + a_tile[a] - 1;  // rows past the extent use the last window
        const int st_l = na_window_start(ql, ksz[a], p.stride[a], extent[a], c);
        const int st_f = na_window_start(qf, ksz[a], p.stride[a], extent[a], c);
        flo = st_l;
        fhi = na_window_end(qf, st_f, ksz[a], extent[a], c) - 1;
      } else {
        const int j0 = a_first[a], j1 = j0 + a_tile[a] - 1;
        if (j1 >= extent[a]) {
          flo = 1;  // the tile holds padding keys: never whole
          fhi = 0;
        } else {
          flo = na_first_query_attending(j1, ksz[a], p.stride[a], extent[a], q_extent[a], c);
          fhi = na_last_query_attending(j0, ksz[a], p.stride[a], extent[a], q_extent[a], c);
        }
      }
      full_t0[a] = na_max(na_ceil_div(na_max(flo, 0), b_sub[a]), box_tile0[a]);
      full_t1[a] = na_min((fhi + 1) / b_sub[a], box_tile0[a] + box_n[a]);  // one past the last whole tile
      if (fhi < 0 || full_t1[a] < full_t0[a]) full_t1[a] = full_t0[a];
    }
  }

  // ---- this lane's stationary row -----------------------------------------------------------------
  const int r_in = rw * 32 + l32;  // row inside the tile: dimension 0 fastest
  int a_off[3];
  a_off[0] = r_in % a_tile[0];
  a_off[1] = (r_in / a_tile[0]) % a_tile[1];
  a_off[2] = r_in / (a_tile[0] * a_tile[1]);
  // Row of the tensors / index into lse and delta: position in the permuted sequence, or the
  // token of the lane's coordinate in the original layout.
  // (original layout: a row past the end of its dilation group works on the group's last row and stores nothing)
  int a_crd[3];
  bool a_valid = true;
#pragma unroll
  for (int a = 0; a < 3; ++a) {
    const int c = a_first[a] + a_off[a];
    const int e = KV_STATIONARY ? extent[a] : q_extent[a];
    a_valid = a_valid && (c < e || !p.fused);
    a_crd[a] = p.fused ? na_min(c, e - 1) : c;
  }
  const int a_tok = group_tok + a_crd[0] * tok_step[0] + a_crd[1] * tok_step[1] + a_crd[2] * tok_step[2];
  const int64_t batch_row0 = p.fused ? int64_t(bg / p.num_groups) * p.tokens : 0;  // first row of the batch entry (original layout)
  const int64_t a_row = p.fused ? batch_row0 + a_tok : (seq_row_a + int64_t(at) * AT + r_in);
  const int64_t a_stride = int64_t(heads_a) * D;
  const int64_t b_stride = int64_t(heads_b) * D;
  const float kLog2e = 1.4426950408889634f;

  typedef T tx4 __attribute__((ext_vector_type(4)));
  auto store_rows = [&](void* dst, const f32x16_t (&acc)[DB], float mul) {
    if (!a_valid) return;
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
  auto store_results = [&](const f32x16_t (&a1)[DB], const f32x16_t (&a2)[DB], float scale1) {
    if constexpr (ROLE == kBwdDQ) store_rows(p.dq, a1, scale1);
    if constexpr (ROLE == kBwdDKV) store_rows(p.dk, a1, scale1);
    if constexpr (PAIR) {
      if (part) store_rows(p.dk, a2, scale1);  // a dS wave accumulates dK where a P wave accumulates dV
      else store_rows(p.dv, a2, scale1 == 0.f ? 0.f : 1.f);
    } else if constexpr (HAS_PV) {
      store_rows(p.dv, a2, scale1 == 0.f ? 0.f : 1.f);
    }
  };

  f32x16_t acc1[DB], acc2[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc1[db][r] = acc2[db][r] = 0.f;

  if (empty) {
    // padding rows, or rows nothing attends: their gradients are zero
    store_results(acc1, acc2, 0.f);
    return;
  }

  // stationary operand fragments: row r_in, elements 16*ks + 8*g .. +7
  // (paired role: K for the P waves, V for the dS waves)
  const T* x1 = reinterpret_cast<const T*>(KV_STATIONARY ? ((PAIR && part) ? p.v : p.k) : p.q) + a_row * a_stride +
                int64_t(head_a) * D + g * 8;
  const T* x2 = reinterpret_cast<const T*>(KV_STATIONARY ? p.v : p.d_out) + a_row * a_stride + int64_t(head_a) * D + g * 8;
  vec8 x1f[KSTEPS], x2f[HAS_DS ? KSTEPS : 1];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) {
    x1f[ks] = *reinterpret_cast<const vec8*>(x1 + ks * 16);
    if constexpr (!KV_STATIONARY) x1f[ks] = scale_query_fragment<T>(x1f[ks], p.scale * kLog2e);
    if constexpr (HAS_DS) x2f[ks] = *reinterpret_cast<const vec8*>(x2 + ks * 16);
  }

  // mask state of the lane
  int wst[3] = {0, 0, 0}, wen[3] = {0, 0, 0};  // dQ role: window of the lane's query
  uint32_t key_packed = 0;                     // other roles: in-tile coordinates of the lane's key
  float lse_l = 0.f, delta_l = 0.f;
  if constexpr (!KV_STATIONARY) {
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int c = a_crd[a];
      wst[a] = na_window_start(c, ksz[a], p.stride[a], extent[a], p.causal[a] != 0);
      wen[a] = na_window_end(c, wst[a], ksz[a], extent[a], p.causal[a] != 0);
    }
    const int64_t stat_idx = p.fused ? (int64_t(bg / p.num_groups) * p.heads_q + head_a) * p.tokens + a_tok
                                     : stat_row_q + head_a * stat_head_stride + int64_t(at) * AT + r_in;
    lse_l = p.lse[stat_idx] * kLog2e;
    delta_l = p.delta[stat_idx];
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
  const T* y1_all = reinterpret_cast<const T*>(KV_STATIONARY ? p.qs : p.k);
  const T* y2_all = reinterpret_cast<const T*>(KV_STATIONARY ? p.d_out : p.v);

  // row (permuted) or token offset (original layout) of position r (dimension 0 fastest) of a streamed tile
  auto sub_pos = [&](int r) {
    if (!p.fused) return r;
    const int t0 = r % b_sub[0];
    r /= b_sub[0];
    return t0 * tok_step[0] + (r % b_sub[1]) * tok_step[1] + (r / b_sub[1]) * tok_step[2];
  };
  // copy i of a thread moves chunk P = i * NT + tid of the tile (row P / CPR, LDS slot P % CPR)
  uint32_t off_u[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int P = i * NT + tid;
    const int row = P / CPR, slot = P % CPR;
    off_u[i] = uint32_t(sub_pos(row)) * uint32_t(b_stride * 2) + uint32_t(L::u_slot(row, slot) * 16);
  }

  struct Tile {
    int origin[3];  // coordinate of the tile's first token (a tile moved back from the group's edge: of the first one gathered)
    int lead[3];    // ... whose first lead[a] positions along dimension a belong to the tile before it
    int row0;       // its first row in the streamed side's permuted sequence
    int head_b;
  };
  // The streamed tiles in visiting order: dimension 2 fastest, dimension 0 slowest; the
  // key-stationary roles walk the box once per query head of the key head's group.  The box is
  // walked twice: first the tiles that need the element mask (the box minus the inner box of
  // whole tiles, see full_t0), then the whole ones (the inner box itself).
  const int total = box_n[0] * box_n[1] * box_n[2];
  const int n_whole = (full_t1[0] - full_t0[0]) * (full_t1[1] - full_t0[1]) * (full_t1[2] - full_t0[2]);
  const int head_b0 = KV_STATIONARY ? head_a * rep : head_a / rep;
  int wc[3], walk_head = 0;  // position of the walk in absolute tile coordinates
  // one step inside the box of the pass (WHOLE: the inner box, else the whole box)
  auto step = [&](auto whole_tag) {
    constexpr bool WHOLE = decltype(whole_tag)::value;
    auto lo = [&](int a) { return WHOLE ? full_t0[a] : box_tile0[a]; };
    auto hi = [&](int a) { return WHOLE ? full_t1[a] : box_tile0[a] + box_n[a]; };
    if (++wc[2] == hi(2)) {
      wc[2] = lo(2);
      if (++wc[1] == hi(1)) {
        wc[1] = lo(1);
        if (++wc[0] == hi(0)) {
          wc[0] = lo(0);
          ++walk_head;
        }
      }
    }
  };
  // masked pass: a position at the start of a run of whole tiles jumps to the run's end
  auto skip_whole = [&]() {
    while (n_whole > 0 && wc[2] == full_t0[2] && wc[1] >= full_t0[1] && wc[1] < full_t1[1] && wc[0] >= full_t0[0] &&
           wc[0] < full_t1[0]) {
      wc[2] = full_t1[2] - 1;
      step(std::false_type{});
    }
  };
  auto start_walk = [&](auto whole_tag) {
    constexpr bool WHOLE = decltype(whole_tag)::value;
#pragma unroll
    for (int a = 0; a < 3; ++a) wc[a] = WHOLE ? full_t0[a] : box_tile0[a];
    walk_head = 0;
    if constexpr (!WHOLE) skip_whole();
  };
  // descriptor of the current position, then on to the next one; `more` = tiles of this pass still
  // to come after this one (past the last one the position is never used)
  auto next_tile = [&](auto whole_tag, bool more) {
    constexpr bool WHOLE = decltype(whole_tag)::value;
    Tile t;
    int cc[3], half = 0;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      t.origin[a] = wc[a] * b_sub[a];
      t.lead[a] = 0;
      if (p.edge) {
        const int moved = na_min(t.origin[a], (KV_STATIONARY ? q_extent[a] : extent[a]) - b_sub[a]);
        t.lead[a] = t.origin[a] - moved;
        t.origin[a] = moved;
      }
      const bool split = (a == split_dim);
      half |= split ? (wc[a] & 1) : 0;
      cc[a] = split ? (wc[a] >> 1) : wc[a];
    }
    t.row0 = p.fused ? group_tok + t.origin[0] * tok_step[0] + t.origin[1] * tok_step[1] + t.origin[2] * tok_step[2]
                     : (cc[0] + b_tiled[0] * (cc[1] + b_tiled[1] * cc[2])) * AT + half * BT;
    t.head_b = KV_STATIONARY ? head_b0 + walk_head : head_b0;
    if (more) {
      step(whole_tag);
      if constexpr (!WHOLE) skip_whole();
    }
    return t;
  };

  // in-tile coordinates of streamed position `lane` (the window tables below are built by wave 0)
  int qo[3];
  qo[0] = lane % b_sub[0];
  qo[1] = (lane / b_sub[0]) % b_sub[1];
  qo[2] = lane / (b_sub[0] * b_sub[1]);

  const uint32_t lds_y1 = uint32_t(__builtin_amdgcn_readfirstlane(int(lds_address(sY1))));
  const uint32_t lds_y2 = uint32_t(__builtin_amdgcn_readfirstlane(int(lds_address(sY2))));
  const uint32_t stat_off = uint32_t(sub_pos(lane)) * 4u;  // byte offset of streamed row `lane` in lse / delta (head-major)
  // the window tables of a masked streamed tile (key-stationary roles, wave 0)
  auto build_tables = [&](const Tile& t, int stage, bool masked) {
    if constexpr (KV_STATIONARY) {
      if (wave == 0 && masked) {
        // per streamed query: its window relative to this workgroup's key tile
        uint32_t addc = 0, subc = 0;
        bool valid = true;
#pragma unroll
        for (int a = 0; a < 3; ++a) {
          const int qc = t.origin[a] + qo[a];
          valid = valid && (qc < q_extent[a]) && (qo[a] >= t.lead[a]);
          const int st = na_window_start(qc, ksz[a], p.stride[a], extent[a], p.causal[a] != 0);
          const int en = na_window_end(qc, st, ksz[a], extent[a], p.causal[a] != 0);
          const int lo = na_min(na_max(st - a_first[a], 0), a_tile[a]);
          const int hi = na_min(na_max(en - a_first[a], 0), a_tile[a]);
          addc |= uint32_t(512 - lo) << (10 * a);
          subc |= uint32_t(511 + hi) << (10 * a);
        }
        sTabA[stage * BT + lane] = valid ? addc : 0u;  // no guard bit survives a zero addend
        sTabB[stage * BT + lane] = valid ? subc : 0u;
      }
    }
  };
  // the asynchronous copies of a streamed tile (and of its LSE / delta values) into a stage
  auto issue_copies = [&](const Tile& t, int stage, int stage2) {
    const int64_t row = p.fused ? batch_row0 + t.row0 : seq_row_b + t.row0;
    if constexpr (KV_STATIONARY) {
      // LSE / delta of the tile's 64 queries: one asynchronous 4-byte-per-lane copy each
      // (wave 1, wave 2; the other waves but wave 0 make the same number of copies into a
      // spare row so that every wave counts the same number of outstanding copies per tile)
      const int64_t stat_row0 = p.fused ? (int64_t(bg / p.num_groups) * p.heads_q + t.head_b) * p.tokens + t.row0
                                        : stat_row_q + t.head_b * stat_head_stride + t.row0;
      const float* src = (wave == 2 ? p.delta : p.lse) + stat_row0;
      float* dst = (wave == 1) ? &sLse[stage * BT] : (wave == 2) ? &sDelta[stage * BT] : &sSpare[0];
      if (wave != 0) async_copy4_asm(src, stat_off, lds_address(dst));
    }
    const int64_t elem = row * b_stride + int64_t(t.head_b) * D;
    const uint64_t y1 = uniform64(y1_all + elem), y2 = uniform64(y2_all + elem);
    const uint32_t dst = uint32_t(__builtin_amdgcn_readfirstlane(stage * TILE_BYTES + wave * 1024));
    const uint32_t dst2 = uint32_t(__builtin_amdgcn_readfirstlane(stage2 * TILE_BYTES + wave * 1024));
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      async_copy16_uniform(y1, off_u[i], lds_y1 + dst + uint32_t(i * NT * 16));
      async_copy16_uniform(y2, off_u[i], lds_y2 + dst2 + uint32_t(i * NT * 16));
    }
  };
  auto issue = [&](const Tile& t, int stage, bool masked) {
    build_tables(t, stage, masked);
    issue_copies(t, stage, stage);
  };

  // lane-constant LDS read offsets (same fragment layouts as the forward kernel)
  int k_off[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) k_off[ks] = l32 * ROWB + L::u_slot(l32, ks * 2 + g) * 16;
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
    const s16x4_t lo = lds_read_tr16(s + r0 * ROWB + v_sub + L::u_slot(r0, c) * 16);
    const s16x4_t hi = lds_read_tr16(s + (r0 + 8) * ROWB + v_sub + L::u_slot(r0 + 8, c) * 16);
    return __builtin_bit_cast(vec8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  // One streamed tile: its two 32-row sub-blocks one after the other, each as products (S, dP),
  // probabilities, accumulations.  Only one sub-block's products are live at a time, which keeps
  // the kernel within 256 registers: two workgroups share a CU, and the other wave of a SIMD
  // fills the gaps of this one (a measured 1.2-1.3 x over interleaving the sub-blocks inside
  // one wave per SIMD).  The matrix instructions form one sequence of fenced "slots", each with
  // its operand fragment read from LDS a few slots ahead.
  constexpr int WP = HAS_DS ? 2 : 1;                       // products per k-step (S, dP)
  constexpr int W = (HAS_DS ? 1 : 0) + (HAS_PV ? 1 : 0);   // accumulators fed per transposed fragment position
  constexpr int NP = WP * KSTEPS;                          // product slots per sub-block
  constexpr int N1 = 2 * NP;
  constexpr int NC = 2 * DB * W;                           // accumulation slots per sub-block
  constexpr int G = N1 + 2 * NC;
  constexpr int PF = 2;                                    // fragments read ahead
  // P waves of the paired role: the products of both sub-blocks first, then the accumulations of
  // both, and the probabilities of a sub-block two per slot between the matrix instructions that
  // follow its products (sub-block 0: the products of sub-block 1; sub-block 1: the accumulations
  // of sub-block 0), so that the wave's vector work runs while the matrix pipe does.
  constexpr bool SPREAD = PAIR;
  static_assert(!SPREAD || (NP == 8 && NC == 8), "two of a sub-block's 16 probabilities per slot");
  auto tile_body = [&](auto masked_tag, int stage, int stage2, uint32_t addc, uint32_t subc, int exch, auto&& after_slot) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    (void)exch;  // paired role: which of the two probability buffers this tile writes
    const char* y1 = sY1 + stage * TILE_BYTES;
    const char* y2 = sY2 + stage2 * TILE_BYTES;  // (stage2 differs from stage in the paired role only)

    // slot x of the tile: a product slot (sub-block, index i < NP) or an accumulation slot (i < NC)
    struct Slot {
      bool prod;
      int sb, i;
    };
    auto slot_of = [](int x) constexpr {
      if constexpr (SPREAD) {
        const bool prod = x < 2 * NP;
        const int z = prod ? x : x - 2 * NP, n = prod ? NP : NC;
        return Slot{prod, z / n, z % n};
      } else {
        const int sb = x / (NP + NC), z = x % (NP + NC);
        return Slot{z < NP, sb, z < NP ? z : z - NP};
      }
    };
    auto frag = [&](auto x_tag) {
      constexpr Slot sl = slot_of(decltype(x_tag)::value);
      if constexpr (sl.prod) {
        constexpr int ks = sl.i / WP, which = sl.i % WP;
        return row_frag(which ? y2 : y1, sl.sb, ks);
      } else {
        constexpr int h = sl.i / (DB * W), db = (sl.i / W) % DB;
        constexpr bool to_acc1 = HAS_DS && (sl.i % W == 0);
        return tr_frag(to_acc1 ? y1 : y2, sl.sb, h, db);
      }
    };

    f32x16_t S[NSB], dP[NSB];
    vec8 pf[NSB][2], dsf[NSB][2];
    // tables of the streamed rows, four rows (8*jj + 4*g + i of a sub-block) at a time, read
    // when they are needed (the other wave covers the wait)
    u32x4_t ta, tb;
    f32x4_t ls4, dl4;
    auto load_group = [&](auto gi_tag) {
      constexpr int gi = decltype(gi_tag)::value;  // sub-block * 4 + jj
      if constexpr (gi < 2 * 4) {
        const int e0 = (gi / 4) * 32 + 8 * (gi % 4) + 4 * g;
        if constexpr (KV_STATIONARY) {
          if constexpr (MASKED) {
            ta = *reinterpret_cast<const u32x4_t*>(&sTabA[stage * BT + e0]);
            tb = *reinterpret_cast<const u32x4_t*>(&sTabB[stage * BT + e0]);
          }
          ls4 = *reinterpret_cast<const f32x4_t*>(&sLse[stage * BT + e0]) * kLog2e;
          if constexpr (HAS_DS) dl4 = *reinterpret_cast<const f32x4_t*>(&sDelta[stage * BT + e0]);
        } else if constexpr (MASKED) {
          ta = *reinterpret_cast<const u32x4_t*>(&sTabA[e0]);
        }
      }
    };
    float held_p = 0.f, held_ds = 0.f;
    uint32_t px[PAIR ? 8 : 1];  // paired role: the sub-block's probabilities as fp16 pairs
    auto elem = [&](auto sb_tag, auto r_tag) {
      constexpr int sb = decltype(sb_tag)::value, r = decltype(r_tag)::value;
      constexpr int i = r % 4;
      if constexpr (i == 0) load_group(std::integral_constant<int, sb * 4 + r / 4>{});
      float x;
      if constexpr (KV_STATIONARY) x = fast_exp2(S[sb][r] - ls4[i]);
      else x = fast_exp2(S[sb][r] - lse_l);
      if constexpr (MASKED) {
        uint32_t ok;
        if constexpr (KV_STATIONARY) ok = (key_packed + ta[i]) & (tb[i] - key_packed) & kGuardBits;
        else ok = (ta[i] + addc) & (subc - ta[i]) & kGuardBits;
        x = (ok == kGuardBits) ? x : 0.f;
      }
      float ds = 0.f;
      if constexpr (HAS_DS) {
        if constexpr (KV_STATIONARY) ds = x * (dP[sb][r] - dl4[i]);
        else ds = x * (dP[sb][r] - delta_l);
      }
      if constexpr (r % 2 == 0) {
        pin(x);
        held_p = x;
        if constexpr (HAS_DS) {
          pin(ds);
          held_ds = ds;
        }
      } else {
        if constexpr (PAIR) {
          const h16x2_t h2 = {static_cast<_Float16>(held_p), static_cast<_Float16>(x)};
          px[r / 2] = __builtin_bit_cast(uint32_t, h2);
          if constexpr (r == 15) {
            char* dst = sX + ((((exch * 4 + rw) * NSB + sb) * 2) * 64 + lane) * 16;
            *reinterpret_cast<u32x4_t*>(dst) = u32x4_t{px[0], px[1], px[2], px[3]};
            *reinterpret_cast<u32x4_t*>(dst + 64 * 16) = u32x4_t{px[4], px[5], px[6], px[7]};
          }
        }
        if constexpr (HAS_PV) {
          vec2 p2 = {static_cast<T>(held_p), static_cast<T>(x)};
          uint32_t pb = __builtin_bit_cast(uint32_t, p2);
          pin(pb);
          p2 = __builtin_bit_cast(vec2, pb);
          pf[sb][r / 8][r % 8 - 1] = p2[0];
          pf[sb][r / 8][r % 8] = p2[1];
        }
        if constexpr (HAS_DS) {
          vec2 d2 = {static_cast<T>(held_ds), static_cast<T>(ds)};
          uint32_t db_ = __builtin_bit_cast(uint32_t, d2);
          pin(db_);
          d2 = __builtin_bit_cast(vec2, db_);
          dsf[sb][r / 8][r % 8 - 1] = d2[0];
          dsf[sb][r / 8][r % 8] = d2[1];
        }
      }
    };

    vec8 fr[G];
    for_range<0, PF>([&](auto x_tag) { fr[decltype(x_tag)::value] = frag(x_tag); });
    for_range<0, G>([&](auto x_tag) __attribute__((always_inline)) {
      constexpr int x = decltype(x_tag)::value;
      constexpr Slot sl = slot_of(x);
      constexpr int sb = sl.sb;
      if constexpr (x + PF < G) fr[x + PF] = frag(std::integral_constant<int, x + PF>{});
      if constexpr (sl.prod) {
        constexpr int ks = sl.i / WP, which = sl.i % WP;
        f32x16_t zero;
#pragma unroll
        for (int r = 0; r < 16; ++r) zero[r] = 0.f;
        if constexpr (which == 0) S[sb] = M::run(fr[x], x1f[ks], ks == 0 ? zero : S[sb]);
        else dP[sb] = M::run(fr[x], x2f[ks], ks == 0 ? zero : dP[sb]);
        // all probabilities of the sub-block once its products are complete
        if constexpr (!SPREAD && sl.i == NP - 1) for_range<0, 16>([&](auto r_tag) { elem(std::integral_constant<int, sb>{}, r_tag); });
      } else {
        constexpr int h = sl.i / (DB * W), db = (sl.i / W) % DB;
        constexpr bool to_acc1 = HAS_DS && (sl.i % W == 0);
        if constexpr (to_acc1) acc1[db] = M::run(fr[x], dsf[sb][h], acc1[db]);
        else acc2[db] = M::run(fr[x], pf[sb][h], acc2[db]);
      }
      if constexpr (SPREAD && x >= NP && x < 2 * NP + NC) {
        // two probabilities per slot, between the matrix instructions of the other sub-block
        constexpr int esb = x < 2 * NP ? 0 : 1, r0 = 2 * (x < 2 * NP ? x - NP : x - 2 * NP);
        elem(std::integral_constant<int, esb>{}, std::integral_constant<int, r0>{});
        elem(std::integral_constant<int, esb>{}, std::integral_constant<int, r0 + 1>{});
      }
      after_slot(x_tag);
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // ---- paired role: the dS waves ----------------------------------------------------------------
  // produce: dP^T of the current tile, kept in registers until the next step;
  // consume: dS of the previous tile from its dP^T, its delta and the P waves' probabilities,
  // then dK += dS^T Q with that tile's Q (still in its stage).
  f32x16_t held_dp[NSB];
  auto pair_produce = [&](int stage) __attribute__((always_inline)) {
    const char* y2 = sY2 + stage * TILE_BYTES;
    constexpr int N = NSB * KSTEPS;
    vec8 fr[N];
    for_range<0, PF>([&](auto x_tag) {
      constexpr int x = decltype(x_tag)::value;
      fr[x] = row_frag(y2, x / KSTEPS, x % KSTEPS);
    });
    for_range<0, N>([&](auto x_tag) __attribute__((always_inline)) {
      constexpr int x = decltype(x_tag)::value;
      constexpr int sb = x / KSTEPS, ks = x % KSTEPS;
      if constexpr (x + PF < N) fr[x + PF] = row_frag(y2, (x + PF) / KSTEPS, (x + PF) % KSTEPS);
      f32x16_t zero;
#pragma unroll
      for (int r = 0; r < 16; ++r) zero[r] = 0.f;
      held_dp[sb] = M::run(fr[x], x1f[ks], ks == 0 ? zero : held_dp[sb]);
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  auto pair_consume = [&](int stage, int exch) __attribute__((always_inline)) {
    const char* y1 = sY1 + stage * TILE_BYTES;
    vec8 dsf[NSB][2];
    u32x4_t plo[NSB], phi[NSB];
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb) {
      const char* src = sX + ((((exch * 4 + rw) * NSB + sb) * 2) * 64 + lane) * 16;
      plo[sb] = *reinterpret_cast<const u32x4_t*>(src);
      phi[sb] = *reinterpret_cast<const u32x4_t*>(src + 64 * 16);
    }
    // dS values 4 jj + 2 i2 and + 1 of a sub-block (k = 2 jj + i2)
    f32x4_t dl4;
    auto ds_pair = [&](auto sb_tag, auto k_tag) {
      constexpr int sb = decltype(sb_tag)::value, k = decltype(k_tag)::value;
      constexpr int jj = k / 2, i2 = k % 2, r = 4 * jj + 2 * i2;
      if constexpr (i2 == 0) dl4 = *reinterpret_cast<const f32x4_t*>(&sDelta[stage * BT + sb * 32 + 8 * jj + 4 * g]);
      const uint32_t pw = (r < 8) ? plo[sb][r / 2] : phi[sb][r / 2 - 4];
      const h16x2_t h2 = __builtin_bit_cast(h16x2_t, pw);
      const float d0 = float(h2[0]) * (held_dp[sb][r] - dl4[2 * i2]);
      const float d1 = float(h2[1]) * (held_dp[sb][r + 1] - dl4[2 * i2 + 1]);
      vec2 d2 = {static_cast<T>(d0), static_cast<T>(d1)};
      dsf[sb][r / 8][r % 8] = d2[0];
      dsf[sb][r / 8][r % 8 + 1] = d2[1];
    };
    constexpr int NCB = 2 * DB;  // accumulation slots per sub-block
    constexpr int N = NSB * NCB;
    static_assert(!PAIR || NCB == 8, "one pair of dS values of sub-block 1 per accumulation slot of sub-block 0");
    vec8 fr[N];
    for_range<0, PF>([&](auto x_tag) {
      constexpr int x = decltype(x_tag)::value;
      fr[x] = tr_frag(y1, x / NCB, (x % NCB) / DB, x % DB);
    });
    for_range<0, 8>([&](auto k_tag) { ds_pair(std::integral_constant<int, 0>{}, k_tag); });
    __builtin_amdgcn_sched_barrier(0);
    for_range<0, N>([&](auto x_tag) __attribute__((always_inline)) {
      constexpr int x = decltype(x_tag)::value;
      constexpr int sb = x / NCB, h = (x % NCB) / DB, db = x % DB;
      if constexpr (x + PF < N) {
        constexpr int y = x + PF;
        fr[y] = tr_frag(y1, y / NCB, (y % NCB) / DB, y % DB);
      }
      acc2[db] = M::run(fr[x], dsf[sb][h], acc2[db]);
      if constexpr (PAIR && x < NCB) ds_pair(std::integral_constant<int, 1>{}, x_tag);
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  constexpr int CPT = 2 * PER;  // tile copies per thread and tile
  // One pass of the paired role over n_iter tiles: step `it` has the P waves on tile `it` and the
  // dS waves forming dP of tile `it` after finishing tile it - 1; one more step drains the dS
  // waves.  Tiles are copied two steps ahead: tile it + 2 during step `it`, into the Y2 stage of
  // tile it - 1 and the Y1 / table stage of tile it - 2, both last read in step it - 1.  The
  // barrier at the top of a step makes tile `it` and the probabilities of tile it - 1 visible and
  // separates those last reads from the copies that overwrite them.
  auto run_pass_pair = [&](auto masked_tag, auto ds_wave_tag, int n_iter) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    constexpr bool DS_WAVE = decltype(ds_wave_tag)::value;
    if (n_iter <= 0) return;
    start_walk(std::integral_constant<bool, !MASKED>{});
    Tile tn = next_tile(std::integral_constant<bool, !MASKED>{}, 1 < n_iter);
    issue(tn, 0, MASKED && !DS_WAVE);  // wave 0, which builds the window tables, is a P wave
    if (1 < n_iter) {
      tn = next_tile(std::integral_constant<bool, !MASKED>{}, 2 < n_iter);
      issue(tn, 1, MASKED && !DS_WAVE);
    }
    // A wave walks to tile it + 2 and issues its share of the copies where it has vector or
    // scalar work anyway: the dS waves between their two matrix phases, the P waves after the
    // products of their first sub-block; the eight waves then do not queue on the CU's address
    // path together while the matrix pipe idles.
    int s2 = 0;  // it % 3
    for (int it = 0; it <= n_iter; ++it) {
      // this thread's copies of tile `it` have landed once only those of tile it + 1 are
      // outstanding (wave 0 makes one copy less per tile)
      if (it + 1 < n_iter) {
        if (wave != 0) wait_vmcnt<CPT + 1>();
        else wait_vmcnt<CPT>();
      } else {
        wait_vmcnt<0>();
      }
      workgroup_sync();
      const int s2_ahead = s2 == 0 ? 2 : s2 - 1;  // (it + 2) % 3
      auto ahead = [&]() __attribute__((always_inline)) {
        if (it + 2 < n_iter) {
          tn = next_tile(std::integral_constant<bool, !MASKED>{}, it + 3 < n_iter);
          build_tables(tn, (it + 2) & 3, MASKED && !DS_WAVE);
          issue_copies(tn, (it + 2) & 3, s2_ahead);
        }
      };
      if constexpr (DS_WAVE) {
        if (it > 0) pair_consume((it - 1) & 3, (it - 1) & 1);
        ahead();
        if (it < n_iter) pair_produce(s2);
      } else {
        if (it < n_iter) {
          tile_body(masked_tag, it & 3, s2, 0u, 0u, it & 1, [&](auto x_tag) __attribute__((always_inline)) {
            if constexpr (decltype(x_tag)::value == NP - 1) ahead();
          });
        }
      }
      s2 = s2 == 2 ? 0 : s2 + 1;
    }
    wait_vmcnt<0>();
    workgroup_sync();  // stages and probability buffers are free for the next pass
  };

  // ---- pipeline: tile `it` is multiplied while tiles it+1 .. it+NS-1 are in flight ----------------
  // Descriptor queue: d[0] = tile `it`, d[k] = tile it + k.
  auto run_pass = [&](auto masked_tag, int n_iter) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    if (n_iter <= 0) return;
    start_walk(std::integral_constant<bool, !MASKED>{});
    // dQ role, masked pass: origins of the tiles in flight (the lane's mask constants need the
    // origin of the tile being multiplied); og<k> = origin of tile it + k
    constexpr bool NEED_ORIGIN = MASKED && !KV_STATIONARY;
    int og0[3] = {0, 0, 0}, og1[3] = {0, 0, 0}, og2[3] = {0, 0, 0};
    int ld0[3] = {0, 0, 0}, ld1[3] = {0, 0, 0}, ld2[3] = {0, 0, 0};  // ... and their leads
    if (0 < n_iter && NS > 1) {
      const Tile t = next_tile(std::integral_constant<bool, !MASKED>{}, 1 < n_iter);
      issue(t, 0, MASKED);
      if constexpr (NEED_ORIGIN) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
          og0[a] = t.origin[a];
          ld0[a] = t.lead[a];
        }
      }
    }
    if (1 < n_iter && NS > 2) {
      const Tile t = next_tile(std::integral_constant<bool, !MASKED>{}, 2 < n_iter);
      issue(t, 1, MASKED);
      if constexpr (NEED_ORIGIN) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
          og1[a] = t.origin[a];
          ld1[a] = t.lead[a];
        }
      }
    }

    for (int it = 0; it < n_iter; ++it) {
      const int stage = it % NS;
      // this thread's copies of tile `it` have landed once at most those of the later tiles in
      // flight (one tile with three stages, none with two) are outstanding; wave 0 makes one
      // copy less per tile in the key-stationary roles
      if (NS == 3 && it + 1 < n_iter) {
        if (KV_STATIONARY && wave != 0) wait_vmcnt<CPT + 1>();
        else wait_vmcnt<CPT>();
      } else {
        wait_vmcnt<0>();
      }
      workgroup_sync();  // tile `it` and its tables are in LDS; everyone is done with the stage of tile it - 1
      if (it + NS - 1 < n_iter) {
        const Tile t = next_tile(std::integral_constant<bool, !MASKED>{}, it + NS < n_iter);
        issue(t, (it + NS - 1) % NS, MASKED);
        if constexpr (NEED_ORIGIN) {
#pragma unroll
          for (int a = 0; a < 3; ++a) {
            (NS == 3 ? og2[a] : og1[a]) = t.origin[a];
            (NS == 3 ? ld2[a] : ld1[a]) = t.lead[a];
          }
        }
      }

      uint32_t addc = 0, subc = 0;
      if constexpr (NEED_ORIGIN) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
          const int lo = na_min(na_max(wst[a] - og0[a], ld0[a]), b_sub[a]);
          const int hi = na_min(na_max(wen[a] - og0[a], 0), b_sub[a]);
          addc |= uint32_t(512 - lo) << (10 * a);
          subc |= uint32_t(511 + hi) << (10 * a);
        }
      }
      tile_body(masked_tag, stage, stage, addc, subc, 0, [](auto) {});
      if constexpr (NEED_ORIGIN) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
          og0[a] = og1[a];
          og1[a] = og2[a];
          ld0[a] = ld1[a];
          ld1[a] = ld2[a];
        }
      }
    }
    wait_vmcnt<0>();
    workgroup_sync();  // the stages are free for the next pass
  };
  const int heads_walked = KV_STATIONARY ? rep : 1;
  if constexpr (PAIR) {
    // the two kinds of wave run separate copies of the passes (the same barriers in both), so
    // that neither carries the other's registers
    if (part == 0) {
      run_pass_pair(std::true_type{}, std::false_type{}, (total - n_whole) * heads_walked);
      run_pass_pair(std::false_type{}, std::false_type{}, n_whole * heads_walked);
    } else {
      run_pass_pair(std::true_type{}, std::true_type{}, (total - n_whole) * heads_walked);
      run_pass_pair(std::false_type{}, std::true_type{}, n_whole * heads_walked);
    }
  } else {
    run_pass(std::true_type{}, (total - n_whole) * heads_walked);
    run_pass(std::false_type{}, n_whole * heads_walked);
  }

  // dQ = scale * sum_k dS k;  dK = scale * sum_q dS q = ln 2 * sum_q dS q'
  store_results(acc1, acc2, KV_STATIONARY ? 0.6931471805599453f : p.scale);
}

// qs = round(q * scale * log2(e)) for `chunks` runs of 8 elements: the logit operand of the
// key-stationary roles (see scale_query_fragment).
template <typename T>
__global__ void __launch_bounds__(256) scale_queries_kernel(const T* q, T* qs, int64_t chunks, float c_log2) {
  using vec8 = typename Mma<T>::vec8;
  const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (i < chunks)
    *reinterpret_cast<vec8*>(qs + i * 8) = scale_query_fragment<T>(*reinterpret_cast<const vec8*>(q + i * 8), c_log2);
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
