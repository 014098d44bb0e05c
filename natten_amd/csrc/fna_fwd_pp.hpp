// Fused neighborhood attention forward for gfx950 (MI355X), two-group "ping-pong" schedule.
//
// One workgroup = 8 waves = two groups of 4 waves.  Each group owns one 128-row Q tile of the
// same (batch*dilation-group, head) and its own double-buffered LDS ring of K/V tiles filled by
// asynchronous global->LDS loads.  Wave i of group 0 and wave i of group 1 share a SIMD; the
// loop body is cut into four phases separated by workgroup barriers,
//     P0: S^T = K Q^T            (matrix cores)
//     P1: softmax, issue V load  (vector units)
//     P2: O^T += V^T P^T         (matrix cores)
//     P3: issue K load, tile bookkeeping
// and group 1 runs one phase behind group 0, so that on every SIMD one wave is in a matrix
// phase while the other is in a vector / memory phase.
//
// Arithmetic, masking, tile box and softmax convention are those of fna_fwd.hpp (same
// reference citations); only the schedule differs.
#pragma once

#include "fna_fwd.hpp"

namespace natten_amd {

template <int D, int KVT>
struct FnaPpSmem {
  using L = FnaSmem<D, KVT>;
  static constexpr int BYTES = 2 * 2 * 2 * L::TILE_BYTES + KVT * 4;  // groups x stages x {K, V}
};

template <typename T, int D, int KVT>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
fna_fwd_pp_kernel(const FnaParams p) {
  constexpr int NTG = 256;  // threads per group
  constexpr int QT = 128;   // query rows per group
  constexpr int MQ = 1;
  constexpr int KSTEPS = D / 16;
  constexpr int DB = D / 32;
  constexpr int NSB = KVT / 32;
  using L = FnaSmem<D, KVT>;
  constexpr int ROWB = L::ROWB;
  constexpr int CPR = L::CPR;
  constexpr int TILE_BYTES = L::TILE_BYTES;
  constexpr int CHUNKS = KVT * CPR;
  constexpr int PER = (CHUNKS + NTG - 1) / NTG;
  static_assert(CHUNKS % NTG == 0, "every wave of a group issues the same number of copies");
  using M = Mma<T>;
  using vec8 = typename M::vec8;
  using vec2 = typename M::vec2;

  // [group][stage] K and V tiles: one LDS object each, so that the compiler can tell the fill of
  // one stage from the operand reads of another (no conservative wait on loads in flight)
  __shared__ __attribute__((aligned(1024))) char sK00[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sK01[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sV00[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sV01[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sK10[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sK11[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sV10[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sV11[TILE_BYTES];
  __shared__ __attribute__((aligned(16))) uint32_t sTab[KVT];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int group = __builtin_amdgcn_readfirstlane(tid >> 8);
  const int wave = __builtin_amdgcn_readfirstlane((tid >> 6) & 3);  // wave inside its group
  const int gtid = tid & 255;
  const int l32 = lane & 31;
  const int g = lane >> 5;

  // ---- workgroup id -> (batch*group, head, pair of Q tiles) -----------------------------------
  int bg, head, pair_rm;
  {
    const int pid = blockIdx.x;
    const int xcd = pid % kNumXcd;
    const int local = pid / kNumXcd;
    const int grp = (local / p.wg_group) * kNumXcd + xcd;
    const int within = local % p.wg_group;
    if (grp >= p.total_groups) return;
    const int bh = grp / p.groups_per_bh;
    pair_rm = (grp % p.groups_per_bh) * p.wg_group + within;
    if (pair_rm * 2 >= p.num_q_tiles) return;
    bg = bh / p.heads_q;
    head = bh % p.heads_q;
  }
  const int head_kv = head / (p.heads_q / p.heads_kv);

  // in-tile coordinates of every KV position, packed in 10-bit fields (shared by both groups)
  for (int i = tid; i < KVT; i += 512) {
    int r = i;
    const int t0 = r % p.kv_tile[0];
    r /= p.kv_tile[0];
    const int t1 = r % p.kv_tile[1];
    r /= p.kv_tile[1];
    sTab[i] = uint32_t(t0) | (uint32_t(t1) << 10) | (uint32_t(r) << 20);
  }

  // dilation group extents
  int extent[3];
  {
    int gl = bg % p.num_groups;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int gi = gl % p.dil[a];
      gl /= p.dil[a];
      extent[a] = na_group_extent(p.qkv_shape[a], p.dil[a], gi);
    }
  }

  // Q tile `qt_rm` (dimension 0 slowest, causal dimension 0 walked from the far end):
  // coordinates, KV tile box and the window intersection used for the per-tile "full" test
  struct QTileBox {
    int q_first[3], tile0[3], n[3], full_lo[3], full_hi[3];
    int qtile_idx, total;
  };
  auto make_box = [&](int qt_rm) {
    QTileBox b;
    if (qt_rm >= p.num_q_tiles) {
#pragma unroll
      for (int a = 0; a < 3; ++a) b.q_first[a] = b.tile0[a] = b.n[a] = b.full_lo[a] = b.full_hi[a] = 0;
      b.qtile_idx = 0;
      b.total = 0;
      return b;
    }
    int tc[3];
    int t = qt_rm;
    tc[2] = t % p.q_tiled[2];
    t /= p.q_tiled[2];
    tc[1] = t % p.q_tiled[1];
    tc[0] = t / p.q_tiled[1];
    if (p.causal[0]) tc[0] = p.q_tiled[0] - 1 - tc[0];
    b.qtile_idx = tc[0] + p.q_tiled[0] * (tc[1] + p.q_tiled[1] * tc[2]);
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      b.q_first[a] = tc[a] * p.q_tile[a];
      const int qf = b.q_first[a], ql = qf + p.q_tile[a] - 1;
      const bool c = p.causal[a] != 0;
      const int st_f = na_window_start(qf, p.ksize[a], p.stride[a], extent[a], c);
      const int en_f = na_window_end(qf, st_f, p.ksize[a], extent[a], c);
      const int st_l = na_window_start(ql, p.ksize[a], p.stride[a], extent[a], c);
      const int en_l = na_window_end(ql, st_l, p.ksize[a], extent[a], c);
      b.tile0[a] = st_f / p.kv_tile[a];
      b.n[a] = na_ceil_div(en_l, p.kv_tile[a]) - b.tile0[a];
      b.full_lo[a] = st_l;
      b.full_hi[a] = en_f;
    }
    b.total = b.n[0] * b.n[1] * b.n[2];
    return b;
  };
  const QTileBox box = make_box(pair_rm * 2 + group);
  const int other_total = make_box(pair_rm * 2 + (group ^ 1)).total;
  const int total_tiles = box.total;
  const int n_iter = na_max(total_tiles, other_total);  // both groups walk the same number of barriers
  const int qtile_idx = box.qtile_idx;

  const int64_t q_row_stride = int64_t(p.heads_q) * D;
  const int64_t kv_row_stride = int64_t(p.heads_kv) * D;
  const T* qbase = reinterpret_cast<const T*>(p.q) + int64_t(bg) * p.seqlen_q * q_row_stride + int64_t(head) * D;
  const T* kbase = reinterpret_cast<const T*>(p.k) + int64_t(bg) * p.seqlen_kv * kv_row_stride + int64_t(head_kv) * D;
  const T* vbase = reinterpret_cast<const T*>(p.v) + int64_t(bg) * p.seqlen_kv * kv_row_stride + int64_t(head_kv) * D;

  // ---- async tile loads: uniform per-tile base + thread-constant byte offset ------------------
  int ld_row[PER];
  uint32_t ld_koff[PER], ld_voff[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int P = i * NTG + gtid;
    ld_row[i] = P / CPR;
    const int slot = P % CPR;
    ld_koff[i] = uint32_t(ld_row[i]) * uint32_t(kv_row_stride * 2) + uint32_t(L::k_slot(ld_row[i], slot) * 16);
    ld_voff[i] = uint32_t(ld_row[i]) * uint32_t(kv_row_stride * 2) + uint32_t(L::v_slot(ld_row[i], slot) * 16);
  }
  auto issue_tile_load = [&](const T* base, const uint32_t (&off)[PER], char* dst, int kv_row0) {
    const char* tile_base = reinterpret_cast<const char*>(base) + int64_t(kv_row0) * kv_row_stride * 2;
    if (kv_row0 + KVT <= p.seqlen_kv) {
#pragma unroll
      for (int i = 0; i < PER; ++i) async_copy16(tile_base + off[i], dst + (i * NTG + wave * 64) * 16);
    } else {
      // last, partial tile of an unpadded sequence: rows past the end are masked; read the last
      // valid row instead so that no out-of-bounds address is formed
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int grow = na_min(kv_row0 + ld_row[i], p.seqlen_kv - 1);
        const uint32_t in_row = off[i] - uint32_t(ld_row[i]) * uint32_t(kv_row_stride * 2);
        async_copy16(reinterpret_cast<const char*>(base) + int64_t(grow) * kv_row_stride * 2 + in_row,
                     dst + (i * NTG + wave * 64) * 16);
      }
    }
  };

  // KV tile stream of this group's box: dimension 2 fastest, dimension 0 slowest
  struct TileInfo {
    int row0;
    int origin[3];
    bool full;
  };
  int itc[3] = {0, 0, 0};
  auto next_tile = [&]() {
    TileInfo t;
    t.full = true;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      t.origin[a] = (box.tile0[a] + itc[a]) * p.kv_tile[a];
      t.full = t.full && (t.origin[a] >= box.full_lo[a]) && (t.origin[a] + p.kv_tile[a] <= box.full_hi[a]);
    }
    t.row0 = ((box.tile0[0] + itc[0]) + p.kv_tiled[0] * ((box.tile0[1] + itc[1]) + p.kv_tiled[1] * (box.tile0[2] + itc[2]))) * KVT;
    if (++itc[2] == box.n[2]) {
      itc[2] = 0;
      if (++itc[1] == box.n[1]) {
        itc[1] = 0;
        ++itc[0];
      }
    }
    return t;
  };

  // ---- per-lane setup: query row, its window, Q fragments -------------------------------------
  int wst[3], wen[3];
  vec8 qf[KSTEPS];
  {
    int r = wave * 32 + l32;
    const int row = qtile_idx * QT + r;
    int off[3];
    off[0] = r % p.q_tile[0];
    r /= p.q_tile[0];
    off[1] = r % p.q_tile[1];
    off[2] = r / p.q_tile[1];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int c = box.q_first[a] + off[a];
      wst[a] = na_window_start(c, p.ksize[a], p.stride[a], extent[a], p.causal[a] != 0);
      wen[a] = na_window_end(c, wst[a], p.ksize[a], extent[a], p.causal[a] != 0);
    }
    const int row_c = na_min(row, p.seqlen_q - 1);
    const T* qrow = qbase + int64_t(row_c) * q_row_stride + g * 8;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) qf[ks] = *reinterpret_cast<const vec8*>(qrow + ks * 16);
  }

  f32x16_t acc[DB];
  float m_run = -INFINITY, l_run = 0.f;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;
  const float c_log2 = p.scale * 1.4426950408889634f;

  // lane-constant LDS read offsets (see fna_fwd.hpp)
  int k_off[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) k_off[ks] = l32 * ROWB + L::k_slot(l32, ks * 2 + g) * 16;
  const int l16 = lane & 15;
  const int v_e = l16 >> 2, v_j4 = l16 & 3;
  const int v_row = 4 * g + v_e;
  const int v_chunk = (l32 >> 4) * 2 + (v_j4 >> 1);
  const int v_sub = (v_j4 & 1) * 8;

  using Tag0 = std::integral_constant<int, 0>;
  using Tag1 = std::integral_constant<int, 1>;

  auto run = [&](auto group_tag) {
    constexpr int G = decltype(group_tag)::value;
    char* const sK_st0 = G ? sK10 : sK00;
    char* const sK_st1 = G ? sK11 : sK01;
    char* const sV_st0 = G ? sV10 : sV00;
    char* const sV_st1 = G ? sV11 : sV01;

    // prologue: K(0), V(0), K(1) in flight (in this order: the waits below count on it)
    TileInfo cur = next_tile();
    TileInfo nxt = next_tile();
    if (total_tiles > 0) {
      issue_tile_load(kbase, ld_koff, sK_st0, cur.row0);
      issue_tile_load(vbase, ld_voff, sV_st0, cur.row0);
    }
    if (total_tiles > 1) issue_tile_load(kbase, ld_koff, sK_st1, nxt.row0);
    if (total_tiles > 1) wait_vmcnt<2 * PER>(); else wait_vmcnt<0>();  // K(0) has landed (this thread's part)
    if (G == 1) __builtin_amdgcn_s_barrier();  // group 1 runs one phase behind group 0

    f32x16_t S[NSB];
    vec8 pf[NSB][2];
#ifdef NA_X_TIMING
    unsigned long long tacc[10] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    unsigned long long tlast = __builtin_amdgcn_s_memtime();
#define NA_TICK(k) { unsigned long long tn = __builtin_amdgcn_s_memtime(); tacc[k] += tn - tlast; tlast = tn; }
#else
#define NA_TICK(k)
#endif

    auto iteration = [&](auto stage_tag, int j) {
      constexpr int st = decltype(stage_tag)::value;
      char* const sK_cur = st ? sK_st1 : sK_st0;  // K(j); refilled with K(j+2) in P3
      char* const sV_cur = st ? sV_st1 : sV_st0;  // V(j)
      char* const sV_nxt = st ? sV_st0 : sV_st1;  // receives V(j+1) in P1
#ifdef NA_X_ONEGROUP
      const bool active = (j < total_tiles) && (G == 0);
#else
      const bool active = j < total_tiles;
#endif
      const bool has1 = j + 1 < total_tiles;
      const bool has2 = j + 2 < total_tiles;

      // ---- P0: S^T = K(j) Q^T --------------------------------------------------------------
      NA_TICK(8)
      __builtin_amdgcn_s_barrier();
      NA_TICK(0)
#ifdef NA_X_NOQK
      if (active) { for (int sb = 0; sb < NSB; ++sb) for (int r = 0; r < 16; ++r) S[sb][r] = float(j + r); if (has1) wait_vmcnt<PER>(); else wait_vmcnt<0>(); }
      if (false) {
#else
      if (active) {
#endif
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb) {
#pragma unroll
          for (int r = 0; r < 16; ++r) S[sb][r] = 0.f;
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks) {
            const vec8 kf = *reinterpret_cast<const vec8*>(sK_cur + sb * 32 * ROWB + k_off[ks]);
            S[sb] = M::run(kf, qf[ks], S[sb]);
          }
        }
        // keep PD operand reads in flight ahead of the matrix instructions that consume them
        {
          constexpr int NR = NSB * KSTEPS;
          constexpr int PD = NR < 6 ? NR : 6;
          __builtin_amdgcn_sched_group_barrier(0x100, PD, 0);
#pragma unroll
          for (int i = 0; i < NR - PD; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          }
          __builtin_amdgcn_sched_group_barrier(0x008, PD, 0);
        }
        NA_TICK(1)
        // V(j) must have landed before anyone starts P2; K(j+1) may stay in flight
        if (has1) wait_vmcnt<PER>(); else wait_vmcnt<0>();
      }
      NA_TICK(2)

      // ---- P1: softmax of S(j); V(j+1) goes in flight ------------------------------------------
      __builtin_amdgcn_s_barrier();
      NA_TICK(3)
      if (active) {
#ifndef NA_X_NOLOAD
        if (has1) issue_tile_load(vbase, ld_voff, sV_nxt, nxt.row0);
#endif
#ifdef NA_X_NOSOFTMAX
        for (int sb = 0; sb < NSB; ++sb) for (int h = 0; h < 2; ++h) for (int i = 0; i < 8; ++i) pf[sb][h][i] = static_cast<T>(S[sb][8 * h + i]);
      }
      if (false) {
#endif
        if (!cur.full) {
          uint32_t addc = 0, subc = 0;
#pragma unroll
          for (int a = 0; a < 3; ++a) {
            const int lo = na_min(na_max(wst[a] - cur.origin[a], 0), p.kv_tile[a]);
            const int hi = na_min(na_max(wen[a] - cur.origin[a], 0), p.kv_tile[a]);
            addc |= uint32_t(512 - lo) << (10 * a);
            subc |= uint32_t(511 + hi) << (10 * a);
          }
#pragma unroll
          for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
              const u32x4_t tc4 = *reinterpret_cast<const u32x4_t*>(&sTab[sb * 32 + 8 * jj + 4 * g]);
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                const uint32_t tp = tc4[i];
                const uint32_t ok = (tp + addc) & (subc - tp) & kGuardBits;
                S[sb][4 * jj + i] = (ok == kGuardBits) ? S[sb][4 * jj + i] : -INFINITY;
              }
            }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
          for (int r = 0; r < 16; ++r) mx = fmaxf(mx, S[sb][r]);
        mx = cross_half_max(mx);
        const bool grow = (mx - m_run) * c_log2 > kLazyRescaleLog2;
        if (__any(grow)) {
          const float m_new = fmaxf(m_run, mx);
          const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
          const float alpha = fast_exp2((m_run - m_use) * c_log2);
          m_run = m_new;
          l_run *= alpha;
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[db][r] *= alpha;
        }
        const float msc = ((m_run == -INFINITY) ? 0.f : m_run) * c_log2;
        float psum = 0.f;
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            vec8 pv;
#pragma unroll
            for (int i = 0; i < 8; i += 2) {
              vec2 p2;
              p2[0] = static_cast<T>(fast_exp2(S[sb][8 * h + i] * c_log2 - msc));
              p2[1] = static_cast<T>(fast_exp2(S[sb][8 * h + i + 1] * c_log2 - msc));
              psum = M::add2(p2, psum);
              pv[i] = p2[0];
              pv[i + 1] = p2[1];
            }
            pf[sb][h] = pv;
          }
        l_run += psum;
      }

      // ---- P2: O^T += V(j)^T P^T ----------------------------------------------------------------
      NA_TICK(4)
      __builtin_amdgcn_s_barrier();
      NA_TICK(5)
#ifdef NA_X_NOPV
      if (active) { acc[0][0] += float(pf[0][0][0]); if (has1) wait_vmcnt<PER>(); }
      if (false) {
#else
      if (active) {
#endif
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const int r0 = sb * 32 + h * 16 + v_row;
            const char* row_lo = sV_cur + r0 * ROWB + v_sub;
            const char* row_hi = sV_cur + (r0 + 8) * ROWB + v_sub;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
              const int c = db * 4 + v_chunk;
              const s16x4_t lo = lds_read_tr16(row_lo + L::v_slot(r0, c) * 16);
              const s16x4_t hi = lds_read_tr16(row_hi + L::v_slot(r0 + 8, c) * 16);
              const s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
              acc[db] = M::run(__builtin_bit_cast(vec8, both), pf[sb][h], acc[db]);
            }
          }
        {
          constexpr int NM = NSB * 2 * DB;  // matrix instructions, two transpose reads each
          constexpr int PD = NM < 4 ? NM : 4;
          __builtin_amdgcn_sched_group_barrier(0x100, 2 * PD, 0);
#pragma unroll
          for (int i = 0; i < NM - PD; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
          }
          __builtin_amdgcn_sched_group_barrier(0x008, PD, 0);
        }
        // K(j+1) must have landed before anyone starts the next P0; V(j+1) may stay in flight
        if (has1) wait_vmcnt<PER>();
      }

      // ---- P3: K(j+2) goes in flight; next tile descriptor --------------------------------------
      NA_TICK(6)
      __builtin_amdgcn_s_barrier();
      NA_TICK(7)
      const TileInfo t2 = next_tile();
#ifndef NA_X_NOLOAD
      if (has2) issue_tile_load(kbase, ld_koff, sK_cur, t2.row0);
#endif
      cur = nxt;
      nxt = t2;
    };

    for (int j = 0; j < n_iter; j += 2) {
      iteration(Tag0{}, j);
      if (j + 1 < n_iter) iteration(Tag1{}, j + 1);
    }
    if (G == 0) __builtin_amdgcn_s_barrier();  // pairs with group 1's extra barrier at the start
#ifdef NA_X_TIMING
    if ((blockIdx.x == 4000 || blockIdx.x == 9001) && lane == 0)
      printf("blk %d grp %d wave %d tiles %d | barA %llu P0 %llu waitV %llu barB %llu P1 %llu barC %llu P2+wait %llu barD %llu P3 %llu\n", blockIdx.x, G, wave, total_tiles,
             tacc[0] / total_tiles, tacc[1] / total_tiles, tacc[2] / total_tiles, tacc[3] / total_tiles, tacc[4] / total_tiles, tacc[5] / total_tiles, tacc[6] / total_tiles, tacc[7] / total_tiles, tacc[8] / total_tiles);
#endif
  };
  if (group == 0) run(Tag0{}); else run(Tag1{});

  // ---- epilogue: O = acc / rowsum, LSE = ln(rowsum) + scale * rowmax -------------------------
  if (total_tiles == 0) return;  // this group had no Q tile (odd tile count)
  T* obase = reinterpret_cast<T*>(p.o) + int64_t(bg) * p.seqlen_q * q_row_stride + int64_t(head) * D;
  const float l = l_run + __shfl_xor(l_run, 32);
  const float inv = (l > 0.f) ? p.out_scale / l : 0.f;
  const int row = qtile_idx * QT + wave * 32 + l32;
  if (row < p.seqlen_q) {
    T* orow = obase + int64_t(row) * q_row_stride;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        typedef T tx4 __attribute__((ext_vector_type(4)));
        tx4 o4;
#pragma unroll
        for (int i = 0; i < 4; ++i) o4[i] = static_cast<T>(acc[db][4 * j + i] * inv);
        *reinterpret_cast<tx4*>(orow + db * 32 + 8 * j + 4 * g) = o4;
      }
    if (g == 0) {
      const float lse = (l > 0.f) ? (m_run * p.scale + __logf(l)) : -INFINITY;
      p.lse[(int64_t(bg) * p.seqlen_q + row) * p.heads_q + head] = lse;
    }
  }
}

}  // namespace natten_amd
