// Fused neighborhood attention forward for 8-bit float operands (OCP e4m3 / e5m2) on gfx950:
// S^T = K Q^T and O^T = V^T P^T on v_mfma_f32_32x32x64_f8f6f4 (twice the rate of the 16-bit
// instruction), P rounded to e4m3, output bf16.  Same tile walk, masks, lazy rescale, operand
// layouts (token-permuted or original) and workgroup layout as fna_fwd_kernel (fna_fwd.hpp); what
// differs is spelled out below.  Semantics follow the reference's 8-bit forward
// (SHI-Labs/NATTEN csrc/include/natten/cuda/fna_blackwell/collective/
// sm100_fna_fwd_mainloop_tma_warpspecialized.hpp:618-861: probabilities cast to the operand
// type before P V), with two differences that only improve accuracy: P is always e4m3 (also for
// e5m2 operands), and it is scaled by 2^6 before rounding so that small probabilities of long
// rows stay in e4m3's normal range (the scale cancels in O = acc / rowsum).
#pragma once

#include "fna_fwd.hpp"

namespace natten_amd {

typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x8_t __attribute__((ext_vector_type(8)));
typedef int i32x2_t __attribute__((ext_vector_type(2)));

// LDS transpose read of bytes: the 16 lanes of a group each point at 8 consecutive bytes of a
// row (lane 2e+j -> row e, columns 8j..8j+7 of an 8 x 16 block); lane c of the group receives
// column c of the block (rows 0..7).
static __device__ __forceinline__ i32x2_t lds_read_tr8(const char* p) {
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wold-style-cast"
  return __builtin_amdgcn_ds_read_tr8_b64_v2i32((NA_LDS i32x2_t*)(p));
#pragma clang diagnostic pop
}

constexpr float kFp8ProbLog2Scale = 6.0f;   // P is stored as 2^6 * exp(...)
constexpr float kFp8LazyRescaleLog2 = 2.0f; // so that 2^6 * 2^2 = 256 stays below e4m3's 448

// One 32-row query block per wave, 64-key tiles, two waves per SIMD.  D = 64 or 128.
// LDS tile: 64 rows of D bytes, 16-byte chunks XOR-swizzled by (row / rows-per-256-bytes); the
// rows of a V tile are stored in the order the P fragment holds its keys (see v_key_of_lds_row).
// `pid`: the launch position (the workgroup id of a launch with one workgroup per Q tile).
// NOMASK: fully block-sparse launch (see fna_fwd_tile): no mask code, tables or per-wave windows.
template <bool E5M2, int D, int NWAVES, bool NOMASK = false, typename Hook>
static __device__ __forceinline__ void fna_fwd_fp8_tile(const FnaParams& p, const uint32_t pid, Hook&& before_stores) {
  constexpr int KVT = 64;
  constexpr int NT = NWAVES * 64;
  constexpr int QT = NWAVES * 32;
  constexpr int KSTEPS = D / 64;  // MFMAs per 32 x 32 block of logits
  constexpr int DB = D / 32;
  constexpr int NSB = KVT / 32;
  constexpr int ROWB = D;         // bytes per row
  constexpr int CPR = D / 16;     // 16-byte chunks per row
  constexpr int RPL = 256 / ROWB; // rows per 256 bytes
  constexpr int TILE_BYTES = KVT * ROWB;
  constexpr int CHUNKS = KVT * CPR;
  constexpr int PER = CHUNKS / NT;  // async copies per thread per operand per tile
  static_assert(D == 64 || D == 128, "head dims 64 and 128");
  static_assert(PER >= 1 && PER <= 4 && CHUNKS % NT == 0, "tile must split evenly over the waves");
  constexpr int FMT_IN = E5M2 ? 1 : 0;  // operand format code of the MFMA: 0 = e4m3, 1 = e5m2
  auto slot_of = [](int r, int c) { return c ^ ((r / RPL) % CPR); };
  // LDS row rho of a V tile holds key 32*sb + 8*a + 4*g + b with rho = 32*g + 16*sb + 4*a + b: the
  // half-wave g of the P fragment owns exactly the keys of LDS rows 32*g .. 32*g + 31, in order.
  auto v_key_of_lds_row = [](int rho) { return 32 * ((rho >> 4) & 1) + 8 * ((rho >> 2) & 3) + 4 * (rho >> 5) + (rho & 3); };

  __shared__ __attribute__((aligned(1024))) char sK0[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sV0[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sK1[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sV1[TILE_BYTES];
  __shared__ __attribute__((aligned(16))) uint32_t sTab[NOMASK ? 1 : KVT];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction
  const int l32 = lane & 31;
  const int g = lane >> 5;

  // ---- workgroup id -> (batch*group, head, Q tile); groups of Q tiles are dealt to XCDs ------
  int bg, head, qtile_rm;
  {
    // (divisions by launch constants are multiply-shift pairs and shifts, as in fna_fwd_kernel)
    const int xcd = int(pid % kNumXcd);
    const int local = int(pid / kNumXcd);
    const int run = na_div(local, p.d_wg_group);
    const int group = run * kNumXcd + xcd;
    const int within = local - run * p.wg_group;
    if (group >= p.total_groups) return;
    const int bh = na_div(group, p.d_groups_per_bh);
    qtile_rm = (group - bh * p.groups_per_bh) * p.wg_group + within;
    if (qtile_rm >= p.num_q_tiles) return;
    bg = na_div(bh, p.d_heads_q);
    head = bh - bg * p.heads_q;
  }
  const int head_kv = na_div(head, p.d_q_per_kv);
  const int b_orig = na_div(bg, p.d_num_groups);  // batch entry before the dilation groups were folded in

  // ---- workgroup-uniform setup: dilation group, Q tile origin, KV tile box -------------------
  // qtile_rm enumerates Q tiles with dimension 0 slowest; causal dimension 0 is walked from
  // the far end so that the Q tiles with the longest KV loops start first.
  int extent[3], q_first[3], box_org[3], box_n[3];  // box_org: coordinate of the box's first KV tile
  int qtile_idx;  // position of the tile in the permuted sequence (dimension 0 fastest)
  int tok_step[3];  // fused layout: tokens per unit step of a coordinate inside a dilation group
  int group_tok = 0;  // fused layout: token of the dilation group's first element
  {
    int gl = bg - b_orig * p.num_groups;
    int tc[3];
    const int t01 = na_div(qtile_rm, p.d_q_tiled[2]);
    tc[2] = qtile_rm - t01 * p.q_tiled[2];
    tc[0] = na_div(t01, p.d_q_tiled[1]);
    tc[1] = t01 - tc[0] * p.q_tiled[1];
    if (p.causal[0]) tc[0] = p.q_tiled[0] - 1 - tc[0];
    qtile_idx = tc[0] + p.q_tiled[0] * (tc[1] + p.q_tiled[1] * tc[2]);
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int rest = na_div(gl, p.d_dil[a]);
      const int gi = gl - rest * p.dil[a];
      gl = rest;
      extent[a] = p.ext_base[a] + (gi < p.ext_rem[a] ? 1 : 0);  // dilation group gi: one more token while gi < X % d
      tok_step[a] = p.dil[a] * p.tok_stride[a];
      group_tok += gi * p.tok_stride[a];
      q_first[a] = tc[a] << p.q_tile_lg[a];
      const int qf = q_first[a], ql = qf + p.q_tile[a] - 1;
      const bool c = p.causal[a] != 0;
      const int st_f = na_window_start(qf, p.ksize[a], p.stride[a], p.d_stride[a], extent[a], c);
      const int st_l = na_window_start(ql, p.ksize[a], p.stride[a], p.d_stride[a], extent[a], c);
      const int en_l = na_window_end(ql, st_l, p.ksize[a], extent[a], c);
      // original layout: tiles may be laid out from the window's first key (see FnaParams::anchor)
      box_org[a] = p.anchor ? st_f : ((st_f >> p.kv_tile_lg[a]) << p.kv_tile_lg[a]);
      box_n[a] = (en_l - box_org[a] + p.kv_tile[a] - 1) >> p.kv_tile_lg[a];
    }
  }
  const int total_tiles = box_n[0] * box_n[1] * box_n[2];

  // ---- this wave's share of the Q tile ------------------------------------------------------------
  // Lanes take the tile's tokens in row-major order (dimension 0 slowest), 32 consecutive
  // ones per wave, so that a wave covers a compact box of queries; the token's row inside the
  // permuted tile (dimension 0 fastest) follows from its coordinates.  Window starts and ends
  // are monotone in the query coordinate, hence over the wave's bounding box the union of the
  // windows is [start(min), end(max)) and their intersection [start(max), end(min)) per
  // dimension: a KV tile outside the union is skipped by this wave, one inside the
  // intersection needs no mask.
  int wave_lo[3], wave_hi[3], wave_full_lo[3], wave_full_hi[3];
  if constexpr (!NOMASK) {
    const int i0 = wave * 32, i1 = i0 + 31;
    const int lg2 = p.q_tile_lg[2], lg12 = p.q_tile_lg[1] + p.q_tile_lg[2];
    int f[3], l[3];
    f[0] = i0 >> lg12;
    f[1] = (i0 >> lg2) & (p.q_tile[1] - 1);
    f[2] = i0 & (p.q_tile[2] - 1);
    l[0] = i1 >> lg12;
    l[1] = (i1 >> lg2) & (p.q_tile[1] - 1);
    l[2] = i1 & (p.q_tile[2] - 1);
    if (f[0] != l[0]) {
      f[1] = 0;
      l[1] = p.q_tile[1] - 1;
    }
    if (f[0] != l[0] || f[1] != l[1]) {
      f[2] = 0;
      l[2] = p.q_tile[2] - 1;
    }
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      // rows past the end of an unpadded sequence (dense attention) are clamped like the loads
      const int qmin = q_first[a] + f[a], qmax = q_first[a] + na_min(l[a], p.q_tile[a] - 1);
      const bool c = p.causal[a] != 0;
      const int st_min = na_window_start(qmin, p.ksize[a], p.stride[a], p.d_stride[a], extent[a], c);
      const int en_min = na_window_end(qmin, st_min, p.ksize[a], extent[a], c);
      const int st_max = na_window_start(qmax, p.ksize[a], p.stride[a], p.d_stride[a], extent[a], c);
      const int en_max = na_window_end(qmax, st_max, p.ksize[a], extent[a], c);
      wave_lo[a] = st_min;
      wave_hi[a] = en_max;
      wave_full_lo[a] = st_max;
      wave_full_hi[a] = en_min;
    }
  }

  // in-tile coordinates of every KV position, packed in 10-bit fields
  for (int i = tid; i < (NOMASK ? 0 : KVT); i += NT) {
    const int t0 = i & (p.kv_tile[0] - 1);
    const int r1 = i >> p.kv_tile_lg[0];
    const int t1 = r1 & (p.kv_tile[1] - 1);
    sTab[i] = uint32_t(t0) | (uint32_t(t1) << 10) | (uint32_t(r1 >> p.kv_tile_lg[1]) << 20);
  }

  const int64_t q_row_stride = int64_t(p.heads_q) * D;
  const int64_t kv_row_stride = int64_t(p.heads_kv) * D;
  // (row strides are in bytes: one byte per element)
  // first row of this (batch, dilation group): rows are then addressed by permuted row index
  // (permuted layout) or by token offset inside the group (fused layout)
  const int64_t q_row_base = p.fused ? int64_t(b_orig) * p.tokens + group_tok : int64_t(bg) * p.seqlen_q;
  const int64_t kv_row_base = p.fused ? int64_t(b_orig) * p.tokens + group_tok : int64_t(bg) * p.seqlen_kv;
  const uint8_t* qbase = static_cast<const uint8_t*>(p.q) + q_row_base * q_row_stride + int64_t(head) * D;
  const uint8_t* kbase = static_cast<const uint8_t*>(p.k) + kv_row_base * kv_row_stride + int64_t(head_kv) * D;
  const uint8_t* vbase = static_cast<const uint8_t*>(p.v) + kv_row_base * kv_row_stride + int64_t(head_kv) * D;
  // row (permuted) or token offset (fused) of position `r` (dimension 0 fastest) of a KV tile
  auto kv_tile_pos = [&](int r) {
    if (!p.fused) return r;
    const int t0 = r & (p.kv_tile[0] - 1);
    r >>= p.kv_tile_lg[0];
    return t0 * tok_step[0] + (r & (p.kv_tile[1] - 1)) * tok_step[1] + (r >> p.kv_tile_lg[1]) * tok_step[2];
  };


  // ---- async tile loads (see fna_fwd_kernel): copy i of wave w fills LDS chunks (w*PER + i)*64 .. +63
  constexpr int kImmBias = 3 * 1024;
  uint32_t ld_koff[PER], ld_voff[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int P = (wave * PER + i) * 64 + lane;
    const int row = P / CPR, slot = P % CPR;
    const int chunk = slot_of(row, slot);  // XOR swizzles are involutions
    ld_koff[i] = uint32_t(kv_tile_pos(row)) * uint32_t(kv_row_stride) + uint32_t(chunk * 16 + kImmBias - i * 1024);
    ld_voff[i] = uint32_t(kv_tile_pos(v_key_of_lds_row(row))) * uint32_t(kv_row_stride) + uint32_t(chunk * 16 + kImmBias - i * 1024);
  }
  struct TileCopy {
    const char* src;
    uint32_t lds0;
  };
  auto make_copy = [&](const uint8_t* base, char* dst, int kv_row0) {
    TileCopy c;
    kv_row0 = __builtin_amdgcn_readfirstlane(kv_row0);
    c.src = reinterpret_cast<const char*>(base) + int64_t(kv_row0) * kv_row_stride - kImmBias;
    c.lds0 = lds_address(dst) + uint32_t(wave * PER * 1024);
    return c;
  };
  auto copy_one = [&](auto i_tag, const TileCopy& c, const uint32_t (&off)[PER]) {
    constexpr int I = decltype(i_tag)::value;
    if constexpr (I < PER) async_copy16_asm<I * 1024>(c.src, off[I], c.lds0);
  };
  auto issue_tile_load = [&](const uint8_t* base, const uint32_t (&off)[PER], char* dst, int kv_row0) {
    const TileCopy c = make_copy(base, dst, kv_row0);
    copy_one(std::integral_constant<int, 0>{}, c, off);
    copy_one(std::integral_constant<int, 1>{}, c, off);
    copy_one(std::integral_constant<int, 2>{}, c, off);
    copy_one(std::integral_constant<int, 3>{}, c, off);
  };

  // KV tile stream: dimension 2 fastest, dimension 0 slowest.  The load stream runs up to two
  // tiles ahead of the softmax, so tile descriptors are produced in order and handed down.
  struct TileInfo {
    int row0;       // first row of the tile in the permuted KV sequence / token offset of its origin (fused)
    int origin[3];  // coordinate of its first token
    bool full;      // every key of the tile is attended by every query of this wave
    bool skip;      // no key of the tile is attended by any query of this wave
  };
  int itc[3] = {0, 0, 0};
  auto next_tile = [&]() {
    TileInfo t;
    t.full = true;
    t.skip = false;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int org = box_org[a] + (itc[a] << p.kv_tile_lg[a]);
      const int end = org + p.kv_tile[a];
      if constexpr (!NOMASK) {
        t.full = t.full && (org >= wave_full_lo[a]) && (end <= wave_full_hi[a]);  // never when end > extent
        t.skip = t.skip || (end <= wave_lo[a]) || (org >= wave_hi[a]);
      }
      // a tile that would reach past the group is moved back to end at the group's last position
      t.origin[a] = (p.edge == 1 || p.anchor) ? na_min(org, extent[a] - p.kv_tile[a]) : org;
    }
    t.row0 = p.fused ? t.origin[0] * tok_step[0] + t.origin[1] * tok_step[1] + t.origin[2] * tok_step[2]
                     : (((box_org[0] >> p.kv_tile_lg[0]) + itc[0]) +
                        p.kv_tiled[0] * (((box_org[1] >> p.kv_tile_lg[1]) + itc[1]) +
                                         p.kv_tiled[1] * ((box_org[2] >> p.kv_tile_lg[2]) + itc[2]))) * KVT;
    if (++itc[2] == box_n[2]) {
      itc[2] = 0;
      if (++itc[1] == box_n[1]) {
        itc[1] = 0;
        ++itc[0];
      }
    }
    return t;
  };

  using Stage0 = std::integral_constant<int, 0>;
  using Stage1 = std::integral_constant<int, 1>;
  TileInfo cur = next_tile();  // tile 0
  issue_tile_load(kbase, ld_koff, sK0, cur.row0);
  issue_tile_load(vbase, ld_voff, sV0, cur.row0);


  // ---- per-lane setup: this lane's query row, its window, Q fragments ------------------------
  int wst[3], wen[3];
  int q_row;  // row of the permuted sequence / token offset in the group (fused), or -1 for padding
  i32x8_t qf[KSTEPS];
  {
    int r = wave * 32 + l32;  // row-major index inside the tile
    int off[3];
    off[2] = r & (p.q_tile[2] - 1);
    r >>= p.q_tile_lg[2];
    off[1] = r & (p.q_tile[1] - 1);
    off[0] = r >> p.q_tile_lg[1];
    int row = qtile_idx * QT + off[0] + p.q_tile[0] * (off[1] + p.q_tile[1] * off[2]);
    bool valid = row < p.seqlen_q;
    int row_c = na_min(row, p.seqlen_q - 1);
    if (p.fused) {
      row = 0;
      row_c = 0;
      valid = true;
    }
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int c = q_first[a] + off[a];
      if constexpr (!NOMASK) {
        wst[a] = na_window_start(c, p.ksize[a], p.stride[a], p.d_stride[a], extent[a], p.causal[a] != 0);
        wen[a] = na_window_end(c, wst[a], p.ksize[a], extent[a], p.causal[a] != 0);
      }
      if (p.fused) {
        valid = valid && (c < extent[a]);
        row += c * tok_step[a];
        row_c += na_min(c, extent[a] - 1) * tok_step[a];
      }
    }
    q_row = valid ? row : -1;
    // B operand of S^T = K Q^T: lane (query l32, half g) holds head-dim bytes 64*ks + 32*g .. +31
    const uint8_t* qrow = qbase + int64_t(row_c) * q_row_stride + g * 32;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const i32x4_t lo = *reinterpret_cast<const i32x4_t*>(qrow + ks * 64);
      const i32x4_t hi = *reinterpret_cast<const i32x4_t*>(qrow + ks * 64 + 16);
      qf[ks] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
  }

  f32x16_t acc[DB];
  float m_run = -INFINITY, l_run = 0.f;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;
  float sm_scale = p.scale, out_scale = 1.f;
  if (p.q_scale) sm_scale *= p.q_scale[head];
  if (p.k_scale) sm_scale *= p.k_scale[head_kv];
  if (p.v_scale) out_scale = p.v_scale[head_kv];
  const float c_log2 = sm_scale * 1.4426950408889634f;

  // ---- building blocks ---------------------------------------------------------------------------
  // A operand of S^T: lane (key row l32 of sub-block sb, half g) holds head-dim bytes
  // 64*ks + 32*g .. +31 of its key: two 16-byte LDS reads.  Both operands use the same byte ->
  // k-index map, which is all the instruction needs.
  auto k_frag = [&](const char* sK, int s) {  // slot s: sub-block s / KSTEPS, k-step s % KSTEPS
    const int row = (s / KSTEPS) * 32 + l32, c0 = (s % KSTEPS) * 4 + 2 * g;
    const i32x4_t lo = *reinterpret_cast<const i32x4_t*>(sK + row * ROWB + slot_of(row, c0) * 16);
    const i32x4_t hi = *reinterpret_cast<const i32x4_t*>(sK + row * ROWB + slot_of(row, c0 + 1) * 16);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  // A operand of O^T += V^T P^T for the 32 columns of block db: lane (column l32, half g) needs
  // its column of LDS rows 32*g .. 32*g + 31: four transpose reads of 8 rows x 16 columns.
  const int l16 = lane & 15;
  auto v_frag = [&](const char* sV, int db) {
    i32x8_t out;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int row = 32 * g + 8 * m + (l16 >> 1);
      const int chunk = 2 * db + (l32 >> 4);
      const i32x2_t t = lds_read_tr8(sV + row * ROWB + slot_of(row, chunk) * 16 + 8 * (l16 & 1));
      out[2 * m] = t[0];
      out[2 * m + 1] = t[1];
    }
    return out;
  };

  f32x16_t S_a[NSB], S_b[NSB];
  uint32_t pfw[8];    // P fragment: byte 16*sb + r of the lane = its probability for logit (sb, r)
  float msc = 0.f;    // running maximum in the exp2 domain minus the probability scale
  // Row sums are taken from the unrounded probabilities (in float): summing the rounded ones
  // with one more MFMA was measured to be no faster and costs two digits of the LSE.
  float psum[2];
  float held[3];

  // probability of logit v (sub-block v / 16, register v % 16) of the current tile
  auto exp_elem = [&](const f32x16_t (&S_cur)[NSB], int v) {
    const int sb = v / 16, r = v % 16;
    float x = fast_exp2(S_cur[sb][r] * c_log2 - msc);
    psum[r & 1] += x;
    pin(x);
    if (r % 4 == 1) {
      pfw[4 * sb + r / 4] = uint32_t(__builtin_amdgcn_cvt_pk_fp8_f32(held[0], x, 0, false));
      pin(pfw[4 * sb + r / 4]);
    } else if (r % 4 == 3) {
      pfw[4 * sb + r / 4] = uint32_t(__builtin_amdgcn_cvt_pk_fp8_f32(held[2], x, int(pfw[4 * sb + r / 4]), true));
      pin(pfw[4 * sb + r / 4]);
    } else {
      held[r % 4] = x;
    }
  };

  auto apply_mask = [&](f32x16_t (&S)[NSB], const int (&origin)[3]) {
    if constexpr (NOMASK) return;
    uint32_t addc = 0, subc = 0;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      // a tile moved back from the group's edge starts before its place in the tiling: the keys up
      // to there belong to the tile before it
      const int from_box = origin[a] - box_org[a];
      const int lead = (((from_box + p.kv_tile[a] - 1) >> p.kv_tile_lg[a]) << p.kv_tile_lg[a]) - from_box;
      const int lo = na_min(na_max(wst[a] - origin[a], lead), p.kv_tile[a]);
      const int hi = na_min(na_max(wen[a] - origin[a], 0), p.kv_tile[a]);
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
  };
  auto update_max = [&](float mx) {
    mx = cross_half_max(mx);
    const bool grow = (mx - m_run) * c_log2 > kFp8LazyRescaleLog2;
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
    msc = ((m_run == -INFINITY) ? 0.f : m_run) * c_log2 - kFp8ProbLog2Scale;
  };
  auto finish_logits = [&](f32x16_t (&S)[NSB], const bool t_full, const bool t_skip, const int (&t_origin)[3],
                           bool have_max, float mx) {
    if (t_skip) {
      mx = -INFINITY;
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) S[sb][r] = -INFINITY;
    } else if (!t_full || !have_max) {
      if (!t_full) apply_mask(S, t_origin);
      mx = -INFINITY;
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, S[sb][r]);
    }
    update_max(mx);
  };
  auto mfma8 = [&](i32x8_t a, i32x8_t b, f32x16_t c, auto fmt_a, auto fmt_b) {
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, decltype(fmt_a)::value, decltype(fmt_b)::value, 0, 0, 0, 0);
  };
  using FmtIn = std::integral_constant<int, FMT_IN>;
  using FmtP = std::integral_constant<int, 0>;

  // ---- software pipeline (as in fna_fwd_kernel): iteration j = slots of S(j+1) = K(j+1) Q^T,
  // carrying the exponentials of S(j) and the tile copies, then slots of O += P(j) V(j),
  // carrying the row maximum of S(j+1).  The matrix instruction is twice as fast here and the
  // vector work per key the same, so the vector units set the pace.
  constexpr int N_QK = NSB * KSTEPS;
  constexpr int N_PV = DB;
  constexpr int N_ELEMS = NSB * 16;
  TileInfo nxt = next_tile();
  wait_vmcnt<0>();
  workgroup_sync();
  if (1 < total_tiles) issue_tile_load(kbase, ld_koff, sK1, nxt.row0);
  msc = -kFp8ProbLog2Scale;
  {
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
      for (int r = 0; r < 16; ++r) S_a[sb][r] = 0.f;
#pragma unroll
    for (int s = 0; s < N_QK; ++s)
      S_a[s / KSTEPS] = mfma8(k_frag(sK0, s), qf[s % KSTEPS], S_a[s / KSTEPS], FmtIn{}, FmtIn{});
    finish_logits(S_a, cur.full, cur.skip, cur.origin, false, 0.f);
  }

  auto iteration = [&](auto stage_tag, int j) __attribute__((always_inline)) {
    constexpr int st = decltype(stage_tag)::value;
    f32x16_t (&S_cur)[NSB] = st ? S_b : S_a;
    f32x16_t (&S_nxt)[NSB] = st ? S_a : S_b;
    char* sK_cur = st ? sK1 : sK0;
    char* sK_nxt = st ? sK0 : sK1;
    char* sV_cur = st ? sV1 : sV0;
    char* sV_nxt = st ? sV0 : sV1;

    wait_vmcnt<0>();
    workgroup_sync();
    const TileInfo t2 = next_tile();
    const TileCopy ck = make_copy(kbase, sK_cur, (j + 2 < total_tiles) ? t2.row0 : cur.row0);
    const TileCopy cv = make_copy(vbase, sV_nxt, (j + 1 < total_tiles) ? nxt.row0 : cur.row0);

    i32x8_t kf[N_QK];
    kf[0] = k_frag(sK_nxt, 0);
    psum[0] = psum[1] = 0.f;
    auto g1_slot = [&](auto s_tag) __attribute__((always_inline)) {
      constexpr int s = decltype(s_tag)::value;
      if constexpr (s + 1 < N_QK) kf[s + 1] = k_frag(sK_nxt, s + 1);
      if constexpr (s % KSTEPS == 0) {
        f32x16_t zero;
#pragma unroll
        for (int r = 0; r < 16; ++r) zero[r] = 0.f;
        S_nxt[s / KSTEPS] = mfma8(kf[s], qf[s % KSTEPS], zero, FmtIn{}, FmtIn{});
      } else {
        S_nxt[s / KSTEPS] = mfma8(kf[s], qf[s % KSTEPS], S_nxt[s / KSTEPS], FmtIn{}, FmtIn{});
      }
      constexpr int e_lo = (s * N_ELEMS) / N_QK, e_hi = ((s + 1) * N_ELEMS) / N_QK;
#pragma unroll
      for (int e = e_lo; e < e_hi; ++e) exp_elem(S_cur, e);
      pin(psum[0]);
      pin(psum[1]);
      // 2 * PER copies over the slots, K first
      constexpr int c_lo = (s * 2 * PER) / N_QK, c_hi = ((s + 1) * 2 * PER) / N_QK;
      for_range<c_lo, c_hi - c_lo>([&](auto c_tag) {
        constexpr int c = decltype(c_tag)::value;
        if constexpr (c < PER) copy_one(std::integral_constant<int, c>{}, ck, ld_koff);
        else copy_one(std::integral_constant<int, c - PER>{}, cv, ld_voff);
      });
      __builtin_amdgcn_sched_barrier(0);
    };
    __builtin_amdgcn_s_setprio(1);  // as in the 16-bit kernel: the QK slots run at raised wave priority
    for_range<0, N_QK>(g1_slot);
    __builtin_amdgcn_s_setprio(0);

    i32x8_t pf;
#pragma unroll
    for (int i = 0; i < 8; ++i) pf[i] = int(pfw[i]);
    i32x8_t vf[N_PV];
    vf[0] = v_frag(sV_cur, 0);
    float mx0 = -INFINITY, mx1 = -INFINITY;
    auto pv_slot = [&](auto t_tag) __attribute__((always_inline)) {
      constexpr int t = decltype(t_tag)::value;
      if constexpr (t + 1 < N_PV) vf[t + 1] = v_frag(sV_cur, t + 1);
      acc[t] = mfma8(vf[t], pf, acc[t], FmtIn{}, FmtP{});
      constexpr int NV = NSB * 16;
      constexpr int e_lo = (t * NV) / N_PV, e_hi = ((t + 1) * NV) / N_PV;
      static_assert((e_hi - e_lo) % 4 == 0, "row maxima are taken two logits per instruction, on two chains");
#pragma unroll
      for (int e = e_lo; e < e_hi; e += 4) {
        mx0 = fmaxf(fmaxf(mx0, S_nxt[e / 16][e % 16]), S_nxt[(e + 1) / 16][(e + 1) % 16]);
        mx1 = fmaxf(fmaxf(mx1, S_nxt[(e + 2) / 16][(e + 2) % 16]), S_nxt[(e + 3) / 16][(e + 3) % 16]);
      }
      pin(mx0);
      pin(mx1);
      __builtin_amdgcn_sched_barrier(0);
    };
    for_range<0, N_PV>(pv_slot);
    l_run += psum[0] + psum[1];

    if (j + 1 < total_tiles) finish_logits(S_nxt, nxt.full, nxt.skip, nxt.origin, true, fmaxf(mx0, mx1));
    cur = nxt;
    nxt = t2;
  };
  for (int j = 0; j < total_tiles; j += 2) {
    iteration(Stage0{}, j);
    if (j + 1 < total_tiles) iteration(Stage1{}, j + 1);
  }
  wait_vmcnt<0>();  // copies into the unused stage must land before the LDS is released
  before_stores();  // (see fna_fwd_tile)

  // ---- epilogue: O = acc / rowsum (bf16), LSE = ln(rowsum) + scale * rowmax - ln(2^6) ----------
  __bf16* obase = reinterpret_cast<__bf16*>(p.o) + q_row_base * q_row_stride + int64_t(head) * D;
  {
    const float l = l_run + __shfl_xor(l_run, 32);
    const float inv = (l > 0.f) ? out_scale / l : 0.f;
    const int row = q_row;
    if (row >= 0) {
      __bf16* orow = obase + int64_t(row) * q_row_stride;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          typedef __bf16 bx4 __attribute__((ext_vector_type(4)));
          bx4 o4;
#pragma unroll
          for (int i = 0; i < 4; ++i) o4[i] = static_cast<__bf16>(acc[db][4 * j + i] * inv);
          *reinterpret_cast<bx4*>(orow + db * 32 + 8 * j + 4 * g) = o4;
        }
      if (g == 0) {
        const float lse = (l > 0.f) ? (m_run * sm_scale + __logf(l) - kFp8ProbLog2Scale * 0.6931471805599453f) : -INFINITY;
        p.lse[(q_row_base + row) * p.heads_q + head] = lse;
      }
    }
  }
}

template <bool E5M2, int D, int NWAVES, bool NOMASK = false>
__global__ void __launch_bounds__(NWAVES * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
fna_fwd_fp8_kernel(const FnaParams p) {
  fna_fwd_fp8_tile<E5M2, D, NWAVES, NOMASK>(p, blockIdx.x, []() {});
}

// Work-queue form (see fna_fwd_queue_kernel).
template <bool E5M2, int D, int NWAVES, bool NOMASK = false>
__global__ void __launch_bounds__(NWAVES * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
fna_fwd_fp8_queue_kernel(const FnaParams p, uint32_t* __restrict__ queues, const int per_xcd) {
  FnaKernargPtr args = fna_kernarg_params();
  fna_queue_loop(queues, per_xcd, [&](int pid, auto& fetch) __attribute__((always_inline)) {
    fna_fwd_fp8_tile<E5M2, D, NWAVES, NOMASK>(fna_params_for_this_tile(args), uint32_t(pid), fetch);
  });
  (void)p;
}

}  // namespace natten_amd
