// Fused neighborhood attention forward for gfx950 (MI355X).
//
// One workgroup = one Q tile of one (batch*dilation-group, head).  K/V tiles stream through a
// double-buffered LDS ring filled by asynchronous global->LDS loads; S^T = K Q^T and
// O^T = V^T P^T run on 32x32x16 MFMA so that every lane owns exactly one query row: row max
// and row sum are per-lane scalars plus one exchange between the two half-waves.  The softmax
// keeps a stale row maximum and rescales the accumulators only when a row's maximum grew by
// more than 2^8 (exact: the final normalisation uses the same maximum).
//
// The structure it restates (not the code): SHI-Labs/NATTEN
//   csrc/include/natten/cuda/fna_blackwell/collective/fna_fusion.hpp:315-347 (KV tile box per Q tile)
//   csrc/include/natten/cuda/fna_blackwell/collective/fna_fusion.hpp:384-436 (element mask)
//   csrc/include/natten/cuda/fna_blackwell/collective/sm100_fna_fwd_mainloop_tma_warpspecialized.hpp:618-861,
//   :1314-1327 (online softmax in the exp2 domain, O / rowsum, LSE = ln(rowsum) + scale * rowmax)
// Differences by design: KV tiles of the box are visited with dimension 0 slowest (the
// reference visits dimension 0 fastest) and workgroups are laid out so that the Q tiles
// resident on one XCD share their KV tiles in that XCD's L2; every (Q tile, KV tile) pair is
// classified per tile (fully inside all windows -> no mask) instead of once per launch.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include <type_traits>
#include <utility>

#include "na_math.hpp"
#include "work_queue.hpp"

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
  int num_q_tiles;              // q_tiled[0] * q_tiled[1] * q_tiled[2]
  // workgroup layout: consecutive `wg_group` Q tiles (dimension 0 slowest) of one (batch, head)
  // form a group; groups are dealt round-robin to the 8 XCDs
  int wg_group, groups_per_bh, total_groups;
  float scale;  // softmax scale
  // optional per-head dequantisation scales (device arrays or null): logits are multiplied by
  // q_scale[head] * k_scale[head_kv], the output by v_scale[head_kv]
  const float* q_scale;  // [heads_q]
  const float* k_scale;  // [heads_kv]
  const float* v_scale;  // [heads_kv]
  // Operand layout.  fused == 0: q, k, v, o, lse are token-permuted sequences
  // [batch * groups, seqlen, heads, D] (tile rows contiguous).  fused == 1: they are the
  // original tensors [batch, X0, X1, X2, heads, D]; the kernel gathers the rows of a tile itself
  // (every dilation group's extent must be a multiple of the KV tile in each dimension, so
  // that no KV tile reaches past the input).
  int fused;
  // fused == 1 only: some KV tile would reach past a dilation group's extent (extents that are
  // not multiples of dilation x KV tile).  1: every group is at least one KV tile wide in every
  // dimension; such a tile is then gathered from where it ends at the group's last position, and its
  // leading keys (which the tile before it already delivered) are masked.  2: the RAGGED instance,
  // which gathers the tile where it is and clamps the rows that fall outside the group.
  int edge;
  // fused == 1 only: KV tiles are laid out from the first key of the Q tile's window box (per
  // dimension) instead of from multiples of the tile extent, which saves the part of a tile that
  // would lie before the window; a tile that then reaches past the group is moved back as under
  // edge == 1 (every dilation group must be at least one KV tile wide in every dimension).
  int anchor;
  int tok_stride[3];  // tokens per unit step of an original coordinate: X1*X2, X2, 1
  int tokens;         // X0 * X1 * X2
  // Sequence-packed dense attention (RAGGED instances only; null otherwise): `batch` sequences
  // lie back to back in one row range, sequence b owns query rows cu_q[b] .. cu_q[b+1]-1 and
  // key rows cu_kv[b] .. cu_kv[b+1]-1; q_tiled[0] then counts the Q tiles of the longest one.
  const int32_t* cu_q;   // [batch + 1]
  const int32_t* cu_kv;  // [batch + 1]
  int total_q, total_kv;  // rows of the packed operands: offsets that do not fit them are not followed
  // Derived by set_wg_layout(): what the per-workgroup set-up would otherwise divide for.
  // Tile extents are powers of two (log2 below); the other divisors get multiply-shift pairs.
  int q_tile_lg[3], kv_tile_lg[3];
  // log2 extents of the box of 32 queries that a wave's lanes hold (sum 5, each <= q_tile_lg): the Q
  // tile is a grid of such boxes, one per wave and row block.  Chosen per launch (choose_wave_box) so
  // that as many (wave, KV tile) pairs as possible need no element mask.
  int wave_box_lg[3];
  int ext_base[3], ext_rem[3];  // qkv_shape / dil and qkv_shape % dil: extent of dilation group g = base + (g < rem)
  NaDiv d_stride[3], d_dil[3], d_q_tiled[3];
  NaDiv d_wg_group, d_groups_per_bh, d_heads_q, d_q_per_kv, d_num_groups;
  // Split launches only (fna_fwd_split_kernel; 0 otherwise): the KV tiles of every Q tile are dealt
  // to `kv_splits` workgroups in contiguous runs; workgroup `pid` of the grid works on Q-tile
  // position pid % split_grid for split pid / split_grid and stores its partial result (normalised
  // over its own keys, with their LSE) `split` strides into o and lse.
  int kv_splits, split_grid;
  int64_t o_split_stride, lse_split_stride;  // elements of the output type / floats
};

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

#define NA_LDS __attribute__((address_space(3)))
#define NA_GLOBAL __attribute__((address_space(1)))

// Timing-only builds.  NATTEN_AMD_ABLATE (0 in the shipped library) is a mask of parts of the tile
// loop to leave out, to time what each costs on a given machine; every non-zero value computes
// wrong results.  `python -m natten_amd.build --ablate N --output PATH` builds such a library.
#ifndef NATTEN_AMD_ABLATE
#define NATTEN_AMD_ABLATE 0
#endif
constexpr int kAblate = NATTEN_AMD_ABLATE;
enum {
  kAblateMask = 1,      // every tile is taken as fully attended: no element masks
  kAblateCopies = 2,    // no global -> LDS tile copies inside the loop (tiles 0 and 1 are read over and over)
  kAblateSoftmax = 4,   // no exponentials, row sums or conversions: P stays what it was before the loop
  kAblateMax = 8,       // no row maxima, no rescaling
  kAblateBarrier = 16,  // no workgroup barrier per KV tile
  kAblateLdsReads = 32, // matrix operands are read from LDS once per iteration instead of once per instruction
};

template <typename T>
struct Mma;

template <>
struct Mma<__bf16> {
  using vec8 = bf16x8_t;
  using vec2 = bf16x2_t;
  static __device__ __forceinline__ f32x16_t run(vec8 a, vec8 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  // a * b + c into registers of its own (c stays live and untouched).  Written as assembly: from
  // the builtin the compiler first copies c into the destination (sixteen moves) and accumulates
  // in place.  The two wait states cover a dependent matrix instruction issued right behind it.
  static __device__ __forceinline__ f32x16_t run_from(vec8 a, vec8 b, const f32x16_t& c) {
    f32x16_t d;
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3\n\ts_nop 1" : "=&v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
  }
  // c + a.x + a.y
  static __device__ __forceinline__ float add2(vec2 a, float c) {
    const vec2 one = {static_cast<__bf16>(1.0f), static_cast<__bf16>(1.0f)};
    return __builtin_amdgcn_fdot2_f32_bf16(a, one, c, false);
  }
};

template <>
struct Mma<_Float16> {
  using vec8 = f16x8_t;
  using vec2 = f16x2_t;
  static __device__ __forceinline__ f32x16_t run(vec8 a, vec8 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x16_t run_from(vec8 a, vec8 b, const f32x16_t& c) {
    f32x16_t d;
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3\n\ts_nop 1" : "=&v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
  }
  static __device__ __forceinline__ float add2(vec2 a, float c) {
    const vec2 one = {static_cast<_Float16>(1.0f), static_cast<_Float16>(1.0f)};
    return __builtin_amdgcn_fdot2(a, one, c, false);
  }
};

// The logit operand of a query row: q' = round(q * scale * log2(e)) in the operand type (the
// factor is formed in float, one multiplication per element, one rounding), clamped to the type's
// finite range (only fp16 has one that a finite product can leave).  The forward kernel and every
// role of the backward form their logits from q', so that they agree to the last bit of the operand.
template <typename T>
static __device__ __forceinline__ typename Mma<T>::vec8 scale_query_fragment(typename Mma<T>::vec8 raw, float c_log2) {
  typename Mma<T>::vec8 out;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float x = float(raw[e]) * c_log2;
    if constexpr (std::is_same<T, _Float16>::value) x = fminf(fmaxf(x, -65504.f), 65504.f);
    out[e] = static_cast<T>(x);
  }
  return out;
}

// LDS transpose read: the 16 lanes of a group each point at 4 consecutive 16-bit elements of
// a row (lane 4e+j -> row e, columns 4j..4j+3 of a 4x16 block); lane c of the group receives
// column c of the block (rows 0..3).
static __device__ __forceinline__ s16x4_t lds_read_tr16(const char* p) {
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wold-style-cast"
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((NA_LDS s16x4_t*)(p));
#pragma clang diagnostic pop
}

// Asynchronous 16-byte-per-lane copy global -> LDS, written as inline assembly so that the
// compiler does not see an LDS write in flight (it would otherwise make every later LDS read
// wait for the copy): lane i's 16 bytes from `base + voff (+ IMM)` land at LDS address
// `lds_addr + IMM + 16 * i`.  Completion is tracked by the vector memory counter; ordering
// against LDS reads of the same bytes is the caller's business (workgroup barriers).
template <int IMM>
static __device__ __forceinline__ void async_copy16_asm(const void* base, uint32_t voff, uint32_t lds_addr) {
  // base and lds_addr are wave-uniform by construction; say so, so that they are always
  // handed over in scalar registers
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  const uint64_t ub = (uint64_t(uint32_t(__builtin_amdgcn_readfirstlane(int(b >> 32)))) << 32) |
                      uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(b))));
  base = reinterpret_cast<const void*>(ub);
  lds_addr = uint32_t(__builtin_amdgcn_readfirstlane(int(lds_addr)));
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2 offset:%3"
      :
      : "s"(lds_addr), "v"(voff), "s"(base), "n"(IMM)
      : "memory", "m0");
}

// The 4-byte-per-lane form: lane i's dword from `base + voff` lands at LDS address `lds_addr + 4 * i`.
static __device__ __forceinline__ void async_copy4_asm(const void* base, uint32_t voff, uint32_t lds_addr) {
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  const uint64_t ub = (uint64_t(uint32_t(__builtin_amdgcn_readfirstlane(int(b >> 32)))) << 32) |
                      uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(b))));
  base = reinterpret_cast<const void*>(ub);
  lds_addr = uint32_t(__builtin_amdgcn_readfirstlane(int(lds_addr)));
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dword %1, %2"
      :
      : "s"(lds_addr), "v"(voff), "s"(base)
      : "memory", "m0");
}

// The same copy for callers whose `base` and `lds_addr` already live in scalar registers
// (made uniform once per tile with readfirstlane), which saves three moves per copy.
static __device__ __forceinline__ void async_copy16_uniform(uint64_t base, uint32_t voff, uint32_t lds_addr) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2"
      :
      : "s"(lds_addr), "v"(voff), "s"(base)
      : "memory", "m0");
}

static __device__ __forceinline__ uint64_t uniform64(const void* p) {
  const uint64_t b = reinterpret_cast<uint64_t>(p);
  return (uint64_t(uint32_t(__builtin_amdgcn_readfirstlane(int(b >> 32)))) << 32) |
         uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(b))));
}

static __device__ __forceinline__ uint32_t lds_address(const void* p) {
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wold-style-cast"
  return (uint32_t)(uintptr_t)((NA_LDS const char*)(p));
#pragma clang diagnostic pop
}

// s_waitcnt vmcnt(N) only (expcnt / lgkmcnt left at their maxima), gfx9 encoding
template <int N>
static __device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 0xF) | ((N >> 4) << 14));
}

// Workgroup barrier that every wave enters with its own LDS operations complete (s_waitcnt
// lgkmcnt(0); vmcnt and expcnt are left alone).  __syncthreads() leaves that wait to the compiler's
// bookkeeping of outstanding operations, and on one path of the work-queue loop -- thread 0 stores the
// workgroup's next position to LDS, nothing else touches LDS, the loop returns to the barrier at
// its top -- the generated code had no wait at all: a wave on another SIMD could then read the
// word before the store had been performed and work on the position the slot held two tiles
// earlier.  Written out, the wait costs nothing where nothing is outstanding.
static __device__ __forceinline__ void workgroup_sync() {
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __syncthreads();
}

// calls f(std::integral_constant<int, LO + i>{}) for i = 0 .. N-1, in order
template <int LO, typename F, int... Is>
static __device__ __forceinline__ void for_range_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, LO + Is>{}), ...);
}
template <int LO, int N, typename F>
static __device__ __forceinline__ void for_range(F&& f) {
  for_range_impl<LO>(f, std::make_integer_sequence<int, N>{});
}

// Keeps the computation of x at this point of the instruction stream: the empty statement
// is a use the compiler can neither remove nor move into a later basic block.
static __device__ __forceinline__ void pin(float& x) { asm volatile("" : "+v"(x)); }
static __device__ __forceinline__ void pin(uint32_t& x) { asm volatile("" : "+v"(x)); }

static __device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// max of x over the lane pair (l, l ^ 32): v_permlane32_swap exchanges the upper half of its
// first register with the lower half of its second, after which every lane holds both values
// of its pair.  Written as inline assembly (with the wait states the instruction needs around
// it) because the two-result builtin is miscompiled when both inputs are the same value.
static __device__ __forceinline__ float cross_half_max(float x) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return fmaxf(fmaxf(a, b), x);
}

constexpr uint32_t kGuardBits = (1u << 9) | (1u << 19) | (1u << 29);
// a row's running maximum may lag the true one by up to this many powers of two
constexpr float kLazyRescaleLog2 = 8.0f;

// LDS layout of one K or V tile: KVT rows of D 16-bit elements, unpadded, with the 16-byte
// chunks of each row XOR-swizzled so that the MFMA operand reads are bank-conflict free:
//   K: chunk c of row r lives in slot c ^ ((r / RPL) % CPR)            (b128 reads down a column of rows)
//   V: chunk c of row r lives in slot c ^ (2 * ((r / RPL) % (CPR/2)))  (transpose reads of 4 rows x 32 bytes)
// CPR = chunks per row, RPL = rows per 256 bytes.
template <int D, int KVT>
struct FnaSmem {
  static constexpr int ROWB = D * 2;
  static constexpr int CPR = D / 8;
  static constexpr int RPL = (16 / CPR) > 0 ? (16 / CPR) : 1;
  static constexpr int TILE_BYTES = KVT * ROWB;
  static constexpr int STAGES = 2;
  static constexpr int BYTES = STAGES * 2 * TILE_BYTES + KVT * 4;  // static LDS of the kernel
  static __host__ __device__ constexpr int k_slot(int r, int c) { return c ^ ((r / RPL) % CPR); }
  static __host__ __device__ constexpr int v_slot(int r, int c) { return c ^ (2 * ((r / RPL) % (CPR / 2))); }
  // One layout that serves both kinds of read (the backward kernels read the same tile both
  // ways): the XOR pattern runs through the even values over the first half of a 16-row period
  // (what the transpose reads need) and through the odd ones over the second half (so that the
  // 16 rows of a b128 column read still hit 16 different slots).
  static __host__ __device__ constexpr int u_slot(int r, int c) {
    return c ^ ((2 * ((r / RPL) % (CPR / 2))) | (((r / RPL) / (CPR / 2)) & 1));
  }
};

// MQ 32-row query blocks per wave.  MQ = 1 runs two waves per SIMD (256 registers each);
// MQ = 2 one wave per SIMD (512 registers: accumulators and Q fragments can sit in the
// accumulation registers) and reads every K / V fragment from LDS once for two MFMAs.
// RAGGED: seqlen_kv is not a multiple of KVT (dense attention on unpadded sequences); the tile
// copies then clamp their rows and are issued at the top of an iteration instead of one per slot.
// The work of one workgroup on one Q tile; `pid` is the position of that tile in the launch order
// (what blockIdx.x is when every Q tile has a workgroup of its own).  `before_stores()` is called
// once, after the last KV tile and before the results are stored: nothing of this wave is in flight
// at that point (the work-queue launch fetches its next position there, so that the wait for the
// fetch does not include the stores); a call that returns early does not make it.
// NOMASK: the launch is fully block-sparse (the host has checked that every KV tile a Q tile visits is
// attended in full by every query of that Q tile: reference fna_fusion.hpp:503-593); the instance then
// holds no mask code, tables or per-wave windows at all.
template <typename T, int D, int NWAVES, int MQ, bool RAGGED, int KVT, bool SPLIT = false, bool NOMASK = false, typename Hook>
static __device__ __forceinline__ void fna_fwd_tile(const FnaParams& p, const int pid_in, Hook&& before_stores) {
  // split launches: which run of the Q tile's KV tiles this workgroup takes
  const int split = SPLIT ? pid_in / p.split_grid : 0;
  const int pid = SPLIT ? pid_in - split * p.split_grid : pid_in;
  constexpr int NT = NWAVES * 64;
  constexpr int QT = NWAVES * MQ * 32;
  constexpr int KSTEPS = D / 16;
  constexpr int DB = D / 32;
  constexpr int NSB = KVT / 32;
  using L = FnaSmem<D, KVT>;
  constexpr int ROWB = L::ROWB;
  constexpr int CPR = L::CPR;
  constexpr int TILE_BYTES = L::TILE_BYTES;
  constexpr int CHUNKS = KVT * CPR;             // 16-byte chunks per operand tile
  constexpr int PER = (CHUNKS + NT - 1) / NT;   // async copies per thread per operand per tile
  static_assert(CHUNKS % 64 == 0, "a tile must be a whole number of wave-wide copies");
  using M = Mma<T>;
  using vec8 = typename M::vec8;
  using vec2 = typename M::vec2;

  // One LDS object per stage and operand: distinct objects let the compiler see that the
  // asynchronous fill of one stage does not alias the operand reads of the other, so those
  // reads do not wait for the fill.
  __shared__ __attribute__((aligned(1024))) char sK0[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sV0[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sK1[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char sV1[TILE_BYTES];
  // What the element mask of a PARTIAL tile needs (absent from NOMASK instances), kept in LDS and read
  // where such a tile is met -- in registers for the whole loop these values would push the loop's own
  // out to spill lanes:
  //   sKeys[a][g][x]  the keys of a tile whose coordinate along dimension a is >= x, one bit per key:
  //                   the 32 bits that the lanes of wave half g hold logits for (na_lane_half_bits)
  //   sWin[row]    window of the Q tile's query `row` (row-major): start and end per dimension
  //   sGeo[a]      KV tile extent along dimension a
  constexpr int MASK_ROWS = NOMASK ? 1 : KVT + 1;
  __shared__ __attribute__((aligned(16))) uint32_t sKeys[NOMASK ? 1 : 3][2][MASK_ROWS];
  __shared__ __attribute__((aligned(16))) int sWin[NOMASK ? 1 : NWAVES * MQ * 32][8];
  __shared__ __attribute__((aligned(16))) int sGeo[4];
  static_assert(NOMASK || KVT == 64, "the element mask holds one bit per key of a 64-key tile");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction
  const int l32 = lane & 31;
  const int g = lane >> 5;

  // ---- workgroup id -> (batch*group, head, Q tile); groups of Q tiles are dealt to XCDs ------
  int bg, head, qtile_rm;
  {
    const int xcd = int(uint32_t(pid) % kNumXcd);
    const int local = int(uint32_t(pid) / kNumXcd);
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

  // sequence lengths, window and row range of this batch entry: launch constants, except for
  // sequence-packed dense attention, where every batch entry is a sequence of its own
  int seqlen_q = p.seqlen_q, seqlen_kv = p.seqlen_kv;
  int ksz[3] = {p.ksize[0], p.ksize[1], p.ksize[2]};
  int ext0 = p.ext_base[0];  // extent of dimension 0 before dilation groups (a sequence's own length when packed)
  int64_t q_seq_row0 = int64_t(bg) * p.seqlen_q, kv_seq_row0 = int64_t(bg) * p.seqlen_kv;
  if constexpr (RAGGED) {
    if (p.cu_q != nullptr) {
      const int q0 = p.cu_q[bg], kv0 = p.cu_kv[bg];
      seqlen_q = p.cu_q[bg + 1] - q0;
      seqlen_kv = p.cu_kv[bg + 1] - kv0;
      // a malformed cumulative array (negative, decreasing, past the end) must not become an address
      if (q0 < 0 || kv0 < 0 || seqlen_q < 0 || seqlen_kv < 0 || q0 > p.total_q - seqlen_q || kv0 > p.total_kv - seqlen_kv)
        return;
      q_seq_row0 = q0;
      kv_seq_row0 = kv0;
      ksz[0] = seqlen_kv;
      ext0 = seqlen_kv;  // (packed sequences are not dilated)
      // Q tiles are counted for the longest sequence: the ones past the end of this one have nothing to do
      int t0 = qtile_rm;
      if (p.causal[0]) t0 = p.q_tiled[0] - 1 - t0;
      if (t0 * QT >= seqlen_q) return;
      if (seqlen_kv <= 0) {
        // no keys: the softmax runs over an empty set, O = 0 and LSE = -inf
        T* o = reinterpret_cast<T*>(p.o) + (q_seq_row0 * p.heads_q + head) * D;
        for (int i = tid; i < QT * (D / 8); i += NT) {
          const int row = t0 * QT + i / (D / 8);
          if (row < seqlen_q) {
            typedef T tx8 __attribute__((ext_vector_type(8)));
            *reinterpret_cast<tx8*>(o + int64_t(row) * p.heads_q * D + (i % (D / 8)) * 8) = tx8{};
          }
        }
        for (int i = tid; i < QT; i += NT)
          if (t0 * QT + i < seqlen_q) p.lse[(q_seq_row0 + t0 * QT + i) * p.heads_q + head] = -INFINITY;
        return;
      }
    }
  }

  // ---- workgroup-uniform setup: dilation group, Q tile origin, KV tile box -------------------
  // qtile_rm enumerates Q tiles with dimension 0 slowest; causal dimension 0 is walked from
  // the far end so that the Q tiles with the longest KV loops start first.
  int extent[3], q_first[3], box_org[3], box_n[3];  // box_org: coordinate of the box's first KV tile
  const int b_orig = na_div(bg, p.d_num_groups);  // batch entry before the dilation groups were folded in
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
      // dilation group gi holds one more token than the last groups when gi < X % d (reference
      // fna_fusion.hpp:250-256, without its divisions: 0 <= gi < d decides the quotient there)
      extent[a] = (a == 0 ? ext0 : p.ext_base[a]) + (gi < p.ext_rem[a] ? 1 : 0);
      tok_step[a] = p.dil[a] * p.tok_stride[a];
      group_tok += gi * p.tok_stride[a];
      q_first[a] = tc[a] << p.q_tile_lg[a];
      const int qf = q_first[a], ql = qf + p.q_tile[a] - 1;
      const bool c = p.causal[a] != 0;
      const int st_f = na_window_start(qf, ksz[a], p.stride[a], p.d_stride[a], extent[a], c);
      const int st_l = na_window_start(ql, ksz[a], p.stride[a], p.d_stride[a], extent[a], c);
      const int en_l = na_window_end(ql, st_l, ksz[a], extent[a], c);
      box_org[a] = p.anchor ? st_f : ((st_f >> p.kv_tile_lg[a]) << p.kv_tile_lg[a]);
      box_n[a] = (en_l - box_org[a] + p.kv_tile[a] - 1) >> p.kv_tile_lg[a];
    }
  }
  // The tiles this workgroup visits: all of the box, or run `split` of its kv_splits runs.  A run
  // that is empty (a box of fewer tiles than splits) still walks one tile, for the sake of one code
  // path, and stores the result of no keys at all: zeros and an LSE of -inf.
  const int box_tiles = box_n[0] * box_n[1] * box_n[2];
  int first_tile = 0, total_tiles = box_tiles;
  bool empty_split = false;
  if constexpr (SPLIT) {
    first_tile = int(int64_t(split) * box_tiles / p.kv_splits);
    total_tiles = int(int64_t(split + 1) * box_tiles / p.kv_splits) - first_tile;
    if (total_tiles == 0) {
      empty_split = true;
      first_tile = 0;
      total_tiles = 1;
    }
  }

  // ---- this wave's share of the Q tile ------------------------------------------------------------
  // The Q tile is a grid of boxes of 32 queries (extents 2^wave_box_lg, dimension 2 fastest inside a
  // box and across the grid); row block mb of wave w holds box w * MQ + mb, one query per lane of each
  // half of the wave.  With the default box (as much of dimension 2 as fits, then of dimension 1, ...)
  // the lanes take the tile's tokens in row-major order.  The token's row inside the permuted tile
  // (dimension 0 fastest) follows from its coordinates.  Window starts and ends
  // are monotone in the query coordinate, hence over the wave's bounding box the union of the
  // windows is [start(min), end(max)) and their intersection [start(max), end(min)) per
  // dimension: a KV tile outside the union is skipped by this wave, one inside the
  // intersection needs no mask.
  auto box_origin = [&](int block, int (&o)[3]) {
#pragma unroll
    for (int a = 2; a >= 0; --a) {
      const int nb = p.q_tile_lg[a] - p.wave_box_lg[a];  // log2 boxes along this dimension
      o[a] = (block & ((1 << nb) - 1)) << p.wave_box_lg[a];
      block >>= nb;
    }
  };
  int wave_lo[3], wave_hi[3], wave_full_lo[3], wave_full_hi[3];
  if constexpr (!NOMASK) {
    int f[3], l[3];
#pragma unroll
    for (int mb = 0; mb < MQ; ++mb) {
      int o[3];
      box_origin(wave * MQ + mb, o);
#pragma unroll
      for (int a = 0; a < 3; ++a) {
        const int last = o[a] + (1 << p.wave_box_lg[a]) - 1;
        f[a] = mb == 0 ? o[a] : na_min(f[a], o[a]);
        l[a] = mb == 0 ? last : na_max(l[a], last);
      }
    }
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      // rows past the end of an unpadded sequence (dense attention) are clamped like the loads
      const int qmin = q_first[a] + f[a], qmax = q_first[a] + na_min(l[a], p.q_tile[a] - 1);
      const bool c = p.causal[a] != 0;
      const int st_min = na_window_start(qmin, ksz[a], p.stride[a], p.d_stride[a], extent[a], c);
      const int en_min = na_window_end(qmin, st_min, ksz[a], extent[a], c);
      const int st_max = na_window_start(qmax, ksz[a], p.stride[a], p.d_stride[a], extent[a], c);
      const int en_max = na_window_end(qmax, st_max, ksz[a], extent[a], c);
      wave_lo[a] = st_min;
      wave_hi[a] = en_max;
      wave_full_lo[a] = st_max;
      wave_full_hi[a] = en_min;
    }
  }

  if constexpr (!NOMASK) {
    if (tid < 3) sGeo[tid] = p.kv_tile[tid];
    // one row per thread and dimension: keys are numbered with dimension 0 fastest
    int lg_stride = 0;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      if (tid <= p.kv_tile[a]) {
        const uint64_t keys = na_keys_at_or_after(tid, lg_stride, p.kv_tile_lg[a]);
        sKeys[a][0][tid] = na_lane_half_bits(keys, 0);
        sKeys[a][1][tid] = na_lane_half_bits(keys, 1);
      }
      lg_stride += p.kv_tile_lg[a];
    }
  }

  const int64_t q_row_stride = int64_t(p.heads_q) * D;
  const int64_t kv_row_stride = int64_t(p.heads_kv) * D;
  // first row of this (batch, dilation group): rows are then addressed by permuted row index
  // (permuted layout) or by token offset inside the group (fused layout)
  const int64_t q_row_base = p.fused ? int64_t(b_orig) * p.tokens + group_tok : q_seq_row0;
  const int64_t kv_row_base = p.fused ? int64_t(b_orig) * p.tokens + group_tok : kv_seq_row0;
  const T* qbase = reinterpret_cast<const T*>(p.q) + q_row_base * q_row_stride + int64_t(head) * D;
  const T* kbase = reinterpret_cast<const T*>(p.k) + kv_row_base * kv_row_stride + int64_t(head_kv) * D;
  const T* vbase = reinterpret_cast<const T*>(p.v) + kv_row_base * kv_row_stride + int64_t(head_kv) * D;
  // row (permuted) or token offset (fused) of position `r` (dimension 0 fastest) of a KV tile
  auto kv_tile_pos = [&](int r) {
    if (!p.fused) return r;
    const int t0 = r & (p.kv_tile[0] - 1);
    r >>= p.kv_tile_lg[0];
    return t0 * tok_step[0] + (r & (p.kv_tile[1] - 1)) * tok_step[1] + (r >> p.kv_tile_lg[1]) * tok_step[2];
  };

  // ---- async tile loads -------------------------------------------------------------------------
  // Copy i of wave w fills LDS chunks (w*PER + i)*64 .. +63 of the tile (chunk P: row P / CPR,
  // slot P % CPR).  Its global address is a per-tile uniform base (first row of the tile) plus
  // a byte offset that never changes for the thread, so a tile load costs no vector address
  // arithmetic.  Up to four copies share one M0 value through the instruction's immediate
  // offset (which the hardware adds to the LDS and to the global address alike: it is taken off
  // the per-lane offset again), and copy i + 4 lies a whole number of swizzle periods (16 rows
  // or more) below copy i, so it reuses that copy's per-lane offset on a shifted base.
  constexpr int NOFF = PER < 4 ? PER : 4;
  constexpr int kImmBias = 3 * 1024;  // largest immediate offset of a copy
  constexpr int ROWS_PER_4 = 256 / CPR;  // rows between copy i and copy i + 4
  // Copy i + 4 (only waves with eight copies have one) sets one more bit of the tile position;
  // tile extents are powers of two, so that bit moves one coordinate by a fixed amount and the
  // row (permuted) or token (fused) distance to copy i is the same for every lane.
  const int64_t bytes_per_4 = int64_t(kv_tile_pos(ROWS_PER_4 % KVT)) * (kv_row_stride * 2);
  int ld_row[NOFF];
  uint32_t ld_koff[NOFF], ld_voff[NOFF];
#pragma unroll
  for (int i = 0; i < NOFF; ++i) {
    const int P = (wave * PER + i) * 64 + lane;
    ld_row[i] = P / CPR;
    const int slot = P % CPR;
    // XOR swizzles are involutions: slot -> source chunk uses the same function
    const uint32_t pos = uint32_t(kv_tile_pos(ld_row[i]));
    ld_koff[i] = pos * uint32_t(kv_row_stride * 2) + uint32_t(L::k_slot(ld_row[i], slot) * 16);
    ld_voff[i] = pos * uint32_t(kv_row_stride * 2) + uint32_t(L::v_slot(ld_row[i], slot) * 16);
    if constexpr (!RAGGED) {
      // the instruction adds its immediate i * 1024 to the global address as well: take it off
      // here, on top of a bias that keeps the offset non-negative and is taken off the tile base
      ld_koff[i] += uint32_t(kImmBias - i * 1024);
      ld_voff[i] += uint32_t(kImmBias - i * 1024);
    }
  }
  // One operand tile in flight: uniform source base, LDS destination of this wave's share.
  struct TileCopy {
    const char* src;  // first row of the tile (this head)
    uint32_t lds0;    // LDS byte address of this wave's first chunk
    int row0;
    int lim[3];       // original layout: positions of the tile that lie inside the dilation group, per dimension
    bool inside;      // the whole tile lies inside the sequence / the dilation group
  };
  auto make_copy = [&](const T* base, char* dst, int kv_row0, const int (&origin)[3]) {
    TileCopy c;
    kv_row0 = __builtin_amdgcn_readfirstlane(kv_row0);  // uniform by construction; keeps the base in scalar registers
    c.src = reinterpret_cast<const char*>(base) + int64_t(kv_row0) * kv_row_stride * 2 - (RAGGED ? 0 : kImmBias);
    c.lds0 = lds_address(dst) + uint32_t(wave * PER * 1024);
    c.row0 = kv_row0;
    c.inside = true;
    if constexpr (RAGGED) {
      if (p.fused) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
          c.lim[a] = na_min(extent[a] - origin[a], p.kv_tile[a]);
          c.inside = c.inside && (c.lim[a] == p.kv_tile[a]);
        }
      } else {
        c.inside = kv_row0 + KVT <= seqlen_kv;
      }
    }
    return c;
  };
  // issues copy I (0 <= I < PER) of a tile; V_LAYOUT selects the LDS swizzle of the operand
  auto copy_one = [&](auto i_tag, const TileCopy& c, const uint32_t (&off)[NOFF], auto v_tag) {
    constexpr int I = decltype(i_tag)::value;
    constexpr bool V_LAYOUT = decltype(v_tag)::value;
    if constexpr (I < PER) {
      if (CHUNKS % (NT * PER) == 0 || (wave * PER + I) * 64 < CHUNKS) {
        constexpr int IMM = (I % 4) * 1024;
        const char* src = c.src + int64_t(I / 4) * bytes_per_4;
        uint32_t voff = off[I % 4];
        if constexpr (RAGGED) {
          if (!c.inside) {
            if (p.fused) {
              // a tile that reaches past its dilation group (original layout): positions beyond
              // the group's extent are masked; gather the group's last row along that dimension
              // instead, so that no address outside the tensor is formed.  The LDS placement
              // (and with it the order of every sum) stays that of the whole tile.
              const int P = (wave * PER + I) * 64 + lane;
              const int r = P / CPR, slot = P % CPR;
              int t0 = r & (p.kv_tile[0] - 1);
              const int r1 = r >> p.kv_tile_lg[0];
              int t1 = r1 & (p.kv_tile[1] - 1), t2 = r1 >> p.kv_tile_lg[1];
              t0 = na_min(t0, c.lim[0] - 1);
              t1 = na_min(t1, c.lim[1] - 1);
              t2 = na_min(t2, c.lim[2] - 1);
              const uint32_t pos = uint32_t(t0 * tok_step[0] + t1 * tok_step[1] + t2 * tok_step[2]);
              voff = pos * uint32_t(kv_row_stride * 2) + uint32_t((V_LAYOUT ? L::v_slot(r, slot) : L::k_slot(r, slot)) * 16);
              src = c.src;
            } else {
              // last, partial tile of an unpadded sequence: rows past the end are masked; read the
              // last valid row instead so that no out-of-bounds address is formed
              const int over = na_max(c.row0 + ld_row[I % 4] + (I / 4) * ROWS_PER_4 - (seqlen_kv - 1), 0);
              voff -= uint32_t(over) * uint32_t(kv_row_stride * 2);
            }
          }
          // the clamped per-lane offset may be smaller than the immediate: take the immediate
          // off the uniform base instead
          src -= IMM;
        }
        async_copy16_asm<IMM>(src, voff, c.lds0 + uint32_t((I / 4) * 4096));
      }
    }
  };
  static_assert(PER <= 8, "tile copy is written for at most eight copies per thread");
  auto issue_tile_load = [&](const T* base, const uint32_t (&off)[NOFF], char* dst, int kv_row0, const int (&origin)[3],
                             auto v_tag) {
    const TileCopy c = make_copy(base, dst, kv_row0, origin);
    copy_one(std::integral_constant<int, 0>{}, c, off, v_tag);
    copy_one(std::integral_constant<int, 1>{}, c, off, v_tag);
    copy_one(std::integral_constant<int, 2>{}, c, off, v_tag);
    copy_one(std::integral_constant<int, 3>{}, c, off, v_tag);
    copy_one(std::integral_constant<int, 4>{}, c, off, v_tag);
    copy_one(std::integral_constant<int, 5>{}, c, off, v_tag);
    copy_one(std::integral_constant<int, 6>{}, c, off, v_tag);
    copy_one(std::integral_constant<int, 7>{}, c, off, v_tag);
  };

  // KV tile stream: dimension 2 fastest, dimension 0 slowest.  The load stream runs up to two
  // tiles ahead of the softmax, so tile descriptors are produced in order and handed down.
  struct TileInfo {
    int row0;       // first row of the tile in the permuted KV sequence / token offset of its origin (fused)
    int origin[3];  // coordinate of its first token (a tile moved back from the group's edge: of the first one gathered)
    bool full;      // every key of the tile is attended by every query of this wave
    bool skip;      // no key of the tile is attended by any query of this wave
    int lead[3];    // a tile moved back from the group's edge: its first lead[a] positions belong to the tile before it
  };
  int itc[3] = {0, 0, 0};
  if constexpr (SPLIT) {
    itc[2] = first_tile % box_n[2];
    const int rest = first_tile / box_n[2];
    itc[1] = rest % box_n[1];
    itc[0] = rest / box_n[1];
  }
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
      t.lead[a] = org - t.origin[a];
    }
    // (both forms are a handful of scalar operations: computed side by side and selected, a branch costs more)
    const int row0_fused = t.origin[0] * tok_step[0] + t.origin[1] * tok_step[1] + t.origin[2] * tok_step[2];
    const int row0_permuted = (((box_org[0] >> p.kv_tile_lg[0]) + itc[0]) +
                               p.kv_tiled[0] * (((box_org[1] >> p.kv_tile_lg[1]) + itc[1]) +
                                                p.kv_tiled[1] * ((box_org[2] >> p.kv_tile_lg[2]) + itc[2]))) * KVT;
    t.row0 = p.fused ? row0_fused : row0_permuted;
    if (++itc[2] == box_n[2]) {
      itc[2] = 0;
      if (++itc[1] == box_n[1]) {
        itc[1] = 0;
        ++itc[0];
      }
    }
    if constexpr (NOMASK || (kAblate & kAblateMask) != 0) {
      t.full = true;
      t.skip = false;
    }
    return t;
  };

  using Stage0 = std::integral_constant<int, 0>;
  using Stage1 = std::integral_constant<int, 1>;
  TileInfo cur = next_tile();  // tile 0
  using KLayout = std::false_type;
  using VLayout = std::true_type;
  issue_tile_load(kbase, ld_koff, sK0, cur.row0, cur.origin, KLayout{});
  issue_tile_load(vbase, ld_voff, sV0, cur.row0, cur.origin, VLayout{});

  float sm_scale = p.scale, out_scale = 1.f;
  if (p.q_scale) sm_scale *= p.q_scale[head];
  if (p.k_scale) sm_scale *= p.k_scale[head_kv];
  if (p.v_scale) out_scale = p.v_scale[head_kv];
  const float c_log2 = sm_scale * 1.4426950408889634f;

  // ---- per-lane setup: this lane's query rows, their windows, Q fragments ---------------------
  int q_row[MQ];     // this lane's row of the permuted sequence / token offset in the group (fused), or -1
  vec8 qf[MQ][KSTEPS];
#pragma unroll
  for (int mb = 0; mb < MQ; ++mb) {
    int off[3];  // the lane's query inside the tile: its box's origin plus its place in the box
    box_origin(wave * MQ + mb, off);
    {
      int r = l32;
#pragma unroll
      for (int a = 2; a >= 0; --a) {
        off[a] += r & ((1 << p.wave_box_lg[a]) - 1);
        r >>= p.wave_box_lg[a];
      }
    }
    int row = qtile_idx * QT + off[0] + p.q_tile[0] * (off[1] + p.q_tile[1] * off[2]);
    bool valid = row < seqlen_q;
    int row_c = na_min(row, seqlen_q - 1);
    if (p.fused) {
      // queries past the end of the dilation group are padding: computed on a clamped copy, never stored
      row = 0;
      row_c = 0;
      valid = true;
    }
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int c = q_first[a] + off[a];
      if (p.fused) {
        valid = valid && (c < extent[a]);
        row += c * tok_step[a];
        row_c += na_min(c, extent[a] - 1) * tok_step[a];
      }
      if constexpr (!NOMASK) {
        // this query's window (padding queries: that of the last real one), for the element masks
        if (g == 0) {
          const int qc = na_min(c, extent[a] - 1);
          const bool cs = p.causal[a] != 0;
          const int ws = na_window_start(qc, ksz[a], p.stride[a], p.d_stride[a], extent[a], cs);
          sWin[(wave * MQ + mb) * 32 + l32][2 * a] = ws;
          sWin[(wave * MQ + mb) * 32 + l32][2 * a + 1] = na_window_end(qc, ws, ksz[a], extent[a], cs);
        }
      }
    }
    q_row[mb] = valid ? row : -1;
    const T* qrow = qbase + int64_t(row_c) * q_row_stride + g * 8;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const vec8 raw = *reinterpret_cast<const vec8*>(qrow + ks * 16);
      // The query row carries the softmax scale (in the exp2 domain) into the matrix product, so
      // that the logits leave the matrix pipe ready for exp2: q' = round(q * scale * log2(e)).
      // Rounding q' to the operand type moves a logit by about 2^-9 (bf16) / 2^-12 (fp16) of
      // |q||k| scale / sqrt(D) -- the size of the operands' own rounding.
      qf[mb][ks] = scale_query_fragment<T>(raw, c_log2);
    }
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

  // lane-constant LDS read offsets
  int k_off[KSTEPS];  // K operand: row l32 (+32*sb), chunk 2*ks+g
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) k_off[ks] = l32 * ROWB + L::k_slot(l32, ks * 2 + g) * 16;
  // V operand: transpose read of rows (4g + e) [+8], 4 columns at 16*(l32/16) + 4*j4 of a 32-column block
  const int l16 = lane & 15;
  const int v_e = l16 >> 2, v_j4 = l16 & 3;
  const int v_row = 4 * g + v_e;
  const int v_chunk = (l32 >> 4) * 2 + (v_j4 >> 1);  // 16-byte chunk inside the 64-byte column block
  const int v_sub = (v_j4 & 1) * 8;

  // ---- building blocks ---------------------------------------------------------------------------
  // The lane owns query row l32 of each of its wave's MQ row blocks and, per 32-key sub-block,
  // the 16 key rows 8*(r/4) + 4*g + r%4.  One "slot" below is one operand fragment read from
  // LDS, the MQ MFMAs that use it, and the vector work that is to run in their shadow; slots are
  // fenced so that the compiler keeps that interleaving (a 32x32x16 MFMA occupies the matrix pipe
  // for 32 cycles but only one issue cycle, and up to six ordinary vector instructions of the
  // same wave issue behind it for free).
  constexpr int N_QK = NSB * KSTEPS;        // slots of S^T = K Q^T
  constexpr int N_PV = NSB * 2 * DB;        // slots of O^T += V^T P^T
  constexpr int PF_K = 2, PF_V = 2;         // operand fragments read ahead of their MFMAs
  static_assert(NSB % 2 == 0 && N_QK > PF_K && N_PV > PF_V, "tile too small for the schedule");

  // QK slot s multiplies k-step s % KSTEPS of sub-block s / KSTEPS (a sub-block's logits only
  // occupy registers once its first slot is reached)
  auto k_frag = [&](const char* sK, int s) {
    return *reinterpret_cast<const vec8*>(sK + (s / KSTEPS) * 32 * ROWB + k_off[s % KSTEPS]);
  };
  // PV slot t: sub-block t / (2*DB), 16-key half (t / DB) % 2, 32-column block t % DB
  auto v_frag = [&](const char* sV, int t) {
    const int r0 = (t / (2 * DB)) * 32 + ((t / DB) % 2) * 16 + v_row;
    const int c = (t % DB) * 4 + v_chunk;
    const s16x4_t lo = lds_read_tr16(sV + r0 * ROWB + v_sub + L::v_slot(r0, c) * 16);
    const s16x4_t hi = lds_read_tr16(sV + (r0 + 8) * ROWB + v_sub + L::v_slot(r0 + 8, c) * 16);
    return __builtin_bit_cast(vec8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  // Logits are kept in the exp2 domain and relative to the row's running maximum: the matrix
  // product starts from the accumulator value -m (sixteen registers per row block that only
  // change when the maximum moves), so the probabilities are exp2 of what the matrix pipe returns.
  f32x16_t S_a[MQ][NSB], S_b[MQ][NSB];  // logits of the current / coming tile, swapping roles every iteration
  vec8 pf[MQ][NSB][2];
  f32x16_t c_init[MQ];          // -(running maximum), 0 while it is -inf: accumulator input of S = K Q^T
  float psum[MQ][2];
  if constexpr ((kAblate & kAblateSoftmax) != 0) {
    // probability-like operands (values in (0, 1]) in place of the ones the loop would form
#pragma unroll
    for (int mb = 0; mb < MQ; ++mb)
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int e = 0; e < 8; ++e)
            pf[mb][sb][h][e] = static_cast<T>(fast_exp2(-fabsf(float(qf[mb][(sb * 2 + h) % KSTEPS][e]))));
  }

  // Element e of the current tile's probabilities: row block e % MQ, logit v = e / MQ of the lane
  // (sub-block v / 16, register v % 16): exp2(c*s - c*m), summed in float; every second
  // element of a row block rounds its pair to T.
  float held[MQ];
  auto exp_elem = [&](const f32x16_t (&S_cur)[MQ][NSB], int e) {
    if constexpr ((kAblate & kAblateSoftmax) != 0) {
      asm volatile("" ::"v"(S_cur[e % MQ][(e / MQ) / 16][(e / MQ) % 16]));  // the logits stay in use
      return;
    }
    const int mb = e % MQ, v = e / MQ;
    const int sb = v / 16, r = v % 16;
    float x = fast_exp2(S_cur[mb][sb][r]);
    psum[mb][r & 1] += x;
    if (r % 2 == 0) {
      pin(x);
      held[mb] = x;
    } else {
      vec2 p2 = {static_cast<T>(held[mb]), static_cast<T>(x)};
      uint32_t bits = __builtin_bit_cast(uint32_t, p2);
      pin(bits);
      p2 = __builtin_bit_cast(vec2, bits);
      pf[mb][sb][r / 8][r % 8 - 1] = p2[0];
      pf[mb][sb][r / 8][r % 8] = p2[1];
    }
  };
  // Elements are spread evenly over the slots that precede the last 16-key block of O += P V
  // (whose P fragment is the last to be completed): cumulative count after global slot x.
  constexpr int N_ELEMS = MQ * NSB * 16;
  constexpr int EXP_SLOTS = N_QK + N_PV - DB;
  auto elems_done = [](int x) constexpr {
    const int n = (N_ELEMS * (x + 1) + EXP_SLOTS - 1) / EXP_SLOTS;
    return x < 0 ? 0 : (n > N_ELEMS ? N_ELEMS : n);
  };

  // Element mask of a PARTIAL tile for row block mb.  Per dimension the lane's window, relative to the
  // tile origin and clamped to the tile, selects two rows of sKeys (keys at or after its start, keys at
  // or after its end); the AND over the dimensions has one bit per logit of the lane: bit 16 sb + r
  // for logit r of sub-block sb.  A tile moved back from the group's edge starts before its place in
  // the tiling (the box origin plus a multiple of the tile extent): the keys up to there (`lead`)
  // belong to the tile before it.  All six rows are read at once (one register each), so that a
  // masked tile waits for LDS twice -- the windows, then the rows -- and not once per dimension.
  auto mask_bits = [&](int mb, const int (&origin)[3], const int (&lead)[3]) __attribute__((always_inline)) {
    uint32_t bits = ~uint32_t(0);
    if constexpr (!NOMASK) {
      typedef int i32x4 __attribute__((ext_vector_type(4)));
      typedef int i32x2 __attribute__((ext_vector_type(2)));
      const int row = (wave * MQ + mb) * 32 + l32;
      const i32x4 w01 = *reinterpret_cast<const i32x4*>(&sWin[row][0]);
      const i32x2 w2 = *reinterpret_cast<const i32x2*>(&sWin[row][4]);
      const int ws[3] = {w01[0], w01[2], w2[0]}, we[3] = {w01[1], w01[3], w2[1]};
      int lo[3], hi[3];
#pragma unroll
      for (int a = 0; a < 3; ++a) {
        const int kt = sGeo[a];
        lo[a] = na_min(na_max(ws[a] - origin[a], lead[a]), kt);
        hi[a] = na_min(na_max(we[a] - origin[a], 0), kt);
      }
      uint32_t from[3], upto[3];
#pragma unroll
      for (int a = 0; a < 3; ++a) {
        from[a] = sKeys[a][g][lo[a]];
        upto[a] = sKeys[a][g][hi[a]];
      }
#pragma unroll
      for (int a = 0; a < 3; ++a) bits &= from[a] & ~upto[a];
    }
    return bits;
  };
  // logit r of sub-block sb: kept where its bit is set, else -inf; two instructions (the
  // sign-extended bit, a bitwise select) and no condition codes
  auto mask_elem = [&](f32x16_t (&S)[NSB], int sb, int r, const uint32_t lane_bits) __attribute__((always_inline)) {
    const uint32_t keep = uint32_t(__builtin_amdgcn_sbfe(int(lane_bits), 16 * sb + r, 1));  // 0 or ~0
    const float logit = S[sb][r];  // (a copy: a bit cast of the vector element itself reads element 0)
    const uint32_t bits = __builtin_bit_cast(uint32_t, logit);
    S[sb][r] = __builtin_bit_cast(float, (bits & keep) | (~keep & 0xff800000u));
  };
  auto apply_mask = [&](f32x16_t (&S)[NSB], int mb, const int (&origin)[3], const int (&lead)[3]) __attribute__((always_inline)) {
    if constexpr (!NOMASK) {
      const uint32_t lane_bits = mask_bits(mb, origin, lead);
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) mask_elem(S, sb, r, lane_bits);
    }
  };

  // adopts the maximum `mx` of the lane's half row of the coming tile (relative to the running
  // maximum, like the logits `S` themselves): the running maximum is only moved (and the logits of
  // that tile, O and the row sum shifted / rescaled) when some row of the wave outgrew it by 2^8
  auto update_max = [&](int mb, float mx, f32x16_t (&S)[NSB]) __attribute__((always_inline)) {
    mx = cross_half_max(mx);
    const bool first = (m_run[mb] == -INFINITY) && (mx != -INFINITY);
    const bool grow = first || (mx > kLazyRescaleLog2);
    if (__builtin_expect(__any(grow), 0)) {
      // rows still at -inf take their first maximum as it is (it may be negative) and have
      // nothing accumulated yet; the others only grow
      const bool was_inf = m_run[mb] == -INFINITY;
      const float shift = was_inf ? ((mx == -INFINITY) ? 0.f : mx) : fmaxf(mx, 0.f);
      const float alpha = was_inf ? 1.f : fast_exp2(-shift);
      if (mx != -INFINITY) m_run[mb] = (was_inf ? 0.f : m_run[mb]) + shift;
      l_run[mb] *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mb][db][r] *= alpha;
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) S[sb][r] -= shift;
      const float c = (m_run[mb] == -INFINITY) ? 0.f : -m_run[mb];
#pragma unroll
      for (int r = 0; r < 16; ++r) c_init[mb][r] = c;
    }
    // one home for the sixteen registers on both paths (otherwise the compiler keeps a second
    // copy of them alive and copies one to the other in every iteration)
    asm volatile("" : "+v"(c_init[mb]));
  };
  // masks (PARTIAL tiles) and maxima of a whole tile of logits, outside the slots
  auto finish_logits = [&](f32x16_t (&S)[MQ][NSB], const TileInfo& t, bool have_max, const float (&mx_in)[MQ]) __attribute__((always_inline)) {
    // One test on the way of a tile that needs nothing (attended in full, maxima at hand): every
    // wave-uniform branch in the tile loop costs about a hundredth of its time.
    const bool t_full = t.full, t_skip = t.skip;
    const bool plain = t_full && !t_skip && have_max;
#pragma unroll
    for (int mb = 0; mb < MQ; ++mb) {
      float mx = mx_in[mb];
      if (__builtin_expect(!plain, 0)) {
        if (t_skip) {
          // none of this wave's queries attends the tile: every logit is masked
          mx = -INFINITY;
#pragma unroll
          for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
            for (int r = 0; r < 16; ++r) S[mb][sb][r] = -INFINITY;
        } else {
          if (!t_full) apply_mask(S[mb], mb, t.origin, t.lead);
          mx = -INFINITY;
#pragma unroll
          for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, S[mb][sb][r]);
        }
      }
      update_max(mb, mx, S[mb]);
    }
  };

  // ---- software pipeline --------------------------------------------------------------------
  // Iteration j: (G1) the slots of S(j+1) = K(j+1) Q^T, with the asynchronous copies of K(j+2)
  // and V(j+1); (G2, G3) the slots of O += P(j) V(j), the second half with the row maxima of
  // S(j+1).  The exponentials of S(j) are spread evenly over all of them.
  // LDS: K(j) and V(j) live in stage j % 2.
  TileInfo nxt = next_tile();  // tile 1 (a descriptor past the box is never used)
  wait_vmcnt<0>();
  workgroup_sync();  // K(0), V(0), the mask tables and the queries' windows are in LDS
  if (1 < total_tiles) issue_tile_load(kbase, ld_koff, sK1, nxt.row0, nxt.origin, KLayout{});
#pragma unroll
  for (int mb = 0; mb < MQ; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) c_init[mb][r] = 0.f;
  {
#pragma unroll
    for (int mb = 0; mb < MQ; ++mb)
#pragma unroll
      for (int sb = 0; sb < NSB; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) S_a[mb][sb][r] = 0.f;
#pragma unroll
    for (int s = 0; s < N_QK; ++s) {
      const vec8 kf = k_frag(sK0, s);
#pragma unroll
      for (int mb = 0; mb < MQ; ++mb) S_a[mb][s / KSTEPS] = M::run(kf, qf[mb][s % KSTEPS], S_a[mb][s / KSTEPS]);
    }
    const float none[MQ] = {};
    finish_logits(S_a, cur, false, none);
  }

  // CUR / NXT: this wave attends keys of tile j / tile j + 1; an inactive tile only takes part
  // in the copies and the barrier.
  auto iteration = [&](auto stage_tag, auto cur_tag, auto nxt_tag, int j) __attribute__((always_inline)) {
    constexpr int st = decltype(stage_tag)::value;
    constexpr bool CUR = decltype(cur_tag)::value, NXT = decltype(nxt_tag)::value;
    constexpr bool SPREAD = !RAGGED;
    f32x16_t (&S_cur)[MQ][NSB] = st ? S_b : S_a;
    f32x16_t (&S_nxt)[MQ][NSB] = st ? S_a : S_b;
    char* sK_cur = st ? sK1 : sK0;  // held K(j): free, receives K(j+2)
    char* sK_nxt = st ? sK0 : sK1;  // holds K(j+1)
    char* sV_cur = st ? sV1 : sV0;  // holds V(j)
    char* sV_nxt = st ? sV0 : sV1;  // held V(j-1): free, receives V(j+1)

    wait_vmcnt<0>();   // this thread's copies of K(j+1) and V(j) have landed
    if constexpr ((kAblate & kAblateBarrier) == 0)
      workgroup_sync();   // ... and everyone's; everyone is done reading K(j) and V(j-1)
    const TileInfo t2 = next_tile();
    // Past the end of the box the spread copies re-read the current tile into the free stage
    // (never used), which keeps the slots below free of control flow.
    // (the spread copies only exist without RAGGED, where a tile's origin is not looked at)
    const TileCopy ck = make_copy(kbase, sK_cur, (j + 2 < total_tiles) ? t2.row0 : cur.row0, cur.origin);
    const TileCopy cv = make_copy(vbase, sV_nxt, (j + 1 < total_tiles) ? nxt.row0 : cur.row0, cur.origin);
    if constexpr (!SPREAD && (kAblate & kAblateCopies) == 0) {
      if (j + 2 < total_tiles) issue_tile_load(kbase, ld_koff, sK_cur, t2.row0, t2.origin, KLayout{});
      if (j + 1 < total_tiles) issue_tile_load(vbase, ld_voff, sV_nxt, nxt.row0, nxt.origin, VLayout{});
    }

    // -- G1 ------------------------------------------------------------------------------------
    vec8 kf[N_QK];
    if constexpr (NXT) {
#pragma unroll
      for (int s = 0; s < PF_K; ++s) kf[s] = k_frag(sK_nxt, s);
    }
#pragma unroll
    for (int mb = 0; mb < MQ; ++mb) psum[mb][0] = psum[mb][1] = 0.f;
    auto g1_slot = [&](auto s_tag) __attribute__((always_inline)) {
      constexpr int s = decltype(s_tag)::value;
      if constexpr (NXT) {
        if constexpr (s + PF_K < N_QK) {
          if constexpr ((kAblate & kAblateLdsReads) == 0 || s + PF_K < 4) kf[s + PF_K] = k_frag(sK_nxt, s + PF_K);
          else kf[s + PF_K] = kf[(s + PF_K) % 4];
        }
#pragma unroll
        for (int mb = 0; mb < MQ; ++mb) {
          if constexpr (s % KSTEPS == 0) {
            S_nxt[mb][s / KSTEPS] = M::run_from(kf[s], qf[mb][s % KSTEPS], c_init[mb]);
          } else {
            S_nxt[mb][s / KSTEPS] = M::run(kf[s], qf[mb][s % KSTEPS], S_nxt[mb][s / KSTEPS]);
          }
        }
      }
      constexpr int e_lo = elems_done(s - 1), e_hi = elems_done(s);
      if constexpr (CUR && e_hi > e_lo) {
#pragma unroll
        for (int e = e_lo; e < e_hi; ++e) exp_elem(S_cur, e);
#pragma unroll
        for (int mb = 0; mb < MQ; ++mb) {
          pin(psum[mb][0]);
          pin(psum[mb][1]);
        }
      }
      if constexpr (SPREAD && (kAblate & kAblateCopies) == 0) {
        // 2 * PER copies spread over the first half of the slots, K first
        constexpr int c_lo = (s * 2 * PER * 2) / N_QK, c_hi = ((s + 1) * 2 * PER * 2) / N_QK;
        for_range<c_lo, c_hi - c_lo>([&](auto c_tag) {
          constexpr int c = decltype(c_tag)::value;
          if constexpr (c < PER) copy_one(std::integral_constant<int, c>{}, ck, ld_koff, KLayout{});
          else if constexpr (c < 2 * PER) copy_one(std::integral_constant<int, c - PER>{}, cv, ld_voff, VLayout{});
        });
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    // The wave runs these slots (the products of the coming tile, the tile copies, most of the
    // current tile's exponentials) at raised priority: when the two waves of a SIMD compete for
    // an issue slot, the one here wins over the one in its accumulation slots (measured: 3.5 %
    // off the kernel time; raising the priority elsewhere, or further, gains nothing).
    __builtin_amdgcn_s_setprio(1);
    for_range<0, N_QK>(g1_slot);
    __builtin_amdgcn_s_setprio(0);

    // -- G2 / G3 -------------------------------------------------------------------------------
    vec8 vf[N_PV];
    if constexpr (CUR) {
#pragma unroll
      for (int t = 0; t < PF_V; ++t) vf[t] = v_frag(sV_cur, t);
    }
    float mx[MQ][2];
#pragma unroll
    for (int mb = 0; mb < MQ; ++mb) mx[mb][0] = mx[mb][1] = -INFINITY;
    auto pv_slot = [&](auto t_tag) __attribute__((always_inline)) {
      constexpr int t = decltype(t_tag)::value;
      // the P fragment of this slot's 16-key block is complete
      static_assert(elems_done(N_QK + (t / DB) * DB - 1) >= MQ * 8 * (t / DB + 1), "exponentials scheduled too late");
      constexpr int x_lo = elems_done(N_QK + t - 1), x_hi = elems_done(N_QK + t);
      if constexpr (CUR) {
        if constexpr (t + PF_V < N_PV) {
          if constexpr ((kAblate & kAblateLdsReads) == 0 || t + PF_V < 4) vf[t + PF_V] = v_frag(sV_cur, t + PF_V);
          else vf[t + PF_V] = vf[(t + PF_V) % 4];
        }
#pragma unroll
        for (int mb = 0; mb < MQ; ++mb)
          acc[mb][t % DB] = M::run(vf[t], pf[mb][t / (2 * DB)][(t / DB) % 2], acc[mb][t % DB]);
        if constexpr (x_hi > x_lo) {
#pragma unroll
          for (int e = x_lo; e < x_hi; ++e) exp_elem(S_cur, e);
#pragma unroll
          for (int mb = 0; mb < MQ; ++mb) {
            pin(psum[mb][0]);
            pin(psum[mb][1]);
          }
        }
      }
      if constexpr (NXT && t >= N_PV / 2 && (kAblate & kAblateMax) == 0) {
        // row maxima of the coming tile (as if unmasked), MQ * NSB * 16 values over N_PV / 2 slots
        constexpr int t3 = t - N_PV / 2;
        constexpr int NV = MQ * NSB * 16;
        constexpr int e_lo = (t3 * NV) / (N_PV / 2), e_hi = ((t3 + 1) * NV) / (N_PV / 2);
#pragma unroll
        for (int e = e_lo; e < e_hi; ++e) {
          const int mb = e / (NSB * 16), i = e % (NSB * 16);
          mx[mb][i % 2] = fmaxf(mx[mb][i % 2], S_nxt[mb][i / 16][i % 16]);
        }
        if constexpr (e_hi > e_lo) {
#pragma unroll
          for (int mb = 0; mb < MQ; ++mb) {
            pin(mx[mb][0]);
            pin(mx[mb][1]);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    if constexpr (CUR || NXT) for_range<0, N_PV>(pv_slot);
    if constexpr (CUR) {
#pragma unroll
      for (int mb = 0; mb < MQ; ++mb) l_run[mb] += psum[mb][0] + psum[mb][1];
    }

    if ((kAblate & kAblateMax) == 0 && NXT && j + 1 < total_tiles) {
      float mxs[MQ];
#pragma unroll
      for (int mb = 0; mb < MQ; ++mb) mxs[mb] = fmaxf(mx[mb][0], mx[mb][1]);
      finish_logits(S_nxt, nxt, true, mxs);
    }
    cur = nxt;
    nxt = t2;
  };
  // A tile this wave has no use for (skip) is still multiplied and then masked entirely:
  // choosing the CUR / NXT variants per iteration at run time costs more registers than the
  // kernel has (the compiler no longer keeps the logits of both stages in place).
  for (int j = 0; j < total_tiles; j += 2) {
    iteration(Stage0{}, std::true_type{}, std::true_type{}, j);
    if (j + 1 < total_tiles) iteration(Stage1{}, std::true_type{}, std::true_type{}, j + 1);
  }
  wait_vmcnt<0>();  // the last iterations' copies into the unused stage must land before the LDS is released
  before_stores();

  // ---- epilogue: O = acc / rowsum, LSE = ln(rowsum) + scale * rowmax -------------------------
  T* obase = reinterpret_cast<T*>(p.o) + q_row_base * q_row_stride + int64_t(head) * D;
  float* lse_base = p.lse;
  if constexpr (SPLIT) {
    obase += split * p.o_split_stride;
    lse_base += split * p.lse_split_stride;
  }
#pragma unroll
  for (int mb = 0; mb < MQ; ++mb) {
    const float l = empty_split ? 0.f : l_run[mb] + __shfl_xor(l_run[mb], 32);
    const float inv = (l > 0.f) ? out_scale / l : 0.f;
    const int row = q_row[mb];
    if (row >= 0) {
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
        const float lse = (l > 0.f) ? (m_run[mb] * 0.6931471805599453f + __logf(l)) : -INFINITY;
        lse_base[(q_row_base + row) * p.heads_q + head] = lse;
      }
    }
  }
}

template <typename T, int D, int NWAVES, int MQ, bool RAGGED, int KVT, bool NOMASK = false>
__global__ void __launch_bounds__(NWAVES * 64) __attribute__((amdgpu_waves_per_eu(MQ == 1 ? 2 : 1, MQ == 1 ? 2 : 1)))
fna_fwd_kernel(const FnaParams p) {
  fna_fwd_tile<T, D, NWAVES, MQ, RAGGED, KVT, false, NOMASK>(p, int(blockIdx.x), []() {});
}

// Split launch: kv_splits workgroups per Q tile, each on a contiguous run of the tile's KV tiles,
// each storing a partial result; a two-way merge per extra split combines them.  For problems with
// fewer Q tiles than the chip keeps workgroups resident: a lone workgroup's tile loop is bound by
// its own instruction issue, not by anything it shares, so two on half the tiles each take about
// half the time.
template <typename T, int D, int NWAVES, int MQ, bool RAGGED, int KVT>
__global__ void __launch_bounds__(NWAVES * 64) __attribute__((amdgpu_waves_per_eu(MQ == 1 ? 2 : 1, MQ == 1 ? 2 : 1)))
fna_fwd_split_kernel(const FnaParams p) {
  fna_fwd_tile<T, D, NWAVES, MQ, RAGGED, KVT, true>(p, int(blockIdx.x), []() {});
}

// Work-queue launch: as many workgroups as the chip keeps resident, each taking Q tiles until
// none is left.  Workgroup i runs on XCD i % 8 (the dispatcher deals workgroups to XCDs in turn),
// and launch position `local * 8 + x` is what the one-tile-per-workgroup launch runs on XCD x:
// every XCD has a queue of its own over its `per_xcd` positions in the same order, so the tiles
// resident on an XCD share K/V in its L2 as before; a workgroup whose queue has run dry takes from
// the other XCDs' queues, which evens out the tail.  The protocol (counter layout, what a ticket
// means, who resets the counters) is work_queue.hpp's.

// The launch parameters of a work-queue kernel, read anew for every tile.  Left to itself the compiler
// hoists the set-up's reads of launch parameters (and what it derives from them) out of the loop
// over tiles and keeps them in scalar registers across the tile's main loop, whose own scalars then
// go to spill lanes.  A pointer to the kernel argument segment (the parameter block is the first
// argument) that passes through an empty asm statement per tile is a new value each time: the reads
// stay where the tile makes them, still as scalar loads from constant memory.
typedef const FnaParams __attribute__((address_space(4)))* FnaKernargPtr;
static __device__ __forceinline__ FnaKernargPtr fna_kernarg_params() {
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wold-style-cast"
  return (FnaKernargPtr)__builtin_amdgcn_kernarg_segment_ptr();
#pragma clang diagnostic pop
}
static __device__ __forceinline__ const FnaParams& fna_params_for_this_tile(FnaKernargPtr& args) {
  asm volatile("" : "+s"(args));
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wold-style-cast"
  return *(const FnaParams*)args;
#pragma clang diagnostic pop
}

// The loop of a resident workgroup: `tile(pid, fetch)` is run for every launch position the workgroup
// pulls, first from the queue of its own XCD, then from the others'.  `fetch` pulls the position after
// the current one; the tile calls it between its last KV tile and its stores, where the wave has
// nothing in flight, so that the wait for the counter's old value is a wait for that alone (issued
// after the stores it would also wait for their completion); a tile that returns without calling it
// has it called here.  All queue state lives in LDS: nothing of it occupies a register while a tile
// is worked on.
template <typename Tile>
static __device__ __forceinline__ void fna_queue_loop(uint32_t* __restrict__ queues, const int per_xcd, Tile&& tile) {
  __shared__ int s_pos[2];   // s_pos[i & 1]: position of the workgroup's i-th tile (-1: none is left)
  __shared__ int s_victim;   // queues found empty so far: the home queue first, then the others in turn
  const int home = int(blockIdx.x) % kNumXcd;
  // thread 0: the next position (-1: every queue is empty).  The wait for the counter's old value is
  // written out as a wait for everything outstanding rather than left to the compiler's count of
  // the operations it knows about: the tile copies are issued from assembly statements it does not see.
  // (Vector memory operations of a wave complete in issue order, so operations it does not count can
  // only make its counted waits longer, never shorter; a full wait does not depend on that either.)
  auto take = [&]() __attribute__((always_inline)) {
    int victim = s_victim, pos = -1;
    while (victim < kNumXcd) {
      const uint32_t ticket = atomicAdd(&queues[queue_counter_word(home, victim)], 1u);
      wait_vmcnt<0>();
      pos = queue_position(home, victim, ticket, per_xcd);  // an empty queue counts into `victim`
      if (pos >= 0) break;
    }
    s_victim = victim;
    return pos;
  };
  if (threadIdx.x == 0) {
    s_victim = 0;
    s_pos[0] = take();
  }
  for (int i = 0;; i ^= 1) {
    // s_pos[i] is written, everyone has read s_pos[i ^ 1] and is done with the LDS of the previous tile
    workgroup_sync();
    const int pid = __builtin_amdgcn_readfirstlane(s_pos[i]);
    if (pid < 0) break;
    bool fetched = false;
    auto fetch = [&]() __attribute__((always_inline)) {
      if (threadIdx.x == 0) s_pos[i ^ 1] = take();
      fetched = true;
    };
    tile(pid, fetch);
    if (!fetched) fetch();
  }
  // The last workgroup to leave puts the counters back to zero, so that the next launch finds them
  // as it needs them.  (Every other workgroup has seen all queues empty by then: its counter
  // increments, whose old values it waited for, are complete.)
  if (threadIdx.x == 0) {
    const uint32_t left = atomicAdd(&queues[kQueueDoneWord], 1u);
    if (queue_last_one_out(left, gridDim.x)) {
      for (int x = 0; x < kNumXcd; ++x) __hip_atomic_store(&queues[x * kQueueStride], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&queues[kQueueDoneWord], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

template <typename T, int D, int NWAVES, int MQ, bool RAGGED, int KVT, bool NOMASK = false>
__global__ void __launch_bounds__(NWAVES * 64) __attribute__((amdgpu_waves_per_eu(MQ == 1 ? 2 : 1, MQ == 1 ? 2 : 1)))
fna_fwd_queue_kernel(const FnaParams p, uint32_t* __restrict__ queues, const int per_xcd) {
  FnaKernargPtr args = fna_kernarg_params();
  fna_queue_loop(queues, per_xcd, [&](int pid, auto& fetch) __attribute__((always_inline)) {
    fna_fwd_tile<T, D, NWAVES, MQ, RAGGED, KVT, false, NOMASK>(fna_params_for_this_tile(args), pid, fetch);
  });
  (void)p;
}

// clears the queue counters (a kernel rather than a memset so that callers may capture the launch pair in a graph)
__global__ void fna_queue_clear_kernel(uint32_t* queues) {
  if (threadIdx.x < kQueueWords) queues[threadIdx.x] = 0;
}

// ---- host side of the launch geometry (kept with the kernels: the two must agree) -----------------

// Workgroup layout: Q tiles are enumerated with dimension 0 slowest; a group is a run of about
// as many consecutive Q tiles as one XCD keeps resident (32 CUs x 2 workgroups), made of whole
// dimension-0 slabs when possible, so that the tiles resident on an XCD overlap in their KV boxes.
// `tiles_per_wg` Q tiles share a workgroup (consecutive tiles of the enumeration) and an XCD keeps
// about 64 Q tiles resident either way (32 CUs x 2 single-tile workgroups or x 1 two-tile workgroup).
// The box of 32 queries that a wave holds (FnaParams::wave_box_lg).  A (wave, KV tile) pair needs
// the element mask unless the tile lies inside the windows of all of the wave's queries or outside
// all of them, and both conditions factor over the dimensions: the number of pairs that need none is
// a product of per-dimension sums over Q tiles, boxes and KV tiles, cheap to count on the host with
// the kernels' own window and box arithmetic.  Of the boxes that fit the Q tile the one with the
// fewest pairs that need the mask is taken; the row-major box (as much of dimension 2 as fits, then
// dimension 1, then 0) on ties, and for sequence-packed launches, whose extents only the device knows.
inline void choose_wave_box(FnaParams& p) {
  int best[3], left = 5;
  for (int a = 2; a >= 0; --a) {
    best[a] = p.q_tile_lg[a] < left ? p.q_tile_lg[a] : left;
    left -= best[a];
  }
  for (int a = 0; a < 3; ++a) p.wave_box_lg[a] = best[a];
  if (p.cu_q) return;
  // the boxes that fit the Q tile; with one (every 1-D problem) there is nothing to choose
  int cand[21][3], n_cand = 0;
  for (int w0 = 0; w0 <= 5 && w0 <= p.q_tile_lg[0]; ++w0)
    for (int w1 = 0; w0 + w1 <= 5 && w1 <= p.q_tile_lg[1]; ++w1) {
      const int w2 = 5 - w0 - w1;
      if (w2 > p.q_tile_lg[2]) continue;
      cand[n_cand][0] = w0;
      cand[n_cand][1] = w1;
      cand[n_cand][2] = w2;
      ++n_cand;
    }
  if (n_cand <= 1) return;
  // the same geometry as the call before (a model calls a layer over and over): the same answer
  struct Key {
    int v[3][7];
    int anchor;
    bool operator==(const Key& o) const { return memcmp(this, &o, sizeof(Key)) == 0; }
  };
  Key key;
  memset(&key, 0, sizeof(key));
  for (int a = 0; a < 3; ++a) {
    const int vals[7] = {p.ext_base[a], p.ext_rem[a], p.ksize[a], p.stride[a], p.causal[a], p.q_tile[a], p.kv_tile[a]};
    for (int i = 0; i < 7; ++i) key.v[a][i] = vals[i];
  }
  key.anchor = p.anchor;
  thread_local Key last_key;
  thread_local int last_box[3] = {-1, -1, -1};
  if (last_box[0] >= 0 && key == last_key) {
    for (int a = 0; a < 3; ++a) p.wave_box_lg[a] = last_box[a];
    return;
  }
  // per dimension and box extent: (wave box, KV tile) pairs attended in full / attended at all,
  // summed over the Q tiles (tile counts in closed form: the cost is Q tiles x boxes per dimension)
  double full[3][6], some[3][6];
  for (int a = 0; a < 3; ++a) {
    const int L = p.ext_base[a] + (p.ext_rem[a] ? 1 : 0), kt = p.kv_tile[a], qt = p.q_tile[a];
    const bool causal = p.causal[a] != 0;
    for (int wb = 0; wb <= 5; ++wb) {
      full[a][wb] = some[a][wb] = 0;
      if (wb > p.q_tile_lg[a]) continue;
      const int box = 1 << wb;
      for (int q0 = 0; q0 < L; q0 += qt) {
        const int q_last = na_min(q0 + qt - 1, L - 1);
        const int st_f = na_window_start(q0, p.ksize[a], p.stride[a], L, causal);
        const int st_l = na_window_start(q_last, p.ksize[a], p.stride[a], L, causal);
        const int en_l = na_window_end(q_last, st_l, p.ksize[a], L, causal);
        const int org = (p.anchor && L >= kt) ? st_f : (st_f / kt) * kt;
        const int tiles = (en_l - org + kt - 1) / kt;
        for (int b0 = 0; b0 < qt; b0 += box) {
          const int qmin = na_min(q0 + b0, L - 1), qmax = na_min(q0 + b0 + box - 1, L - 1);
          const int st_min = na_window_start(qmin, p.ksize[a], p.stride[a], L, causal);
          const int st_max = na_window_start(qmax, p.ksize[a], p.stride[a], L, causal);
          const int en_min = na_window_end(qmin, st_min, p.ksize[a], L, causal);
          const int en_max = na_window_end(qmax, st_max, p.ksize[a], L, causal);
          // tile t covers [org + t kt, org + (t + 1) kt).  Attended in full: it starts at or after
          // st_max and ends at or before min(en_min, L).  Attended at all: it ends after st_min and
          // starts before en_max.  (org <= st_min: the box starts at or before every window.)
          const int f_lo = (st_max - org + kt - 1) / kt, f_hi = na_min((na_min(en_min, L) - org) / kt, tiles);
          const int s_lo = (st_min - org) / kt, s_hi = na_min((en_max - org + kt - 1) / kt, tiles);
          full[a][wb] += na_max(f_hi - f_lo, 0);
          some[a][wb] += na_max(s_hi - s_lo, 0);
        }
      }
    }
  }
  auto masked = [&](const int* w) {
    return some[0][w[0]] * some[1][w[1]] * some[2][w[2]] - full[0][w[0]] * full[1][w[1]] * full[2][w[2]];
  };
  double best_masked = masked(best);
  for (int c = 0; c < n_cand; ++c) {
    const double m = masked(cand[c]);
    if (m < best_masked * 0.9999999 - 0.5) {
      best_masked = m;
      for (int a = 0; a < 3; ++a) p.wave_box_lg[a] = cand[c][a];
    }
  }
  last_key = key;
  for (int a = 0; a < 3; ++a) last_box[a] = p.wave_box_lg[a];
}

inline void set_wg_layout(FnaParams& p, int tiles_per_wg = 1) {
  p.num_q_tiles = p.q_tiled[0] * p.q_tiled[1] * p.q_tiled[2];
  const int slab = p.q_tiled[1] * p.q_tiled[2];
  int rows = (64 + slab / 2) / slab;
  if (rows < 1) rows = 1;
  if (rows > p.q_tiled[0]) rows = p.q_tiled[0];
  const int units = (p.num_q_tiles + tiles_per_wg - 1) / tiles_per_wg;
  p.wg_group = (slab * rows + tiles_per_wg - 1) / tiles_per_wg;
  if (p.wg_group > units) p.wg_group = units;
  // Few tiles in all (one head, a small input): groups of that size would leave XCDs without work
  // while others hold several workgroups per CU; smaller groups give every XCD its share.
  const long long bh = (long long)p.batch * p.heads_q;
  if (bh * ((units + p.wg_group - 1) / p.wg_group) < kNumXcd) {
    int want = int((kNumXcd + bh - 1) / bh);  // groups per (batch, head) pair
    if (want > units) want = units;
    p.wg_group = (units + want - 1) / want;
  }
  p.groups_per_bh = (units + p.wg_group - 1) / p.wg_group;
  p.total_groups = p.batch * p.heads_q * p.groups_per_bh;
  // what the kernels' set-up would otherwise divide for (every forward launch comes through here)
  for (int a = 0; a < 3; ++a) {
    p.q_tile_lg[a] = p.kv_tile_lg[a] = 0;
    while ((1 << p.q_tile_lg[a]) < p.q_tile[a]) ++p.q_tile_lg[a];
    while ((1 << p.kv_tile_lg[a]) < p.kv_tile[a]) ++p.kv_tile_lg[a];
    p.ext_base[a] = p.qkv_shape[a] / p.dil[a];
    p.ext_rem[a] = p.qkv_shape[a] % p.dil[a];
    p.d_stride[a] = na_make_div(p.stride[a]);
    p.d_dil[a] = na_make_div(p.dil[a]);
    p.d_q_tiled[a] = na_make_div(p.q_tiled[a]);
  }
  choose_wave_box(p);
  p.d_wg_group = na_make_div(p.wg_group);
  p.d_groups_per_bh = na_make_div(p.groups_per_bh);
  p.d_heads_q = na_make_div(p.heads_q);
  p.d_q_per_kv = na_make_div(p.heads_q / p.heads_kv);
  p.d_num_groups = na_make_div(p.num_groups);
}

// tile extents must be powers of two (every factorisation of the supported token counts is)
inline bool fna_tiles_are_powers_of_two(const FnaParams& p) {
  for (int a = 0; a < 3; ++a)
    if ((p.q_tile[a] & (p.q_tile[a] - 1)) || (p.kv_tile[a] & (p.kv_tile[a] - 1))) return false;
  return true;
}

}  // namespace natten_amd
