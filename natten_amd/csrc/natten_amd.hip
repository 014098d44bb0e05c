// C ABI of the MI355X fused neighborhood attention forward path (see include/natten_amd.h).
// Host-side argument validation, kernel selection and launches; no framework types.

#include "../../include/natten_amd.h"

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>
#include <type_traits>

#include "fna_bwd.hpp"
#include "fna_fwd.hpp"
#include "fna_fwd_f32.hpp"
#include "fna_fwd_fp8.hpp"
#include "merge.hpp"
#include "mfma_probe.hpp"
#include "na_math.hpp"
#include "tokperm.hpp"

using namespace natten_amd;

// Queue counters of natten_amd_fna_forward_fused_static, the entry point for callers that cannot
// allocate: every GPU the library runs on holds this array (512 bytes) until the process ends.
// The name is a host-side stand-in, not a device address: host code only ever uses the
// per-device address hipGetSymbolAddress returns for it (static_scratch()).  No `used`
// attribute: the compiler gives the device-side symbol external binding because host code names
// it, and with the attribute it stays local, where the runtime's lookup by name cannot find it.
static __device__ __align__(256) uint32_t scratch[kQueueWords];

namespace {

thread_local char g_error[512] = "";

int fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return 1;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail("%s: launch failed: %s", what, hipGetErrorString(e));
  return 0;
}

int prod3(const int* x) { return x[0] * x[1] * x[2]; }

struct TileConfig {
  int q_tile, kv_tile;
};

// (Q tile, KV tile) sizes in tokens that have a kernel instance.
const TileConfig kTileConfigs[] = {{128, 64}, {256, 64}, {64, 64}};
constexpr int kNumTileConfigs = sizeof(kTileConfigs) / sizeof(kTileConfigs[0]);

// Workgroups a work-queue launch starts: two per compute unit (what the kernel's LDS and register
// use keep resident), a multiple of the XCD count; the device's figure is read once.
int resident_workgroups() {
  static std::atomic<int> cached[64] = {};  // (threads that race here compute the same value)
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 512;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) cus = 256;
    n = (2 * cus / kNumXcd) * kNumXcd;
    if (n < kNumXcd) n = kNumXcd;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// The counters of a work-queue launch (null: one workgroup per Q tile).  Every work-queue kernel
// leaves the counters at zero when its last workgroup ends; `clear_first` clears them by a kernel
// before the launch, for memory whose contents are not known.
struct WorkQueue {
  uint32_t* counters = nullptr;
  bool clear_first = true;
};

template <typename T, int D, int NWAVES, int MQ, bool RAGGED, int KVT, bool NOMASK = false>
int launch_fna(const FnaParams& p, hipStream_t stream, WorkQueue queues = {}) {
  constexpr int QT = NWAVES * MQ * 32;
  if (!fna_tiles_are_powers_of_two(p)) return fail("fna_forward: tile extents must be powers of two");
  if ((p.seqlen_q + QT - 1) / QT != p.num_q_tiles) return fail("fna_forward: internal tile count mismatch");
  const long long wgs = (long long)((p.total_groups + kNumXcd - 1) / kNumXcd) * kNumXcd * p.wg_group;
  if (wgs > 0x7fffffffLL) return fail("fna_forward: problem needs more than 2^31 workgroups");
  if (queues.counters != nullptr) {
    const long long resident = resident_workgroups();
    if (queues.clear_first) hipLaunchKernelGGL(fna_queue_clear_kernel, dim3(1), dim3(kQueueWords), 0, stream, queues.counters);
    hipLaunchKernelGGL((fna_fwd_queue_kernel<T, D, NWAVES, MQ, RAGGED, KVT, NOMASK>),
                       dim3((unsigned)(wgs < resident ? wgs : resident)), dim3(NWAVES * 64), 0, stream, p, queues.counters,
                       int(wgs / kNumXcd));
    return check_launch("fna_forward (work queue)");
  }
  if (p.kv_splits > 1) {
    // kv_splits workgroups per Q-tile position, split slowest (positions keep their XCDs: wgs is a multiple of 8)
    if constexpr (NWAVES == 4 && MQ == 1 && KVT == 64) {
      if (wgs * p.kv_splits > 0x7fffffffLL) return fail("fna_forward: problem needs more than 2^31 workgroups");
      FnaParams ps = p;
      ps.split_grid = int(wgs);
      hipLaunchKernelGGL((fna_fwd_split_kernel<T, D, NWAVES, MQ, RAGGED, KVT>), dim3((unsigned)(wgs * p.kv_splits)),
                         dim3(NWAVES * 64), 0, stream, ps);
      return check_launch("fna_forward (split)");
    } else {
      return fail("fna_forward: KV splits exist for Q tiles of 128 and KV tiles of 64 tokens");
    }
  }
  hipLaunchKernelGGL((fna_fwd_kernel<T, D, NWAVES, MQ, RAGGED, KVT, NOMASK>), dim3((unsigned)wgs), dim3(NWAVES * 64), 0, stream,
                     p);
  return check_launch("fna_forward");
}

// Whether the launch is fully block-sparse: every Q tile is whole (no padding queries), all its
// queries share one window in every dimension, and the KV tiles laid out for it cover that window
// exactly, so that every (Q tile, KV tile) pair the kernel visits is attended in full and the
// instance without any mask code gives the same bits.  The role of the reference's
// fully_block_sparse (csrc/include/natten/cuda/fna_blackwell/collective/fna_fusion.hpp:503-593),
// evaluated from the kernel's own window and box arithmetic.  Needs set_wg_layout() to have run.
bool fully_block_sparse(const FnaParams& p) {
  if (p.cu_q != nullptr || p.edge != 0 || p.kv_splits > 1) return false;
  for (int a = 0; a < 3; ++a) {
    // dilation groups come in at most two extents
    for (int ext = p.ext_base[a] + (p.ext_rem[a] > 0 ? 1 : 0); ext >= p.ext_base[a]; --ext) {
      if (ext < 1 || ext % p.q_tile[a] != 0) return false;
      const bool c = p.causal[a] != 0;
      for (int qf = 0; qf < ext; qf += p.q_tile[a]) {
        const int ql = qf + p.q_tile[a] - 1;
        const int st_f = na_window_start(qf, p.ksize[a], p.stride[a], p.d_stride[a], ext, c);
        const int st_l = na_window_start(ql, p.ksize[a], p.stride[a], p.d_stride[a], ext, c);
        const int en_f = na_window_end(qf, st_f, p.ksize[a], ext, c);
        const int en_l = na_window_end(ql, st_l, p.ksize[a], ext, c);
        // (start and end are monotone in the query: equal at both ends means equal throughout)
        if (st_f != st_l || en_f != en_l) return false;
        const int org = p.anchor ? st_f : ((st_f >> p.kv_tile_lg[a]) << p.kv_tile_lg[a]);
        if (org != st_f || (en_l - org) % p.kv_tile[a] != 0) return false;
      }
    }
  }
  return true;
}

template <bool E5M2, int D, bool NOMASK>
int launch_fna_fp8_instance(const FnaParams& p, hipStream_t stream, WorkQueue queues) {
  constexpr int QT = 128;
  if (!fna_tiles_are_powers_of_two(p)) return fail("fna_forward: tile extents must be powers of two");
  if ((p.seqlen_q + QT - 1) / QT != p.num_q_tiles) return fail("fna_forward: internal tile count mismatch");
  const long long wgs = (long long)((p.total_groups + kNumXcd - 1) / kNumXcd) * kNumXcd * p.wg_group;
  if (wgs > 0x7fffffffLL) return fail("fna_forward: problem needs more than 2^31 workgroups");
  if (queues.counters != nullptr) {
    const long long resident = resident_workgroups();
    if (queues.clear_first) hipLaunchKernelGGL(fna_queue_clear_kernel, dim3(1), dim3(kQueueWords), 0, stream, queues.counters);
    hipLaunchKernelGGL((fna_fwd_fp8_queue_kernel<E5M2, D, 4, NOMASK>), dim3((unsigned)(wgs < resident ? wgs : resident)),
                       dim3(256), 0, stream, p, queues.counters, int(wgs / kNumXcd));
    return check_launch("fna_forward (work queue)");
  }
  hipLaunchKernelGGL((fna_fwd_fp8_kernel<E5M2, D, 4, NOMASK>), dim3((unsigned)wgs), dim3(256), 0, stream, p);
  return check_launch("fna_forward");
}

template <bool E5M2, int D>
int launch_fna_fp8(const FnaParams& p, hipStream_t stream, WorkQueue queues) {
  if (fully_block_sparse(p)) return launch_fna_fp8_instance<E5M2, D, true>(p, stream, queues);
  return launch_fna_fp8_instance<E5M2, D, false>(p, stream, queues);
}

template <typename T, int D>
int dispatch_tiles(const FnaParams& p, int qt, int kvt, hipStream_t stream, WorkQueue queues) {
  if (p.seqlen_kv % kvt != 0 || p.cu_q != nullptr || p.edge == 2) {
    // key sequences that end inside a tile: dense attention on unpadded or packed sequences only
    if (qt == 128 && kvt == 64) return launch_fna<T, D, 4, 1, true, 64>(p, stream);
    return fail("fna_forward: seqlen_kv (%d) must be a multiple of the KV tile (%d tokens)", p.seqlen_kv, kvt);
  }
  // the work-queue launch exists for the default tile pair; the others launch a workgroup per Q tile
  if (qt == 128 && kvt == 64) {
    if (fully_block_sparse(p)) return launch_fna<T, D, 4, 1, false, 64, true>(p, stream, queues);
    return launch_fna<T, D, 4, 1, false, 64>(p, stream, queues);
  }
  if (qt == 256 && kvt == 64) return launch_fna<T, D, 8, 1, false, 64>(p, stream);
  if (qt == 64 && kvt == 64) return launch_fna<T, D, 2, 1, false, 64>(p, stream);
  return fail("fna_forward: no kernel for Q tile of %d and KV tile of %d tokens", qt, kvt);
}

template <typename T>
int dispatch_head_dim(const FnaParams& p, int head_dim, int qt, int kvt, hipStream_t stream, WorkQueue queues) {
  switch (head_dim) {
    case 32: return dispatch_tiles<T, 32>(p, qt, kvt, stream, queues);
    case 64: return dispatch_tiles<T, 64>(p, qt, kvt, stream, queues);
    case 128: return dispatch_tiles<T, 128>(p, qt, kvt, stream, queues);
  }
  return fail("fna_forward: head_dim must be 32, 64 or 128, got %d", head_dim);
}

int dispatch_dtype(const FnaParams& p, int dtype, int head_dim, int qt, int kvt, hipStream_t stream,
                   WorkQueue queues = {}) {
  switch (dtype) {
    case NATTEN_AMD_F16: return dispatch_head_dim<_Float16>(p, head_dim, qt, kvt, stream, queues);
    case NATTEN_AMD_BF16: return dispatch_head_dim<__bf16>(p, head_dim, qt, kvt, stream, queues);
  }
  if (p.kv_splits > 1) return fail("fna_forward: KV splits need fp16 / bf16 operands, got dtype code %d", dtype);
  if (dtype == NATTEN_AMD_F8E4M3 || dtype == NATTEN_AMD_F8E5M2) {
    // 8-bit float operands, bf16 output: one kernel configuration
    if (qt != 128 || kvt != 64)
      return fail("fna_forward: 8-bit float operands need a Q tile of 128 and a KV tile of 64 tokens, got %d and %d", qt,
                  kvt);
    if (p.seqlen_kv % kvt != 0)
      return fail("fna_forward: seqlen_kv (%d) must be a multiple of the KV tile (%d tokens)", p.seqlen_kv, kvt);
    if (head_dim != 64 && head_dim != 128)
      return fail("fna_forward: 8-bit float operands need head_dim 64 or 128, got %d", head_dim);
    const bool e5m2 = dtype == NATTEN_AMD_F8E5M2;
    if (head_dim == 128)
      return e5m2 ? launch_fna_fp8<true, 128>(p, stream, queues) : launch_fna_fp8<false, 128>(p, stream, queues);
    return e5m2 ? launch_fna_fp8<true, 64>(p, stream, queues) : launch_fna_fp8<false, 64>(p, stream, queues);
  }
  if (dtype == NATTEN_AMD_F32) {
    // float32 operands and output: one plain kernel configuration on token-permuted sequences
    if (qt != 128 || kvt != 64)
      return fail("fna_forward: float32 operands need a Q tile of 128 and a KV tile of 64 tokens, got %d and %d", qt, kvt);
    if (p.fused || p.cu_q != nullptr) return fail("fna_forward: float32 operands run on token-permuted sequences only");
    if (p.seqlen_kv % kvt != 0)
      return fail("fna_forward: seqlen_kv (%d) must be a multiple of the KV tile (%d tokens)", p.seqlen_kv, kvt);
    if (p.q_scale || p.k_scale || p.v_scale) return fail("fna_forward: float32 operands take no dequantisation scales");
    if ((p.seqlen_q + qt - 1) / qt != p.num_q_tiles) return fail("fna_forward: internal tile count mismatch");
    const long long wgs = (long long)p.num_q_tiles * p.heads_q * p.batch;
    if (wgs > 0x7fffffffLL) return fail("fna_forward: problem needs more than 2^31 workgroups");
    switch (head_dim) {
      case 32: hipLaunchKernelGGL((fna_fwd_f32_kernel<32>), dim3((unsigned)wgs), dim3(256), 0, stream, p); break;
      case 64: hipLaunchKernelGGL((fna_fwd_f32_kernel<64>), dim3((unsigned)wgs), dim3(256), 0, stream, p); break;
      case 128: hipLaunchKernelGGL((fna_fwd_f32_kernel<128>), dim3((unsigned)wgs), dim3(256), 0, stream, p); break;
      default: return fail("fna_forward: unsupported head_dim %d", head_dim);
    }
    return check_launch("fna_forward (float32)");
  }
  return fail("fna_forward: unsupported dtype code %d", dtype);
}

int check_common(const char* what, const void* q, const void* k, const void* v, const void* out, const float* lse,
                 int batch, int seqlen_q, int seqlen_kv, int heads_q, int heads_kv, int head_dim) {
  if (!q || !k || !v || !out || !lse) return fail("%s: null pointer argument", what);
  if (batch < 1 || seqlen_q < 1 || seqlen_kv < 1 || heads_q < 1 || heads_kv < 1)
    return fail("%s: batch, sequence lengths and head counts must be positive", what);
  if (heads_q % heads_kv != 0)
    return fail("%s: heads_kv (%d) must divide heads_q (%d)", what, heads_kv, heads_q);
  if (head_dim != 32 && head_dim != 64 && head_dim != 128)
    return fail("%s: head_dim must be 32, 64 or 128, got %d", what, head_dim);
  if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
       reinterpret_cast<uintptr_t>(out)) & 15)
    return fail("%s: q, k, v and out must be 16-byte aligned", what);
  return 0;
}

// Shared by the permuted and the fused entry points: checks the neighborhood parameters and fills
// everything but the operand layout.  q_shape / kv_shape: padded per-group token layouts.
int fill_fna_params(const char* what, FnaParams& p, int na_dim, const int* q_shape, const int* kv_shape,
                    const int32_t* qkv_shape, const int32_t* kernel_size, const int32_t* stride,
                    const int32_t* dilation, const int32_t* is_causal, const int32_t* q_tile_shape,
                    const int32_t* kv_tile_shape) {
  memset(&p, 0, sizeof(p));
  p.num_groups = 1;
  for (int a = 0; a < 3; ++a) {
    const bool used = a < na_dim;
    p.qkv_shape[a] = used ? qkv_shape[a] : 1;
    p.ksize[a] = used ? kernel_size[a] : 1;
    p.stride[a] = used ? stride[a] : 1;
    p.dil[a] = used ? dilation[a] : 1;
    p.causal[a] = used ? (is_causal[a] != 0) : 0;
    p.q_tile[a] = used ? q_tile_shape[a] : 1;
    p.kv_tile[a] = used ? kv_tile_shape[a] : 1;
    const int qs = used ? q_shape[a] : 1, ks = used ? kv_shape[a] : 1;
    if (p.qkv_shape[a] < 1 || p.dil[a] < 1 || p.stride[a] < 1 || p.q_tile[a] < 1 || p.kv_tile[a] < 1 ||
        (used && p.ksize[a] < 2))
      return fail("%s: invalid parameter along dimension %d", what, a);
    if (p.ksize[a] * p.dil[a] > p.qkv_shape[a])
      return fail("%s: kernel_size * dilation exceeds the input along dimension %d (%d * %d > %d)", what, a,
                  p.ksize[a], p.dil[a], p.qkv_shape[a]);
    if (p.stride[a] > p.ksize[a])
      return fail("%s: stride exceeds kernel_size along dimension %d (%d > %d)", what, a, p.stride[a], p.ksize[a]);
    if (qs % p.q_tile[a] != 0 || ks % p.kv_tile[a] != 0)
      return fail("%s: padded layouts must be multiples of the tile shapes (dimension %d)", what, a);
    const int need = na_ceil_div(p.qkv_shape[a], p.dil[a]);
    if (qs < need || ks < need)
      return fail("%s: q_shape / kv_shape smaller than the dilation group extent along dimension %d", what, a);
    if (p.kv_tile[a] > 512) return fail("%s: KV tile extent above 512 along dimension %d", what, a);
    p.q_tiled[a] = qs / p.q_tile[a];
    p.kv_tiled[a] = ks / p.kv_tile[a];
    p.num_groups *= p.dil[a];
  }
  p.tok_stride[2] = 1;
  p.tok_stride[1] = p.qkv_shape[2];
  p.tok_stride[0] = p.qkv_shape[2] * p.qkv_shape[1];
  return 0;
}

// The queue counters of a work-queue launch inside the caller's workspace (nullptr: launch a
// workgroup per Q tile).  rc != 0 on a workspace that cannot hold them.
int queue_workspace(const char* what, int run_persistent, void* workspace, uint64_t workspace_bytes, WorkQueue* queues) {
  *queues = WorkQueue{};
  if (!run_persistent) return 0;
  if (run_persistent != 1 && run_persistent != 2) return fail("%s: run_persistent must be 0, 1 or 2, got %d", what, run_persistent);
  if (!workspace || workspace_bytes < uint64_t(kQueueWords) * 4 || (reinterpret_cast<uintptr_t>(workspace) & 63))
    return fail("%s: run_persistent needs a 64-byte aligned device workspace of at least %d bytes (got %p, %llu bytes)", what,
                kQueueWords * 4, workspace, (unsigned long long)workspace_bytes);
  queues->counters = static_cast<uint32_t*>(workspace);
  queues->clear_first = run_persistent == 1;  // 2: the caller vouches for zeros (what every launch leaves behind)
  return 0;
}

int fused_geometry(const char* what, FnaParams& p, bool sixteen_bit, int na_dim, int heads_kv, int head_dim,
                   const int32_t* qkv_shape, const int32_t* kernel_size, const int32_t* stride, const int32_t* dilation,
                   const int32_t* is_causal, const int32_t* q_tile_shape, const int32_t* kv_tile_shape, int anchor_kv_tiles,
                   long long* tokens_out);
}  // namespace

extern "C" {

int natten_amd_abi_version(void) { return 16; }

uint64_t natten_amd_fna_forward_workspace_bytes(void) { return uint64_t(kQueueWords) * 4; }

const char* natten_amd_last_error(void) { return g_error; }

int natten_amd_window(int query, int kernel_size, int stride, int extent, int is_causal, int32_t* start, int32_t* end) {
  g_error[0] = 0;
  if (!start || !end) return fail("window: null pointer argument");
  if (query < 0 || kernel_size < 1 || stride < 1 || extent < 1)
    return fail("window: query >= 0, kernel_size, stride and extent >= 1 expected");
  // the arithmetic the kernels' set-up runs: stride division by multiply and shift
  *start = na_window_start(query, kernel_size, stride, na_make_div(stride), extent, is_causal != 0);
  *end = na_window_end(query, *start, kernel_size, extent, is_causal != 0);
  return 0;
}

int natten_amd_tile_key_mask(const int32_t* kv_tile_shape, const int32_t* lo, const int32_t* hi, uint64_t* mask) {
  g_error[0] = 0;
  if (!kv_tile_shape || !lo || !hi || !mask) return fail("tile_key_mask: null pointer argument");
  int lg[3], keys = 1;
  for (int a = 0; a < 3; ++a) {
    lg[a] = 0;
    while ((1 << lg[a]) < kv_tile_shape[a]) ++lg[a];
    if (kv_tile_shape[a] < 1 || (1 << lg[a]) != kv_tile_shape[a])
      return fail("tile_key_mask: tile extents must be powers of two, got %d", kv_tile_shape[a]);
    if (lo[a] < 0 || hi[a] < 0 || lo[a] > kv_tile_shape[a] || hi[a] > kv_tile_shape[a])
      return fail("tile_key_mask: bounds must lie in 0 .. extent along dimension %d", a);
    keys *= kv_tile_shape[a];
  }
  if (keys != 64) return fail("tile_key_mask: the tile must hold 64 keys, got %d", keys);
  // the rows the kernels keep in LDS (per half of the wave: the bits its lanes hold logits for) and
  // how their element mask combines them
  uint32_t half[2] = {~uint32_t(0), ~uint32_t(0)};
  int lg_stride = 0;
  for (int a = 0; a < 3; ++a) {
    for (int g = 0; g < 2; ++g)
      half[g] &= na_lane_half_bits(na_keys_at_or_after(lo[a], lg_stride, lg[a]), g) &
                 ~na_lane_half_bits(na_keys_at_or_after(hi[a], lg_stride, lg[a]), g);
    lg_stride += lg[a];
  }
  *mask = na_keys_of_lane_halves(half[0], half[1]);
  return 0;
}

int natten_amd_fna_fully_block_sparse(int na_dim, const int32_t* qkv_shape, const int32_t* kernel_size,
                                      const int32_t* stride, const int32_t* dilation, const int32_t* is_causal,
                                      const int32_t* q_tile_shape, const int32_t* kv_tile_shape, int anchor_kv_tiles,
                                      int32_t* result) {
  g_error[0] = 0;
  if (na_dim < 1 || na_dim > 3) return fail("fna_fully_block_sparse: na_dim must be 1, 2 or 3, got %d", na_dim);
  if (!result) return fail("fna_fully_block_sparse: null pointer argument");
  FnaParams p;
  long long tokens = 0;
  if (int rc = fused_geometry("fna_fully_block_sparse", p, true, na_dim, 1, 32, qkv_shape, kernel_size, stride, dilation,
                              is_causal, q_tile_shape, kv_tile_shape, anchor_kv_tiles, &tokens))
    return rc;
  p.batch = p.num_groups;
  p.heads_q = p.heads_kv = 1;
  set_wg_layout(p, 1);
  *result = fully_block_sparse(p) ? 1 : 0;
  return 0;
}

int natten_amd_fna_wave_box(int na_dim, const int32_t* qkv_shape, const int32_t* kernel_size, const int32_t* stride,
                            const int32_t* dilation, const int32_t* is_causal, const int32_t* q_tile_shape,
                            const int32_t* kv_tile_shape, int anchor_kv_tiles, int32_t* box) {
  g_error[0] = 0;
  if (na_dim < 1 || na_dim > 3) return fail("fna_wave_box: na_dim must be 1, 2 or 3, got %d", na_dim);
  if (!box) return fail("fna_wave_box: null pointer argument");
  FnaParams p;
  long long tokens = 0;
  if (int rc = fused_geometry("fna_wave_box", p, true, na_dim, 1, 32, qkv_shape, kernel_size, stride, dilation, is_causal,
                              q_tile_shape, kv_tile_shape, anchor_kv_tiles, &tokens))
    return rc;
  p.batch = p.num_groups;
  p.heads_q = p.heads_kv = 1;
  set_wg_layout(p, 1);
  for (int a = 0; a < na_dim; ++a) box[a] = 1 << p.wave_box_lg[a];
  return 0;
}

int natten_amd_fna_supported_tiles(int dtype, int head_dim, int32_t* q_sizes, int32_t* kv_sizes, int capacity) {
  if (dtype == NATTEN_AMD_F8E4M3 || dtype == NATTEN_AMD_F8E5M2) {
    if (head_dim != 64 && head_dim != 128) return 0;
    if (capacity > 0 && q_sizes) q_sizes[0] = 128;
    if (capacity > 0 && kv_sizes) kv_sizes[0] = 64;
    return 1;
  }
  if (dtype == NATTEN_AMD_F32) {
    if (head_dim != 32 && head_dim != 64 && head_dim != 128) return 0;
    if (capacity > 0 && q_sizes) q_sizes[0] = 128;
    if (capacity > 0 && kv_sizes) kv_sizes[0] = 64;
    return 1;
  }
  if (dtype != NATTEN_AMD_F16 && dtype != NATTEN_AMD_BF16) return 0;
  if (head_dim != 32 && head_dim != 64 && head_dim != 128) return 0;
  for (int i = 0; i < kNumTileConfigs && i < capacity; ++i) {
    if (q_sizes) q_sizes[i] = kTileConfigs[i].q_tile;
    if (kv_sizes) kv_sizes[i] = kTileConfigs[i].kv_tile;
  }
  return kNumTileConfigs;
}

int natten_amd_fna_forward(const void* q, const void* k, const void* v, void* out, float* lse, int dtype, int na_dim,
                           int batch, int seqlen_q, int seqlen_kv, int heads_q, int heads_kv, int head_dim,
                           const int32_t* q_shape, const int32_t* kv_shape, const int32_t* qkv_shape,
                           const int32_t* kernel_size, const int32_t* stride, const int32_t* dilation,
                           const int32_t* is_causal, const int32_t* q_tile_shape, const int32_t* kv_tile_shape,
                           float scale, const float* q_scale, const float* k_scale, const float* v_scale,
                           int run_persistent, void* workspace, uint64_t workspace_bytes, void* stream) {
  g_error[0] = 0;
  if (na_dim < 1 || na_dim > 3) return fail("fna_forward: na_dim must be 1, 2 or 3, got %d", na_dim);
  WorkQueue queues;
  if (int rc = queue_workspace("fna_forward", run_persistent, workspace, workspace_bytes, &queues)) return rc;
  if (int rc = check_common("fna_forward", q, k, v, out, lse, batch, seqlen_q, seqlen_kv, heads_q, heads_kv, head_dim))
    return rc;
  if (!q_shape || !kv_shape || !qkv_shape || !kernel_size || !stride || !dilation || !is_causal || !q_tile_shape ||
      !kv_tile_shape)
    return fail("fna_forward: null shape argument");
  FnaParams p;
  if (int rc = fill_fna_params("fna_forward", p, na_dim, q_shape, kv_shape, qkv_shape, kernel_size, stride, dilation,
                               is_causal, q_tile_shape, kv_tile_shape))
    return rc;
  int qs[3] = {1, 1, 1}, ks[3] = {1, 1, 1};
  for (int a = 0; a < na_dim; ++a) {
    qs[a] = q_shape[a];
    ks[a] = kv_shape[a];
  }
  if (prod3(qs) != seqlen_q || prod3(ks) != seqlen_kv)
    return fail("fna_forward: seqlen_q / seqlen_kv do not match q_shape / kv_shape (%d vs %d, %d vs %d)", prod3(qs),
                seqlen_q, prod3(ks), seqlen_kv);
  if (batch % p.num_groups != 0)
    return fail("fna_forward: batch (%d) is not a multiple of the number of dilation groups (%d)", batch, p.num_groups);
  p.q = q;
  p.k = k;
  p.v = v;
  p.o = out;
  p.lse = lse;
  p.batch = batch;
  p.heads_q = heads_q;
  p.heads_kv = heads_kv;
  p.seqlen_q = seqlen_q;
  p.seqlen_kv = seqlen_kv;
  p.scale = scale;
  p.q_scale = q_scale;
  p.k_scale = k_scale;
  p.v_scale = v_scale;
  set_wg_layout(p, 1);
  return dispatch_dtype(p, dtype, head_dim, prod3(p.q_tile), prod3(p.kv_tile), static_cast<hipStream_t>(stream), queues);
}

namespace {
// The part of natten_amd_fna_forward_fused that needs no operands: checks the shapes and fills the
// launch geometry of the one-launch route (`sixteen_bit`: fp16 / bf16 operands, which take any extent).
int fused_geometry(const char* what, FnaParams& p, bool sixteen_bit, int na_dim, int heads_kv, int head_dim,
                   const int32_t* qkv_shape, const int32_t* kernel_size, const int32_t* stride, const int32_t* dilation,
                   const int32_t* is_causal, const int32_t* q_tile_shape, const int32_t* kv_tile_shape, int anchor_kv_tiles,
                   long long* tokens_out) {
  if (!qkv_shape || !kernel_size || !stride || !dilation || !is_causal || !q_tile_shape || !kv_tile_shape)
    return fail("%s: null shape argument", what);
  int qs[3] = {1, 1, 1}, ks[3] = {1, 1, 1};
  long long tokens = 1;
  // Extents that are not multiples of dilation x KV tile: some KV tile would reach past its
  // dilation group.  1: every group is at least a KV tile wide everywhere, any kernel instance will
  // do (such tiles are gathered from one tile extent before the group's end).  2: a group is
  // narrower than the KV tile somewhere, only the instance that clamps its gathers will do.
  int edge = 0;
  for (int a = 0; a < na_dim; ++a) {
    if (qkv_shape[a] < 1 || dilation[a] < 1 || q_tile_shape[a] < 1 || kv_tile_shape[a] < 1)
      return fail("%s: invalid parameter along dimension %d", what, a);
    // dilation groups may differ in extent by one; the padded per-group layouts cover the largest
    const int ext = na_ceil_div(qkv_shape[a], dilation[a]);
    if (qkv_shape[a] % dilation[a] != 0 || ext % kv_tile_shape[a] != 0) edge = edge > 1 ? edge : 1;
    if (qkv_shape[a] / dilation[a] < kv_tile_shape[a]) edge = 2;
    qs[a] = na_ceil_div(ext, q_tile_shape[a]) * q_tile_shape[a];
    ks[a] = na_ceil_div(ext, kv_tile_shape[a]) * kv_tile_shape[a];
    tokens *= qkv_shape[a];
  }
  if (edge != 0) {
    long long qt = 1, kvt = 1;
    for (int a = 0; a < na_dim; ++a) {
      qt *= q_tile_shape[a];
      kvt *= kv_tile_shape[a];
    }
    if (edge == 2 && !sixteen_bit)
      return fail("%s: a dilation group narrower than the KV tile needs fp16 / bf16 operands; use the token-permuted "
                  "entry point", what);
    if (edge == 2 && (qt != 128 || kvt != 64))
      return fail("%s: a dilation group narrower than the KV tile needs tiles of 128 x 64 tokens (got %lld x %lld); use "
                  "the token-permuted entry point", what, qt, kvt);
  }
  if (tokens > 0x7fffffffLL) return fail("%s: more than 2^31 tokens per batch", what);
  if (int rc = fill_fna_params(what, p, na_dim, qs, ks, qkv_shape, kernel_size, stride, dilation, is_causal, q_tile_shape,
                               kv_tile_shape))
    return rc;
  // per-lane byte offsets inside a KV tile are 32-bit
  long long span = 0;
  for (int a = 0; a < 3; ++a) span += (long long)(p.kv_tile[a] - 1) * p.dil[a] * p.tok_stride[a];
  if ((span + 1) * heads_kv * head_dim * 2 + 8192 >= 0x7fffffffLL)  // (16-bit rows; 8-bit ones are shorter)
    return fail("%s: a KV tile spans more than 2^31 bytes of the input; use the token-permuted entry point", what);
  p.seqlen_q = prod3(qs);
  p.seqlen_kv = prod3(ks);
  p.fused = 1;
  p.edge = edge;
  // tiles laid out from the window's first key: needs every dilation group at least a KV tile wide
  p.anchor = (anchor_kv_tiles != 0 && edge != 2) ? 1 : 0;
  for (int a = 0; a < na_dim; ++a)
    if (qkv_shape[a] / dilation[a] < kv_tile_shape[a]) p.anchor = 0;
  p.tokens = int(tokens);
  *tokens_out = tokens;
  return 0;
}

// natten_amd_fna_forward_fused after its workspace has been resolved (`queues` == nullptr: a workgroup per Q tile)
int fna_forward_fused_impl(const void* q, const void* k, const void* v, void* out, float* lse, int dtype, int na_dim,
                           int batch, int heads_q, int heads_kv, int head_dim, const int32_t* qkv_shape,
                           const int32_t* kernel_size, const int32_t* stride, const int32_t* dilation,
                           const int32_t* is_causal, const int32_t* q_tile_shape, const int32_t* kv_tile_shape,
                           float scale, const float* q_scale, const float* k_scale, const float* v_scale,
                           int anchor_kv_tiles, WorkQueue queues, void* stream, int kv_splits = 1) {
  FnaParams p;
  long long tokens = 0;
  if (heads_kv < 1 || head_dim < 1) return fail("fna_forward_fused: head counts and head_dim must be positive");
  if (int rc = fused_geometry("fna_forward_fused", p, dtype == NATTEN_AMD_F16 || dtype == NATTEN_AMD_BF16, na_dim, heads_kv,
                              head_dim, qkv_shape, kernel_size, stride, dilation, is_causal, q_tile_shape, kv_tile_shape,
                              anchor_kv_tiles, &tokens))
    return rc;
  if (int rc = check_common("fna_forward_fused", q, k, v, out, lse, batch, p.seqlen_q, p.seqlen_kv, heads_q, heads_kv,
                            head_dim))
    return rc;
  p.q = q;
  p.k = k;
  p.v = v;
  p.o = out;
  p.lse = lse;
  p.batch = batch * p.num_groups;
  p.heads_q = heads_q;
  p.heads_kv = heads_kv;
  p.scale = scale;
  p.q_scale = q_scale;
  p.k_scale = k_scale;
  p.v_scale = v_scale;
  if (kv_splits > 1) {
    // out and lse hold kv_splits results of the full shape, one after the other
    p.kv_splits = kv_splits;
    p.o_split_stride = (int64_t)batch * tokens * heads_q * head_dim;
    p.lse_split_stride = (int64_t)batch * tokens * heads_q;
  }
  set_wg_layout(p, 1);
  return dispatch_dtype(p, dtype, head_dim, prod3(p.q_tile), prod3(p.kv_tile), static_cast<hipStream_t>(stream), queues);
}
}  // namespace

int natten_amd_fna_forward_fused(const void* q, const void* k, const void* v, void* out, float* lse, int dtype,
                                 int na_dim, int batch, int heads_q, int heads_kv, int head_dim,
                                 const int32_t* qkv_shape, const int32_t* kernel_size, const int32_t* stride,
                                 const int32_t* dilation, const int32_t* is_causal, const int32_t* q_tile_shape,
                                 const int32_t* kv_tile_shape, float scale, const float* q_scale,
                                 const float* k_scale, const float* v_scale, int anchor_kv_tiles, int run_persistent,
                                 void* workspace, uint64_t workspace_bytes, void* stream) {
  g_error[0] = 0;
  if (na_dim < 1 || na_dim > 3) return fail("fna_forward_fused: na_dim must be 1, 2 or 3, got %d", na_dim);
  WorkQueue queues;
  if (int rc = queue_workspace("fna_forward_fused", run_persistent, workspace, workspace_bytes, &queues)) return rc;
  return fna_forward_fused_impl(q, k, v, out, lse, dtype, na_dim, batch, heads_q, heads_kv, head_dim, qkv_shape,
                                kernel_size, stride, dilation, is_causal, q_tile_shape, kv_tile_shape, scale, q_scale,
                                k_scale, v_scale, anchor_kv_tiles, queues, stream);
}

int natten_amd_fna_forward_fused_split(const void* q, const void* k, const void* v, void* out_parts, float* lse_parts,
                                       int dtype, int na_dim, int batch, int heads_q, int heads_kv, int head_dim,
                                       const int32_t* qkv_shape, const int32_t* kernel_size, const int32_t* stride,
                                       const int32_t* dilation, const int32_t* is_causal,
                                       const int32_t* q_tile_shape, const int32_t* kv_tile_shape, float scale,
                                       int anchor_kv_tiles, int kv_splits, void* stream) {
  g_error[0] = 0;
  const char* what = "fna_forward_fused_split";
  if (na_dim < 1 || na_dim > 3) return fail("%s: na_dim must be 1, 2 or 3, got %d", what, na_dim);
  if (kv_splits < 2 || kv_splits > 8) return fail("%s: kv_splits must be 2 .. 8, got %d", what, kv_splits);
  if (dtype != NATTEN_AMD_F16 && dtype != NATTEN_AMD_BF16)
    return fail("%s: KV splits need fp16 / bf16 operands, got dtype code %d", what, dtype);
  if (!q_tile_shape || !kv_tile_shape) return fail("%s: null shape argument", what);
  long long qt = 1, kvt = 1;
  for (int a = 0; a < na_dim; ++a) {
    qt *= q_tile_shape[a];
    kvt *= kv_tile_shape[a];
  }
  if (qt != 128 || kvt != 64)
    return fail("%s: KV splits exist for Q tiles of 128 and KV tiles of 64 tokens, got %lld and %lld", what, qt, kvt);
  return fna_forward_fused_impl(q, k, v, out_parts, lse_parts, dtype, na_dim, batch, heads_q, heads_kv, head_dim, qkv_shape,
                                kernel_size, stride, dilation, is_causal, q_tile_shape, kv_tile_shape, scale, nullptr,
                                nullptr, nullptr, anchor_kv_tiles, WorkQueue{}, stream, kv_splits);
}

namespace {
// Device address of `scratch` on the current device, looked up once per device (each GPU holds
// its own copy of the array at its own address); nullptr + error message on failure.
uint32_t* static_scratch(const char* what) {
  constexpr int kMaxDevices = 64;
  static uint32_t* ptrs[kMaxDevices] = {};
  static std::mutex lock;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    fail("%s: cannot identify the current device (%s, device %d)", what, hipGetErrorString(e), dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> guard(lock);
  if (ptrs[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      fail("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", what, dev, hipGetErrorString(e));
      return nullptr;
    }
    ptrs[dev] = static_cast<uint32_t*>(ptr);
  }
  return ptrs[dev];
}
}  // namespace

int natten_amd_fna_forward_fused_static(const void* q, const void* k, const void* v, void* out, float* lse, int dtype,
                                        int na_dim, int batch, int heads_q, int heads_kv, int head_dim,
                                        const int32_t* qkv_shape, const int32_t* kernel_size, const int32_t* stride,
                                        const int32_t* dilation, const int32_t* is_causal,
                                        const int32_t* q_tile_shape, const int32_t* kv_tile_shape, float scale,
                                        const float* q_scale, const float* k_scale, const float* v_scale,
                                        void* stream) {
  g_error[0] = 0;
  const char* what = "fna_forward_fused_static";
  if (na_dim < 1 || na_dim > 3) return fail("%s: na_dim must be 1, 2 or 3, got %d", what, na_dim);
  if (!qkv_shape || !q_tile_shape || !kv_tile_shape) return fail("%s: null shape argument", what);
  // only the work-queue kernel uses the scratch array: 16-bit operands, 128 x 64 token tiles
  if (dtype != NATTEN_AMD_F16 && dtype != NATTEN_AMD_BF16)
    return fail("%s: the work-queue kernel takes fp16 / bf16 operands, got dtype code %d", what, dtype);
  long long qt = 1, kvt = 1, q_tiles = 1;
  for (int a = 0; a < na_dim; ++a) {
    if (q_tile_shape[a] < 1 || kv_tile_shape[a] < 1 || qkv_shape[a] < 1 || !dilation || dilation[a] < 1)
      return fail("%s: invalid parameter along dimension %d", what, a);
    qt *= q_tile_shape[a];
    kvt *= kv_tile_shape[a];
    const long long ext = (qkv_shape[a] + dilation[a] - 1) / dilation[a];
    q_tiles *= (ext + q_tile_shape[a] - 1) / q_tile_shape[a] * dilation[a];
  }
  if (qt != 128 || kvt != 64)
    return fail("%s: the work-queue kernel exists for Q tiles of 128 and KV tiles of 64 tokens, got %lld and %lld", what, qt,
                kvt);
  // the queues hold 32-bit positions: at most 2^28 Q tiles per queue (2^31 in all); the array itself never grows
  if (batch < 1 || heads_q < 1 || q_tiles * batch * heads_q > (1LL << 31) - 4096)
    return fail("%s: %lld Q tiles x %d x %d exceed the 2^31 positions the static queues can count", what, q_tiles, batch,
                heads_q);
  WorkQueue queues;  // (cleared by a kernel before every launch: the array is shared by all callers on this GPU)
  queues.counters = static_scratch(what);
  if (queues.counters == nullptr) return 1;
  return fna_forward_fused_impl(q, k, v, out, lse, dtype, na_dim, batch, heads_q, heads_kv, head_dim, qkv_shape,
                                kernel_size, stride, dilation, is_causal, q_tile_shape, kv_tile_shape, scale, q_scale,
                                k_scale, v_scale, /*anchor_kv_tiles=*/1, queues, stream);
}

int natten_amd_attention_forward(const void* q, const void* k, const void* v, void* out, float* lse, int dtype,
                                 int batch, int seqlen_q, int seqlen_kv, int heads_q, int heads_kv, int head_dim,
                                 int is_causal, float scale, const float* q_scale, const float* k_scale,
                                 const float* v_scale, void* stream) {
  g_error[0] = 0;
  if (int rc = check_common("attention_forward", q, k, v, out, lse, batch, seqlen_q, seqlen_kv, heads_q, heads_kv,
                            head_dim))
    return rc;
  // Dense attention is the 1-D neighborhood problem whose window is the whole key sequence:
  // non-causal windows are [0, seqlen_kv), causal ones [0, min(i + 1, seqlen_kv)).
  constexpr int QT = 128, KVT = 64;
  FnaParams p;
  memset(&p, 0, sizeof(p));
  for (int a = 0; a < 3; ++a) {
    p.qkv_shape[a] = p.ksize[a] = p.stride[a] = p.dil[a] = p.q_tile[a] = p.kv_tile[a] = p.q_tiled[a] = p.kv_tiled[a] = 1;
  }
  if (seqlen_kv < 2) {
    // a one-key window is the unused-dimension case of the window arithmetic (k = 1)
    p.ksize[0] = 1;
  } else {
    p.ksize[0] = seqlen_kv;
  }
  p.qkv_shape[0] = seqlen_kv;
  p.causal[0] = is_causal != 0;
  p.q_tile[0] = QT;
  p.kv_tile[0] = KVT;
  p.q_tiled[0] = na_ceil_div(seqlen_q, QT);
  p.kv_tiled[0] = na_ceil_div(seqlen_kv, KVT);
  p.num_groups = 1;
  p.q = q;
  p.k = k;
  p.v = v;
  p.o = out;
  p.lse = lse;
  p.batch = batch;
  p.heads_q = heads_q;
  p.heads_kv = heads_kv;
  p.seqlen_q = seqlen_q;
  p.seqlen_kv = seqlen_kv;
  p.scale = scale;
  p.q_scale = q_scale;
  p.k_scale = k_scale;
  p.v_scale = v_scale;
  set_wg_layout(p, 1);
  return dispatch_dtype(p, dtype, head_dim, QT, KVT, static_cast<hipStream_t>(stream));
}

int natten_amd_attention_forward_varlen(const void* q, const void* k, const void* v, void* out, float* lse, int dtype,
                                        int num_seqs, int total_seqlen_q, int total_seqlen_kv, int max_seqlen_q,
                                        int max_seqlen_kv, int heads_q, int heads_kv, int head_dim,
                                        const int32_t* cumulative_seqlen_q, const int32_t* cumulative_seqlen_kv,
                                        int is_causal, float scale, const float* q_scale, const float* k_scale,
                                        const float* v_scale, void* stream) {
  g_error[0] = 0;
  const char* what = "attention_forward_varlen";
  if (int rc = check_common(what, q, k, v, out, lse, num_seqs, total_seqlen_q, total_seqlen_kv, heads_q, heads_kv,
                            head_dim))
    return rc;
  if (!cumulative_seqlen_q || !cumulative_seqlen_kv) return fail("%s: null cumulative sequence length array", what);
  if (max_seqlen_q < 1 || max_seqlen_kv < 1 || max_seqlen_q > total_seqlen_q || max_seqlen_kv > total_seqlen_kv)
    return fail("%s: maximum sequence lengths (%d, %d) must lie in 1 .. total (%d, %d)", what, max_seqlen_q,
                max_seqlen_kv, total_seqlen_q, total_seqlen_kv);
  if (dtype != NATTEN_AMD_F16 && dtype != NATTEN_AMD_BF16)
    return fail("%s: only 16-bit float operands are supported, got dtype code %d", what, dtype);
  constexpr int QT = 128, KVT = 64;
  FnaParams p;
  memset(&p, 0, sizeof(p));
  for (int a = 0; a < 3; ++a) {
    p.qkv_shape[a] = p.ksize[a] = p.stride[a] = p.dil[a] = p.q_tile[a] = p.kv_tile[a] = p.q_tiled[a] = p.kv_tiled[a] = 1;
  }
  // one batch entry per sequence; the kernel reads every sequence's own lengths (window =
  // its whole key sequence) from the cumulative arrays, the launch is sized for the longest
  p.ksize[0] = max_seqlen_kv;
  p.qkv_shape[0] = max_seqlen_kv;
  p.causal[0] = is_causal != 0;
  p.q_tile[0] = QT;
  p.kv_tile[0] = KVT;
  p.q_tiled[0] = na_ceil_div(max_seqlen_q, QT);
  p.kv_tiled[0] = na_ceil_div(max_seqlen_kv, KVT);
  p.num_groups = 1;
  p.q = q;
  p.k = k;
  p.v = v;
  p.o = out;
  p.lse = lse;
  p.batch = num_seqs;
  p.heads_q = heads_q;
  p.heads_kv = heads_kv;
  p.seqlen_q = max_seqlen_q;
  p.seqlen_kv = max_seqlen_kv;
  p.scale = scale;
  p.q_scale = q_scale;
  p.k_scale = k_scale;
  p.v_scale = v_scale;
  p.cu_q = cumulative_seqlen_q;
  p.cu_kv = cumulative_seqlen_kv;
  p.total_q = total_seqlen_q;
  p.total_kv = total_seqlen_kv;
  set_wg_layout(p, 1);
  return dispatch_dtype(p, dtype, head_dim, QT, KVT, static_cast<hipStream_t>(stream));
}

// ---- backward ---------------------------------------------------------------------------------

extern "C++" {
template <typename T, int D, bool VARLEN>
static int launch_bwd(const FnaBwdParams& params, hipStream_t stream) {
  FnaBwdParams p = params;
  // grids are padded to a multiple of the 8 XCDs: each XCD takes a contiguous eighth of the tiles
  auto grid = [](long long wgs) { return (wgs + kNumXcd - 1) / kNumXcd * kNumXcd; };
  const long long wg_q = grid((long long)p.batch * p.heads_q * prod3(p.q_tiled));
  long long wg_kv = grid((long long)p.batch * p.heads_kv * prod3(p.kv_tiled));
  if constexpr (D == 128) {
    // paired role (one workgroup per CU, 32 resident per XCD): runs of about 32 key tiles, a whole
    // number of dimension-0 slabs or an even part of one, dealt round-robin to the XCDs
    const int slab = p.kv_tiled[1] * p.kv_tiled[2];
    int run;
    if (slab >= 32) {
      const int parts = (slab + 16) / 32;
      run = (slab + parts - 1) / parts;
    } else {
      int rows = (32 + slab / 2) / slab;
      if (rows > p.kv_tiled[0]) rows = p.kv_tiled[0];
      run = slab * rows;
    }
    p.kv_wg_run = run;
    const long long runs = ((long long)p.batch * p.heads_kv * prod3(p.kv_tiled) + run - 1) / run;
    wg_kv = (runs + kNumXcd - 1) / kNumXcd * kNumXcd * run;
  }
  if (wg_q > 0x7fffffffLL || wg_kv > 0x7fffffffLL) return fail("fna_backward: problem needs more than 2^31 workgroups");
  const int roles = p.roles ? p.roles : 3;
  if (roles & 2) {
    // The key-stationary launch streams the queries as the forward kernel multiplied them: scaled
    // and rounded once, into the workspace.  It runs before the dQ launch, so that the workspace
    // may be the dq buffer.
    const long long q_rows = p.cu_q ? (long long)p.seqlen_q
                                    : p.fused ? (long long)(p.batch / p.num_groups) * p.tokens : (long long)p.batch * p.seqlen_q;
    const long long chunks = q_rows * p.heads_q * (D / 8);
    const long long blocks = (chunks + 255) / 256;
    if (blocks > 0x7fffffffLL) return fail("fna_backward: problem needs more than 2^31 workgroups");
    hipLaunchKernelGGL((scale_queries_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream, static_cast<const T*>(p.q),
                       static_cast<T*>(const_cast<void*>(p.qs)), (int64_t)chunks, p.scale * 1.4426950408889634f);
    if (int rc = check_launch("fna_backward (scaled queries)")) return rc;
    if constexpr (D == 128) {
      // dK and dV by wave pairs (eight waves per workgroup): one wave's registers cannot hold the
      // accumulators, fragments and products of both
      hipLaunchKernelGGL((fna_bwd_kernel<T, D, kBwdPair, VARLEN>), dim3((unsigned)wg_kv), dim3(512), 0, stream, p);
    } else {
      hipLaunchKernelGGL((fna_bwd_kernel<T, D, kBwdDKV, VARLEN>), dim3((unsigned)wg_kv), dim3(256), 0, stream, p);
    }
    if (int rc = check_launch("fna_backward (dK, dV)")) return rc;
  }
  if (roles & 1) {
    hipLaunchKernelGGL((fna_bwd_kernel<T, D, kBwdDQ, VARLEN>), dim3((unsigned)wg_q), dim3(256), 0, stream, p);
    if (int rc = check_launch("fna_backward (dQ)")) return rc;
  }
  return 0;
}

template <typename T>
static int dispatch_bwd_head_dim(const FnaBwdParams& p, int head_dim, hipStream_t stream) {
  const bool varlen = p.cu_q != nullptr;  // sequence-packed dense attention
  switch (head_dim) {
    case 32: return varlen ? launch_bwd<T, 32, true>(p, stream) : launch_bwd<T, 32, false>(p, stream);
    case 64: return varlen ? launch_bwd<T, 64, true>(p, stream) : launch_bwd<T, 64, false>(p, stream);
    case 128: return varlen ? launch_bwd<T, 128, true>(p, stream) : launch_bwd<T, 128, false>(p, stream);
  }
  return fail("fna_backward: head_dim must be 32, 64 or 128, got %d", head_dim);
}

static int dispatch_bwd(const FnaBwdParams& p, int dtype, int head_dim, hipStream_t stream) {
  switch (dtype) {
    case NATTEN_AMD_F16: return dispatch_bwd_head_dim<_Float16>(p, head_dim, stream);
    case NATTEN_AMD_BF16: return dispatch_bwd_head_dim<__bf16>(p, head_dim, stream);
  }
  return fail("fna_backward: only 16-bit float operands are supported, got dtype code %d", dtype);
}
}  // extern "C++"

// last dimension of extent > 1 (0 for a one-token tile)
static int split_dim_of(const int* tile) {
  int s = 0;
  for (int a = 0; a < 3; ++a)
    if (tile[a] > 1) s = a;
  return s;
}

static int check_bwd_pointers(const char* what, const void* q, const void* k, const void* v, const void* d_out,
                              const float* lse, const float* delta, void* dq, void* dk, void* dv, void* q_scaled,
                              int roles) {
  if (!q || !k || !v || !d_out || !lse || !delta || !dq || !dk || !dv) return fail("%s: null pointer argument", what);
  if ((roles & 2) && !q_scaled) return fail("%s: the dk / dv launch needs the q_scaled workspace", what);
  if (q_scaled == q) return fail("%s: q_scaled must not be q itself (the dq launch reads the unscaled queries)", what);
  if (reinterpret_cast<uintptr_t>(q_scaled) & 15) return fail("%s: q_scaled must be 16-byte aligned", what);
  const uintptr_t all = reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                        reinterpret_cast<uintptr_t>(d_out) | reinterpret_cast<uintptr_t>(dq) |
                        reinterpret_cast<uintptr_t>(dk) | reinterpret_cast<uintptr_t>(dv);
  if (all & 15) return fail("%s: q, k, v, d_out, dq, dk and dv must be 16-byte aligned", what);
  return 0;
}

int natten_amd_fna_backward(const void* q, const void* k, const void* v, const void* d_out, const float* lse,
                            const float* delta, void* dq, void* dk, void* dv, void* q_scaled, int dtype, int na_dim,
                            int batch, int seqlen_q, int seqlen_kv, int heads_q, int heads_kv, int head_dim,
                            const int32_t* q_shape, const int32_t* kv_shape, const int32_t* qkv_shape,
                            const int32_t* kernel_size, const int32_t* stride, const int32_t* dilation,
                            const int32_t* is_causal, const int32_t* q_tile_shape, const int32_t* kv_tile_shape,
                            float scale, void* stream) {
  g_error[0] = 0;
  const char* what = "fna_backward";
  if (int rc = check_bwd_pointers(what, q, k, v, d_out, lse, delta, dq, dk, dv, q_scaled, 3)) return rc;
  if (int rc = check_common(what, q, k, v, dq, lse, batch, seqlen_q, seqlen_kv, heads_q, heads_kv, head_dim)) return rc;
  if (na_dim < 1 || na_dim > 3) return fail("%s: na_dim must be 1, 2 or 3, got %d", what, na_dim);
  if (!q_shape || !kv_shape || !qkv_shape || !kernel_size || !stride || !dilation || !is_causal || !q_tile_shape ||
      !kv_tile_shape)
    return fail("%s: null shape argument", what);
  FnaParams f;
  if (int rc = fill_fna_params(what, f, na_dim, q_shape, kv_shape, qkv_shape, kernel_size, stride, dilation, is_causal,
                               q_tile_shape, kv_tile_shape))
    return rc;
  if (prod3(f.q_tile) != 128 || prod3(f.kv_tile) != 128)
    return fail("%s: Q and KV tiles must hold 128 tokens each, got %d and %d", what, prod3(f.q_tile), prod3(f.kv_tile));
  FnaBwdParams p;
  memset(&p, 0, sizeof(p));
  p.q_split = split_dim_of(f.q_tile);
  p.kv_split = split_dim_of(f.kv_tile);
  if (f.q_tile[p.q_split] % 2 != 0 || f.kv_tile[p.kv_split] % 2 != 0)
    return fail("%s: the last tile extent above 1 must be even", what);
  int groups = 1;
  for (int a = 0; a < 3; ++a) {
    p.qkv_shape[a] = f.qkv_shape[a];
    p.ksize[a] = f.ksize[a];
    p.stride[a] = f.stride[a];
    p.dil[a] = f.dil[a];
    p.causal[a] = f.causal[a];
    p.q_tile[a] = f.q_tile[a];
    p.kv_tile[a] = f.kv_tile[a];
    p.q_tiled[a] = f.q_tiled[a];
    p.kv_tiled[a] = f.kv_tiled[a];
    groups *= f.dil[a];
  }
  if (batch % groups != 0) return fail("%s: batch (%d) must be a multiple of prod(dilation) (%d)", what, batch, groups);
  if (seqlen_q != prod3(p.q_tiled) * 128 || seqlen_kv != prod3(p.kv_tiled) * 128)
    return fail("%s: sequence lengths (%d, %d) do not match the padded layouts (%d, %d)", what, seqlen_q, seqlen_kv,
                prod3(p.q_tiled) * 128, prod3(p.kv_tiled) * 128);
  p.q = q;
  p.qs = q_scaled;
  p.k = k;
  p.v = v;
  p.d_out = d_out;
  p.lse = lse;
  p.delta = delta;
  p.dq = dq;
  p.dk = dk;
  p.dv = dv;
  p.batch = batch;
  p.heads_q = heads_q;
  p.heads_kv = heads_kv;
  p.seqlen_q = seqlen_q;
  p.seqlen_kv = seqlen_kv;
  p.num_groups = groups;
  p.q_extent0 = 0;
  p.scale = scale;
  return dispatch_bwd(p, dtype, head_dim, static_cast<hipStream_t>(stream));
}

int natten_amd_fna_backward_fused(const void* q, const void* k, const void* v, const void* d_out, const float* lse,
                                  const float* delta, void* dq, void* dk, void* dv, void* q_scaled, int dtype, int na_dim,
                                  int batch, int heads_q, int heads_kv, int head_dim, const int32_t* qkv_shape,
                                  const int32_t* kernel_size, const int32_t* stride, const int32_t* dilation,
                                  const int32_t* is_causal, const int32_t* q_tile_shape, const int32_t* kv_tile_shape,
                                  float scale, int roles, void* stream) {
  g_error[0] = 0;
  const char* what = "fna_backward_fused";
  if (roles < 1 || roles > 3) return fail("%s: roles must be 1 (dq), 2 (dk and dv) or 3 (all), got %d", what, roles);
  if (int rc = check_bwd_pointers(what, q, k, v, d_out, lse, delta, dq, dk, dv, q_scaled, roles)) return rc;
  if (na_dim < 1 || na_dim > 3) return fail("%s: na_dim must be 1, 2 or 3, got %d", what, na_dim);
  if (!qkv_shape || !kernel_size || !stride || !dilation || !is_causal || !q_tile_shape || !kv_tile_shape)
    return fail("%s: null shape argument", what);
  // Per-group layouts, padded to whole tiles.  Extents that are not multiples of dilation x tile are
  // taken as long as every dilation group is at least one tile wide (either side's) in every
  // dimension: tiles that would reach past a group are then moved back or clamped by the kernels.
  int q_group_shape[3] = {1, 1, 1}, kv_group_shape[3] = {1, 1, 1}, edge = 0;
  long long tokens = 1;
  for (int a = 0; a < na_dim; ++a) {
    if (qkv_shape[a] < 1 || dilation[a] < 1 || q_tile_shape[a] < 1 || kv_tile_shape[a] < 1)
      return fail("%s: invalid parameter along dimension %d", what, a);
    if (qkv_shape[a] % (dilation[a] * q_tile_shape[a]) != 0 || qkv_shape[a] % (dilation[a] * kv_tile_shape[a]) != 0) edge = 1;
    if (qkv_shape[a] / dilation[a] < q_tile_shape[a] || qkv_shape[a] / dilation[a] < kv_tile_shape[a])
      return fail("%s: a dilation group of dimension %d (%d tokens / dilation %d) is narrower than a tile (%d, %d); use "
                  "the token-permuted entry point",
                  what, a, qkv_shape[a], dilation[a], q_tile_shape[a], kv_tile_shape[a]);
    const int ext = na_ceil_div(qkv_shape[a], dilation[a]);
    q_group_shape[a] = na_ceil_div(ext, q_tile_shape[a]) * q_tile_shape[a];
    kv_group_shape[a] = na_ceil_div(ext, kv_tile_shape[a]) * kv_tile_shape[a];
    tokens *= qkv_shape[a];
  }
  if (tokens > 0x7fffffffLL) return fail("%s: more than 2^31 tokens", what);
  FnaParams f;
  if (int rc = fill_fna_params(what, f, na_dim, q_group_shape, kv_group_shape, qkv_shape, kernel_size, stride, dilation,
                               is_causal, q_tile_shape, kv_tile_shape))
    return rc;
  if (!fna_tiles_are_powers_of_two(f)) return fail("%s: tile extents must be powers of two", what);
  if (int rc = check_common(what, q, k, v, dq, lse, batch, int(tokens), int(tokens), heads_q, heads_kv, head_dim)) return rc;
  // per-lane byte offsets inside a tile are 32-bit
  long long span_q = 0, span_kv = 0;
  for (int a = 0; a < 3; ++a) {
    span_q += (long long)(f.q_tile[a] - 1) * f.dil[a] * f.tok_stride[a];
    span_kv += (long long)(f.kv_tile[a] - 1) * f.dil[a] * f.tok_stride[a];
  }
  if ((span_q + 1) * heads_q * head_dim * 2 + 8192 >= 0x7fffffffLL || (span_kv + 1) * heads_kv * head_dim * 2 + 8192 >= 0x7fffffffLL)
    return fail("%s: a tile spans more than 2^31 bytes of the tensors; use the token-permuted entry point", what);
  if (prod3(f.q_tile) != 128 || prod3(f.kv_tile) != 128)
    return fail("%s: Q and KV tiles must hold 128 tokens each, got %d and %d", what, prod3(f.q_tile), prod3(f.kv_tile));
  FnaBwdParams p;
  memset(&p, 0, sizeof(p));
  p.q_split = split_dim_of(f.q_tile);
  p.kv_split = split_dim_of(f.kv_tile);
  if (f.q_tile[p.q_split] % 2 != 0 || f.kv_tile[p.kv_split] % 2 != 0)
    return fail("%s: the last tile extent above 1 must be even", what);
  int groups = 1;
  for (int a = 0; a < 3; ++a) {
    p.qkv_shape[a] = f.qkv_shape[a];
    p.ksize[a] = f.ksize[a];
    p.stride[a] = f.stride[a];
    p.dil[a] = f.dil[a];
    p.causal[a] = f.causal[a];
    p.q_tile[a] = f.q_tile[a];
    p.kv_tile[a] = f.kv_tile[a];
    p.q_tiled[a] = f.q_tiled[a];
    p.kv_tiled[a] = f.kv_tiled[a];
    p.tok_stride[a] = f.tok_stride[a];
    groups *= f.dil[a];
  }
  p.q = q;
  p.qs = q_scaled;
  p.k = k;
  p.v = v;
  p.d_out = d_out;
  p.lse = lse;
  p.delta = delta;
  p.dq = dq;
  p.dk = dk;
  p.dv = dv;
  p.batch = batch * groups;
  p.heads_q = heads_q;
  p.heads_kv = heads_kv;
  p.seqlen_q = prod3(p.q_tiled) * 128;
  p.seqlen_kv = prod3(p.kv_tiled) * 128;
  p.num_groups = groups;
  p.q_extent0 = 0;
  p.scale = scale;
  p.fused = 1;
  p.edge = edge;
  p.tokens = int(tokens);
  p.roles = roles;
  return dispatch_bwd(p, dtype, head_dim, static_cast<hipStream_t>(stream));
}

int natten_amd_attention_backward(const void* q, const void* k, const void* v, const void* d_out, const float* lse,
                                  const float* delta, void* dq, void* dk, void* dv, void* q_scaled, int dtype, int batch,
                                  int seqlen_q, int seqlen_kv, int padded_seqlen_q, int padded_seqlen_kv, int heads_q,
                                  int heads_kv, int head_dim, int is_causal, float scale, void* stream) {
  g_error[0] = 0;
  const char* what = "attention_backward";
  if (int rc = check_bwd_pointers(what, q, k, v, d_out, lse, delta, dq, dk, dv, q_scaled, 3)) return rc;
  if (int rc = check_common(what, q, k, v, dq, lse, batch, seqlen_q, seqlen_kv, heads_q, heads_kv, head_dim)) return rc;
  if (padded_seqlen_q % 128 != 0 || padded_seqlen_kv % 128 != 0 || padded_seqlen_q < seqlen_q ||
      padded_seqlen_kv < seqlen_kv)
    return fail("%s: padded sequence lengths (%d, %d) must be multiples of 128 that cover (%d, %d)", what,
                padded_seqlen_q, padded_seqlen_kv, seqlen_q, seqlen_kv);
  // the 1-D neighborhood problem whose window is the whole key sequence, with its own query count
  FnaBwdParams p;
  memset(&p, 0, sizeof(p));
  for (int a = 0; a < 3; ++a) {
    p.qkv_shape[a] = p.ksize[a] = p.stride[a] = p.dil[a] = p.q_tile[a] = p.kv_tile[a] = p.q_tiled[a] = p.kv_tiled[a] = 1;
  }
  p.qkv_shape[0] = seqlen_kv;
  p.ksize[0] = seqlen_kv;
  p.causal[0] = is_causal != 0;
  p.q_tile[0] = p.kv_tile[0] = 128;
  p.q_tiled[0] = padded_seqlen_q / 128;
  p.kv_tiled[0] = padded_seqlen_kv / 128;
  p.q_extent0 = seqlen_q;
  p.q = q;
  p.qs = q_scaled;
  p.k = k;
  p.v = v;
  p.d_out = d_out;
  p.lse = lse;
  p.delta = delta;
  p.dq = dq;
  p.dk = dk;
  p.dv = dv;
  p.batch = batch;
  p.heads_q = heads_q;
  p.heads_kv = heads_kv;
  p.seqlen_q = padded_seqlen_q;
  p.seqlen_kv = padded_seqlen_kv;
  p.num_groups = 1;
  p.scale = scale;
  return dispatch_bwd(p, dtype, head_dim, static_cast<hipStream_t>(stream));
}

int natten_amd_attention_backward_varlen(const void* q, const void* k, const void* v, const void* d_out,
                                         const float* lse, const float* delta, void* dq, void* dk, void* dv,
                                         void* q_scaled, int dtype, int num_seqs, int rows_q, int rows_kv, const int32_t* cu_seqlens_q,
                                         const int32_t* cu_seqlens_kv, const int32_t* padded_cu_seqlens_q,
                                         const int32_t* padded_cu_seqlens_kv, int max_seqlen_q, int max_seqlen_kv,
                                         int heads_q, int heads_kv, int head_dim, int is_causal, float scale,
                                         void* stream) {
  g_error[0] = 0;
  const char* what = "attention_backward_varlen";
  if (int rc = check_bwd_pointers(what, q, k, v, d_out, lse, delta, dq, dk, dv, q_scaled, 3)) return rc;
  if (int rc = check_common(what, q, k, v, dq, lse, num_seqs, rows_q, rows_kv, heads_q, heads_kv, head_dim)) return rc;
  if (!cu_seqlens_q || !cu_seqlens_kv || !padded_cu_seqlens_q || !padded_cu_seqlens_kv)
    return fail("%s: null cumulative length argument", what);
  if (rows_q % 128 != 0 || rows_kv % 128 != 0)
    return fail("%s: the padded row counts (%d, %d) must be multiples of 128", what, rows_q, rows_kv);
  if (max_seqlen_q < 1 || max_seqlen_kv < 1 || max_seqlen_q > rows_q || max_seqlen_kv > rows_kv)
    return fail("%s: max_seqlen_q / max_seqlen_kv (%d, %d) must lie in 1 .. the row counts (%d, %d)", what,
                max_seqlen_q, max_seqlen_kv, rows_q, rows_kv);
  // per sequence: the 1-D neighborhood problem whose window is the whole key sequence
  FnaBwdParams p;
  memset(&p, 0, sizeof(p));
  for (int a = 0; a < 3; ++a) {
    p.qkv_shape[a] = p.ksize[a] = p.stride[a] = p.dil[a] = p.q_tile[a] = p.kv_tile[a] = p.q_tiled[a] = p.kv_tiled[a] = 1;
  }
  p.qkv_shape[0] = p.ksize[0] = max_seqlen_kv;  // replaced per sequence inside the kernel
  p.q_extent0 = max_seqlen_q;
  p.causal[0] = is_causal != 0;
  p.q_tile[0] = p.kv_tile[0] = 128;
  p.q_tiled[0] = (max_seqlen_q + 127) / 128;
  p.kv_tiled[0] = (max_seqlen_kv + 127) / 128;
  p.q = q;
  p.qs = q_scaled;
  p.k = k;
  p.v = v;
  p.d_out = d_out;
  p.lse = lse;
  p.delta = delta;
  p.dq = dq;
  p.dk = dk;
  p.dv = dv;
  p.batch = num_seqs;
  p.heads_q = heads_q;
  p.heads_kv = heads_kv;
  p.seqlen_q = rows_q;
  p.seqlen_kv = rows_kv;
  p.num_groups = 1;
  p.scale = scale;
  p.cu_q = cu_seqlens_q;
  p.cu_kv = cu_seqlens_kv;
  p.pcu_q = padded_cu_seqlens_q;
  p.pcu_kv = padded_cu_seqlens_kv;
  return dispatch_bwd(p, dtype, head_dim, static_cast<hipStream_t>(stream));
}

int natten_amd_query_range(int key_first, int key_last, int kernel_size, int stride, int extent, int num_queries,
                           int is_causal, int32_t* first_query, int32_t* last_query) {
  g_error[0] = 0;
  if (!first_query || !last_query) return fail("query_range: null pointer argument");
  if (kernel_size < 1 || stride < 1 || extent < 1 || num_queries < 1 || kernel_size > extent || stride > kernel_size ||
      key_first < 0 || key_last < key_first || key_last >= extent)
    return fail("query_range: invalid argument");
  *first_query = na_first_query_attending(key_first, kernel_size, stride, extent, num_queries, is_causal != 0);
  *last_query = na_last_query_attending(key_last, kernel_size, stride, extent, num_queries, is_causal != 0);
  return 0;
}

int natten_amd_compute_delta(const void* out, const void* d_out, float* delta, int dtype, int64_t items, int head_dim,
                             void* stream) {
  g_error[0] = 0;
  if (!out || !d_out || !delta) return fail("compute_delta: null pointer argument");
  if (items < 0) return fail("compute_delta: negative item count");
  if ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(d_out)) & 15)
    return fail("compute_delta: out and d_out must be 16-byte aligned");
  if (items == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define NA_DELTA_LAUNCH(TYPE, DD)                                                                              \
  do {                                                                                                         \
    const int64_t blocks = (items * ((DD) / 8) + 255) / 256;                                                   \
    if (blocks > 0x7fffffffLL) return fail("compute_delta: too many rows");                                    \
    hipLaunchKernelGGL((delta_kernel<TYPE, DD>), dim3((unsigned)blocks), dim3(256), 0, s,                      \
                       static_cast<const TYPE*>(out), static_cast<const TYPE*>(d_out), delta, items);          \
  } while (0)
#define NA_DELTA_DTYPE(DD)                                              \
  do {                                                                  \
    if (dtype == NATTEN_AMD_F16) NA_DELTA_LAUNCH(_Float16, DD);         \
    else if (dtype == NATTEN_AMD_BF16) NA_DELTA_LAUNCH(__bf16, DD);     \
    else return fail("compute_delta: unsupported dtype code %d", dtype); \
  } while (0)
  switch (head_dim) {
    case 32: NA_DELTA_DTYPE(32); break;
    case 64: NA_DELTA_DTYPE(64); break;
    case 128: NA_DELTA_DTYPE(128); break;
    default: return fail("compute_delta: head_dim must be 32, 64 or 128, got %d", head_dim);
  }
#undef NA_DELTA_DTYPE
#undef NA_DELTA_LAUNCH
  return check_launch("compute_delta");
}

// widen: 0 = copy the payload, NATTEN_AMD_F8E4M3 / NATTEN_AMD_F8E5M2 = 8-bit float source, bf16 destination
static int tokperm_common(const char* what, bool unpermute, int widen, const void* src, void* dst, int elem_bytes, int na_dim,
                          int batch, int heads, int head_dim, const int32_t* token_layout, const int32_t* tile_shape,
                          const int32_t* dilation, int flip, void* stream) {
  g_error[0] = 0;
  if (!src || !dst) return fail("%s: null pointer argument", what);
  if (na_dim < 1 || na_dim > 3) return fail("%s: na_dim must be 1, 2 or 3, got %d", what, na_dim);
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8)
    return fail("%s: elem_bytes must be 1, 2, 4 or 8, got %d", what, elem_bytes);
  if (batch < 1 || heads < 1 || head_dim < 1) return fail("%s: batch, heads and head_dim must be positive", what);
  if (!token_layout || !tile_shape || !dilation) return fail("%s: null shape argument", what);
  TokPermParams p;
  memset(&p, 0, sizeof(p));
  p.src = static_cast<const char*>(src);
  p.dst = static_cast<char*>(dst);
  p.na_dim = na_dim;
  p.batch = batch;
  p.num_groups = 1;
  p.perm_len = 1;
  p.orig_len = 1;
  p.row_bytes = int64_t(heads) * head_dim * elem_bytes;
  int R[3] = {1, 1, 1};
  for (int a = 0; a < na_dim; ++a) {
    if (token_layout[a] < 1 || tile_shape[a] < 1 || dilation[a] < 1)
      return fail("%s: token_layout, tile_shape and dilation must be positive (dimension %d)", what, a);
    p.layout[a] = token_layout[a];
    p.tile[a] = tile_shape[a];
    p.dil[a] = dilation[a];
    R[a] = na_ceil_div(na_ceil_div(token_layout[a], tile_shape[a]), dilation[a]);
    p.num_groups *= dilation[a];
    p.perm_len *= int64_t(R[a]) * tile_shape[a];
    p.orig_len *= token_layout[a];
  }
  for (int i = 0; i < na_dim; ++i) {
    const int a = flip ? i : na_dim - 1 - i;  // slot i (fastest first) -> original dimension
    p.t_dim[i] = a;
    p.t_size[i] = p.tile[a];
    p.r_size[i] = R[a];
    p.g_size[i] = p.dil[a];
  }
  const uintptr_t align = reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst) | uintptr_t(p.row_bytes);
  if (widen) {
    if (p.row_bytes % 8 != 0 || reinterpret_cast<uintptr_t>(src) % 8 != 0 || reinterpret_cast<uintptr_t>(dst) % 16 != 0)
      return fail("%s: heads * head_dim must be a multiple of 8, src 8-byte and dst 16-byte aligned", what);
  }
  const int vec = widen ? 8 : (align % 16 == 0) ? 16 : (align % 4 == 0) ? 4 : (align % 2 == 0) ? 2 : 1;
  const int64_t total = int64_t(batch) * p.num_groups * p.perm_len * (p.row_bytes / vec);
  int64_t blocks = (total + 255) / 256;
  const int64_t cap = 256 * 64;  // grid-stride beyond this many workgroups
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define NA_TOKPERM_LAUNCH(VEC)                                                                    \
  do {                                                                                            \
    if (unpermute)                                                                                \
      hipLaunchKernelGGL((tokperm_kernel<VEC, true>), dim3(unsigned(blocks)), dim3(256), 0, s, p);  \
    else                                                                                          \
      hipLaunchKernelGGL((tokperm_kernel<VEC, false>), dim3(unsigned(blocks)), dim3(256), 0, s, p); \
  } while (0)
  if (widen == NATTEN_AMD_F8E5M2) {
    hipLaunchKernelGGL((tokperm_widen_kernel<true>), dim3(unsigned(blocks)), dim3(256), 0, s, p);
    return check_launch(what);
  } else if (widen) {
    hipLaunchKernelGGL((tokperm_widen_kernel<false>), dim3(unsigned(blocks)), dim3(256), 0, s, p);
    return check_launch(what);
  }
  if (vec == 16 && p.row_bytes >= 256) {
    // a wave per token row
    const int64_t rows = int64_t(batch) * p.num_groups * p.perm_len;
    int64_t wgs = (rows + 3) / 4;
    if (wgs > 256 * 32) wgs = 256 * 32;
    if (unpermute)
      hipLaunchKernelGGL(tokperm_rows_kernel<true>, dim3(unsigned(wgs)), dim3(256), 0, s, p);
    else
      hipLaunchKernelGGL(tokperm_rows_kernel<false>, dim3(unsigned(wgs)), dim3(256), 0, s, p);
    return check_launch(what);
  }
  switch (vec) {
    case 16: NA_TOKPERM_LAUNCH(16); break;
    case 4: NA_TOKPERM_LAUNCH(4); break;
    case 2: NA_TOKPERM_LAUNCH(2); break;
    default: NA_TOKPERM_LAUNCH(1); break;
  }
#undef NA_TOKPERM_LAUNCH
  return check_launch(what);
}

int natten_amd_token_permute(const void* src, void* dst, int elem_bytes, int na_dim, int batch, int heads,
                             int head_dim, const int32_t* token_layout, const int32_t* tile_shape,
                             const int32_t* dilation, int flip_tiled_dims, void* stream) {
  return tokperm_common("token_permute", false, 0, src, dst, elem_bytes, na_dim, batch, heads, head_dim, token_layout,
                        tile_shape, dilation, flip_tiled_dims, stream);
}

int natten_amd_token_unpermute(const void* src, void* dst, int elem_bytes, int na_dim, int batch, int heads,
                               int head_dim, const int32_t* token_layout, const int32_t* tile_shape,
                               const int32_t* dilation, int flip_tiled_dims, void* stream) {
  return tokperm_common("token_unpermute", true, 0, src, dst, elem_bytes, na_dim, batch, heads, head_dim, token_layout,
                        tile_shape, dilation, flip_tiled_dims, stream);
}

int natten_amd_token_permute_widen(const void* src, void* dst, int src_dtype, int na_dim, int batch, int heads,
                                   int head_dim, const int32_t* token_layout, const int32_t* tile_shape,
                                   const int32_t* dilation, int flip_tiled_dims, void* stream) {
  if (src_dtype != NATTEN_AMD_F8E4M3 && src_dtype != NATTEN_AMD_F8E5M2) {
    g_error[0] = 0;
    return fail("token_permute_widen: src_dtype must be an 8-bit float code, got %d", src_dtype);
  }
  return tokperm_common("token_permute_widen", false, src_dtype, src, dst, 1, na_dim, batch, heads, head_dim,
                        token_layout, tile_shape, dilation, flip_tiled_dims, stream);
}

int natten_amd_merge_attentions(const void* o0, const float* lse0, const void* o1, const float* lse1, void* out,
                                float* lse_out, int dtype, int64_t rows, int head_dim, void* stream) {
  g_error[0] = 0;
  if (!o0 || !lse0 || !o1 || !lse1 || !out || !lse_out) return fail("merge_attentions: null pointer argument");
  if (rows < 1 || head_dim < 1) return fail("merge_attentions: rows and head_dim must be positive");
  if (lse_out == lse0 || lse_out == lse1) return fail("merge_attentions: lse_out must not alias an input");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // eight elements per thread where head dim and alignment allow 16-byte accesses
  const uintptr_t align = reinterpret_cast<uintptr_t>(o0) | reinterpret_cast<uintptr_t>(o1) | reinterpret_cast<uintptr_t>(out);
  const bool wide = head_dim % 8 == 0 && align % (dtype == NATTEN_AMD_F32 ? 32 : 16) == 0;
  const int64_t total = rows * (wide ? head_dim / 8 : head_dim);
  int64_t blocks = (total + 255) / 256;
  if (blocks > 256 * 64) blocks = 256 * 64;
#define NA_MERGE_LAUNCH(T, VEC)                                                                                     \
  hipLaunchKernelGGL((merge_kernel<T, VEC>), dim3(unsigned(blocks)), dim3(256), 0, s, static_cast<const T*>(o0), lse0, \
                     static_cast<const T*>(o1), lse1, static_cast<T*>(out), lse_out, rows, head_dim)
  switch (dtype) {
    case NATTEN_AMD_F16:
      if (wide) NA_MERGE_LAUNCH(_Float16, 8); else NA_MERGE_LAUNCH(_Float16, 1);
      break;
    case NATTEN_AMD_BF16:
      if (wide) NA_MERGE_LAUNCH(__bf16, 8); else NA_MERGE_LAUNCH(__bf16, 1);
      break;
    case NATTEN_AMD_F32:
      if (wide) NA_MERGE_LAUNCH(float, 8); else NA_MERGE_LAUNCH(float, 1);
      break;
    default:
      return fail("merge_attentions: unsupported dtype code %d", dtype);
  }
#undef NA_MERGE_LAUNCH
  return check_launch("merge_attentions");
}

int natten_amd_merge_attention_parts(const void* parts, const float* lse_parts, int num_parts, void* out, float* lse_out,
                                     int dtype, int64_t rows, int head_dim, void* stream) {
  g_error[0] = 0;
  if (!parts || !lse_parts || !out || !lse_out) return fail("merge_attention_parts: null pointer argument");
  if (rows < 1 || head_dim < 1) return fail("merge_attention_parts: rows and head_dim must be positive");
  if (num_parts < 1 || num_parts > 64) return fail("merge_attention_parts: num_parts must be 1 .. 64, got %d", num_parts);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uintptr_t align = reinterpret_cast<uintptr_t>(parts) | reinterpret_cast<uintptr_t>(out);
  const bool wide = head_dim % 8 == 0 && align % (dtype == NATTEN_AMD_F32 ? 32 : 16) == 0;
  const int64_t total = rows * (wide ? head_dim / 8 : head_dim);
  int64_t blocks = (total + 255) / 256;
  if (blocks > 256 * 64) blocks = 256 * 64;
  const int64_t part_stride = rows * head_dim;
#define NA_MERGE_LAUNCH(T, VEC)                                                                                      \
  hipLaunchKernelGGL((merge_parts_kernel<T, VEC>), dim3(unsigned(blocks)), dim3(256), 0, s, static_cast<const T*>(parts), \
                     lse_parts, num_parts, part_stride, static_cast<T*>(out), lse_out, rows, head_dim)
  switch (dtype) {
    case NATTEN_AMD_F16:
      if (wide) NA_MERGE_LAUNCH(_Float16, 8); else NA_MERGE_LAUNCH(_Float16, 1);
      break;
    case NATTEN_AMD_BF16:
      if (wide) NA_MERGE_LAUNCH(__bf16, 8); else NA_MERGE_LAUNCH(__bf16, 1);
      break;
    case NATTEN_AMD_F32:
      if (wide) NA_MERGE_LAUNCH(float, 8); else NA_MERGE_LAUNCH(float, 1);
      break;
    default:
      return fail("merge_attention_parts: unsupported dtype code %d", dtype);
  }
#undef NA_MERGE_LAUNCH
  return check_launch("merge_attention_parts");
}

int natten_amd_mfma_probe(const void* operands, float* sink, uint64_t* clocks, int iters, int fma_per_mfma,
                          void* stream) {
  g_error[0] = 0;
  if (!operands || !sink || !clocks) return fail("mfma_probe: null pointer argument");
  if (iters < 1) return fail("mfma_probe: iters must be positive");
  hipStream_t s = static_cast<hipStream_t>(stream);
  unsigned long long* c = reinterpret_cast<unsigned long long*>(clocks);
  switch (fma_per_mfma) {
    case 0:
      hipLaunchKernelGGL(mfma_probe_kernel<0>, dim3(kProbeBlocks), dim3(kProbeThreads), 0, s, operands, sink, c, iters);
      break;
    case 4:
      hipLaunchKernelGGL(mfma_probe_kernel<4>, dim3(kProbeBlocks), dim3(kProbeThreads), 0, s, operands, sink, c, iters);
      break;
    default:
      return fail("mfma_probe: fma_per_mfma must be 0 or 4, got %d", fma_per_mfma);
  }
  return check_launch("mfma_probe");
}

}  // extern "C"
