/*
 * natten_amd — C ABI of the MI355X (gfx950) fused neighborhood attention forward path.
 *
 * Every entry point takes plain device pointers and sizes (no framework types), launches on
 * the HIP stream handle it is given (NULL = default stream), never synchronises and never
 * allocates or frees device memory.  The caller owns all buffers.  Return value: 0 on
 * success, non-zero on error; natten_amd_last_error() then returns a message (thread local).
 *
 * The entry points replace, one for one, the native functions the reference binds with
 * pybind11 for this path (paths relative to the SHI-Labs/NATTEN tree):
 *
 *   natten_amd_fna_forward      <- blackwell_na{1,2,3}d_forward
 *                                  csrc/include/natten/blackwell_fna.h:36-52, csrc/natten.cpp:39-160
 *   natten_amd_fna_forward_fused<- the reference driver's permute + kernel + unpermute sequence,
 *                                  src/natten/backends/blackwell_fna.py:99-164, in one launch
 *   natten_amd_fna_forward_fused_split <- the same forward for small grids: several workgroups per
 *                                  Q tile, partial results merged by natten_amd_merge_attention_parts
 *   natten_amd_token_permute    <- token_permute_{1,2,3}d   csrc/include/natten/token_permute.h:34-52
 *   natten_amd_token_permute_widen <- the same, for e4m3 / e5m2 operands (writes bf16)
 *   natten_amd_token_unpermute  <- token_unpermute_{1,2,3}d csrc/include/natten/token_permute.h:54-74
 *   natten_amd_attention_forward<- blackwell_fmha_forward   csrc/include/natten/blackwell_fmha.h
 *                                  (dense attention used for additional keys/values and for
 *                                  kernel_size == input size)
 *   natten_amd_attention_forward_varlen <- the same function with cumulative_seqlen_Q / _KV,
 *                                  max_seqlen_Q / _KV (csrc/include/natten/blackwell_fmha.h:34-50)
 *   natten_amd_fna_backward     <- blackwell_na{1,2,3}d_backward
 *                                  csrc/include/natten/blackwell_fna.h:92-160
 *   natten_amd_fna_backward_fused <- the reference driver's permutes + backward + unpermutes,
 *                                  src/natten/backends/blackwell_fna.py:205-297, without the copies
 *   natten_amd_attention_backward <- blackwell_fmha_backward csrc/include/natten/blackwell_fmha.h:52-73
 *                                  (fixed-length batches)
 *   natten_amd_attention_backward_varlen <- the same function with cumulative_seqlen_Q / _KV,
 *                                  max_seqlen_Q / _KV (csrc/include/natten/blackwell_fmha.h:52-73)
 *   natten_amd_compute_delta    <- compute_delta            csrc/include/natten/compute_delta.h:33-36
 *   natten_amd_merge_attentions <- the elementwise merge of src/natten/attn_merge.py:48-105
 *                                  (the reference runs it as framework ops; here it is one kernel)
 *   natten_amd_merge_attention_parts <- the same merge over any number of partial results at once
 */
#ifndef NATTEN_AMD_H_
#define NATTEN_AMD_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types of Q/K/V (`dtype` arguments). */
#define NATTEN_AMD_F16 0
#define NATTEN_AMD_BF16 1
#define NATTEN_AMD_F8E4M3 2 /* OCP e4m3fn operands, bf16 output */
#define NATTEN_AMD_F32 3    /* float32 operands and output (natten_amd_fna_forward), merge payloads */
#define NATTEN_AMD_F8E5M2 4 /* OCP e5m2 operands, bf16 output */

/* ABI version; bumped whenever a signature changes. */
int natten_amd_abi_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char* natten_amd_last_error(void);

/*
 * Fused neighborhood attention forward on token-permuted operands.
 *
 *   q   [batch, seqlen_q,  heads_q,  head_dim]   contiguous
 *   k,v [batch, seqlen_kv, heads_kv, head_dim]   contiguous, heads_q % heads_kv == 0
 *   out [batch, seqlen_q,  heads_q,  head_dim]   dtype of q (bf16 for 8-bit float operands)
 *   lse [batch, seqlen_q,  heads_q]              float32, natural log of the sum of exp(scale*q.k)
 *
 * `batch` already includes the dilation groups (batch index = b * prod(dilation) + group,
 * group decoded with dimension 0 fastest).  q_shape / kv_shape are the padded per-group token
 * layouts the permuted sequences were built from (seqlen = product), qkv_shape the original
 * token layout.  All shape-like arrays hold `na_dim` entries.  Tiles are multi-dimensional;
 * their element counts must be a supported (Q tile, KV tile) pair, see
 * natten_amd_fna_supported_tiles().  head_dim must be 32, 64 or 128 (64 or 128 for 8-bit floats).
 *
 * q_scale [heads_q], k_scale [heads_kv], v_scale [heads_kv] are optional device arrays of
 * per-head dequantisation scales (NULL = 1): logits are scale * q_scale[h] * k_scale[hkv] * q.k,
 * the output is multiplied by v_scale[hkv], and lse is the log-sum-exp of those logits.
 *
 * 8-bit float operands (dtype F8E4M3 / F8E5M2; the reference passes such tensors to this same
 * entry point, csrc/src/blackwell_fna_forward.cu:81-222) are multiplied by the 8-bit matrix
 * instruction with the probabilities rounded to e4m3, as the reference rounds them to the operand
 * type; tiles must be 128 x 64 tokens.  A more accurate, slower route for the same operands:
 * widen them to bf16 while permuting (natten_amd_token_permute_widen, exact) and call this
 * function with dtype BF16 and the scales.
 *
 * float32 operands (dtype F32; the reference's tests run float32 at atol 1e-4,
 * tests/test_fna.py:107-131): tiles of 128 x 64 tokens, head_dim 32, 64 or 128, no scales; products,
 * sums and softmax in float32 (P not rounded), output float32.  This entry point only (no one-launch
 * form, no backward).
 *
 * run_persistent (the reference's `run_persistent` argument, blackwell_fna.h:52, scheduler
 * csrc/include/natten/cuda/fmha_blackwell/kernel/fmha_tile_scheduler.hpp:146-149): non-zero
 * launches as many workgroups as the device keeps resident, which take Q tiles from per-XCD work
 * queues until none is left, instead of one workgroup per Q tile; results are bit-identical.
 * The queues are counters in `workspace`: device memory owned by the caller, 64-byte aligned,
 * at least natten_amd_fna_forward_workspace_bytes() bytes, free for reuse once the work queued on
 * `stream` by this call has run.  run_persistent == 1: the launch clears them first (by a kernel,
 * so the call may be captured in a graph): any memory will do.  run_persistent == 2: the caller
 * vouches that they are zero, which is how every work-queue launch leaves them (its last workgroup
 * resets them): a workspace zeroed once and then only handed to these launches, one at a time,
 * needs no clearing again, and the call is a single kernel launch.  (A launch that did not run to
 * completion leaves counts behind; a later call in this mode on that workspace would then skip Q
 * tiles without any error: after a failed or aborted launch, clear the workspace or use mode 1.)
 * Two calls must not use one workspace concurrently.  Tile
 * pairs other than 128 x 64 tokens and float32 operands ignore the flag.  run_persistent == 0:
 * workspace may be NULL.
 */
uint64_t natten_amd_fna_forward_workspace_bytes(void);
int natten_amd_fna_forward(const void* q, const void* k, const void* v, void* out, float* lse,
                           int dtype, int na_dim, int batch, int seqlen_q, int seqlen_kv,
                           int heads_q, int heads_kv, int head_dim, const int32_t* q_shape,
                           const int32_t* kv_shape, const int32_t* qkv_shape,
                           const int32_t* kernel_size, const int32_t* stride,
                           const int32_t* dilation, const int32_t* is_causal,
                           const int32_t* q_tile_shape, const int32_t* kv_tile_shape, float scale,
                           const float* q_scale, const float* k_scale, const float* v_scale,
                           int run_persistent, void* workspace, uint64_t workspace_bytes,
                           void* stream);

/*
 * The same function in one launch on the ORIGINAL tensors: q [batch, *qkv_shape, heads_q,
 * head_dim], k / v [batch, *qkv_shape, heads_kv, head_dim], out like q, lse [batch, *qkv_shape,
 * heads_q].  The kernel gathers the rows of each tile from the input and scatters its results,
 * so the three token permutes and two unpermutes around natten_amd_fna_forward (what the
 * reference's driver runs as separate operations, src/natten/backends/blackwell_fna.py:99-164)
 * disappear.  Which extents are taken:
 *   - every qkv_shape[a] a multiple of dilation[a] * kv_tile_shape[a] (no KV tile reaches past
 *     its dilation group): every dtype but float32 and every tile pair; with anchor_kv_tiles == 0
 *     the results are bit-identical to the permuted path with the same tile shapes;
 *   - any other extent whose dilation groups are all at least one KV tile wide in every dimension
 *     (fp16 / bf16 and 8-bit float operands): a tile that would reach past its dilation group is
 *     gathered from one tile extent before the group's end and its leading keys, which the tile
 *     before it delivered, are masked (sums then run in another order than on the permuted path);
 *   - a dilation group narrower than the KV tile in some dimension: fp16 / bf16 operands with tiles
 *     of 128 x 64 tokens only (the instance that clamps its gathers).
 * Anything else returns an error that says which rule was missed, and the caller uses the
 * permuted path.  A KV tile must span less than 2^31 bytes of the input.  dtype, tiles, head_dim,
 * scales, run_persistent and workspace as in natten_amd_fna_forward.
 *
 * anchor_kv_tiles != 0: the KV tiles of a Q tile are laid out from the first key of its window
 * box (per dimension) instead of from multiples of the KV tile extent -- there is no permuted
 * layout to follow here -- so no tile lies partly before the window: fewer tiles are visited
 * whenever window starts are not multiples of the tile extent (stride 1, or strides that do not
 * divide the tile).  Needs every dilation group at least one KV tile wide in every dimension and
 * is ignored otherwise.  Sums run in a different order than with anchor_kv_tiles == 0, which is
 * bit-identical to the permuted path where the tiles divide the extents.
 */
int natten_amd_fna_forward_fused(const void* q, const void* k, const void* v, void* out,
                                 float* lse, int dtype, int na_dim, int batch, int heads_q,
                                 int heads_kv, int head_dim, const int32_t* qkv_shape,
                                 const int32_t* kernel_size, const int32_t* stride,
                                 const int32_t* dilation, const int32_t* is_causal,
                                 const int32_t* q_tile_shape, const int32_t* kv_tile_shape,
                                 float scale, const float* q_scale, const float* k_scale,
                                 const float* v_scale, int anchor_kv_tiles, int run_persistent,
                                 void* workspace, uint64_t workspace_bytes, void* stream);

/*
 * natten_amd_fna_forward_fused for problems with fewer Q tiles than the chip keeps workgroups
 * resident (few heads, small inputs, long windows): the same operation
 * (blackwell_na{1,2,3}d_forward, csrc/include/natten/blackwell_fna.h:36-52, with the driver's
 * permutes folded in) launched with kv_splits (2 .. 8) workgroups per Q tile, each on a
 * contiguous run of the tile's KV tiles.  out_parts [kv_splits][batch, *qkv_shape, heads_q,
 * head_dim] and lse_parts [kv_splits][batch, *qkv_shape, heads_q] receive one partial result per
 * run, normalised over the keys of that run, with their log-sum-exp (zeros and -inf for a query
 * none of whose keys lie in the run); natten_amd_merge_attention_parts combines them
 * (src/natten/attn_merge.py:48-105 is the arithmetic).  fp16 / bf16 operands, Q
 * tiles of 128 and KV tiles of 64 tokens, no dequantisation scales; other arguments as in
 * natten_amd_fna_forward_fused.
 */
int natten_amd_fna_forward_fused_split(const void* q, const void* k, const void* v, void* out_parts,
                                       float* lse_parts, int dtype, int na_dim, int batch,
                                       int heads_q, int heads_kv, int head_dim,
                                       const int32_t* qkv_shape, const int32_t* kernel_size,
                                       const int32_t* stride, const int32_t* dilation,
                                       const int32_t* is_causal, const int32_t* q_tile_shape,
                                       const int32_t* kv_tile_shape, float scale,
                                       int anchor_kv_tiles, int kv_splits, void* stream);

/*
 * natten_amd_fna_forward_fused with run_persistent = 1 for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
 * it has no counterpart in the reference.  The queue counters live in a 512-byte array inside
 * the library's device image instead of a workspace, and the call allocates and frees nothing
 * (no hipMalloc / hipFree, no allocating library routine).  Operands, results and arguments
 * are those of natten_amd_fna_forward_fused; limits: fp16 / bf16 operands, Q tiles of 128 and
 * KV tiles of 64 tokens (the work-queue kernel's), at most 2^31 - 4096 Q tiles over all
 * (batch, head) pairs; anything else is refused with an error.  Results are bit-identical to
 * natten_amd_fna_forward_fused with anchor_kv_tiles = 1.  Every call on a GPU shares that GPU's array (the launch clears
 * it first, with a kernel): calls that overlap in time on one GPU -- on different streams or
 * from different threads -- race on the queues and must not be made; calls queued on one
 * stream are fine.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress, once per device): make one call on the device eagerly before the entry
 * point is used on a stream that is capturing a graph.
 */
int natten_amd_fna_forward_fused_static(const void* q, const void* k, const void* v, void* out,
                                        float* lse, int dtype, int na_dim, int batch, int heads_q,
                                        int heads_kv, int head_dim, const int32_t* qkv_shape,
                                        const int32_t* kernel_size, const int32_t* stride,
                                        const int32_t* dilation, const int32_t* is_causal,
                                        const int32_t* q_tile_shape, const int32_t* kv_tile_shape,
                                        float scale, const float* q_scale, const float* k_scale,
                                        const float* v_scale, void* stream);

/*
 * Host arithmetic only (no device call): the window [*start, *end) of key coordinates that query
 * coordinate `query` attends along one dimension of a dilation group of `extent` tokens --
 * csrc/include/natten/cuda/fna_blackwell/collective/fna_fusion.hpp:88-123 (get_win_start /
 * get_win_end), evaluated with the same routine the forward kernels' set-up uses (the stride's
 * division replaced by a multiply and a shift), so that tests can pin it against the oracle.
 */
int natten_amd_window(int query, int kernel_size, int stride, int extent, int is_causal,
                      int32_t* start, int32_t* end);

/*
 * Host arithmetic only: the keys of a 64-key KV tile (numbered with dimension 0 fastest, extents
 * kv_tile_shape[0..2], powers of two) whose in-tile coordinates lie in [lo[a], hi[a]) along every
 * dimension, one bit per key -- the element mask the forward kernels apply to a partially attended
 * tile (csrc/include/natten/cuda/fna_blackwell/collective/fna_fusion.hpp:384-436 tests the same
 * condition coordinate by coordinate), built from the same per-dimension rows the kernels keep in
 * LDS, so that tests can pin it against a brute-force decode.
 */
int natten_amd_tile_key_mask(const int32_t* kv_tile_shape, const int32_t* lo, const int32_t* hi,
                             uint64_t* mask);

/*
 * Host arithmetic only: *result = 1 when natten_amd_fna_forward_fused would run this problem with
 * the kernel instance that holds no mask code (every KV tile a Q tile visits is attended in full
 * by all of its queries), the launch-level predicate of
 * csrc/include/natten/cuda/fna_blackwell/collective/fna_fusion.hpp:503-593 (fully_block_sparse).
 */
int natten_amd_fna_fully_block_sparse(int na_dim, const int32_t* qkv_shape,
                                      const int32_t* kernel_size, const int32_t* stride,
                                      const int32_t* dilation, const int32_t* is_causal,
                                      const int32_t* q_tile_shape, const int32_t* kv_tile_shape,
                                      int anchor_kv_tiles, int32_t* result);

/*
 * Host arithmetic only: the box of 32 queries (extents per dimension, product 32) that one wave of
 * the 16-bit forward kernels holds for this problem.  A Q tile is a grid of such boxes; a (wave, KV
 * tile) pair needs the element mask unless the tile lies inside the windows of all of the wave's
 * queries or outside all of them, and the launch takes the box with the fewest pairs that do (the
 * row-major box on ties).  No counterpart in the reference, whose threads own rows of a fixed
 * layout.
 */
int natten_amd_fna_wave_box(int na_dim, const int32_t* qkv_shape, const int32_t* kernel_size,
                            const int32_t* stride, const int32_t* dilation,
                            const int32_t* is_causal, const int32_t* q_tile_shape,
                            const int32_t* kv_tile_shape, int anchor_kv_tiles, int32_t* box);

/*
 * Supported tile sizes (tokens per tile).  Writes up to `capacity` pairs
 * (q_tile_size, kv_tile_size) for the given dtype / head_dim and returns how many exist.
 */
int natten_amd_fna_supported_tiles(int dtype, int head_dim, int32_t* q_sizes, int32_t* kv_sizes,
                                   int capacity);

/*
 * Dense attention forward (optional top-left causal mask) on unpermuted operands.
 *   q [batch, seqlen_q, heads_q, head_dim], k/v [batch, seqlen_kv, heads_kv, head_dim],
 *   out like q, lse [batch, seqlen_q, heads_q] float32.  Any seqlen >= 1.
 * q_scale / k_scale / v_scale as in natten_amd_fna_forward.
 */
int natten_amd_attention_forward(const void* q, const void* k, const void* v, void* out,
                                 float* lse, int dtype, int batch, int seqlen_q, int seqlen_kv,
                                 int heads_q, int heads_kv, int head_dim, int is_causal,
                                 float scale, const float* q_scale, const float* k_scale,
                                 const float* v_scale, void* stream);

/*
 * Dense attention forward on sequence-packed operands (variable-length batches).
 *   q / out [total_seqlen_q, heads_q, head_dim], k / v [total_seqlen_kv, heads_kv, head_dim],
 *   lse [total_seqlen_q, heads_q] float32.  Sequence b (0 <= b < num_seqs) owns query rows
 *   cumulative_seqlen_q[b] .. cumulative_seqlen_q[b+1]-1 and key rows likewise; the two int32
 *   arrays of num_seqs + 1 entries live in device memory.  max_seqlen_* bound the sequence
 *   lengths (the launch is sized from them; rows of a longer sequence would not be computed).
 *   The causal mask is top-left aligned per sequence.  A sequence without keys gets
 *   out = 0 and lse = -inf.  Rows that belong to no sequence are not written.
 *   16-bit float operands only.
 */
int natten_amd_attention_forward_varlen(const void* q, const void* k, const void* v, void* out,
                                        float* lse, int dtype, int num_seqs, int total_seqlen_q,
                                        int total_seqlen_kv, int max_seqlen_q, int max_seqlen_kv,
                                        int heads_q, int heads_kv, int head_dim,
                                        const int32_t* cumulative_seqlen_q,
                                        const int32_t* cumulative_seqlen_kv, int is_causal,
                                        float scale, const float* q_scale, const float* k_scale,
                                        const float* v_scale, void* stream);

/*
 * Host-only helper (no GPU work): the interval of query coordinates 0 .. num_queries-1 whose
 * window meets the key coordinates key_first .. key_last of one dimension of `extent` keys:
 * what the dK/dV kernel iterates over per KV tile (the role of get_trip_count in
 * csrc/include/natten/cuda/fna_blackwell/collective/fna_fusion_bwd.hpp:256-318).  An empty
 * interval comes back as *first_query > *last_query.
 */
int natten_amd_query_range(int key_first, int key_last, int kernel_size, int stride, int extent,
                           int num_queries, int is_causal, int32_t* first_query,
                           int32_t* last_query);

/*
 * delta[i] = sum_d out[i, d] * d_out[i, d] for `items` rows of head_dim contiguous elements
 * (any layout whose last dimension is head_dim: items = batch * tokens * heads).  float32 result.
 */
int natten_amd_compute_delta(const void* out, const void* d_out, float* delta, int dtype,
                             int64_t items, int head_dim, void* stream);

/*
 * Fused neighborhood attention backward on token-permuted operands.
 *   q, d_out, dq [batch, seqlen_q, heads_q, head_dim]; k, v, dk, dv [batch, seqlen_kv, heads_kv,
 *   head_dim], permuted like the forward operands (dimension 0 fastest inside a tile, dilation
 *   groups folded into batch); lse, delta float32, permuted the same way and then stored
 *   head-major, [batch, heads_q, seqlen_q] (the kernels read 64 consecutive rows of one head at
 *   a time); lse from the forward pass (natural log), delta from natten_amd_compute_delta.
 *   Both tile shapes must hold 128 tokens and their last extent above 1 must be even; q_shape /
 *   kv_shape are the padded per-group layouts (multiples of the tiles), seqlen = their product.
 * dq, dk, dv are written completely (padding rows get zeros); nothing is accumulated through
 * memory, results are deterministic.  The gradient of the LSE output is not propagated (as in
 * the reference).  16-bit float operands, head_dim 32 / 64 / 128.
 *
 * q_scaled (all four backward entry points): workspace of q's shape and type.  The forward
 * kernel multiplies the keys with q' = round(q * scale * log2(e)) (rounded to the operand type
 * once), so that its logits need no further scaling; the backward forms its logits from the same
 * q', which makes its probabilities exp(logit - LSE) those the forward normalised (they sum to
 * one over a query's window).  The launch that writes dq scales the query rows it holds in
 * registers; the launch that writes dk and dv streams q' and first writes it to q_scaled with
 * one pass over q.  The call makes the dk / dv launch first and the dq launch last, so q_scaled
 * may be the dq buffer itself (for a call that only makes the dk / dv launch: if dq is written
 * afterwards); it must not be q.  May be null for a call that only makes the dq launch.
 */
int natten_amd_fna_backward(const void* q, const void* k, const void* v, const void* d_out,
                            const float* lse, const float* delta, void* dq, void* dk, void* dv,
                            void* q_scaled, int dtype, int na_dim, int batch, int seqlen_q, int seqlen_kv,
                            int heads_q, int heads_kv, int head_dim, const int32_t* q_shape,
                            const int32_t* kv_shape, const int32_t* qkv_shape,
                            const int32_t* kernel_size, const int32_t* stride,
                            const int32_t* dilation, const int32_t* is_causal,
                            const int32_t* q_tile_shape, const int32_t* kv_tile_shape, float scale,
                            void* stream);

/*
 * The same backward on the original tensors: q, d_out, dq [batch, *qkv_shape, heads_q, head_dim],
 * k, v, dk, dv [batch, *qkv_shape, heads_kv, head_dim], lse and delta head-major
 * [batch, heads_q, prod(qkv_shape)].  The kernels gather and scatter the rows of their tiles
 * themselves, which replaces the six token permutes and three unpermutes of the reference's
 * backward driver (src/natten/backends/blackwell_fna.py:205-297).  Where every extent is a
 * multiple of dilation x tile for both tile shapes the results are bit-identical to that
 * sequence.  Other extents are taken as long as every dilation group is at least one tile wide
 * (both tile shapes) in every dimension: rows of a tile past the end of its dilation group are
 * computed on a clamped copy and not stored, a streamed tile that would reach past the group is
 * gathered from one tile extent before its end and its leading rows, which the tile before it
 * delivered, take no part (sums then run in another order than on permuted operands).  Narrower
 * groups return an error: use natten_amd_fna_backward on permuted operands.
 *
 * roles: 3 makes both launches; 1 only the one that writes dq, 2 only the one that writes dk and
 * dv (the other results are left untouched).  With no permuted layout to share, the two launches
 * need not use the same tile shapes: the dq launch streams half KV tiles past a Q tile, the
 * dk / dv launch half Q tiles past a KV tile, and the shapes that visit the fewest tiles differ
 * (a caller makes one call per role, each with that role's shapes).
 */
int natten_amd_fna_backward_fused(const void* q, const void* k, const void* v, const void* d_out,
                                  const float* lse, const float* delta, void* dq, void* dk,
                                  void* dv, void* q_scaled, int dtype, int na_dim, int batch, int heads_q,
                                  int heads_kv, int head_dim, const int32_t* qkv_shape,
                                  const int32_t* kernel_size, const int32_t* stride,
                                  const int32_t* dilation, const int32_t* is_causal,
                                  const int32_t* q_tile_shape, const int32_t* kv_tile_shape,
                                  float scale, int roles, void* stream);

/*
 * Dense attention backward (optional top-left causal mask).  Operands as above (lse and delta
 * head-major) with sequences zero-padded to padded_seqlen_q / padded_seqlen_kv rows (multiples
 * of 128); seqlen_q / seqlen_kv are the true lengths.
 */
int natten_amd_attention_backward(const void* q, const void* k, const void* v, const void* d_out,
                                  const float* lse, const float* delta, void* dq, void* dk,
                                  void* dv, void* q_scaled, int dtype, int batch, int seqlen_q, int seqlen_kv,
                                  int padded_seqlen_q, int padded_seqlen_kv, int heads_q,
                                  int heads_kv, int head_dim, int is_causal, float scale,
                                  void* stream);

/*
 * Dense attention backward of a sequence-packed batch, one set of launches for all sequences.
 * The operands hold the `num_seqs` sequences back to back, each zero-padded to a multiple of
 * 128 rows: q, d_out, dq [1, rows_q, heads_q, head_dim], k, v, dk, dv [1, rows_kv, heads_kv,
 * head_dim], lse and delta head-major [1, heads_q, rows_q]; rows_q and rows_kv are multiples
 * of 128.  All four cumulative arrays are device int32 [num_seqs + 1]: sequence b has
 * cu_seqlens_q[b+1] - cu_seqlens_q[b] queries, which are rows padded_cu_seqlens_q[b] ... of the
 * operands (padded_cu_seqlens_* count padded lengths: multiples of 128, each covering the
 * sequence); keys likewise.  max_seqlen_q / max_seqlen_kv bound the sequence lengths (they size
 * the grid; rows of longer sequences would be left out).  Rows of dq, dk, dv outside every
 * sequence's padded range are not written.  A sequence whose offsets do not fit the row counts
 * is skipped by the kernels (the host cannot see the device arrays).  No host synchronisation.
 */
int natten_amd_attention_backward_varlen(const void* q, const void* k, const void* v,
                                         const void* d_out, const float* lse, const float* delta,
                                         void* dq, void* dk, void* dv, void* q_scaled, int dtype, int num_seqs,
                                         int rows_q, int rows_kv, const int32_t* cu_seqlens_q,
                                         const int32_t* cu_seqlens_kv,
                                         const int32_t* padded_cu_seqlens_q,
                                         const int32_t* padded_cu_seqlens_kv, int max_seqlen_q,
                                         int max_seqlen_kv, int heads_q, int heads_kv,
                                         int head_dim, int is_causal, float scale, void* stream);

/*
 * Token permute: src [batch, *token_layout, heads, head_dim] -> dst
 * [batch * prod(dilation), prod(ceil(ceil(X/t)/d) * t), heads, head_dim]; padding rows are
 * zero.  Payload is copied verbatim (`elem_bytes` bytes per element, any type).
 */
int natten_amd_token_permute(const void* src, void* dst, int elem_bytes, int na_dim, int batch,
                             int heads, int head_dim, const int32_t* token_layout,
                             const int32_t* tile_shape, const int32_t* dilation,
                             int flip_tiled_dims, void* stream);

/*
 * Token permute of an 8-bit float tensor (src_dtype F8E4M3 or F8E5M2) that writes bf16: same
 * index map as natten_amd_token_permute, every element converted exactly (all e4m3 / e5m2
 * values are bf16 values; NaN stays NaN).  heads * head_dim must be a multiple of 8.
 * With token_layout = {seqlen}, tile_shape = {1}, dilation = {1} it is a plain widening copy.
 * The reference permutes the 8-bit payload verbatim (csrc/include/natten/token_permute.h:34-52)
 * and multiplies in 8 bits; here the operands are widened on the permute's HBM pass and the
 * products are taken in bf16.
 */
int natten_amd_token_permute_widen(const void* src, void* dst, int src_dtype, int na_dim,
                                   int batch, int heads, int head_dim,
                                   const int32_t* token_layout, const int32_t* tile_shape,
                                   const int32_t* dilation, int flip_tiled_dims, void* stream);

/* Inverse of natten_amd_token_permute; padding rows of `src` are dropped. */
int natten_amd_token_unpermute(const void* src, void* dst, int elem_bytes, int na_dim, int batch,
                               int heads, int head_dim, const int32_t* token_layout,
                               const int32_t* tile_shape, const int32_t* dilation,
                               int flip_tiled_dims, void* stream);

/*
 * Merge two partial attentions over disjoint key sets of the same queries:
 *   out = o0 - sigmoid(lse1 - lse0) * (o0 - o1),  lse = lse0 - logsigmoid(lse0 - lse1)
 * o0/o1/out [rows, head_dim] of `dtype` (F16/BF16/F32), lse0/lse1/lse_out [rows] float32,
 * rows = batch * seqlen * heads.  out may alias o0; lse_out must not alias lse0 or lse1
 * (several lanes of a row read both while one writes the result; aliasing is rejected).
 */
int natten_amd_merge_attentions(const void* o0, const float* lse0, const void* o1,
                                const float* lse1, void* out, float* lse_out, int dtype,
                                int64_t rows, int head_dim, void* stream);

/*
 * The same merge over num_parts (1 .. 64) partial attentions that lie one after the other:
 * parts [num_parts][rows, head_dim], lse_parts [num_parts][rows] -- the layout
 * natten_amd_fna_forward_fused_split writes.  out = sum_i exp(lse_i - lse) parts_i,
 * lse = log sum_i exp(lse_i), in float32 and rounded once: what src/natten/attn_merge.py:48-105
 * computes by merging two at a time, without the roundings in between.  A row all of whose parts
 * hold no key (lse -inf) gives zeros and -inf.
 */
int natten_amd_merge_attention_parts(const void* parts, const float* lse_parts, int num_parts,
                                     void* out, float* lse_out, int dtype, int64_t rows,
                                     int head_dim, void* stream);

/*
 * Diagnostic without a counterpart in the reference: sustained rate of the bf16 matrix
 * instruction the fused kernel is built on.  256 workgroups of 256 threads (one wave per SIMD
 * of an MI355X) each run `iters` x 16 v_mfma_f32_32x32x16_bf16 (interleaved with `fma_per_mfma`
 * = 0 or 4 independent v_fma_f32 each) on operands read once from `operands`.
 *   operands: 256 * 256 * 128 bytes of bf16 values (random values show the rate the power
 *             limit allows; constant ones the rate at the highest clock)
 *   sink:     256 * 256 floats, written
 *   clocks:   2 * 256 uint64, written: per workgroup, shader cycles and 100 MHz ticks spent
 * Work per launch: 256 * 4 * iters * 16 * 32768 FLOP; time it on the stream.
 */
int natten_amd_mfma_probe(const void* operands, float* sink, uint64_t* clocks, int iters,
                          int fma_per_mfma, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* NATTEN_AMD_H_ */
