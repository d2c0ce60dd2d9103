/*
 * mi_ep.h -- C ABI of the MI355X (gfx950) expert-parallel dispatch core.
 *
 * One GPU; the reference's "ranks" are partitions of this GPU's HBM.  Every
 * pointer is a device pointer unless stated otherwise, every call enqueues on
 * `stream` (a hipStream_t passed as void*, NULL = the null stream) and returns
 * without synchronising.  The caller owns every buffer.  Return value: 0 on
 * success, a negative MI_EP_E* code for bad arguments, a positive hipError_t
 * when the HIP runtime reports one.  Nothing here exits the process.
 *
 * Reference files are cited relative to the reference tree's datasets/ folder.
 */
#ifndef MI_EP_H_
#define MI_EP_H_

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI_EP_ABI_VERSION 3

#define MI_EP_OK 0
#define MI_EP_EINVAL (-22)    /* argument out of range or NULL where required */
#define MI_EP_ENOSPC (-28)    /* workspace too small */
#define MI_EP_ETIMEDOUT (-110) /* device-side bounded wait expired (mi_ep_workspace_status) */
#define MI_EP_E2BIG (-7)      /* shape exceeds the static scratch of mi_ep_dispatch_layout_static */

/* Limits.  Ranks and top-k follow the reference's constructor checks
 * (example042_deepep_dispatch_layout/nv/empty_deepep_dispatch_layout.cu:43,46,96-107). */
#define MI_EP_MAX_RANKS 8
#define MI_EP_MAX_TOPK 8
#define MI_EP_MAX_EXPERTS 1024

int mi_ep_abi_version(void);
const char* mi_ep_strerror(int code);

/*
 * Dispatch layout, exact kernel-level signature of
 * example042_deepep_dispatch_layout/nv/empty_deepep_dispatch_layout.cu:48-58
 * (deepep_get_dispatch_layout_kernel) plus the stream of
 * DeepepDispatchLayout::compute (:110-132).
 *   topk_idx                  int64[num_tokens, num_topk]; < 0 = masked slot
 *   num_tokens_per_rank       int32[num_ranks]   one per (token, rank) pair
 *   num_tokens_per_rdma_rank  accepted and ignored (always NULL in the reference)
 *   num_tokens_per_expert     int32[num_experts] every valid slot counts
 *   is_token_in_rank          bool[num_tokens, num_ranks]
 * Outputs are overwritten, not accumulated into (the reference benchmark never
 * re-zeroes them, :313-329).  Needs no workspace.
 */
int mi_ep_get_dispatch_layout(const int64_t* topk_idx, int* num_tokens_per_rank,
                              int* num_tokens_per_rdma_rank, int* num_tokens_per_expert,
                              bool* is_token_in_rank, int num_tokens, int num_topk, int num_ranks,
                              int num_experts, void* stream);

/*
 * Workspace of the fused layout kernel below.  It must be initialised once
 * (mi_ep_workspace_init) before its first use; every later call leaves it ready
 * for the next.  Calls that share one workspace must not overlap in time.
 * It must be 8-byte aligned; with 16-byte alignment (any hipMalloc result) grids
 * of up to a few dozen tiles scan their tiles' totals with wide loads, which is
 * about 2 us faster per launch.
 * The three calls that take a workspace pointer below (init, status, set_wait_limit) also accept
 * MI_EP_STATIC_SCRATCH: the library's own scratch of mi_ep_dispatch_layout_static on the device
 * `stream` belongs to (workspace_bytes is ignored then).  That scratch starts initialised;
 * initialising it again clears a reported time-out.
 */
#define MI_EP_STATIC_SCRATCH ((void*)(size_t)256)
size_t mi_ep_workspace_bytes(int num_tokens, int num_topk, int num_experts, int num_ranks);
int mi_ep_workspace_init(void* workspace, size_t workspace_bytes, void* stream);
/* Synchronises `stream`, then reports MI_EP_ETIMEDOUT if any launch on this
 * workspace gave up a bounded device-side wait since the last init. */
int mi_ep_workspace_status(const void* workspace, void* stream);

/* Bounds the device-side waits of later mi_ep_dispatch_layout launches on THIS workspace: a wait
 * gives up at its max_polls-th unsuccessful poll in a row (0 restores the default of about four
 * million, a few seconds).  Enqueue-only; mi_ep_workspace_init resets it to the default.  A launch
 * whose wait expires still terminates; its outputs are then unspecified, dispatch calls fed with
 * them write no row outside the destination buffer, and the workspace reports MI_EP_ETIMEDOUT until
 * it is initialised again: check mi_ep_workspace_status before trusting the outputs of a launch that
 * may have timed out.  The reference's counterpart is the kNumTimeoutCycles template argument of
 * dispatch_impl (example080_deepep_jit_dispatch_payload/nv/empty_deepep_jit_dispatch_payload.cu:29,122-143). */
int mi_ep_workspace_set_wait_limit(void* workspace, unsigned int max_polls, void* stream);

/* What the destination-order copy kernel assumes of a device, as the runtime reports it for the
 * device `stream` belongs to (the current device for NULL): compute units, accelerator dies
 * (XCCs) and bytes of L2 per die; any pointer may be NULL.  The kernel is tuned for 8 dies that
 * take workgroups round-robin and 4 MiB of L2 each; on anything else (another partition mode,
 * another part) mi_ep_dispatch takes the token-order kernel unless told otherwise. */
int mi_ep_device_traits(int* compute_units, int* dies, int* l2_bytes, void* stream);
/* The kernel mi_ep_dispatch picks by itself for a shape when route_order is given, on a device
 * with these traits (from mi_ep_device_traits): MI_EP_DISPATCH_BY_TOKEN or
 * MI_EP_DISPATCH_BY_DESTINATION (kernel symbols ep_permute_kernel and ep_permute_tiles_kernel), or
 * MI_EP_EINVAL.  Touches no device. */
int mi_ep_dispatch_schedule_for(int num_tokens, int num_topk, int num_experts, int row_bytes, int dies,
                                int l2_bytes);

/*
 * Fused single-pass layout: everything the reference spreads over
 *   example042 (counts + flags, empty_deepep_dispatch_layout.cu:48-86),
 *   example047 (per-channel inclusive prefix, empty_deepep_intranode_notify_dispatch.cu:132-143),
 *   example078 (deterministic slots, empty_deepep_jit_dispatch_deterministic_prologue.cu:27-43),
 *   example080 notify role (histogram, aligned exclusive expert psum, inclusive rank
 *   psum, empty_deepep_jit_dispatch_payload.cu:78-107,197-239).
 * Outputs:
 *   num_tokens_per_rank / num_tokens_per_expert / is_token_in_rank   as above
 *   expert_offsets      int32[num_experts + 1]; off[0] = 0,
 *                       off[e+1] = off[e] + round_up(count[e], expert_alignment)
 *   psum_rank_rows      int32[num_ranks]; inclusive rows of partitions 0..r
 *   channel_prefix_matrix int32[num_ranks, num_channels]; tokens flagged for rank r in
 *                       token tiles 0..c (tile bounds as get_channel_task_range, :73-79)
 *   rank_prefix_matrix  int32[num_ranks, num_ranks], source-major: [src, dst] = tokens of source
 *                       chunks 0..src flagged for rank dst, the tokens taken as num_ranks contiguous
 *                       chunks of ceil(num_tokens / num_ranks) (the same range rule, :73-79), one per
 *                       source rank: rank_prefix_matrix_copy of notify_dispatch
 *                       (empty_deepep_intranode_notify_dispatch.cu:112-143, checked at :352-384),
 *                       which the reference gathers from R GPUs and this GPU's partitions provide
 *                       in the same launch as the channel matrix; row num_ranks - 1 equals
 *                       num_tokens_per_rank
 *   slot_rel            int32[num_tokens, num_topk]; position of route (t,k) inside its
 *                       expert segment in (token, slot) order, -1 for non-routes
 *   rank_slot_idx       int32[num_tokens, num_topk]; the prologue's own output format
 *                       (dst_buffer_slot_idx, example078 .cu:36-40): for the first slot of every
 *                       distinct destination rank of a token, rank_slot_base + the number of
 *                       earlier tokens sent to that rank; -1 for masked slots and for further
 *                       slots on a rank the token already reaches.  rank_slot_base stands for
 *                       scaleup_rank_idx * kNumMaxTokensPerRank.
 *   route_order         int32[mi_ep_route_order_bytes / 16, 4]; per tile of 256 consecutive
 *                       tokens (tile j owns entries [j*256*K, (j+1)*256*K)), the tile's routes as
 *                       {t*K + k, expert, slot_rel, t} sorted by (expert, slot_rel), followed by
 *                       its non-routes as {t*K + k, -1, -1, t} in (token, slot) order; entries
 *                       past the last token's are not written.  It lets mi_ep_dispatch write
 *                       recv_x in destination order (no counterpart in the reference, whose
 *                       senders push token by token; the nearest relative is the sorted pull
 *                       list of example056 compute_dispatch_indices, :521-564).  16-byte aligned.
 *   tile_rank_counts    int32[ceil(num_tokens / 256), num_ranks]; tokens of each 256-token tile
 *                       flagged for each rank: the one-GPU form of rank_count_buffer[sm, rank]
 *                       (example078 .cu:20,34-35), a tile standing for an SM's share of the tokens
 *   copied_topk_idx     int64[num_tokens, num_topk]; verbatim copy of topk_idx for the handle to
 *                       keep (example080 .cu:33)
 *   cumulative_expert_stats  int32[num_experts], NOT overwritten: every launch adds its
 *                       num_tokens_per_expert (unaligned counts) to it
 *                       (cumulative_local_expert_recv_stats, example080 .cu:35,211-212)
 * Any of the outputs from expert_offsets on may be NULL.
 */
int mi_ep_dispatch_layout(const int64_t* topk_idx, int num_tokens, int num_topk, int num_ranks,
                          int num_experts, int expert_alignment, int num_channels,
                          int* num_tokens_per_rank, int* num_tokens_per_expert,
                          bool* is_token_in_rank, int* expert_offsets, int* psum_rank_rows,
                          int* channel_prefix_matrix, int* rank_prefix_matrix, int* slot_rel,
                          int* rank_slot_idx, int rank_slot_base, int* route_order, int* tile_rank_counts,
                          int64_t* copied_topk_idx, int* cumulative_expert_stats, void* workspace,
                          size_t workspace_bytes, void* stream);
/*
 * mi_ep_dispatch_layout without a workspace argument and without any allocation.  It has no
 * counterpart in the reference; it is for callers that cannot allocate device memory or carry a
 * workspace: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * The look-back status words live in a static device array inside the library (2 MiB + 256 bytes
 * on every GPU the library runs on, held until the process ends).  Same arguments, outputs and
 * results as mi_ep_dispatch_layout.
 *   limit    ceil(num_tokens / 256) * (num_experts + num_ranks) <= MI_EP_STATIC_LAYOUT_STATUS_WORDS
 *            (254 000 tokens at 256 experts, 65 000 at 1024); beyond it the call returns
 *            MI_EP_E2BIG and launches nothing.
 *   timeout_report  NULL, or one int32 of device memory that the caller has set to 0: receives
 *            MI_EP_ETIMEDOUT if a bounded device-side wait of this launch expires (the outputs are
 *            then unspecified); never written otherwise.  With or without it,
 *            mi_ep_workspace_status(MI_EP_STATIC_SCRATCH, stream) reports an expired wait since the
 *            scratch was last initialised, mi_ep_workspace_set_wait_limit(MI_EP_STATIC_SCRATCH, ...)
 *            bounds the waits and mi_ep_workspace_init(MI_EP_STATIC_SCRATCH, 0, stream) clears the
 *            report.
 * Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU (two
 * streams, two threads) race and give unspecified results; calls ordered on one stream, or
 * otherwise serialised, are safe back to back whatever their shapes.  The array used is the one
 * of the device `stream` belongs to (of the current device for NULL), whatever device is current.
 * The first call on a device resolves the array's address (hipGetSymbolAddress, which may load the
 * code object): make it outside graph capture; the address does not outlive a hipDeviceReset.
 * Calls hipMalloc / hipFree never.
 */
#define MI_EP_STATIC_LAYOUT_STATUS_WORDS 262144
int mi_ep_dispatch_layout_static(const int64_t* topk_idx, int num_tokens, int num_topk, int num_ranks,
                                 int num_experts, int expert_alignment, int num_channels,
                                 int* num_tokens_per_rank, int* num_tokens_per_expert,
                                 bool* is_token_in_rank, int* expert_offsets, int* psum_rank_rows,
                                 int* channel_prefix_matrix, int* rank_prefix_matrix, int* slot_rel,
                                 int* rank_slot_idx, int rank_slot_base, int* route_order,
                                 int* tile_rank_counts, int64_t* copied_topk_idx,
                                 int* cumulative_expert_stats, int* timeout_report, void* stream);
/* Bytes of route_order for this shape. */
size_t mi_ep_route_order_bytes(int num_tokens, int num_topk);

/*
 * Dispatch (permute): the payload role of dispatch_impl
 * (example080_deepep_jit_dispatch_payload/nv/empty_deepep_jit_dispatch_payload.cu:31-44,241-256)
 * fused with dispatch_copy_epilogue_impl in expand mode
 * (example081_deepep_jit_dispatch_copy_epilogue/nv/empty_deepep_jit_dispatch_copy_epilogue.cu:22-60).
 * Row slot_map[t,k] = expert_offsets[e] + slot_rel[t,k] of every output receives
 * token t's input; segment e is rows [off[e], off[e+1]).
 *   x            [num_tokens, row_bytes] opaque bytes (bf16 or fp8); row_bytes % 16 == 0,
 *                x and recv_x 16-byte aligned
 *   x_scales     float[num_tokens, num_scales] or NULL (num_scales = 0)
 *   topk_weights float[num_tokens, num_topk] or NULL
 *   recv_x       [capacity_rows, row_bytes]
 *   recv_scales  float[capacity_rows, num_scales] or NULL
 *   recv_src_map int32[capacity_rows]: source token of each row; -1 for pad rows
 *   recv_topk_idx     int64[capacity_rows] or NULL: expert owning the row; -1 pad
 *   recv_topk_weights float[capacity_rows] or NULL: gate weight of the row's route; 0 pad
 *   slot_map     int32[num_tokens, num_topk]: absolute row of each route, -1 non-routes
 * Rows >= capacity_rows are never written.  With expert_alignment > 1 the pad rows' map entries
 * are written (source -1, expert -1, weight 0) by further workgroups of the same launch; their
 * payload and scales are left untouched, as the reference's receive buffer is (its harness pads to
 * 128 rows and only reads the received ones, example080 build_and_run.py:718,728-748).
 * num_tokens_per_expert (from the layout call) locates the pad rows and may be NULL when
 * expert_alignment == 1.
 *   flags        0, or an OR of
 *                MI_EP_DISPATCH_ZERO_PAD_PAYLOAD  also zero-fill the payload and scales of pad rows,
 *                  for consumers that read whole aligned segments.  At alignment 128 the fill is a
 *                  fifth of the copy's bytes.
 *                MI_EP_DISPATCH_BY_TOKEN / MI_EP_DISPATCH_BY_DESTINATION  (at most one) the copy
 *                  kernel to use instead of the one chosen by shape and device; by destination needs
 *                  route_order.  Results are identical.
 *   route_order  the layout call's table for the same topk_idx, or NULL.  The outputs are the
 *                same either way; with it, large shapes are copied in destination order
 *                (adjacent rows of recv_x written together, sources re-read from the L2 of the
 *                die that owns the tile), which the HBM write path takes ~14 % faster than
 *                rows scattered token by token.
 */
#define MI_EP_DISPATCH_ZERO_PAD_PAYLOAD 1
#define MI_EP_DISPATCH_BY_TOKEN 2
#define MI_EP_DISPATCH_BY_DESTINATION 4
int mi_ep_dispatch(const void* x, const float* x_scales, const int64_t* topk_idx,
                   const float* topk_weights, const int* expert_offsets, const int* slot_rel,
                   const int* route_order, const int* num_tokens_per_expert, int num_tokens, int num_topk,
                   int num_experts, int expert_alignment, int row_bytes, int num_scales,
                   void* recv_x, float* recv_scales, int* recv_src_map, int64_t* recv_topk_idx,
                   float* recv_topk_weights, int* slot_map, int capacity_rows, int flags,
                   void* stream);

/*
 * The same call with the scale factors addressed through strides, as the reference's dispatch
 * takes them (sf_token_stride, sf_hidden_stride, example080 .cu:40; recv_sf_token_stride,
 * recv_sf_hidden_stride, example081 .cu:31): element j of row r sits at
 * base[r * token_stride + j * hidden_stride], strides counted in 4-byte elements (a float, or
 * a pack of four 8-bit exponents: the copy does not look inside).  mi_ep_dispatch is this call
 * with strides (num_scales, 1) on both sides.  Column-major scale tensors, which the reference's
 * TMA-aligned layouts use, are (1, padded row count).
 */
int mi_ep_dispatch_strided_scales(const void* x, const float* x_scales, long long x_scales_token_stride,
                                  long long x_scales_hidden_stride, const int64_t* topk_idx,
                                  const float* topk_weights, const int* expert_offsets, const int* slot_rel,
                                  const int* route_order, const int* num_tokens_per_expert, int num_tokens,
                                  int num_topk, int num_experts, int expert_alignment, int row_bytes,
                                  int num_scales, void* recv_x, float* recv_scales,
                                  long long recv_scales_token_stride, long long recv_scales_hidden_stride,
                                  int* recv_src_map, int64_t* recv_topk_idx, float* recv_topk_weights,
                                  int* slot_map, int capacity_rows, int flags, void* stream);

/*
 * Dispatch de-duplicated by destination rank: the reference's own receive format (payload role
 * of dispatch_impl, example080_deepep_jit_dispatch_payload/nv/empty_deepep_jit_dispatch_payload.cu:31-44,
 * 241-256, then dispatch_copy_epilogue_impl without expansion,
 * example081_deepep_jit_dispatch_copy_epilogue/nv/empty_deepep_jit_dispatch_copy_epilogue.cu:22-60).
 * A token sends ONE row to every rank that owns at least one of its experts; rank r receives its
 * rows in token order at [psum_rank_tokens[r-1], psum_rank_tokens[r]).
 *   rank_slot_idx, rank_slot_base, num_tokens_per_rank   from mi_ep_dispatch_layout for the same topk_idx
 *   expand_slot_map   NULL, or the slot_map of mi_ep_dispatch (rows of the expanded buffer)
 *   recv_x / recv_scales   [capacity_rows, row_bytes] / float[capacity_rows, num_scales] or NULL
 *   recv_topk_idx     int64[capacity_rows, num_topk] or NULL: the token's expert ids that live on
 *                     the row's rank (minus rank * E/R when local_expert_ids != 0), -1 elsewhere
 *   recv_topk_weights float[capacity_rows, num_topk] or NULL: the weights of those slots (1 when
 *                     topk_weights is NULL), 0 elsewhere
 *   recv_src_metadata int32[capacity_rows, 2 + num_topk] or NULL: {source_token_base + t, rank,
 *                     then per slot the expanded row of the route when its expert lives on the
 *                     rank and expand_slot_map is given, else -1} (column 0 as the reference's
 *                     harness reads it, example080 build_and_run.py:733; source_token_base stands
 *                     for rank_idx * num_max_tokens_per_rank)
 *   rank_row_map      int32[num_tokens, num_topk]: the row that carries route (t,k); slots that
 *                     share a rank share a row; -1 for non-routes and dropped rows
 *   psum_rank_tokens  int32[num_ranks]: inclusive rows per rank
 *                     (psum_num_recv_tokens_per_scaleup_rank, :734)
 *   combine_map       int32[num_tokens, num_topk] or NULL: rank_row_map on the first slot of
 *                     every distinct rank of the token, -1 elsewhere: each received row once.
 *                     mi_ep_combine(y, rows, combine_map, topk_weights = NULL, ...) is then the
 *                     reference's combine of this format (an ordered sum of the ranks' rows)
 * Rows at or beyond capacity_rows are dropped; min(num_topk, num_ranks) * num_tokens always fit.
 * mi_ep_dispatch_ranks_strided_scales is the same call with the scale factors addressed through
 * (token, hidden) strides in 4-byte elements on both sides, as the reference's epilogue takes them
 * (recv_sf_token_stride, recv_sf_hidden_stride, example081 .cu:31); mi_ep_dispatch_ranks is that
 * call with strides (num_scales, 1).
 * mi_ep_combine_rank_weights returns what travelled with the rows, gathered back per route:
 * combined_topk_weights[t,k] = recv_topk_weights[rank_row_map[t,k], k] (0 for non-routes;
 * example082 build_and_run.py:765) and combined_topk_idx[t,k] = recv_topk_idx[rank_row_map[t,k], k]
 * as stored (-1 for non-routes; combined_topk_idx of the reduce epilogue, example083 .cu:26).
 * Either pair of pointers may be NULL, not both.
 */
int mi_ep_dispatch_ranks(const void* x, const float* x_scales, const int64_t* topk_idx,
                         const float* topk_weights, const int* rank_slot_idx, int rank_slot_base,
                         const int* num_tokens_per_rank, const int* expand_slot_map, int num_tokens,
                         int num_topk, int num_ranks, int num_experts, int row_bytes, int num_scales,
                         int source_token_base, int local_expert_ids, void* recv_x, float* recv_scales,
                         int64_t* recv_topk_idx, float* recv_topk_weights, int* recv_src_metadata,
                         int* rank_row_map, int* combine_map, int* psum_rank_tokens, int capacity_rows,
                         void* stream);
int mi_ep_dispatch_ranks_strided_scales(const void* x, const float* x_scales, long long x_scales_token_stride,
                                        long long x_scales_hidden_stride, const int64_t* topk_idx,
                                        const float* topk_weights, const int* rank_slot_idx, int rank_slot_base,
                                        const int* num_tokens_per_rank, const int* expand_slot_map,
                                        int num_tokens, int num_topk, int num_ranks, int num_experts,
                                        int row_bytes, int num_scales, int source_token_base,
                                        int local_expert_ids, void* recv_x, float* recv_scales,
                                        long long recv_scales_token_stride, long long recv_scales_hidden_stride,
                                        int64_t* recv_topk_idx, float* recv_topk_weights,
                                        int* recv_src_metadata, int* rank_row_map, int* combine_map,
                                        int* psum_rank_tokens, int capacity_rows, void* stream);
int mi_ep_combine_rank_weights(const float* recv_topk_weights, const int64_t* recv_topk_idx,
                               const int* rank_row_map, int num_tokens, int num_topk, int num_rows,
                               float* combined_topk_weights, int64_t* combined_topk_idx, void* stream);

/*
 * Pull-mode dispatch with a map from an earlier dispatch (the reference's cached mode,
 * kCachedMode of dispatch_copy_epilogue_impl,
 * example081_deepep_jit_dispatch_copy_epilogue/nv/empty_deepep_jit_dispatch_copy_epilogue.cu:11,
 * and the token pull of the ThunderKittens MoE example,
 * example056_thunderkitten_moe_dispatch_gemm_easy, kernel spec at :181-202): row i of
 * recv_x / recv_scales becomes a byte copy of token recv_src_map[i]; rows whose map entry is
 * negative (pads) or not below num_tokens are zero-filled.  No routing tables are read.
 * Same size and alignment rules as mi_ep_dispatch.
 *   ready_counters  NULL, or int32[ceil(num_rows / rows_per_counter)] that the caller has zeroed:
 *                   counter i is incremented once (device-scope release) for every row of block
 *                   i, pads included, after the row is in place; a consumer on another stream
 *                   may read block i once the counter equals the block's row count.  This is the
 *                   per-row-block arrival barrier of the same example (:196-202, ROW_BLOCK = 128).
 */
int mi_ep_dispatch_cached(const void* x, const float* x_scales, const int* recv_src_map,
                          int num_rows, int num_tokens, int row_bytes, int num_scales,
                          void* recv_x, float* recv_scales, int* ready_counters,
                          int rows_per_counter, void* stream);

/*
 * The same map in the ThunderKittens example's format
 * (example056_thunderkitten_moe_dispatch_gemm_easy compute_dispatch_indices, :521-564):
 * pull_indices[i] = {source rank, token index inside that rank} with tokens_per_source_rank
 * consecutive tokens per source rank, {-1, -1} for pad rows.  int32[num_rows, 2].
 */
int mi_ep_pull_indices(const int* recv_src_map, int num_rows, int tokens_per_source_rank,
                       int* pull_indices, void* stream);

/*
 * Combine: combine_impl + combine_reduce_epilogue_impl
 * (example082_deepep_jit_combine/nv/empty_deepep_jit_combine.cu:28-67,
 *  example083_deepep_jit_combine_reduce_epilogue/nv/empty_deepep_jit_combine_reduce_epilogue.cu:23-53).
 *   combined_x[t,h] = bf16( sum_k w[t,k] * y[slot_map[t,k], h] + bias_0[t,h] + bias_1[t,h] )
 * accumulated in fp32, slots ascending, one fused multiply-add per row, one
 * rounding to bf16 at the end.  topk_weights == NULL gives the reference's plain
 * ordered sum.  hidden % 8 == 0; y, biases and combined_x 16-byte aligned.
 *   y            bf16[num_rows, hidden] expert outputs in dispatch row order; map entries
 *                that are negative or not below num_rows are not routes
 *   bias_0/1     bf16[num_tokens, hidden] or NULL
 *   recv_topk_weights / combined_topk_weights   both NULL, or float[rows] in and
 *                float[num_tokens, num_topk] out: the weights that travelled with the
 *                rows, gathered back per route (0 for non-routes)
 *   recv_topk_idx / combined_topk_idx   both NULL, or int64[rows] in and
 *                int64[num_tokens, num_topk] out: the expert ids that travelled with the rows
 *                (-1 for non-routes; combined_topk_idx, example083 .cu:26)
 *   flags        0, or MI_EP_COMBINE_STREAM_OUTPUT.  By default an output of up to 120 MiB is
 *                written through into the GPU's memory-side cache (256 MB), where the operator
 *                that consumes it next finds it and from where it reaches HBM later; the kernel
 *                itself is then almost a pure read stream (about 5 % faster on large shapes).
 *                Of a larger output only the leading part that leaves that cache room for an
 *                input of the output's size is written through (nothing from 240 MiB on).
 *                With the flag the whole output is streamed straight to HBM: the choice for an
 *                output that nothing reads soon, since lines that fall out of that cache during
 *                other memory-bound kernels cost those more than the flag costs this one.  The
 *                results are identical.
 */
#define MI_EP_COMBINE_STREAM_OUTPUT 1
int mi_ep_combine(const void* y, int num_rows, const int* slot_map, const float* topk_weights,
                  const void* bias_0, const void* bias_1, const float* recv_topk_weights,
                  const int64_t* recv_topk_idx, int num_tokens, int num_topk, int hidden,
                  void* combined_x, float* combined_topk_weights, int64_t* combined_topk_idx,
                  int flags, void* stream);

/*
 * Host-pointer twins: the same operations with every pointer in ordinary host memory.  Each call
 * allocates device buffers, copies inputs over, runs the kernels above on the null stream, copies
 * the outputs back and returns after synchronising; errors as above.  They serve callers without a
 * device-side pipeline (the reference's harnesses keep their data in host vectors between
 * hipMemcpy calls, example042 .cu:243-293); transfers dominate their time.
 *   mi_ep_host_get_dispatch_layout  twin of mi_ep_get_dispatch_layout
 *   mi_ep_host_dispatch_layout      twin of mi_ep_dispatch_layout: same arguments and outputs without
 *                                   the workspace; cumulative_expert_stats is read and written
 *                                   (the running totals continue from the caller's values);
 *                                   route_order entries past the last token come back as zeros
 *   mi_ep_host_dispatch             layout + dispatch in one call: the layout outputs
 *                                   (num_tokens_per_rank / _expert, is_token_in_rank, any of them
 *                                   may be NULL) and expert_offsets come back with the permuted
 *                                   rows; only the first min(expert_offsets[E], capacity_rows)
 *                                   rows of the recv_* arrays are written
 *   mi_ep_host_dispatch_ranks       layout + mi_ep_dispatch_ranks in one call (the reference's own
 *                                   receive format, example081 .cu:22-60): num_tokens_per_rank (may
 *                                   be NULL), the per-row arrays (recv_topk_idx, recv_topk_weights,
 *                                   recv_src_metadata: any may be NULL), rank_row_map, combine_map
 *                                   (may be NULL) and psum_rank_tokens come back; only the first
 *                                   min(psum_rank_tokens[R-1], capacity_rows) rows are written
 *   mi_ep_host_dispatch_cached      twin of mi_ep_dispatch_cached (without arrival counters)
 *   mi_ep_host_combine              twin of mi_ep_combine (without the travelled weights)
 */
int mi_ep_host_get_dispatch_layout(const int64_t* topk_idx, int* num_tokens_per_rank,
                                   int* num_tokens_per_rdma_rank, int* num_tokens_per_expert,
                                   bool* is_token_in_rank, int num_tokens, int num_topk, int num_ranks,
                                   int num_experts);
int mi_ep_host_dispatch_layout(const int64_t* topk_idx, int num_tokens, int num_topk, int num_ranks,
                               int num_experts, int expert_alignment, int num_channels,
                               int* num_tokens_per_rank, int* num_tokens_per_expert, bool* is_token_in_rank,
                               int* expert_offsets, int* psum_rank_rows, int* channel_prefix_matrix,
                               int* rank_prefix_matrix, int* slot_rel, int* rank_slot_idx, int rank_slot_base,
                               int* route_order, int* tile_rank_counts, int64_t* copied_topk_idx,
                               int* cumulative_expert_stats);
int mi_ep_host_dispatch(const void* x, const float* x_scales, const int64_t* topk_idx,
                        const float* topk_weights, int num_tokens, int num_topk, int num_ranks,
                        int num_experts, int expert_alignment, int row_bytes, int num_scales,
                        int* num_tokens_per_rank, int* num_tokens_per_expert, bool* is_token_in_rank,
                        int* expert_offsets, void* recv_x, float* recv_scales, int* recv_src_map,
                        int64_t* recv_topk_idx, float* recv_topk_weights, int* slot_map,
                        int capacity_rows);
int mi_ep_host_dispatch_ranks(const void* x, const float* x_scales, const int64_t* topk_idx,
                              const float* topk_weights, int num_tokens, int num_topk, int num_ranks,
                              int num_experts, int row_bytes, int num_scales, int source_token_base,
                              int local_expert_ids, int* num_tokens_per_rank, void* recv_x,
                              float* recv_scales, int64_t* recv_topk_idx, float* recv_topk_weights,
                              int* recv_src_metadata, int* rank_row_map, int* combine_map,
                              int* psum_rank_tokens, int capacity_rows);
int mi_ep_host_dispatch_cached(const void* x, const float* x_scales, const int* recv_src_map, int num_rows,
                               int num_tokens, int row_bytes, int num_scales, void* recv_x,
                               float* recv_scales);
int mi_ep_host_combine(const void* y, int num_rows, const int* slot_map, const float* topk_weights,
                       const void* bias_0, const void* bias_1, int num_tokens, int num_topk, int hidden,
                       void* combined_x);

/*
 * 16-byte streaming copy used as the measured HBM ceiling next to the nominal
 * peak; same access width as example077_GPU_vectorized_copy_widths (16-byte loads).
 * bytes % 16 == 0.
 */
int mi_ep_copy_yardstick(void* dst, const void* src, size_t bytes, void* stream);
/* The same stream split in two: read-only (every 16-byte vector is loaded and folded into one
 * word; *sink is written only if that word equals a fixed magic value, which keeps the loads
 * alive without adding write traffic) and write-only (a fill).  They bound what a read-heavy
 * (combine) and a write-heavy (permute) kernel can reach.  bytes % 16 == 0; sink is 4 bytes of
 * device memory. */
int mi_ep_read_yardstick(const void* src, size_t bytes, void* sink, void* stream);
int mi_ep_write_yardstick(void* dst, size_t bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MI_EP_H_ */
