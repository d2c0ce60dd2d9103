/*
 * ep_oracle.c -- CPU restatement of the MoE dispatch-layout / permute / combine path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker that the HIP kernels are
 * compared against and the CPU baseline that the benchmark times beside them.
 * Nothing in the shipped library links, loads or calls it.
 *
 * Every function restates, from its definition, an operation of the reference
 * (paths relative to the reference tree, datasets/ prefix omitted):
 *
 *   ep_oracle_layout            example042_deepep_dispatch_layout/nv/
 *                               empty_deepep_dispatch_layout.cu:208-234 (cpuReference)
 *   ep_oracle_expert_offsets    example080_deepep_jit_dispatch_payload/nv/
 *                               empty_deepep_jit_dispatch_payload.cu:197-239
 *                               (align, inclusive rank psum, exclusive expert psum)
 *   ep_oracle_slot_maps         example078_deepep_jit_dispatch_deterministic_prologue/nv/
 *                               empty_deepep_jit_dispatch_deterministic_prologue.cu:27-43
 *                               (deterministic slots: earlier work is the prefix),
 *                               generalised from destination ranks to expert segments
 *   ep_oracle_rank_slots        example078 ... deterministic_prologue.cu:27-43, in its own output format
 *   ep_oracle_route_order       no reference kernel: the per-tile stable sort of routes by expert that
 *                               the destination-order copy walks (nearest relative: example056 :521-564)
 *   ep_oracle_channel_prefix    example047_deepep_intranode_notify_dispatch/nv/
 *                               empty_deepep_intranode_notify_dispatch.cu:73-79,386-406
 *   ep_oracle_rank_prefix       same file :352-360
 *   ep_oracle_permute           example081_deepep_jit_dispatch_copy_epilogue/nv/
 *                               empty_deepep_jit_dispatch_copy_epilogue.cu:22-60
 *                               (payload, scales, weights and source metadata per row)
 *   ep_oracle_permute_ranks     example080 .cu:31-44,241-256 + example081 .cu:22-60 without expansion:
 *                               one row per (token, destination rank), K ids / weights and the
 *                               source metadata per row
 *   ep_oracle_gather_rows,
 *   ep_oracle_pull_indices      example056_thunderkitten_moe_dispatch_gemm_easy/nv/
 *                               empty_thunderkitten_moe_dispatch_gemm.cu:181-202,521-564
 *                               and the cached mode of the copy epilogue (example081 .cu:11)
 *   ep_oracle_combine           example083_deepep_jit_combine_reduce_epilogue/nv/
 *                               empty_deepep_jit_combine_reduce_epilogue.cu:23-53
 *                               (fp32 accumulate over up to K rows, two biases, bf16 out)
 *   ep_oracle_gather_weights,
 *   ep_oracle_gather_idx        the same epilogue's combined_topk_weights / combined_topk_idx (:25-26):
 *                               what travelled with each route's row, read back per (token, slot);
 *                               ep_oracle_gather_rank_side the same for the per-rank format's [rows, K] tables
 *   ep_oracle_tile_rank_counts  example078 .cu:20,34-35 (rank_count_buffer[sm, rank]) with a block of
 *                               consecutive tokens standing for an SM's share
 *   ep_oracle_accumulate_stats  example080 .cu:35,211-212 (cumulative_local_expert_recv_stats += counts)
 *
 * Pinning (what checks this file, beyond the kernels agreeing with it):
 *   layout           the reference's 13 closed-form correctness cases with
 *                    number-theoretic expected counts, plus a numpy bincount/unique
 *                    brute force (tests/test_oracle_layout.py)
 *   expert offsets   numpy cumsum; off[E] == N; partition sums
 *   slot maps        numpy stable argsort by expert id (the map IS a stable sort)
 *   rank slots       numpy: exclusive cumsum of the rank flags + first-occurrence mask
 *   route order      numpy lexsort per tile; positions agree with the slot maps
 *   channel prefix   closed form for the reference's routeDst pattern
 *   rank prefix      numpy cumsum over axis 0
 *   permute          numpy fancy-index gather
 *   permute by rank  numpy: rows of rank r = x[flag[:, r]] in token order, masks from the ids;
 *                    the reference harness's own checks (example080 build_and_run.py:728-748)
 *   pull indices     the closed form of the ThunderKittens example's own generator
 *   combine          exact rational arithmetic rounded once per fma (python ints),
 *                    integer-valued exact sums, K=1 copy, closed forms
 *   gather idx / rank side   numpy fancy indexing with a mask
 *   tile rank counts numpy add.reduceat over the flag matrix; column sums == per-rank counts
 *   accumulate stats numpy += over several calls
 *   bf16 codec       exhaustive against torch.bfloat16 (fixtures in tests/golden)
 * Parity unpinned: the order in which two bias rows are added in the reference's
 * combine epilogue (its arithmetic lives in the un-vendored DeepEP tree); this
 * file defines it as acc + bias_0 + bias_1 after the top-k loop.  Also unpinned, for the
 * same reason: column 1 of recv_src_metadata (defined here as the destination rank) and
 * whether recv_topk_idx holds global or rank-local expert ids (both offered).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#define EP_MAX_RANKS 8

/* ---- bf16 codec ------------------------------------------------------- */

float ep_oracle_bf16_to_f32(uint16_t v) {
  uint32_t u = (uint32_t)v << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* Round to nearest, ties to even; NaN stays NaN (quiet bit forced). */
uint16_t ep_oracle_f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

void ep_oracle_f32_to_bf16_array(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = ep_oracle_f32_to_bf16(in[i]);
}

void ep_oracle_bf16_to_f32_array(const uint16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = ep_oracle_bf16_to_f32(in[i]);
}

/* ---- layout ----------------------------------------------------------- */

static inline int route_valid(int64_t e, int num_experts) {
  return e >= 0 && e < (int64_t)num_experts;
}

/*
 * Per-expert counts count every valid slot; the per-rank flag and count are one
 * per (token, rank) pair however many of the token's slots land on that rank.
 * Slots with idx < 0 (masked) or idx >= num_experts are not routes.
 */
int ep_oracle_layout(const int64_t* topk_idx, int num_tokens, int num_topk, int num_ranks,
                     int num_experts, int* num_tokens_per_rank, int* num_tokens_per_expert,
                     uint8_t* is_token_in_rank) {
  if (num_ranks <= 0 || num_ranks > EP_MAX_RANKS || num_topk <= 0 || num_experts <= 0 ||
      num_experts % num_ranks != 0 || num_tokens < 0)
    return -22;
  const int per_rank = num_experts / num_ranks;
  memset(num_tokens_per_rank, 0, sizeof(int) * (size_t)num_ranks);
  memset(num_tokens_per_expert, 0, sizeof(int) * (size_t)num_experts);
  for (int t = 0; t < num_tokens; ++t) {
    uint8_t seen[EP_MAX_RANKS] = {0};
    for (int k = 0; k < num_topk; ++k) {
      int64_t e = topk_idx[(size_t)t * num_topk + k];
      if (!route_valid(e, num_experts)) continue;
      num_tokens_per_expert[e] += 1;
      seen[e / per_rank] = 1;
    }
    for (int r = 0; r < num_ranks; ++r) {
      is_token_in_rank[(size_t)t * num_ranks + r] = seen[r];
      num_tokens_per_rank[r] += seen[r];
    }
  }
  return 0;
}

/*
 * off[0] = 0, off[e+1] = off[e] + round_up(cnt[e], align): exclusive over aligned
 * counts, length E+1, last element = padded row total.  psum_rank_rows[r] is the
 * inclusive number of rows owned by partitions 0..r (= off[(r+1) * E/R]).
 */
int ep_oracle_expert_offsets(const int* num_tokens_per_expert, int num_experts, int num_ranks,
                             int expert_alignment, int* expert_offsets, int* psum_rank_rows) {
  if (expert_alignment < 1 || num_ranks <= 0 || num_experts % num_ranks != 0) return -22;
  const int per_rank = num_experts / num_ranks;
  int run = 0;
  expert_offsets[0] = 0;
  for (int e = 0; e < num_experts; ++e) {
    int c = num_tokens_per_expert[e];
    int padded = (c + expert_alignment - 1) / expert_alignment * expert_alignment;
    run += padded;
    expert_offsets[e + 1] = run;
  }
  if (psum_rank_rows)
    for (int r = 0; r < num_ranks; ++r) psum_rank_rows[r] = expert_offsets[(r + 1) * per_rank];
  return 0;
}

/*
 * Routes are enumerated by (token ascending, slot ascending).  Route (t,k) with
 * expert e takes row off[e] + (number of earlier routes with expert e).
 *   slot_rel[t,k]  position inside the expert segment, -1 for non-routes
 *   slot_map[t,k]  absolute row, -1 for non-routes
 *   src_map[row]   source token of the row, -1 for pad rows
 *   src_k[row]     source slot of the row, -1 for pad rows
 * Any output pointer may be NULL.  `fill` is scratch of num_experts ints.
 */
int ep_oracle_slot_maps(const int64_t* topk_idx, int num_tokens, int num_topk, int num_experts,
                        const int* expert_offsets, int* slot_rel, int* slot_map, int* src_map,
                        int* src_k, int* fill) {
  memset(fill, 0, sizeof(int) * (size_t)num_experts);
  const int total = expert_offsets[num_experts];
  if (src_map)
    for (int i = 0; i < total; ++i) src_map[i] = -1;
  if (src_k)
    for (int i = 0; i < total; ++i) src_k[i] = -1;
  for (int t = 0; t < num_tokens; ++t) {
    for (int k = 0; k < num_topk; ++k) {
      size_t i = (size_t)t * num_topk + k;
      int64_t e = topk_idx[i];
      if (!route_valid(e, num_experts)) {
        if (slot_rel) slot_rel[i] = -1;
        if (slot_map) slot_map[i] = -1;
        continue;
      }
      int rel = fill[e]++;
      int row = expert_offsets[e] + rel;
      if (slot_rel) slot_rel[i] = rel;
      if (slot_map) slot_map[i] = row;
      if (src_map) src_map[row] = t;
      if (src_k) src_k[row] = k;
    }
  }
  return 0;
}

/*
 * The deterministic prologue's own table (example078 .cu:36-40): per destination rank, tokens
 * take slots in token order; out[t,k] = base + slot for the first slot k of token t that
 * reaches the rank, -1 for non-routes and for further slots on the same rank.
 */
int ep_oracle_rank_slots(const int64_t* topk_idx, int num_tokens, int num_topk, int num_ranks,
                         int num_experts, int base, int* out) {
  if (num_ranks <= 0 || num_ranks > EP_MAX_RANKS || num_experts % num_ranks != 0) return -22;
  const int per_rank = num_experts / num_ranks;
  int next_slot[EP_MAX_RANKS] = {0};
  for (int t = 0; t < num_tokens; ++t) {
    int taken[EP_MAX_RANKS] = {0};
    for (int k = 0; k < num_topk; ++k) {
      size_t i = (size_t)t * num_topk + k;
      int64_t e = topk_idx[i];
      out[i] = -1;
      if (!route_valid(e, num_experts)) continue;
      int r = (int)(e / per_rank);
      if (taken[r]) continue;
      taken[r] = 1;
      out[i] = base + next_slot[r]++;
    }
  }
  return 0;
}

/*
 * Routes of every tile of `tile_tokens` consecutive tokens in destination order: a stable
 * counting sort of the tile's routes by expert (so by position in the expert's segment),
 * non-routes after them in (token, slot) order.  Entry i of tile j sits at
 * out[(j * tile_tokens * K + i) * 4 ..] = {t*K + k, expert, slot_rel, t}, with expert and
 * slot_rel -1 for non-routes; entries past the last token's are left untouched.  This is the
 * sender-side counterpart of the sorted pull list the ThunderKittens example builds
 * (example056 compute_dispatch_indices, :521-564), restricted to one tile.
 * `scratch` holds 2 * num_experts ints.
 */
int ep_oracle_route_order(const int64_t* topk_idx, int num_tokens, int num_topk, int num_experts,
                          int tile_tokens, int* out, int* scratch) {
  if (tile_tokens <= 0) return -22;
  int* seen = scratch;                 /* routes of expert e in earlier tokens */
  int* next = scratch + num_experts;   /* next position of expert e inside the tile's list */
  memset(seen, 0, sizeof(int) * (size_t)num_experts);
  for (int t0 = 0; t0 < num_tokens; t0 += tile_tokens) {
    const int t1 = t0 + tile_tokens < num_tokens ? t0 + tile_tokens : num_tokens;
    int* list = out + (size_t)(t0 / tile_tokens) * tile_tokens * num_topk * 4;
    memset(next, 0, sizeof(int) * (size_t)num_experts);
    for (size_t i = (size_t)t0 * num_topk; i < (size_t)t1 * num_topk; ++i)
      if (route_valid(topk_idx[i], num_experts)) next[topk_idx[i]]++;
    int total = 0;
    for (int e = 0; e < num_experts; ++e) {
      int c = next[e];
      next[e] = total;
      total += c;
    }
    int masked = total;
    for (size_t i = (size_t)t0 * num_topk; i < (size_t)t1 * num_topk; ++i) {
      int64_t e = topk_idx[i];
      int* entry;
      if (route_valid(e, num_experts)) {
        entry = list + 4 * (size_t)next[e]++;
        entry[1] = (int)e;
        entry[2] = seen[e]++;
      } else {
        entry = list + 4 * (size_t)masked++;
        entry[1] = -1;
        entry[2] = -1;
      }
      entry[0] = (int)i;
      entry[3] = (int)(i / (size_t)num_topk);
    }
  }
  return 0;
}

/*
 * Token tile c of C covers [min(tpc*c, T), min(tpc*c + tpc, T)) with
 * tpc = ceil(T / C); out[r, c] = number of tokens flagged for rank r in tiles 0..c.
 */
int ep_oracle_channel_prefix(const uint8_t* is_token_in_rank, int num_tokens, int num_ranks,
                             int num_channels, int* channel_prefix_matrix) {
  if (num_channels <= 0) return -22;
  const int tpc = (num_tokens + num_channels - 1) / num_channels;
  for (int r = 0; r < num_ranks; ++r) {
    int run = 0;
    for (int c = 0; c < num_channels; ++c) {
      int start = tpc * c < num_tokens ? tpc * c : num_tokens;
      int end = start + tpc < num_tokens ? start + tpc : num_tokens;
      for (int t = start; t < end; ++t) run += is_token_in_rank[(size_t)t * num_ranks + r] != 0;
      channel_prefix_matrix[r * num_channels + c] = run;
    }
  }
  return 0;
}

/* out[src, dst] = sum over s <= src of counts[s, dst]. */
void ep_oracle_rank_prefix(const int* counts, int num_ranks, int* out) {
  for (int dst = 0; dst < num_ranks; ++dst) {
    int run = 0;
    for (int src = 0; src < num_ranks; ++src) {
      run += counts[src * num_ranks + dst];
      out[src * num_ranks + dst] = run;
    }
  }
}

/* ---- permute ---------------------------------------------------------- */

/*
 * Row `row` of every output is a byte copy of the source token's input; pad rows
 * (src_map < 0) are zero in every output.  x_scales / topk_weights and their
 * outputs may be NULL.  recv_topk_idx[row] is the expert that owns the row.
 */
int ep_oracle_permute(const void* x, int row_bytes, const float* x_scales, int num_scales,
                      const int64_t* topk_idx, const float* topk_weights, int num_topk,
                      const int* src_map, const int* src_k, int num_rows, void* recv_x,
                      float* recv_scales, int64_t* recv_topk_idx, float* recv_topk_weights,
                      int num_threads) {
  const uint8_t* xin = (const uint8_t*)x;
  uint8_t* xout = (uint8_t*)recv_x;
  if (num_threads < 1) num_threads = 1;
#pragma omp parallel for num_threads(num_threads) schedule(static)
  for (int row = 0; row < num_rows; ++row) {
    int t = src_map[row];
    if (t < 0) {
      memset(xout + (size_t)row * row_bytes, 0, (size_t)row_bytes);
      if (recv_scales) memset(recv_scales + (size_t)row * num_scales, 0, sizeof(float) * (size_t)num_scales);
      if (recv_topk_idx) recv_topk_idx[row] = -1;
      if (recv_topk_weights) recv_topk_weights[row] = 0.0f;
      continue;
    }
    memcpy(xout + (size_t)row * row_bytes, xin + (size_t)t * row_bytes, (size_t)row_bytes);
    if (recv_scales)
      memcpy(recv_scales + (size_t)row * num_scales, x_scales + (size_t)t * num_scales,
             sizeof(float) * (size_t)num_scales);
    size_t i = (size_t)t * num_topk + src_k[row];
    if (recv_topk_idx) recv_topk_idx[row] = topk_idx[i];
    if (recv_topk_weights) recv_topk_weights[row] = topk_weights[i];
  }
  return 0;
}

/*
 * Dispatch de-duplicated by destination rank, the format of the reference's own dispatch
 * (payload role of dispatch_impl, example080 .cu:31-44,241-256, followed by the copy epilogue
 * without expansion, example081 .cu:22-60): a token sends ONE row to every rank that owns at
 * least one of its experts.  Rank r receives its rows in token order at
 * [psum[r-1], psum[r]) (psum inclusive, as psum_num_recv_tokens_per_scaleup_rank).  Per row n
 * of token t on rank r:
 *   recv_x / recv_scales   byte copy of the token's input
 *   recv_topk_idx[n,k]     topk_idx[t,k] if that expert lives on r (minus r * E/R when
 *                          local_expert_ids), else -1
 *   recv_topk_weights[n,k] topk_weights[t,k] where recv_topk_idx[n,k] >= 0, else 0
 *   recv_src_metadata[n,:] {source_token_base + t, r, then per slot k the row of route (t,k) in
 *                          the expanded buffer (expand_slot_map, may be NULL) where the expert
 *                          lives on r, else -1}
 * and per token: rank_row_map[t,k] = the row that carries route (t,k) (-1 for non-routes;
 * slots that share a rank share a row).  Rows at or beyond capacity_rows are dropped.
 * Outputs other than recv_x and rank_row_map may be NULL.
 */
int ep_oracle_permute_ranks(const void* x, int row_bytes, const float* x_scales, int num_scales,
                            const int64_t* topk_idx, const float* topk_weights, int num_tokens,
                            int num_topk, int num_ranks, int num_experts, int source_token_base,
                            int local_expert_ids, const int* expand_slot_map, int capacity_rows,
                            void* recv_x, float* recv_scales, int64_t* recv_topk_idx,
                            float* recv_topk_weights, int* recv_src_metadata, int* rank_row_map,
                            int* psum_rank_tokens) {
  if (num_ranks <= 0 || num_ranks > EP_MAX_RANKS || num_experts % num_ranks != 0) return -22;
  const int per_rank = num_experts / num_ranks;
  const int stride = 2 + num_topk;
  const uint8_t* xin = (const uint8_t*)x;
  uint8_t* xout = (uint8_t*)recv_x;
  int count[EP_MAX_RANKS] = {0}, base[EP_MAX_RANKS + 1] = {0}, next[EP_MAX_RANKS] = {0};
  for (int t = 0; t < num_tokens; ++t) {
    int hit[EP_MAX_RANKS] = {0};
    for (int k = 0; k < num_topk; ++k) {
      int64_t e = topk_idx[(size_t)t * num_topk + k];
      if (route_valid(e, num_experts)) hit[e / per_rank] = 1;
    }
    for (int r = 0; r < num_ranks; ++r) count[r] += hit[r];
  }
  for (int r = 0; r < num_ranks; ++r) {
    base[r + 1] = base[r] + count[r];
    if (psum_rank_tokens) psum_rank_tokens[r] = base[r + 1];
  }
  for (int t = 0; t < num_tokens; ++t) {
    int row_of[EP_MAX_RANKS];
    for (int r = 0; r < num_ranks; ++r) row_of[r] = -2;  /* not reached */
    for (int k = 0; k < num_topk; ++k) {
      size_t i = (size_t)t * num_topk + k;
      int64_t e = topk_idx[i];
      rank_row_map[i] = -1;
      if (!route_valid(e, num_experts)) continue;
      int r = (int)(e / per_rank);
      if (row_of[r] == -2) {
        int row = base[r] + next[r]++;
        row_of[r] = row < capacity_rows ? row : -1;
      }
      rank_row_map[i] = row_of[r];
    }
    for (int r = 0; r < num_ranks; ++r) {
      int row = row_of[r];
      if (row < 0) continue;
      memcpy(xout + (size_t)row * row_bytes, xin + (size_t)t * row_bytes, (size_t)row_bytes);
      if (recv_scales)
        memcpy(recv_scales + (size_t)row * num_scales, x_scales + (size_t)t * num_scales,
               sizeof(float) * (size_t)num_scales);
      if (recv_src_metadata) {
        recv_src_metadata[(size_t)row * stride + 0] = source_token_base + t;
        recv_src_metadata[(size_t)row * stride + 1] = r;
      }
      for (int k = 0; k < num_topk; ++k) {
        size_t i = (size_t)t * num_topk + k;
        int64_t e = topk_idx[i];
        int local = route_valid(e, num_experts) && (int)(e / per_rank) == r;
        if (recv_topk_idx)
          recv_topk_idx[(size_t)row * num_topk + k] = local ? e - (local_expert_ids ? (int64_t)r * per_rank : 0) : -1;
        if (recv_topk_weights)
          recv_topk_weights[(size_t)row * num_topk + k] = local ? (topk_weights ? topk_weights[i] : 1.0f) : 0.0f;
        if (recv_src_metadata)
          recv_src_metadata[(size_t)row * stride + 2 + k] = (local && expand_slot_map) ? expand_slot_map[i] : -1;
      }
    }
  }
  return 0;
}

/*
 * Pull-mode (cached) dispatch: row i is a byte copy of token src_map[i]; rows whose entry is
 * negative or not below num_tokens are zero (example081 .cu:11 kCachedMode; example056
 * thunderkitten_moe_dispatch_gemm_easy kernel spec :181-202).
 */
int ep_oracle_gather_rows(const void* x, int row_bytes, const float* x_scales, int num_scales,
                          const int* src_map, int num_rows, int num_tokens, void* recv_x,
                          float* recv_scales) {
  const uint8_t* xin = (const uint8_t*)x;
  uint8_t* xout = (uint8_t*)recv_x;
  for (int row = 0; row < num_rows; ++row) {
    int t = src_map[row];
    if (t < 0 || t >= num_tokens) {
      memset(xout + (size_t)row * row_bytes, 0, (size_t)row_bytes);
      if (recv_scales) memset(recv_scales + (size_t)row * num_scales, 0, sizeof(float) * (size_t)num_scales);
      continue;
    }
    memcpy(xout + (size_t)row * row_bytes, xin + (size_t)t * row_bytes, (size_t)row_bytes);
    if (recv_scales)
      memcpy(recv_scales + (size_t)row * num_scales, x_scales + (size_t)t * num_scales,
             sizeof(float) * (size_t)num_scales);
  }
  return 0;
}

/*
 * {source rank, token inside the rank} per row, {-1,-1} for pads
 * (example056 compute_dispatch_indices, :521-564).
 */
void ep_oracle_pull_indices(const int* src_map, int num_rows, int tokens_per_source_rank, int* out) {
  for (int row = 0; row < num_rows; ++row) {
    int t = src_map[row];
    out[2 * row] = t < 0 ? -1 : t / tokens_per_source_rank;
    out[2 * row + 1] = t < 0 ? -1 : t % tokens_per_source_rank;
  }
}

/* ---- combine ---------------------------------------------------------- */

/*
 * out[t,h] = bf16_rne( ((sum over k ascending, slot_map[t,k] >= 0, of
 *                        fmaf(w[t,k], y[slot_map[t,k], h], acc)) + b0[t,h]) + b1[t,h] )
 * with w = 1 when topk_weights is NULL (then fmaf(1, y, acc) == acc + y exactly
 * rounded, the reference's plain ordered sum).  A token with no routes gives zeros
 * (plus biases).  y, bias_0, bias_1 and out are bf16 bit patterns.
 */
int ep_oracle_combine(const uint16_t* y, const int* slot_map, const float* topk_weights,
                      const uint16_t* bias_0, const uint16_t* bias_1, int num_tokens,
                      int num_topk, int hidden, uint16_t* combined_x, int num_threads) {
  if (num_threads < 1) num_threads = 1;
#pragma omp parallel for num_threads(num_threads) schedule(static)
  for (int t = 0; t < num_tokens; ++t) {
    float acc[256];
    for (int h0 = 0; h0 < hidden; h0 += 256) {
      int hn = hidden - h0 < 256 ? hidden - h0 : 256;
      for (int h = 0; h < hn; ++h) acc[h] = 0.0f;
      for (int k = 0; k < num_topk; ++k) {
        int row = slot_map[(size_t)t * num_topk + k];
        if (row < 0) continue;
        float w = topk_weights ? topk_weights[(size_t)t * num_topk + k] : 1.0f;
        const uint16_t* yr = y + (size_t)row * hidden + h0;
        for (int h = 0; h < hn; ++h) acc[h] = fmaf(w, ep_oracle_bf16_to_f32(yr[h]), acc[h]);
      }
      if (bias_0)
        for (int h = 0; h < hn; ++h)
          acc[h] = acc[h] + ep_oracle_bf16_to_f32(bias_0[(size_t)t * hidden + h0 + h]);
      if (bias_1)
        for (int h = 0; h < hn; ++h)
          acc[h] = acc[h] + ep_oracle_bf16_to_f32(bias_1[(size_t)t * hidden + h0 + h]);
      for (int h = 0; h < hn; ++h)
        combined_x[(size_t)t * hidden + h0 + h] = ep_oracle_f32_to_bf16(acc[h]);
    }
  }
  return 0;
}

/* combined_topk_weights[t,k] = recv_topk_weights[slot_map[t,k]], 0 for non-routes. */
void ep_oracle_gather_weights(const float* recv_topk_weights, const int* slot_map, int num_tokens,
                              int num_topk, float* combined_topk_weights) {
  for (size_t i = 0; i < (size_t)num_tokens * num_topk; ++i)
    combined_topk_weights[i] = slot_map[i] >= 0 ? recv_topk_weights[slot_map[i]] : 0.0f;
}

/* combined_topk_idx[t,k] = recv_topk_idx[slot_map[t,k]], -1 for non-routes. */
void ep_oracle_gather_idx(const int64_t* recv_topk_idx, const int* slot_map, int num_tokens, int num_topk,
                          int64_t* combined_topk_idx) {
  for (size_t i = 0; i < (size_t)num_tokens * num_topk; ++i)
    combined_topk_idx[i] = slot_map[i] >= 0 ? recv_topk_idx[slot_map[i]] : -1;
}

/* The per-rank format keeps K weights and K ids per row: route (t,k) reads column k of the row
 * that carries it (rank_row_map[t,k]); 0 / -1 for non-routes.  Either output may be NULL. */
void ep_oracle_gather_rank_side(const float* recv_topk_weights, const int64_t* recv_topk_idx,
                                const int* rank_row_map, int num_tokens, int num_topk, int num_rows,
                                float* combined_topk_weights, int64_t* combined_topk_idx) {
  for (int t = 0; t < num_tokens; ++t)
    for (int k = 0; k < num_topk; ++k) {
      size_t i = (size_t)t * num_topk + k;
      int row = rank_row_map[i];
      int live = row >= 0 && row < num_rows;
      if (combined_topk_weights) combined_topk_weights[i] = live ? recv_topk_weights[(size_t)row * num_topk + k] : 0.0f;
      if (combined_topk_idx) combined_topk_idx[i] = live ? recv_topk_idx[(size_t)row * num_topk + k] : -1;
    }
}

/* counts[b, r] = tokens of block b (tile_tokens consecutive tokens) flagged for rank r. */
int ep_oracle_tile_rank_counts(const uint8_t* is_token_in_rank, int num_tokens, int num_ranks,
                               int tile_tokens, int* counts) {
  if (tile_tokens <= 0 || num_ranks <= 0 || num_tokens < 0) return -1;
  int tiles = (num_tokens + tile_tokens - 1) / tile_tokens;
  memset(counts, 0, sizeof(int) * (size_t)tiles * num_ranks);
  for (int t = 0; t < num_tokens; ++t)
    for (int r = 0; r < num_ranks; ++r)
      if (is_token_in_rank[(size_t)t * num_ranks + r]) ++counts[(size_t)(t / tile_tokens) * num_ranks + r];
  return 0;
}

/* stats[e] += num_tokens_per_expert[e]: the running per-expert totals a caller keeps over launches. */
void ep_oracle_accumulate_stats(const int* num_tokens_per_expert, int num_experts, int* stats) {
  for (int e = 0; e < num_experts; ++e) stats[e] += num_tokens_per_expert[e];
}

/* Per-expert constant scale used by the round-trip workload: rows of expert e are
 * multiplied by (1 + e / denom) in fp32 and rounded to bf16 once. */
void ep_oracle_scale_rows_by_expert(const uint16_t* in, const int* expert_offsets, int num_experts,
                                    int hidden, float denom, uint16_t* out, int num_threads) {
  if (num_threads < 1) num_threads = 1;
#pragma omp parallel for num_threads(num_threads) schedule(dynamic, 1)
  for (int e = 0; e < num_experts; ++e) {
    float s = 1.0f + (float)e / denom;
    for (int row = expert_offsets[e]; row < expert_offsets[e + 1]; ++row)
      for (int h = 0; h < hidden; ++h) {
        size_t i = (size_t)row * hidden + h;
        out[i] = ep_oracle_f32_to_bf16(ep_oracle_bf16_to_f32(in[i]) * s);
      }
  }
}
