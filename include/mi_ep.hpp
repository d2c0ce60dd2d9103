// mi_ep.hpp -- C++ host surface over the C ABI of mi_ep.h.
//
// Mirrors the reference's host classes so that its harnesses read the same with
// hipStream_t in place of cudaStream_t:
//   DeepepDispatchLayout   example042_deepep_dispatch_layout/nv/empty_deepep_dispatch_layout.cu:88-139
//                          (constructor checks :96-107, compute :110-132, print-and-exit :29-37)
//   ExpertParallelBuffer   the one-GPU analogue of DeepEP's ElasticBuffer as the JIT examples
//                          drive it (example080_deepep_jit_dispatch_payload/nv/build_and_run.py:683-725,
//                          example082_deepep_jit_combine/nv/build_and_run.py:751-765)
// Header-only; link against libmi_ep.so and the HIP runtime.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "mi_ep.h"

namespace mi_ep {

using TopkIdx = int64_t;  // negative = masked slot (reference :39)

// Print file:line and the error text, then exit: the reference's CUDA_CHECK convention.
#define MI_EP_HIP_CHECK(call)                                                            \
  do {                                                                                   \
    hipError_t _e = (call);                                                              \
    if (_e != hipSuccess) {                                                              \
      std::fprintf(stderr, "HIP error %s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(_e)); \
      std::exit(EXIT_FAILURE);                                                           \
    }                                                                                    \
  } while (0)

#define MI_EP_CHECK(call)                                                                \
  do {                                                                                   \
    int _c = (call);                                                                     \
    if (_c != MI_EP_OK) {                                                                \
      std::fprintf(stderr, "mi_ep error %s:%d: %s\n", __FILE__, __LINE__, mi_ep_strerror(_c)); \
      std::exit(EXIT_FAILURE);                                                           \
    }                                                                                    \
  } while (0)

inline void check_routing_shape(int num_topk, int num_ranks, int num_experts) {
  if (num_ranks <= 0 || num_ranks > MI_EP_MAX_RANKS) {
    std::fprintf(stderr, "num_ranks must be in [1, %d]\n", MI_EP_MAX_RANKS);
    std::exit(EXIT_FAILURE);
  }
  if (num_topk <= 0 || num_topk > MI_EP_MAX_TOPK) {
    std::fprintf(stderr, "num_topk must be in [1, %d]\n", MI_EP_MAX_TOPK);
    std::exit(EXIT_FAILURE);
  }
  if (num_experts <= 0 || num_experts % num_ranks != 0) {
    std::fprintf(stderr, "num_experts must be divisible by num_ranks\n");
    std::exit(EXIT_FAILURE);
  }
  if (num_experts > MI_EP_MAX_EXPERTS) {
    std::fprintf(stderr, "num_experts must be at most %d\n", MI_EP_MAX_EXPERTS);
    std::exit(EXIT_FAILURE);
  }
}

// Counts and flags; stores four ints, owns nothing, compute() enqueues and returns.
class DeepepDispatchLayout {
 public:
  DeepepDispatchLayout(int num_tokens, int num_topk, int num_ranks, int num_experts)
      : num_tokens_(num_tokens), num_topk_(num_topk), num_ranks_(num_ranks), num_experts_(num_experts) {
    check_routing_shape(num_topk_, num_ranks_, num_experts_);
  }

  void compute(const TopkIdx* d_topk_idx, int* d_num_tokens_per_rank, int* d_num_tokens_per_expert,
               bool* d_is_token_in_rank, hipStream_t stream = 0) const {
    MI_EP_CHECK(mi_ep_get_dispatch_layout(d_topk_idx, d_num_tokens_per_rank, nullptr,
                                          d_num_tokens_per_expert, d_is_token_in_rank, num_tokens_,
                                          num_topk_, num_ranks_, num_experts_, stream));
  }

 private:
  int num_tokens_ = 0;
  int num_topk_ = 0;
  int num_ranks_ = 0;
  int num_experts_ = 0;
};

// What dispatch hands to combine (the reference's `handle`): all device memory, owned by the buffer.
struct DispatchHandle {
  int num_tokens = 0;
  int expert_alignment = 1;
  int* num_tokens_per_rank = nullptr;    // [R]
  int* num_tokens_per_expert = nullptr;  // [E]
  bool* is_token_in_rank = nullptr;      // [T, R]
  int* expert_offsets = nullptr;         // [E + 1]
  int* psum_rank_rows = nullptr;         // [R]
  int* channel_prefix_matrix = nullptr;  // [R, C] (C = num_channels of the buffer, may be 0)
  int* rank_prefix_matrix = nullptr;     // [R, R] source-major, the notify example's rank_prefix_matrix_copy
  int* slot_rel = nullptr;               // [T, K]
  int* rank_slot_idx = nullptr;          // [T, K] the deterministic prologue's table (base 0)
  int* route_order = nullptr;            // [tiles * 256 * K, 4] routes in destination order
  int* tile_rank_counts = nullptr;       // [tiles, R] the prologue's rank_count_buffer, a tile per SM share
  int64_t* copied_topk_idx = nullptr;    // [T, K] the layout kernel's own copy of topk_idx
  int* slot_map = nullptr;               // [T, K]
  int* recv_src_map = nullptr;           // [capacity]
  int64_t* recv_topk_idx = nullptr;      // [capacity]
  float* recv_topk_weights = nullptr;    // [capacity]
  // per-rank receive format (dispatch_ranks)
  int* rank_row_map = nullptr;           // [T, K] row carrying each route
  int* rank_combine_map = nullptr;       // [T, K] each received row once
  int* psum_rank_tokens = nullptr;       // [R] inclusive rows per rank
};

// Owns the layout workspace and the handle's index arrays; payload buffers stay with the caller.
// One buffer serves one stream at a time.
class ExpertParallelBuffer {
 public:
  ExpertParallelBuffer(int num_max_tokens, int num_topk, int num_experts, int num_ranks,
                       int expert_alignment = 1, int num_channels = 0)
      : max_tokens_(num_max_tokens), num_topk_(num_topk), num_experts_(num_experts), num_ranks_(num_ranks),
        num_channels_(num_channels) {
    check_routing_shape(num_topk, num_ranks, num_experts);
    if (expert_alignment < 1) {
      std::fprintf(stderr, "expert_alignment must be positive\n");
      std::exit(EXIT_FAILURE);
    }
    h_.expert_alignment = expert_alignment;
    capacity_ = num_max_tokens * num_topk + num_experts * (expert_alignment - 1);
    workspace_bytes_ = mi_ep_workspace_bytes(num_max_tokens > 0 ? num_max_tokens : 1, num_topk, num_experts, num_ranks);
    const size_t tk = static_cast<size_t>(num_max_tokens) * num_topk;
    MI_EP_HIP_CHECK(hipMalloc(&workspace_, workspace_bytes_));
    MI_EP_HIP_CHECK(hipMalloc(&h_.num_tokens_per_rank, sizeof(int) * num_ranks));
    MI_EP_HIP_CHECK(hipMalloc(&h_.num_tokens_per_expert, sizeof(int) * num_experts));
    MI_EP_HIP_CHECK(hipMalloc(&h_.is_token_in_rank, static_cast<size_t>(num_max_tokens) * num_ranks + 1));
    MI_EP_HIP_CHECK(hipMalloc(&h_.expert_offsets, sizeof(int) * (num_experts + 1)));
    MI_EP_HIP_CHECK(hipMalloc(&h_.psum_rank_rows, sizeof(int) * num_ranks));
    if (num_channels > 0)
      MI_EP_HIP_CHECK(hipMalloc(&h_.channel_prefix_matrix, sizeof(int) * num_ranks * num_channels));
    MI_EP_HIP_CHECK(hipMalloc(&h_.rank_prefix_matrix, sizeof(int) * num_ranks * num_ranks));
    MI_EP_HIP_CHECK(hipMalloc(&h_.slot_rel, sizeof(int) * (tk + 1)));
    MI_EP_HIP_CHECK(hipMalloc(&h_.rank_slot_idx, sizeof(int) * (tk + 1)));
    MI_EP_HIP_CHECK(hipMalloc(&h_.rank_row_map, sizeof(int) * (tk + 1)));
    MI_EP_HIP_CHECK(hipMalloc(&h_.rank_combine_map, sizeof(int) * (tk + 1)));
    MI_EP_HIP_CHECK(hipMalloc(&h_.psum_rank_tokens, sizeof(int) * num_ranks));
    MI_EP_HIP_CHECK(hipMalloc(&h_.route_order, mi_ep_route_order_bytes(num_max_tokens, num_topk) + 16));
    MI_EP_HIP_CHECK(hipMalloc(&h_.tile_rank_counts, sizeof(int) * ((num_max_tokens + 255) / 256 + 1) * num_ranks));
    MI_EP_HIP_CHECK(hipMalloc(&h_.copied_topk_idx, sizeof(int64_t) * (tk + 1)));
    MI_EP_HIP_CHECK(hipMalloc(&h_.slot_map, sizeof(int) * (tk + 1)));
    MI_EP_HIP_CHECK(hipMalloc(&h_.recv_src_map, sizeof(int) * (capacity_ + 1)));
    MI_EP_HIP_CHECK(hipMalloc(&h_.recv_topk_idx, sizeof(int64_t) * (capacity_ + 1)));
    MI_EP_HIP_CHECK(hipMalloc(&h_.recv_topk_weights, sizeof(float) * (capacity_ + 1)));
    MI_EP_CHECK(mi_ep_workspace_init(workspace_, workspace_bytes_, nullptr));
    MI_EP_HIP_CHECK(hipStreamSynchronize(nullptr));
  }

  ~ExpertParallelBuffer() {
    void* owned[] = {workspace_, h_.num_tokens_per_rank, h_.num_tokens_per_expert, h_.is_token_in_rank,
                     h_.expert_offsets, h_.psum_rank_rows, h_.channel_prefix_matrix, h_.slot_rel,
                     h_.rank_slot_idx, h_.rank_row_map, h_.rank_combine_map, h_.psum_rank_tokens,
                     h_.route_order, h_.slot_map, h_.recv_src_map, h_.recv_topk_idx, h_.recv_topk_weights,
                     h_.tile_rank_counts, h_.copied_topk_idx, h_.rank_prefix_matrix};
    for (void* p : owned)
      if (p != nullptr) (void)hipFree(p);
  }

  ExpertParallelBuffer(const ExpertParallelBuffer&) = delete;
  ExpertParallelBuffer& operator=(const ExpertParallelBuffer&) = delete;

  int capacity_rows() const { return capacity_; }
  const DispatchHandle& handle() const { return h_; }
  // Running per-expert totals (int32[E], device memory of the caller): every later layout call adds
  // its counts (the reference's cumulative_local_expert_recv_stats); nullptr switches it off.
  void set_cumulative_expert_stats(int* d_stats) { cumulative_expert_stats_ = d_stats; }

  // Fused layout: counts, flags, offsets, per-route segment positions, the rank prefix matrix (and
  // channel prefixes when the buffer has channels).
  // with_rank_slots also fills rank_slot_idx, the deterministic prologue's per-rank slot table.
  const DispatchHandle& get_dispatch_layout(const TopkIdx* d_topk_idx, int num_tokens, hipStream_t stream = 0,
                                            bool with_rank_slots = false) {
    check_tokens(num_tokens);
    h_.num_tokens = num_tokens;
    MI_EP_CHECK(mi_ep_dispatch_layout(d_topk_idx, num_tokens, num_topk_, num_ranks_, num_experts_,
                                      h_.expert_alignment, num_channels_, h_.num_tokens_per_rank,
                                      h_.num_tokens_per_expert, h_.is_token_in_rank, h_.expert_offsets,
                                      h_.psum_rank_rows, h_.channel_prefix_matrix, h_.rank_prefix_matrix, h_.slot_rel,
                                      with_rank_slots ? h_.rank_slot_idx : nullptr, /*rank_slot_base=*/0, h_.route_order,
                                      h_.tile_rank_counts, h_.copied_topk_idx, cumulative_expert_stats_,
                                      workspace_, workspace_bytes_, stream));
    return h_;
  }

  // Layout + permute.  recv_x / recv_scales hold capacity_rows() rows; scales may be null.
  // flags: MI_EP_DISPATCH_* (pad payload zeroed, copy kernel forced).
  const DispatchHandle& dispatch(const void* d_x, const float* d_scales, const TopkIdx* d_topk_idx,
                                 const float* d_topk_weights, int num_tokens, int row_bytes, int num_scales,
                                 void* d_recv_x, float* d_recv_scales, hipStream_t stream = 0,
                                 int flags = 0) {
    get_dispatch_layout(d_topk_idx, num_tokens, stream);
    MI_EP_CHECK(mi_ep_dispatch(d_x, d_scales, d_topk_idx, d_topk_weights, h_.expert_offsets, h_.slot_rel,
                               h_.route_order, h_.num_tokens_per_expert, num_tokens, num_topk_, num_experts_,
                               h_.expert_alignment, row_bytes, num_scales, d_recv_x, d_recv_scales,
                               h_.recv_src_map, h_.recv_topk_idx, h_.recv_topk_weights, h_.slot_map,
                               capacity_, flags, stream));
    return h_;
  }

  // The reference's own receive format: one row per (token, destination rank), ranks' rows in token
  // order.  Outputs hold rank_capacity_rows() rows; any of the three side arrays may be null.
  // source_token_base stands for rank_idx * num_max_tokens_per_rank in the metadata's column 0.
  const DispatchHandle& dispatch_ranks(const void* d_x, const float* d_scales, const TopkIdx* d_topk_idx,
                                       const float* d_topk_weights, int num_tokens, int row_bytes,
                                       int num_scales, int source_token_base, bool local_expert_ids,
                                       void* d_recv_x, float* d_recv_scales, int64_t* d_recv_topk_idx,
                                       float* d_recv_topk_weights, int* d_recv_src_metadata,
                                       hipStream_t stream = 0) {
    get_dispatch_layout(d_topk_idx, num_tokens, stream, /*with_rank_slots=*/true);
    MI_EP_CHECK(mi_ep_dispatch_ranks(d_x, d_scales, d_topk_idx, d_topk_weights, h_.rank_slot_idx, 0,
                                     h_.num_tokens_per_rank, nullptr, num_tokens, num_topk_, num_ranks_,
                                     num_experts_, row_bytes, num_scales, source_token_base,
                                     local_expert_ids ? 1 : 0, d_recv_x, d_recv_scales, d_recv_topk_idx,
                                     d_recv_topk_weights, d_recv_src_metadata, h_.rank_row_map,
                                     h_.rank_combine_map, h_.psum_rank_tokens, rank_capacity_rows(), stream));
    return h_;
  }
  int rank_capacity_rows() const { return max_tokens_ * (num_topk_ < num_ranks_ ? num_topk_ : num_ranks_); }

  // The reference's combine of that format: the ordered sum of the rows a token sent out (+ biases).
  void combine_ranks(const void* d_y, int num_rows, const void* d_bias_0, const void* d_bias_1, int hidden,
                     void* d_combined_x, hipStream_t stream = 0) const {
    MI_EP_CHECK(mi_ep_combine(d_y, num_rows, h_.rank_combine_map, nullptr, d_bias_0, d_bias_1, nullptr, nullptr,
                              h_.num_tokens, num_topk_, hidden, d_combined_x, nullptr, nullptr, /*flags=*/0, stream));
  }

  // combined_x[t] = bf16(sum_k w[t,k] * y[slot_map[t,k]] + bias_0 + bias_1); null weights = plain sum.
  // d_y holds num_rows rows (capacity_rows() when it is the buffer dispatch filled).
  // d_combined_topk_weights / d_combined_topk_idx (optional) receive the weights / expert ids that
  // travelled with the rows.
  void combine(const void* d_y, int num_rows, const float* d_topk_weights, const void* d_bias_0,
               const void* d_bias_1, int hidden, void* d_combined_x,
               float* d_combined_topk_weights = nullptr, hipStream_t stream = 0,
               int64_t* d_combined_topk_idx = nullptr) const {
    MI_EP_CHECK(mi_ep_combine(d_y, num_rows, h_.slot_map, d_topk_weights, d_bias_0, d_bias_1,
                              d_combined_topk_weights != nullptr ? h_.recv_topk_weights : nullptr,
                              d_combined_topk_idx != nullptr ? h_.recv_topk_idx : nullptr, h_.num_tokens,
                              num_topk_, hidden, d_combined_x, d_combined_topk_weights, d_combined_topk_idx,
                              /*flags=*/0, stream));
  }

  // Synchronises the stream; exits if a device-side bounded wait ever expired.
  void check_status(hipStream_t stream = 0) const { MI_EP_CHECK(mi_ep_workspace_status(workspace_, stream)); }

 private:
  void check_tokens(int num_tokens) const {
    if (num_tokens < 0 || num_tokens > max_tokens_) {
      std::fprintf(stderr, "num_tokens must be in [0, %d]\n", max_tokens_);
      std::exit(EXIT_FAILURE);
    }
  }

  int max_tokens_, num_topk_, num_experts_, num_ranks_, num_channels_;
  int capacity_ = 0;
  void* workspace_ = nullptr;
  size_t workspace_bytes_ = 0;
  int* cumulative_expert_stats_ = nullptr;
  DispatchHandle h_;
};

}  // namespace mi_ep
