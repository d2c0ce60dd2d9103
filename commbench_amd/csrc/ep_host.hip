// Host-pointer twins of the device entry points: every pointer is ordinary host memory.
// Each call allocates device buffers, copies the inputs over, runs the same kernels through
// the device entry points, copies the outputs back and synchronises.  They are a convenience
// for callers without a device-side pipeline (a harness that holds numpy arrays, a first
// integration step); the transfers dominate, so nothing here is a measured path.
#include "../../include/mi_ep.h"

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace {

// Device buffers that free themselves; `ok` turns false on the first failed allocation or copy.
struct Staging {
  hipError_t err = hipSuccess;
  void* owned[24];
  int count = 0;

  ~Staging() {
    for (int i = 0; i < count; ++i) (void)hipFree(owned[i]);
  }
  bool ok() const { return err == hipSuccess; }

  template <typename T>
  T* alloc(size_t n) {
    if (!ok()) return nullptr;
    if (count == static_cast<int>(sizeof(owned) / sizeof(owned[0]))) {
      err = hipErrorOutOfMemory;
      return nullptr;
    }
    void* p = nullptr;
    err = hipMalloc(&p, (n > 0 ? n : 1) * sizeof(T) + 16);
    if (err != hipSuccess) return nullptr;
    owned[count++] = p;
    return static_cast<T*>(p);
  }
  template <typename T>
  T* upload(const T* host, size_t n) {
    if (host == nullptr) return nullptr;
    T* d = alloc<T>(n);
    if (ok() && n > 0) err = hipMemcpy(d, host, n * sizeof(T), hipMemcpyHostToDevice);
    return d;
  }
  template <typename T>
  void download(T* host, const T* dev, size_t n) {
    if (ok() && host != nullptr && n > 0) err = hipMemcpy(host, dev, n * sizeof(T), hipMemcpyDeviceToHost);
  }
  int status(int code) const {
    if (code != MI_EP_OK) return code;
    return err == hipSuccess ? MI_EP_OK : static_cast<int>(err);
  }
};

int sync_status(int code) {
  if (code != MI_EP_OK) return code;
  const hipError_t e = hipStreamSynchronize(nullptr);
  return e == hipSuccess ? MI_EP_OK : static_cast<int>(e);
}

}  // namespace

extern "C" {

int mi_ep_host_get_dispatch_layout(const int64_t* topk_idx, int* num_tokens_per_rank,
                                   int* num_tokens_per_rdma_rank, int* num_tokens_per_expert,
                                   bool* is_token_in_rank, int num_tokens, int num_topk, int num_ranks,
                                   int num_experts) {
  (void)num_tokens_per_rdma_rank;
  if (num_tokens < 0 || num_topk <= 0 || num_ranks <= 0 || num_experts <= 0) return MI_EP_EINVAL;
  if (num_tokens_per_rank == nullptr || num_tokens_per_expert == nullptr) return MI_EP_EINVAL;
  if (num_tokens > 0 && (topk_idx == nullptr || is_token_in_rank == nullptr)) return MI_EP_EINVAL;
  Staging s;
  const size_t tk = static_cast<size_t>(num_tokens) * num_topk;
  const size_t tr = static_cast<size_t>(num_tokens) * num_ranks;
  const int64_t* d_topk = s.upload(topk_idx, tk);
  int* d_rank = s.alloc<int>(num_ranks);
  int* d_expert = s.alloc<int>(num_experts);
  bool* d_flags = s.alloc<bool>(tr);
  if (!s.ok()) return s.status(MI_EP_OK);
  int code = mi_ep_get_dispatch_layout(d_topk, d_rank, nullptr, d_expert, d_flags, num_tokens, num_topk,
                                       num_ranks, num_experts, nullptr);
  code = sync_status(code);
  if (code != MI_EP_OK) return code;
  s.download(num_tokens_per_rank, d_rank, num_ranks);
  s.download(num_tokens_per_expert, d_expert, num_experts);
  s.download(is_token_in_rank, d_flags, tr);
  return s.status(MI_EP_OK);
}

int mi_ep_host_dispatch_layout(const int64_t* topk_idx, int num_tokens, int num_topk, int num_ranks,
                               int num_experts, int expert_alignment, int num_channels,
                               int* num_tokens_per_rank, int* num_tokens_per_expert, bool* is_token_in_rank,
                               int* expert_offsets, int* psum_rank_rows, int* channel_prefix_matrix,
                               int* rank_prefix_matrix, int* slot_rel, int* rank_slot_idx, int rank_slot_base,
                               int* route_order, int* tile_rank_counts, int64_t* copied_topk_idx,
                               int* cumulative_expert_stats) {
  if (num_tokens < 0 || num_topk <= 0 || num_ranks <= 0 || num_experts <= 0 || expert_alignment < 1)
    return MI_EP_EINVAL;
  if (num_tokens_per_rank == nullptr || num_tokens_per_expert == nullptr) return MI_EP_EINVAL;
  if (num_tokens > 0 && (topk_idx == nullptr || is_token_in_rank == nullptr)) return MI_EP_EINVAL;
  if (channel_prefix_matrix != nullptr && num_channels < 1) return MI_EP_EINVAL;
  const size_t workspace_bytes = mi_ep_workspace_bytes(num_tokens > 0 ? num_tokens : 1, num_topk, num_experts, num_ranks);
  if (workspace_bytes == 0) return MI_EP_EINVAL;

  Staging s;
  const size_t tk = static_cast<size_t>(num_tokens) * num_topk;
  const size_t tr = static_cast<size_t>(num_tokens) * num_ranks;
  const size_t tiles = (static_cast<size_t>(num_tokens) + 255) / 256;
  const size_t order_ints = mi_ep_route_order_bytes(num_tokens, num_topk) / sizeof(int);
  const size_t rc = channel_prefix_matrix != nullptr ? static_cast<size_t>(num_ranks) * num_channels : 0;
  const int64_t* d_topk = s.upload(topk_idx, tk);
  int* d_rank = s.alloc<int>(num_ranks);
  int* d_expert = s.alloc<int>(num_experts);
  bool* d_flags = s.alloc<bool>(tr);
  int* d_off = expert_offsets != nullptr ? s.alloc<int>(static_cast<size_t>(num_experts) + 1) : nullptr;
  int* d_psum = psum_rank_rows != nullptr ? s.alloc<int>(num_ranks) : nullptr;
  int* d_prefix = channel_prefix_matrix != nullptr ? s.alloc<int>(rc) : nullptr;
  const size_t rr = static_cast<size_t>(num_ranks) * num_ranks;
  int* d_rank_prefix = rank_prefix_matrix != nullptr ? s.alloc<int>(rr) : nullptr;
  int* d_slot_rel = slot_rel != nullptr ? s.alloc<int>(tk) : nullptr;
  int* d_rank_slots = rank_slot_idx != nullptr ? s.alloc<int>(tk) : nullptr;
  int* d_order = route_order != nullptr ? s.alloc<int>(order_ints) : nullptr;
  int* d_tile_ranks = tile_rank_counts != nullptr ? s.alloc<int>(tiles * num_ranks) : nullptr;
  int64_t* d_copied = copied_topk_idx != nullptr ? s.alloc<int64_t>(tk) : nullptr;
  // The running statistics continue from the caller's values.
  int* d_stats = cumulative_expert_stats != nullptr
                     ? const_cast<int*>(s.upload(static_cast<const int*>(cumulative_expert_stats), num_experts))
                     : nullptr;
  unsigned char* d_ws = s.alloc<unsigned char>(workspace_bytes);
  if (!s.ok()) return s.status(MI_EP_OK);
  if (d_order != nullptr && order_ints > 0) {
    // Entries past the last token are not written by the kernel: hand back zeros there.
    s.err = hipMemset(d_order, 0, order_ints * sizeof(int));
    if (!s.ok()) return s.status(MI_EP_OK);
  }

  int code = mi_ep_workspace_init(d_ws, workspace_bytes, nullptr);
  if (code == MI_EP_OK)
    code = mi_ep_dispatch_layout(d_topk, num_tokens, num_topk, num_ranks, num_experts, expert_alignment,
                                 num_channels, d_rank, d_expert, d_flags, d_off, d_psum, d_prefix, d_rank_prefix,
                                 d_slot_rel, d_rank_slots, rank_slot_base, d_order, d_tile_ranks, d_copied, d_stats, d_ws,
                                 workspace_bytes, nullptr);
  if (code == MI_EP_OK) code = mi_ep_workspace_status(d_ws, nullptr);  // synchronises
  if (code != MI_EP_OK) return code;
  s.download(num_tokens_per_rank, d_rank, num_ranks);
  s.download(num_tokens_per_expert, d_expert, num_experts);
  s.download(is_token_in_rank, d_flags, tr);
  s.download(expert_offsets, d_off, static_cast<size_t>(num_experts) + 1);
  s.download(psum_rank_rows, d_psum, num_ranks);
  s.download(channel_prefix_matrix, d_prefix, rc);
  s.download(rank_prefix_matrix, d_rank_prefix, rr);
  s.download(slot_rel, d_slot_rel, tk);
  s.download(rank_slot_idx, d_rank_slots, tk);
  s.download(route_order, d_order, order_ints);
  s.download(tile_rank_counts, d_tile_ranks, tiles * num_ranks);
  s.download(copied_topk_idx, d_copied, tk);
  s.download(cumulative_expert_stats, d_stats, num_experts);
  return s.status(MI_EP_OK);
}

int mi_ep_host_dispatch(const void* x, const float* x_scales, const int64_t* topk_idx,
                        const float* topk_weights, int num_tokens, int num_topk, int num_ranks,
                        int num_experts, int expert_alignment, int row_bytes, int num_scales,
                        int* num_tokens_per_rank, int* num_tokens_per_expert, bool* is_token_in_rank,
                        int* expert_offsets, void* recv_x, float* recv_scales, int* recv_src_map,
                        int64_t* recv_topk_idx, float* recv_topk_weights, int* slot_map,
                        int capacity_rows) {
  if (num_tokens < 0 || num_topk <= 0 || num_ranks <= 0 || num_experts <= 0 || expert_alignment < 1)
    return MI_EP_EINVAL;
  if (row_bytes <= 0 || row_bytes % 16 != 0 || num_scales < 0 || capacity_rows < 0) return MI_EP_EINVAL;
  if (expert_offsets == nullptr || recv_src_map == nullptr || slot_map == nullptr) return MI_EP_EINVAL;
  if (num_tokens > 0 && (x == nullptr || topk_idx == nullptr)) return MI_EP_EINVAL;
  if (capacity_rows > 0 && recv_x == nullptr) return MI_EP_EINVAL;
  if ((num_scales > 0) != (recv_scales != nullptr)) return MI_EP_EINVAL;
  if (num_scales > 0 && num_tokens > 0 && x_scales == nullptr) return MI_EP_EINVAL;
  const size_t workspace_bytes = mi_ep_workspace_bytes(num_tokens > 0 ? num_tokens : 1, num_topk, num_experts, num_ranks);
  if (workspace_bytes == 0) return MI_EP_EINVAL;

  Staging s;
  const size_t tk = static_cast<size_t>(num_tokens) * num_topk;
  const size_t tr = static_cast<size_t>(num_tokens) * num_ranks;
  const size_t cap = static_cast<size_t>(capacity_rows);
  const unsigned char* d_x = s.upload(static_cast<const unsigned char*>(x), static_cast<size_t>(num_tokens) * row_bytes);
  const float* d_scales = num_scales > 0 ? s.upload(x_scales, static_cast<size_t>(num_tokens) * num_scales) : nullptr;
  const int64_t* d_topk = s.upload(topk_idx, tk);
  const float* d_w = s.upload(topk_weights, tk);
  int* d_rank = s.alloc<int>(num_ranks);
  int* d_expert = s.alloc<int>(num_experts);
  bool* d_flags = s.alloc<bool>(tr);
  int* d_off = s.alloc<int>(static_cast<size_t>(num_experts) + 1);
  int* d_slot_rel = s.alloc<int>(tk);
  int* d_order = s.alloc<int>(mi_ep_route_order_bytes(num_tokens, num_topk) / sizeof(int));
  unsigned char* d_ws = s.alloc<unsigned char>(workspace_bytes);
  unsigned char* d_recv_x = s.alloc<unsigned char>(cap * row_bytes);
  float* d_recv_scales = num_scales > 0 ? s.alloc<float>(cap * num_scales) : nullptr;
  int* d_src_map = s.alloc<int>(cap);
  int64_t* d_recv_idx = s.alloc<int64_t>(cap);
  float* d_recv_w = s.alloc<float>(cap);
  int* d_slot_map = s.alloc<int>(tk);
  if (!s.ok()) return s.status(MI_EP_OK);

  int code = mi_ep_workspace_init(d_ws, workspace_bytes, nullptr);
  if (code == MI_EP_OK)
    code = mi_ep_dispatch_layout(d_topk, num_tokens, num_topk, num_ranks, num_experts, expert_alignment, 0,
                                 d_rank, d_expert, d_flags, d_off, nullptr, nullptr, nullptr, d_slot_rel, nullptr,
                                 0, d_order, nullptr, nullptr, nullptr, d_ws, workspace_bytes, nullptr);
  if (code == MI_EP_OK)
    code = mi_ep_dispatch(d_x, d_scales, d_topk, d_w, d_off, d_slot_rel, d_order, d_expert, num_tokens,
                          num_topk, num_experts, expert_alignment, row_bytes, num_scales, d_recv_x,
                          d_recv_scales, d_src_map, d_recv_idx, d_recv_w, d_slot_map, capacity_rows,
                          MI_EP_DISPATCH_ZERO_PAD_PAYLOAD, nullptr);  // pad rows come back as zeros
  if (code == MI_EP_OK) code = mi_ep_workspace_status(d_ws, nullptr);  // synchronises
  if (code != MI_EP_OK) return code;

  int total = 0;
  s.download(&total, d_off + num_experts, 1);
  if (!s.ok()) return s.status(MI_EP_OK);
  const size_t rows = static_cast<size_t>(total) < cap ? static_cast<size_t>(total) : cap;
  s.download(num_tokens_per_rank, d_rank, num_ranks);
  s.download(num_tokens_per_expert, d_expert, num_experts);
  s.download(is_token_in_rank, d_flags, tr);
  s.download(expert_offsets, d_off, static_cast<size_t>(num_experts) + 1);
  s.download(static_cast<unsigned char*>(recv_x), d_recv_x, rows * row_bytes);
  if (num_scales > 0) s.download(recv_scales, d_recv_scales, rows * num_scales);
  s.download(recv_src_map, d_src_map, rows);
  s.download(recv_topk_idx, d_recv_idx, rows);
  s.download(recv_topk_weights, d_recv_w, rows);
  s.download(slot_map, d_slot_map, tk);
  return s.status(MI_EP_OK);
}

int mi_ep_host_dispatch_ranks(const void* x, const float* x_scales, const int64_t* topk_idx,
                              const float* topk_weights, int num_tokens, int num_topk, int num_ranks,
                              int num_experts, int row_bytes, int num_scales, int source_token_base,
                              int local_expert_ids, int* num_tokens_per_rank, void* recv_x,
                              float* recv_scales, int64_t* recv_topk_idx, float* recv_topk_weights,
                              int* recv_src_metadata, int* rank_row_map, int* combine_map,
                              int* psum_rank_tokens, int capacity_rows) {
  if (num_tokens < 0 || num_topk <= 0 || num_ranks <= 0 || num_experts <= 0) return MI_EP_EINVAL;
  if (row_bytes <= 0 || row_bytes % 16 != 0 || num_scales < 0 || capacity_rows < 0) return MI_EP_EINVAL;
  if (psum_rank_tokens == nullptr) return MI_EP_EINVAL;
  if (num_tokens > 0 && (x == nullptr || topk_idx == nullptr || rank_row_map == nullptr)) return MI_EP_EINVAL;
  if (capacity_rows > 0 && recv_x == nullptr) return MI_EP_EINVAL;
  if ((num_scales > 0) != (recv_scales != nullptr)) return MI_EP_EINVAL;
  if (num_scales > 0 && num_tokens > 0 && x_scales == nullptr) return MI_EP_EINVAL;
  const size_t workspace_bytes = mi_ep_workspace_bytes(num_tokens > 0 ? num_tokens : 1, num_topk, num_experts, num_ranks);
  if (workspace_bytes == 0) return MI_EP_EINVAL;

  Staging s;
  const size_t tk = static_cast<size_t>(num_tokens) * num_topk;
  const size_t tr = static_cast<size_t>(num_tokens) * num_ranks;
  const size_t cap = static_cast<size_t>(capacity_rows);
  const size_t meta = static_cast<size_t>(2 + num_topk);
  const unsigned char* d_x = s.upload(static_cast<const unsigned char*>(x), static_cast<size_t>(num_tokens) * row_bytes);
  const float* d_scales = num_scales > 0 ? s.upload(x_scales, static_cast<size_t>(num_tokens) * num_scales) : nullptr;
  const int64_t* d_topk = s.upload(topk_idx, tk);
  const float* d_w = s.upload(topk_weights, tk);
  int* d_rank = s.alloc<int>(num_ranks);
  int* d_expert = s.alloc<int>(num_experts);
  bool* d_flags = s.alloc<bool>(tr);
  int* d_rank_slots = s.alloc<int>(tk);
  unsigned char* d_ws = s.alloc<unsigned char>(workspace_bytes);
  unsigned char* d_recv_x = s.alloc<unsigned char>(cap * row_bytes);
  float* d_recv_scales = num_scales > 0 ? s.alloc<float>(cap * num_scales) : nullptr;
  int64_t* d_recv_idx = recv_topk_idx != nullptr ? s.alloc<int64_t>(cap * num_topk) : nullptr;
  float* d_recv_w = recv_topk_weights != nullptr ? s.alloc<float>(cap * num_topk) : nullptr;
  int* d_meta = recv_src_metadata != nullptr ? s.alloc<int>(cap * meta) : nullptr;
  int* d_row_map = s.alloc<int>(tk);
  int* d_combine_map = combine_map != nullptr ? s.alloc<int>(tk) : nullptr;
  int* d_psum = s.alloc<int>(num_ranks);
  if (!s.ok()) return s.status(MI_EP_OK);

  int code = mi_ep_workspace_init(d_ws, workspace_bytes, nullptr);
  if (code == MI_EP_OK)
    code = mi_ep_dispatch_layout(d_topk, num_tokens, num_topk, num_ranks, num_experts, 1, 0, d_rank, d_expert,
                                 d_flags, nullptr, nullptr, nullptr, nullptr, nullptr, d_rank_slots, 0, nullptr,
                                 nullptr, nullptr, nullptr, d_ws, workspace_bytes, nullptr);
  if (code == MI_EP_OK)
    code = mi_ep_dispatch_ranks(d_x, d_scales, d_topk, d_w, d_rank_slots, 0, d_rank, nullptr, num_tokens,
                                num_topk, num_ranks, num_experts, row_bytes, num_scales, source_token_base,
                                local_expert_ids, d_recv_x, d_recv_scales, d_recv_idx, d_recv_w, d_meta,
                                d_row_map, d_combine_map, d_psum, capacity_rows, nullptr);
  if (code == MI_EP_OK) code = mi_ep_workspace_status(d_ws, nullptr);  // synchronises
  if (code != MI_EP_OK) return code;

  int total = 0;
  s.download(&total, d_psum + (num_ranks - 1), 1);
  if (!s.ok()) return s.status(MI_EP_OK);
  const size_t rows = static_cast<size_t>(total) < cap ? static_cast<size_t>(total) : cap;
  s.download(num_tokens_per_rank, d_rank, num_ranks);
  s.download(static_cast<unsigned char*>(recv_x), d_recv_x, rows * row_bytes);
  if (num_scales > 0) s.download(recv_scales, d_recv_scales, rows * num_scales);
  s.download(recv_topk_idx, d_recv_idx, rows * num_topk);
  s.download(recv_topk_weights, d_recv_w, rows * num_topk);
  s.download(recv_src_metadata, d_meta, rows * meta);
  s.download(rank_row_map, d_row_map, tk);
  s.download(combine_map, d_combine_map, tk);
  s.download(psum_rank_tokens, d_psum, num_ranks);
  return s.status(MI_EP_OK);
}

int mi_ep_host_dispatch_cached(const void* x, const float* x_scales, const int* recv_src_map, int num_rows,
                               int num_tokens, int row_bytes, int num_scales, void* recv_x,
                               float* recv_scales) {
  if (num_rows < 0 || num_tokens < 0 || row_bytes <= 0 || row_bytes % 16 != 0 || num_scales < 0)
    return MI_EP_EINVAL;
  if (num_rows > 0 && (recv_src_map == nullptr || recv_x == nullptr)) return MI_EP_EINVAL;
  if (num_rows > 0 && num_tokens > 0 && x == nullptr) return MI_EP_EINVAL;
  if ((num_scales > 0) != (recv_scales != nullptr)) return MI_EP_EINVAL;
  if (num_scales > 0 && num_tokens > 0 && x_scales == nullptr) return MI_EP_EINVAL;
  Staging s;
  const size_t rows = static_cast<size_t>(num_rows);
  const unsigned char* d_x = s.upload(static_cast<const unsigned char*>(x), static_cast<size_t>(num_tokens) * row_bytes);
  const float* d_scales = num_scales > 0 ? s.upload(x_scales, static_cast<size_t>(num_tokens) * num_scales) : nullptr;
  const int* d_map = s.upload(recv_src_map, rows);
  unsigned char* d_recv_x = s.alloc<unsigned char>(rows * row_bytes);
  float* d_recv_scales = num_scales > 0 ? s.alloc<float>(rows * num_scales) : nullptr;
  if (!s.ok()) return s.status(MI_EP_OK);
  int code = mi_ep_dispatch_cached(d_x, d_scales, d_map, num_rows, num_tokens, row_bytes, num_scales, d_recv_x,
                                   d_recv_scales, nullptr, 0, nullptr);
  code = sync_status(code);
  if (code != MI_EP_OK) return code;
  s.download(static_cast<unsigned char*>(recv_x), d_recv_x, rows * row_bytes);
  if (num_scales > 0) s.download(recv_scales, d_recv_scales, rows * num_scales);
  return s.status(MI_EP_OK);
}

int mi_ep_host_combine(const void* y, int num_rows, const int* slot_map, const float* topk_weights,
                       const void* bias_0, const void* bias_1, int num_tokens, int num_topk, int hidden,
                       void* combined_x) {
  if (num_tokens < 0 || num_topk <= 0 || hidden <= 0 || hidden % 8 != 0 || num_rows < 0) return MI_EP_EINVAL;
  if (num_rows > 0 && y == nullptr) return MI_EP_EINVAL;
  if (num_tokens > 0 && (slot_map == nullptr || combined_x == nullptr)) return MI_EP_EINVAL;
  Staging s;
  const size_t tk = static_cast<size_t>(num_tokens) * num_topk;
  const size_t th = static_cast<size_t>(num_tokens) * hidden;
  const uint16_t* d_y = s.upload(static_cast<const uint16_t*>(y), static_cast<size_t>(num_rows) * hidden);
  const int* d_map = s.upload(slot_map, tk);
  const float* d_w = s.upload(topk_weights, tk);
  const uint16_t* d_b0 = s.upload(static_cast<const uint16_t*>(bias_0), th);
  const uint16_t* d_b1 = s.upload(static_cast<const uint16_t*>(bias_1), th);
  uint16_t* d_out = s.alloc<uint16_t>(th);
  if (!s.ok()) return s.status(MI_EP_OK);
  int code = mi_ep_combine(d_y, num_rows, d_map, d_w, d_b0, d_b1, nullptr, nullptr, num_tokens, num_topk,
                           hidden, d_out, nullptr, nullptr, MI_EP_COMBINE_STREAM_OUTPUT, nullptr);  // read back over PCIe next
  code = sync_status(code);
  if (code != MI_EP_OK) return code;
  s.download(static_cast<uint16_t*>(combined_x), d_out, th);
  return s.status(MI_EP_OK);
}

}  // extern "C"
