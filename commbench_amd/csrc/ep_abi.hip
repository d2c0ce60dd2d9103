// extern "C" boundary of the gfx950 dispatch core: argument checks on the host,
// then kernel launches.  No allocation, no synchronisation (except
// mi_ep_workspace_status, which says so) and no mutable process-wide state: what
// varies per caller travels in arguments or in the caller's workspace; the only
// file-scope data are per-device caches of hardware facts that never change.
#include "../../include/mi_ep.h"

#include <atomic>

#include "ep_device.h"

namespace {

using namespace mi_ep;

inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// The reference's constructor checks (example042 .cu:96-107) plus the limits of
// these kernels.
inline bool routing_shape_ok(int num_tokens, int num_topk, int num_ranks, int num_experts) {
  if (num_tokens < 0) return false;
  if (num_ranks <= 0 || num_ranks > MI_EP_MAX_RANKS) return false;
  if (num_topk <= 0 || num_topk > MI_EP_MAX_TOPK) return false;
  if (num_experts <= 0 || num_experts > MI_EP_MAX_EXPERTS) return false;
  if (num_experts % num_ranks != 0) return false;
  if (static_cast<long long>(num_tokens) * num_topk >= (1LL << 30)) return false;
  // A library built for fixed shapes serves those only.
  return fixed::accepts(fixed::kTopk, num_topk) && fixed::accepts(fixed::kExperts, num_experts) &&
         fixed::accepts(fixed::kRanks, num_ranks);
}

inline int num_tiles_for(int num_tokens) { return (num_tokens + kTileTokens - 1) / kTileTokens; }

inline int status_of(hipError_t e) { return e == hipSuccess ? MI_EP_OK : static_cast<int>(e); }

inline bool route_count_ok(int num_tokens, int num_topk) {
  return num_tokens >= 0 && num_topk > 0 && num_topk <= MI_EP_MAX_TOPK && fixed::accepts(fixed::kTopk, num_topk) &&
         static_cast<long long>(num_tokens) * num_topk < (1LL << 30);
}

constexpr int kScheduleFlags = MI_EP_DISPATCH_BY_TOKEN | MI_EP_DISPATCH_BY_DESTINATION;

// ---- scratch of the allocation-free layout entry point ------------------------------------
// One copy per GPU, held until the process ends: the layout workspace (256-byte header + status
// words) for shapes up to MI_EP_STATIC_LAYOUT_STATUS_WORDS status words.  `scratch` is a host-side
// stand-in here; kernels get the device address resolved below.
constexpr size_t kStaticStatusWords = MI_EP_STATIC_LAYOUT_STATUS_WORDS;
constexpr size_t kStaticScratchBytes = sizeof(LayoutWorkspace) + kStaticStatusWords * sizeof(uint64_t);
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
// Device address of `scratch` per device ordinal: resolved on the first call on that device,
// read-only afterwards (every resolver stores the same value).  Like any device address it does not
// outlive a hipDeviceReset of that device.
std::atomic<void*> g_scratch_address[kMaxDevices];

// The static scratch of the device `stream` belongs to (of the current device for the null
// stream): the device the kernels are launched on, whatever device is current.
int static_scratch_of(hipStream_t stream, void** out) {
  int dev = -1;
  hipError_t e = stream != nullptr ? hipStreamGetDevice(stream, &dev) : hipGetDevice(&dev);
  if (e != hipSuccess) return static_cast<int>(e);
  if (dev < 0 || dev >= kMaxDevices) return MI_EP_EINVAL;
  void* p = g_scratch_address[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    // A symbol resolves to the current device's copy of the array: make the stream's device
    // current for the lookup, and put the caller's back.
    int current = -1;
    e = hipGetDevice(&current);
    if (e != hipSuccess) return static_cast<int>(e);
    if (current != dev && (e = hipSetDevice(dev)) != hipSuccess) return static_cast<int>(e);
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (current != dev) {
      const hipError_t back = hipSetDevice(current);
      if (e == hipSuccess) e = back;
    }
    if (e != hipSuccess) return static_cast<int>(e);
    if (p == nullptr) return static_cast<int>(hipErrorInvalidSymbol);
    g_scratch_address[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return MI_EP_OK;
}

// The workspace calls take MI_EP_STATIC_SCRATCH for the library's own scratch.
int resolve_workspace(void** workspace, size_t* workspace_bytes, hipStream_t stream) {
  if (*workspace != MI_EP_STATIC_SCRATCH) return MI_EP_OK;
  const int rc = static_scratch_of(stream, workspace);
  if (rc == MI_EP_OK && workspace_bytes != nullptr) *workspace_bytes = kStaticScratchBytes;
  return rc;
}

// Argument checks and launch shared by mi_ep_dispatch_layout (caller's workspace) and
// mi_ep_dispatch_layout_static (workspace == nullptr and use_static_scratch: the library's static
// scratch on the stream's device, resolved after the argument checks).
int dispatch_layout_on(const int64_t* topk_idx, int num_tokens, int num_topk, int num_ranks,
                       int num_experts, int expert_alignment, int num_channels,
                       int* num_tokens_per_rank, int* num_tokens_per_expert, bool* is_token_in_rank,
                       int* expert_offsets, int* psum_rank_rows, int* channel_prefix_matrix,
                       int* rank_prefix_matrix, int* slot_rel, int* rank_slot_idx, int rank_slot_base,
                       int* route_order,
                       int* tile_rank_counts, int64_t* copied_topk_idx, int* cumulative_expert_stats,
                       void* workspace, size_t workspace_bytes, bool use_static_scratch,
                       int* timeout_report, void* stream) {
  if (!routing_shape_ok(num_tokens, num_topk, num_ranks, num_experts)) return MI_EP_EINVAL;
  // Shapes beyond the static array are refused before anything else is looked at.
  if (use_static_scratch &&
      static_cast<size_t>(num_tiles_for(num_tokens)) * static_cast<size_t>(num_experts + num_ranks) > kStaticStatusWords)
    return MI_EP_E2BIG;
  if (expert_alignment < 1) return MI_EP_EINVAL;
  if (num_tokens_per_rank == nullptr || num_tokens_per_expert == nullptr) return MI_EP_EINVAL;
  if (channel_prefix_matrix != nullptr && (num_channels < 1 || num_channels > 4096)) return MI_EP_EINVAL;
  if (psum_rank_rows != nullptr && expert_offsets == nullptr) return MI_EP_EINVAL;
  // Padded totals must stay inside int32.
  if ((static_cast<long long>(num_tokens) * num_topk +
       static_cast<long long>(num_experts) * (expert_alignment - 1)) >= (1LL << 31))
    return MI_EP_EINVAL;
  if (num_tokens > 0 && (topk_idx == nullptr || is_token_in_rank == nullptr)) return MI_EP_EINVAL;
  if (!aligned16(route_order)) return MI_EP_EINVAL;
  hipStream_t s = as_stream(stream);
  if (use_static_scratch && num_tokens > 0) {
    const int rc = static_scratch_of(s, &workspace);
    if (rc != MI_EP_OK) return rc;
    workspace_bytes = kStaticScratchBytes;
  }

  if (num_tokens == 0) {
    // Nothing to scan: every output is zero.
    hipError_t e = launch_fill_u32(reinterpret_cast<uint32_t*>(num_tokens_per_rank), num_ranks, 0u, s);
    if (e == hipSuccess)
      e = launch_fill_u32(reinterpret_cast<uint32_t*>(num_tokens_per_expert), num_experts, 0u, s);
    if (e == hipSuccess && expert_offsets != nullptr)
      e = launch_fill_u32(reinterpret_cast<uint32_t*>(expert_offsets), num_experts + 1, 0u, s);
    if (e == hipSuccess && psum_rank_rows != nullptr)
      e = launch_fill_u32(reinterpret_cast<uint32_t*>(psum_rank_rows), num_ranks, 0u, s);
    if (e == hipSuccess && channel_prefix_matrix != nullptr)
      e = launch_fill_u32(reinterpret_cast<uint32_t*>(channel_prefix_matrix),
                          static_cast<size_t>(num_ranks) * num_channels, 0u, s);
    if (e == hipSuccess && rank_prefix_matrix != nullptr)
      e = launch_fill_u32(reinterpret_cast<uint32_t*>(rank_prefix_matrix),
                          static_cast<size_t>(num_ranks) * num_ranks, 0u, s);
    return status_of(e);
  }

  if (workspace == nullptr) return MI_EP_EINVAL;
  if ((reinterpret_cast<uintptr_t>(workspace) & 7u) != 0) return MI_EP_EINVAL;
  if (workspace_bytes < mi_ep_workspace_bytes(num_tokens, num_topk, num_experts, num_ranks))
    return MI_EP_ENOSPC;

  LayoutArgs a{};
  a.topk_idx = topk_idx;
  a.num_tokens_per_rank = num_tokens_per_rank;
  a.num_tokens_per_expert = num_tokens_per_expert;
  a.is_token_in_rank = reinterpret_cast<uint8_t*>(is_token_in_rank);
  a.expert_offsets = expert_offsets;
  a.psum_rank_rows = psum_rank_rows;
  a.channel_prefix_matrix = channel_prefix_matrix;
  a.rank_prefix_matrix = rank_prefix_matrix;
  a.slot_rel = slot_rel;
  a.rank_slot_idx = rank_slot_idx;
  a.rank_slot_base = rank_slot_base;
  a.route_order = route_order;
  a.tile_rank_counts = tile_rank_counts;
  a.copied_topk_idx = copied_topk_idx;
  a.cumulative_expert_stats = cumulative_expert_stats;
  a.ws = static_cast<LayoutWorkspace*>(workspace);
  a.timeout_report = timeout_report;
  a.num_tokens = num_tokens;
  a.num_topk = num_topk;
  a.num_ranks = num_ranks;
  a.num_experts = num_experts;
  a.experts_per_rank = num_experts / num_ranks;
  a.expert_alignment = expert_alignment;
  a.num_channels = num_channels;
  a.num_tiles = num_tiles_for(num_tokens);
  // Small grids take static tiles (workgroup b = tile b: one memory round trip less before the first
  // load).  A tile's scan then may wait on a tile whose workgroup has not started, which is harmless as
  // long as that workgroup finds a slot: with at most one tile per eight compute units a launch takes
  // 1/16 of the slots its workgroups could occupy (two fit a compute unit), so that sixteen such
  // launches would have to execute at once, each partly resident, before one could keep another's
  // tiles out -- more than a process has hardware queues.  Larger grids take tickets, which order the
  // tiles by arrival and need no such argument.  The wait is bounded either way.
  DeviceTraits dev{};
  a.static_tiles = (device_traits(s, &dev) == hipSuccess && a.num_tiles * 8 <= dev.compute_units) ? 1 : 0;
  // Grids whose last tile can fetch every predecessor's packed row in two rounds of 16-byte loads do
  // that instead of walking back column by column.
  const long long row_words = (num_experts + 1) / 2 + (num_ranks + 1) / 2;
  a.gather_rows = ((a.num_tiles - 1) * row_words <= kGatherLimitWords && aligned16(workspace)) ? 1 : 0;
  a.expert_bits = 1;
  while ((1 << a.expert_bits) < num_experts) ++a.expert_bits;
  a.inv_topk = ((1u << 19) + num_topk - 1) / num_topk;
  a.inv_experts_per_rank = ((1u << 22) + a.experts_per_rank - 1) / a.experts_per_rank;
  return status_of(launch_layout_fused(a, s));
}

}  // namespace

extern "C" {

int mi_ep_abi_version(void) { return MI_EP_ABI_VERSION; }

const char* mi_ep_strerror(int code) {
  switch (code) {
    case MI_EP_OK: return "ok";
    case MI_EP_EINVAL: return "invalid argument";
    case MI_EP_ENOSPC: return "workspace too small";
    case MI_EP_E2BIG: return "shape exceeds the static scratch of the allocation-free entry point";
    case MI_EP_ETIMEDOUT: return "device-side wait timed out";
    default: break;
  }
  if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
  return "unknown error";
}

int mi_ep_get_dispatch_layout(const int64_t* topk_idx, int* num_tokens_per_rank,
                              int* num_tokens_per_rdma_rank, int* num_tokens_per_expert,
                              bool* is_token_in_rank, int num_tokens, int num_topk, int num_ranks,
                              int num_experts, void* stream) {
  (void)num_tokens_per_rdma_rank;
  if (!routing_shape_ok(num_tokens, num_topk, num_ranks, num_experts)) return MI_EP_EINVAL;
  if (num_tokens_per_rank == nullptr || num_tokens_per_expert == nullptr) return MI_EP_EINVAL;
  if (num_tokens > 0 && (topk_idx == nullptr || is_token_in_rank == nullptr)) return MI_EP_EINVAL;
  return status_of(launch_layout_counts(topk_idx, num_tokens_per_rank, num_tokens_per_expert,
                                        reinterpret_cast<uint8_t*>(is_token_in_rank), num_tokens,
                                        num_topk, num_ranks, num_experts, as_stream(stream)));
}

size_t mi_ep_workspace_bytes(int num_tokens, int num_topk, int num_experts, int num_ranks) {
  if (!routing_shape_ok(num_tokens, num_topk, num_ranks, num_experts)) return 0;
  const size_t tiles = static_cast<size_t>(num_tiles_for(num_tokens));
  return sizeof(LayoutWorkspace) + tiles * static_cast<size_t>(num_experts + num_ranks) * sizeof(uint64_t);
}

int mi_ep_workspace_init(void* workspace, size_t workspace_bytes, void* stream) {
  const int rc = resolve_workspace(&workspace, &workspace_bytes, as_stream(stream));
  if (rc != MI_EP_OK) return rc;
  if (workspace == nullptr || workspace_bytes < sizeof(LayoutWorkspace)) return MI_EP_EINVAL;
  if ((reinterpret_cast<uintptr_t>(workspace) & 7u) != 0) return MI_EP_EINVAL;
  return status_of(launch_fill_u32(static_cast<uint32_t*>(workspace), workspace_bytes / 4, 0u,
                                   as_stream(stream)));
}

int mi_ep_workspace_set_wait_limit(void* workspace, unsigned int max_polls, void* stream) {
  const int rc = resolve_workspace(&workspace, nullptr, as_stream(stream));
  if (rc != MI_EP_OK) return rc;
  if (workspace == nullptr || (reinterpret_cast<uintptr_t>(workspace) & 7u) != 0) return MI_EP_EINVAL;
  LayoutWorkspace* ws = static_cast<LayoutWorkspace*>(workspace);
  return status_of(launch_fill_u32(&ws->wait_limit, 1, max_polls, as_stream(stream)));
}

int mi_ep_workspace_status(const void* workspace, void* stream) {
  void* ws = const_cast<void*>(workspace);
  const int rc = resolve_workspace(&ws, nullptr, as_stream(stream));
  if (rc != MI_EP_OK) return rc;
  if (ws == nullptr) return MI_EP_EINVAL;
  LayoutWorkspace header;
  hipError_t e = hipMemcpyAsync(&header, ws, sizeof(uint64_t) * 2, hipMemcpyDeviceToHost,
                                as_stream(stream));
  if (e != hipSuccess) return static_cast<int>(e);
  e = hipStreamSynchronize(as_stream(stream));
  if (e != hipSuccess) return static_cast<int>(e);
  return header.timed_out != 0 ? MI_EP_ETIMEDOUT : MI_EP_OK;
}

int mi_ep_device_traits(int* compute_units, int* dies, int* l2_bytes, void* stream) {
  DeviceTraits t{};
  const hipError_t e = device_traits(as_stream(stream), &t);
  if (e != hipSuccess) return static_cast<int>(e);
  if (compute_units != nullptr) *compute_units = t.compute_units;
  if (dies != nullptr) *dies = t.dies;
  if (l2_bytes != nullptr) *l2_bytes = t.l2_bytes;
  return MI_EP_OK;
}

int mi_ep_dispatch_schedule_for(int num_tokens, int num_topk, int num_experts, int row_bytes, int dies,
                                int l2_bytes) {
  if (num_tokens < 0 || num_topk <= 0 || num_topk > MI_EP_MAX_TOPK || num_experts <= 0 ||
      num_experts > MI_EP_MAX_EXPERTS || row_bytes <= 0 || row_bytes % 16 != 0)
    return MI_EP_EINVAL;
  PermuteArgs a{};
  a.num_tokens = num_tokens;
  a.num_topk = num_topk;
  a.num_experts = num_experts;
  a.row_vecs = row_bytes / 16;
  DeviceTraits t{};
  t.dies = dies;
  t.l2_bytes = l2_bytes;
  return destination_order_pays(a, t) ? MI_EP_DISPATCH_BY_DESTINATION : MI_EP_DISPATCH_BY_TOKEN;
}

size_t mi_ep_route_order_bytes(int num_tokens, int num_topk) {
  if (num_tokens <= 0 || num_topk <= 0) return 0;
  return static_cast<size_t>(num_tiles_for(num_tokens)) * kTileTokens * num_topk * 4 * sizeof(int);
}

int mi_ep_dispatch_layout(const int64_t* topk_idx, int num_tokens, int num_topk, int num_ranks,
                          int num_experts, int expert_alignment, int num_channels,
                          int* num_tokens_per_rank, int* num_tokens_per_expert,
                          bool* is_token_in_rank, int* expert_offsets, int* psum_rank_rows,
                          int* channel_prefix_matrix, int* rank_prefix_matrix, int* slot_rel,
                          int* rank_slot_idx, int rank_slot_base, int* route_order, int* tile_rank_counts,
                          int64_t* copied_topk_idx, int* cumulative_expert_stats, void* workspace,
                          size_t workspace_bytes, void* stream) {
  return dispatch_layout_on(topk_idx, num_tokens, num_topk, num_ranks, num_experts, expert_alignment,
                            num_channels, num_tokens_per_rank, num_tokens_per_expert, is_token_in_rank,
                            expert_offsets, psum_rank_rows, channel_prefix_matrix, rank_prefix_matrix,
                            slot_rel, rank_slot_idx,
                            rank_slot_base, route_order, tile_rank_counts, copied_topk_idx,
                            cumulative_expert_stats, workspace, workspace_bytes, false, nullptr, stream);
}

int mi_ep_dispatch_layout_static(const int64_t* topk_idx, int num_tokens, int num_topk, int num_ranks,
                                 int num_experts, int expert_alignment, int num_channels,
                                 int* num_tokens_per_rank, int* num_tokens_per_expert,
                                 bool* is_token_in_rank, int* expert_offsets, int* psum_rank_rows,
                                 int* channel_prefix_matrix, int* rank_prefix_matrix, int* slot_rel,
                                 int* rank_slot_idx, int rank_slot_base, int* route_order,
                                 int* tile_rank_counts, int64_t* copied_topk_idx,
                                 int* cumulative_expert_stats, int* timeout_report, void* stream) {
  // Nothing needs clearing between calls: the scratch starts zeroed when the code object is
  // loaded (an initialised workspace), and every launch leaves the ticket word ready for the
  // next and tags its status words with a fresh generation.
  return dispatch_layout_on(topk_idx, num_tokens, num_topk, num_ranks, num_experts, expert_alignment,
                            num_channels, num_tokens_per_rank, num_tokens_per_expert, is_token_in_rank,
                            expert_offsets, psum_rank_rows, channel_prefix_matrix, rank_prefix_matrix,
                            slot_rel, rank_slot_idx,
                            rank_slot_base, route_order, tile_rank_counts, copied_topk_idx,
                            cumulative_expert_stats, nullptr, 0, true, timeout_report, stream);
}

int mi_ep_dispatch_strided_scales(const void* x, const float* x_scales, long long x_scales_token_stride,
                                  long long x_scales_hidden_stride, const int64_t* topk_idx,
                                  const float* topk_weights, const int* expert_offsets, const int* slot_rel,
                                  const int* route_order, const int* num_tokens_per_expert, int num_tokens,
                                  int num_topk, int num_experts, int expert_alignment, int row_bytes,
                                  int num_scales, void* recv_x, float* recv_scales,
                                  long long recv_scales_token_stride, long long recv_scales_hidden_stride,
                                  int* recv_src_map, int64_t* recv_topk_idx, float* recv_topk_weights,
                                  int* slot_map, int capacity_rows, int flags, void* stream) {
  if (!route_count_ok(num_tokens, num_topk)) return MI_EP_EINVAL;
  if (num_experts <= 0 || num_experts > MI_EP_MAX_EXPERTS || expert_alignment < 1) return MI_EP_EINVAL;
  if (row_bytes <= 0 || row_bytes % 16 != 0 || num_scales < 0 || capacity_rows < 0) return MI_EP_EINVAL;
  if (!fixed::accepts(fixed::kExperts, num_experts) || !fixed::accepts(fixed::kRowBytes, row_bytes)) return MI_EP_EINVAL;
  if (expert_offsets == nullptr || recv_src_map == nullptr) return MI_EP_EINVAL;
  if (capacity_rows > 0 && recv_x == nullptr) return MI_EP_EINVAL;
  if (!aligned16(x) || !aligned16(recv_x) || !aligned16(route_order)) return MI_EP_EINVAL;
  if (num_tokens > 0 &&
      (x == nullptr || topk_idx == nullptr || slot_rel == nullptr || slot_map == nullptr))
    return MI_EP_EINVAL;
  if ((num_scales > 0) != (recv_scales != nullptr)) return MI_EP_EINVAL;
  if (num_scales > 0 && num_tokens > 0 && x_scales == nullptr) return MI_EP_EINVAL;
  if (expert_alignment > 1 && num_tokens_per_expert == nullptr) return MI_EP_EINVAL;
  if ((flags & ~(MI_EP_DISPATCH_ZERO_PAD_PAYLOAD | kScheduleFlags)) != 0) return MI_EP_EINVAL;
  if ((flags & kScheduleFlags) == kScheduleFlags) return MI_EP_EINVAL;  // one copy kernel at most
  if ((flags & MI_EP_DISPATCH_BY_DESTINATION) != 0 && route_order == nullptr && num_tokens > 0)
    return MI_EP_EINVAL;
  if (num_scales > 0 && (x_scales_token_stride < 0 || x_scales_hidden_stride < 0 ||
                         recv_scales_token_stride < 0 || recv_scales_hidden_stride < 0))
    return MI_EP_EINVAL;
  // Pad rows are addressed as expert * (alignment - 1) + index in int.
  if (static_cast<long long>(num_experts) * (expert_alignment - 1) >= (1LL << 30)) return MI_EP_EINVAL;

  PermuteArgs a{};
  a.x = static_cast<const vec16*>(x);
  a.x_scales = x_scales;
  a.topk_idx = topk_idx;
  a.topk_weights = topk_weights;
  a.expert_offsets = expert_offsets;
  a.slot_rel = slot_rel;
  a.route_order = route_order;
  a.num_tokens_per_expert = num_tokens_per_expert;
  a.recv_x = static_cast<vec16*>(recv_x);
  a.recv_scales = recv_scales;
  a.recv_src_map = recv_src_map;
  a.recv_topk_idx = recv_topk_idx;
  a.recv_topk_weights = recv_topk_weights;
  a.slot_map = slot_map;
  a.num_tokens = num_tokens;
  a.num_topk = num_topk;
  a.num_experts = num_experts;
  a.row_vecs = row_bytes / 16;
  a.num_scales = num_scales;
  a.capacity_rows = capacity_rows;
  a.xs_token_stride = x_scales_token_stride;
  a.xs_hidden_stride = x_scales_hidden_stride;
  a.rs_token_stride = recv_scales_token_stride;
  a.rs_hidden_stride = recv_scales_hidden_stride;
  a.expert_alignment = expert_alignment;
  a.zero_pad_payload = (flags & MI_EP_DISPATCH_ZERO_PAD_PAYLOAD) != 0 ? 1 : 0;
  const int schedule = (flags & MI_EP_DISPATCH_BY_TOKEN) != 0         ? kPermuteByToken
                       : (flags & MI_EP_DISPATCH_BY_DESTINATION) != 0 ? kPermuteByDestination
                                                                      : kPermuteAuto;
  return status_of(launch_permute(a, schedule, as_stream(stream)));
}

int mi_ep_dispatch(const void* x, const float* x_scales, const int64_t* topk_idx,
                   const float* topk_weights, const int* expert_offsets, const int* slot_rel,
                   const int* route_order, const int* num_tokens_per_expert, int num_tokens, int num_topk,
                   int num_experts, int expert_alignment, int row_bytes, int num_scales,
                   void* recv_x, float* recv_scales, int* recv_src_map, int64_t* recv_topk_idx,
                   float* recv_topk_weights, int* slot_map, int capacity_rows, int flags,
                   void* stream) {
  return mi_ep_dispatch_strided_scales(x, x_scales, num_scales, 1, topk_idx, topk_weights, expert_offsets,
                                       slot_rel, route_order, num_tokens_per_expert, num_tokens, num_topk,
                                       num_experts, expert_alignment, row_bytes, num_scales, recv_x,
                                       recv_scales, num_scales, 1, recv_src_map, recv_topk_idx,
                                       recv_topk_weights, slot_map, capacity_rows, flags, stream);
}

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
                                        int* psum_rank_tokens, int capacity_rows, void* stream) {
  if (!routing_shape_ok(num_tokens, num_topk, num_ranks, num_experts)) return MI_EP_EINVAL;
  if (row_bytes <= 0 || row_bytes % 16 != 0 || num_scales < 0 || capacity_rows < 0) return MI_EP_EINVAL;
  if (!fixed::accepts(fixed::kRowBytes, row_bytes)) return MI_EP_EINVAL;
  if (num_tokens_per_rank == nullptr || psum_rank_tokens == nullptr) return MI_EP_EINVAL;
  if (capacity_rows > 0 && recv_x == nullptr) return MI_EP_EINVAL;
  if (!aligned16(x) || !aligned16(recv_x)) return MI_EP_EINVAL;
  if (num_tokens > 0 &&
      (x == nullptr || topk_idx == nullptr || rank_slot_idx == nullptr || rank_row_map == nullptr))
    return MI_EP_EINVAL;
  if ((num_scales > 0) != (recv_scales != nullptr)) return MI_EP_EINVAL;
  if (num_scales > 0 && num_tokens > 0 && x_scales == nullptr) return MI_EP_EINVAL;
  if (num_scales > 0 && (x_scales_token_stride < 0 || x_scales_hidden_stride < 0 ||
                         recv_scales_token_stride < 0 || recv_scales_hidden_stride < 0))
    return MI_EP_EINVAL;

  RankPermuteArgs a{};
  a.x = static_cast<const vec16*>(x);
  a.x_scales = x_scales;
  a.topk_idx = topk_idx;
  a.topk_weights = topk_weights;
  a.rank_slot_idx = rank_slot_idx;
  a.num_tokens_per_rank = num_tokens_per_rank;
  a.expand_slot_map = expand_slot_map;
  a.recv_x = static_cast<vec16*>(recv_x);
  a.recv_scales = recv_scales;
  a.recv_topk_idx = recv_topk_idx;
  a.recv_topk_weights = recv_topk_weights;
  a.recv_src_metadata = recv_src_metadata;
  a.rank_row_map = rank_row_map;
  a.combine_map = combine_map;
  a.psum_rank_tokens = psum_rank_tokens;
  a.num_tokens = num_tokens;
  a.num_topk = num_topk;
  a.num_ranks = num_ranks;
  a.num_experts = num_experts;
  a.experts_per_rank = num_experts / num_ranks;
  a.row_vecs = row_bytes / 16;
  a.num_scales = num_scales;
  a.capacity_rows = capacity_rows;
  a.rank_slot_base = rank_slot_base;
  a.source_token_base = source_token_base;
  a.local_expert_ids = local_expert_ids != 0;
  a.xs_token_stride = x_scales_token_stride;
  a.xs_hidden_stride = x_scales_hidden_stride;
  a.rs_token_stride = recv_scales_token_stride;
  a.rs_hidden_stride = recv_scales_hidden_stride;
  return status_of(launch_permute_ranks(a, as_stream(stream)));
}

int mi_ep_dispatch_ranks(const void* x, const float* x_scales, const int64_t* topk_idx,
                         const float* topk_weights, const int* rank_slot_idx, int rank_slot_base,
                         const int* num_tokens_per_rank, const int* expand_slot_map, int num_tokens,
                         int num_topk, int num_ranks, int num_experts, int row_bytes, int num_scales,
                         int source_token_base, int local_expert_ids, void* recv_x, float* recv_scales,
                         int64_t* recv_topk_idx, float* recv_topk_weights, int* recv_src_metadata,
                         int* rank_row_map, int* combine_map, int* psum_rank_tokens, int capacity_rows,
                         void* stream) {
  return mi_ep_dispatch_ranks_strided_scales(
      x, x_scales, num_scales, 1, topk_idx, topk_weights, rank_slot_idx, rank_slot_base, num_tokens_per_rank,
      expand_slot_map, num_tokens, num_topk, num_ranks, num_experts, row_bytes, num_scales, source_token_base,
      local_expert_ids, recv_x, recv_scales, num_scales, 1, recv_topk_idx, recv_topk_weights, recv_src_metadata,
      rank_row_map, combine_map, psum_rank_tokens, capacity_rows, stream);
}

int mi_ep_combine_rank_weights(const float* recv_topk_weights, const int64_t* recv_topk_idx,
                               const int* rank_row_map, int num_tokens, int num_topk, int num_rows,
                               float* combined_topk_weights, int64_t* combined_topk_idx, void* stream) {
  if (!route_count_ok(num_tokens, num_topk) || num_rows < 0) return MI_EP_EINVAL;
  if ((recv_topk_weights != nullptr) != (combined_topk_weights != nullptr)) return MI_EP_EINVAL;
  if ((recv_topk_idx != nullptr) != (combined_topk_idx != nullptr)) return MI_EP_EINVAL;
  if (combined_topk_weights == nullptr && combined_topk_idx == nullptr) return MI_EP_EINVAL;
  if (num_tokens > 0 && rank_row_map == nullptr) return MI_EP_EINVAL;
  return status_of(launch_gather_rank_weights(recv_topk_weights, recv_topk_idx, rank_row_map, num_tokens,
                                              num_topk, num_rows, combined_topk_weights, combined_topk_idx,
                                              as_stream(stream)));
}

int mi_ep_dispatch_cached(const void* x, const float* x_scales, const int* recv_src_map,
                          int num_rows, int num_tokens, int row_bytes, int num_scales,
                          void* recv_x, float* recv_scales, int* ready_counters,
                          int rows_per_counter, void* stream) {
  if (num_rows < 0 || num_tokens < 0 || row_bytes <= 0 || row_bytes % 16 != 0 || num_scales < 0)
    return MI_EP_EINVAL;
  if (!aligned16(x) || !aligned16(recv_x)) return MI_EP_EINVAL;
  if (num_rows > 0 && (recv_src_map == nullptr || recv_x == nullptr)) return MI_EP_EINVAL;
  if (num_rows > 0 && num_tokens > 0 && x == nullptr) return MI_EP_EINVAL;
  if ((num_scales > 0) != (recv_scales != nullptr)) return MI_EP_EINVAL;
  if (num_scales > 0 && num_tokens > 0 && x_scales == nullptr) return MI_EP_EINVAL;
  if (ready_counters != nullptr && rows_per_counter <= 0) return MI_EP_EINVAL;
  return status_of(launch_gather_rows(static_cast<const vec16*>(x), x_scales, recv_src_map, num_rows,
                                      num_tokens, row_bytes / 16, num_scales, static_cast<vec16*>(recv_x),
                                      recv_scales, ready_counters, rows_per_counter, as_stream(stream)));
}

int mi_ep_pull_indices(const int* recv_src_map, int num_rows, int tokens_per_source_rank,
                       int* pull_indices, void* stream) {
  if (num_rows < 0 || tokens_per_source_rank <= 0) return MI_EP_EINVAL;
  if (num_rows > 0 && (recv_src_map == nullptr || pull_indices == nullptr)) return MI_EP_EINVAL;
  if ((reinterpret_cast<uintptr_t>(pull_indices) & 7u) != 0) return MI_EP_EINVAL;
  return status_of(launch_pull_indices(recv_src_map, num_rows, tokens_per_source_rank, pull_indices,
                                       as_stream(stream)));
}

int mi_ep_combine(const void* y, int num_rows, const int* slot_map, const float* topk_weights,
                  const void* bias_0, const void* bias_1, const float* recv_topk_weights,
                  const int64_t* recv_topk_idx, int num_tokens, int num_topk, int hidden,
                  void* combined_x, float* combined_topk_weights, int64_t* combined_topk_idx,
                  int flags, void* stream) {
  if (!route_count_ok(num_tokens, num_topk)) return MI_EP_EINVAL;
  if ((flags & ~MI_EP_COMBINE_STREAM_OUTPUT) != 0) return MI_EP_EINVAL;
  if (hidden <= 0 || hidden % 8 != 0 || num_rows < 0 || !fixed::accepts(fixed::kHidden, hidden)) return MI_EP_EINVAL;
  // Units of the staged schedule are counted in int: rows of a group times 16-byte vectors.
  if (static_cast<long long>(hidden) / 8 >= (1LL << 24)) return MI_EP_EINVAL;
  if (num_rows > 0 && y == nullptr) return MI_EP_EINVAL;
  if ((recv_topk_weights != nullptr) != (combined_topk_weights != nullptr)) return MI_EP_EINVAL;
  if ((recv_topk_idx != nullptr) != (combined_topk_idx != nullptr)) return MI_EP_EINVAL;
  if (num_tokens > 0 && (slot_map == nullptr || combined_x == nullptr)) return MI_EP_EINVAL;
  if (!aligned16(y) || !aligned16(bias_0) || !aligned16(bias_1) || !aligned16(combined_x))
    return MI_EP_EINVAL;

  CombineArgs a{};
  a.y = static_cast<const vec16*>(y);
  a.slot_map = slot_map;
  a.topk_weights = topk_weights;
  a.bias_0 = static_cast<const vec16*>(bias_0);
  a.bias_1 = static_cast<const vec16*>(bias_1);
  a.recv_topk_weights = recv_topk_weights;
  a.recv_topk_idx = recv_topk_idx;
  a.combined_x = static_cast<vec16*>(combined_x);
  a.combined_topk_weights = combined_topk_weights;
  a.combined_topk_idx = combined_topk_idx;
  a.num_tokens = num_tokens;
  a.num_topk = num_topk;
  a.num_rows = num_rows;
  a.row_vecs = hidden / 8;
  a.stream_output = (flags & MI_EP_COMBINE_STREAM_OUTPUT) != 0 ? 1 : 0;
  return status_of(launch_combine(a, as_stream(stream)));
}

int mi_ep_copy_yardstick(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes % 16 != 0 || !aligned16(dst) || !aligned16(src)) return MI_EP_EINVAL;
  if (bytes > 0 && (dst == nullptr || src == nullptr)) return MI_EP_EINVAL;
  return status_of(launch_copy_yardstick(static_cast<vec16*>(dst), static_cast<const vec16*>(src),
                                         bytes / 16, as_stream(stream)));
}

int mi_ep_read_yardstick(const void* src, size_t bytes, void* sink, void* stream) {
  if (bytes % 16 != 0 || !aligned16(src) || sink == nullptr) return MI_EP_EINVAL;
  if (bytes > 0 && src == nullptr) return MI_EP_EINVAL;
  return status_of(launch_read_yardstick(static_cast<const vec16*>(src), bytes / 16,
                                         static_cast<uint32_t*>(sink), as_stream(stream)));
}

int mi_ep_write_yardstick(void* dst, size_t bytes, void* stream) {
  if (bytes % 16 != 0 || !aligned16(dst)) return MI_EP_EINVAL;
  if (bytes > 0 && dst == nullptr) return MI_EP_EINVAL;
  return status_of(launch_write_yardstick(static_cast<vec16*>(dst), bytes / 16, as_stream(stream)));
}

}  // extern "C"
