// Permute (dispatch payload) kernels for gfx950.
//
// Three copies with the same outputs but different orders and formats:
//   ep_permute_tiles_kernel   destination order, for long rows on large batches (further down)
//   ep_permute_kernel         token order, everything else
//   ep_permute_ranks_kernel   one row per (token, destination rank), the reference's own format
// plus the pull-mode gathers and the bandwidth yardsticks.  With expert_alignment > 1 the first two
// also write the pad rows of every segment from extra units of the same launch.
//
// ep_permute_kernel: each wavefront owns (token, batch): one batch is up to
// kBatchVecs * 64 consecutive 16-byte vectors of the token's row (1 KiB as launched).  The wave reads
// its batch once into registers and stores it to every row the token was routed
// to, so the source is read once and every destination row is written once.
// Every access of a wave is 1 KiB contiguous.  The first batch of a token also
// carries the per-row side data: block scales, gate weight, owning expert,
// source token, and the absolute slot map.
// Replaces the payload role of dispatch_impl (example080 .cu:241-256) and the
// expand-mode copy epilogue (example081 .cu:22-60); one partition of this GPU's
// HBM stands where the reference has a peer GPU's receive buffer.
#include <atomic>

#include "ep_device.h"

namespace mi_ep {
namespace {

constexpr int kPermuteThreads = 256;  // pull-mode kernels
constexpr int kPermuteWaves = kPermuteThreads / kWave;
// The push kernel: small workgroups of two waves and one vector per lane measured best on
// every row size tried (7, 8 and 14 KiB rows); the kernel is bound by HBM writes, not by
// occupancy, and finer units even out the tail.
constexpr int kPushThreads = 128;
constexpr int kPushWaves = kPushThreads / kWave;
// The destination-order kernel leans on two facts of the GPU it was tuned on: eight accelerator
// dies that take workgroups round-robin, each with a 4 MiB L2.  A tile's source rows must fit that
// L2 with room for the routing tables; on a device that reports anything else (another partition
// mode, another part) the token-order kernel is used.
constexpr int kDies = 8;
constexpr int kDieL2BytesMin = 4 * 1024 * 1024;
constexpr size_t kTileSourceBytesMax = 3840u * 1024u;
constexpr size_t kRowBytesMin = 4u * 1024u;
constexpr size_t kRowWideBytesMax = 12u * 1024u;  // up to this, one workgroup per route row instead of 2 KiB parts
constexpr int kRunRowsMin = 4;
// The first workgroups of a tile pull its source rows into L2, 4 rows per group of workgroups
// (whole step at 8192 x 14 KiB rows with 32 / 64 / 128 groups: 343.1 / 342.2 / 343 us with the source
// cached, 357.8 / 353.8 / 355.7 us with the source read from HBM).
constexpr int kPrefetchGroups = 64;


// The same pointer in the constant address space: for memory that no thread of the launch writes.
template <typename T>
__device__ __forceinline__ const T __attribute__((address_space(4)))* as_constant(const T* p) {
  return reinterpret_cast<const T __attribute__((address_space(4)))*>(reinterpret_cast<uintptr_t>(p));
}

// Pad rows (expert_alignment > 1): item p stands for possible pad row i = p % (align - 1) of expert
// e = p / (align - 1); it exists when off[e] + count[e] + i is still inside the padded segment and
// the capacity.  Returns the row, or -1.
__device__ __forceinline__ int pad_row_of_item(const PermuteArgs& a, const int item) {
  const int per_expert = a.expert_alignment - 1;
  const int e = item / per_expert;
  if (e >= a.num_experts) return -1;
  const int i = item - e * per_expert;
  const int begin = a.expert_offsets[e] + a.num_tokens_per_expert[e];
  int end = a.expert_offsets[e + 1];
  if (end > a.capacity_rows) end = a.capacity_rows;
  const int row = begin + i;
  return (begin >= 0 && row < end) ? row : -1;
}

// Side data of the pad rows, one item per thread: source -1, expert -1, weight 0, and zero scale
// factors when the payload is zeroed too.  Called by `threads` threads numbered `first`...
__device__ __forceinline__ void write_pad_markers(const PermuteArgs& a, const long long first, const long long threads) {
  const long long items = static_cast<long long>(a.num_experts) * (a.expert_alignment - 1);
  for (long long item = first; item < items; item += threads) {
    const int row = pad_row_of_item(a, static_cast<int>(item));
    if (row < 0) continue;
    a.recv_src_map[row] = -1;
    if (a.recv_topk_idx != nullptr) a.recv_topk_idx[row] = -1;
    if (a.recv_topk_weights != nullptr) a.recv_topk_weights[row] = 0.0f;
    if (a.zero_pad_payload && a.recv_scales != nullptr)
      for (int j = 0; j < a.num_scales; ++j)
        a.recv_scales[static_cast<size_t>(row) * a.rs_token_stride + static_cast<size_t>(j) * a.rs_hidden_stride] = 0.0f;
  }
}

template <int kBatchVecs, bool kStreamStores>
__global__ __launch_bounds__(kPushThreads) void ep_permute_kernel(const PermuteArgs args,
                                                                  const int batches_per_row) {
  const PermuteArgs a = fixed::apply(args);
  const int lane = lane_id();
  const int wave = static_cast<int>(threadIdx.x) >> 6;
  const long long unit = static_cast<long long>(blockIdx.x) * kPushWaves + wave;
  const int token = static_cast<int>(unit / batches_per_row);
  const int batch = static_cast<int>(unit - static_cast<long long>(token) * batches_per_row);
  if (token >= a.num_tokens) {
    if (a.expert_alignment <= 1) return;
    // Units past the last token: first the pad rows' side data (one item per lane), then, when the
    // pads are zeroed, one unit per pad item in row order, so that the fill is a linear stream
    // wherever pad rows are adjacent.
    const long long items = static_cast<long long>(a.num_experts) * (a.expert_alignment - 1);
    const long long marker_units = (items + kWave - 1) / kWave;
    const long long u = unit - static_cast<long long>(a.num_tokens) * batches_per_row;
    if (u < marker_units) {
      write_pad_markers(a, u * kWave + lane, marker_units * kWave);
      return;
    }
    if (!a.zero_pad_payload) return;
    const long long item = u - marker_units;   // one wave per pad item zeroes the whole row
    if (item >= items) return;
    const int row = pad_row_of_item(a, static_cast<int>(item));
    if (row < 0) return;
    const vec16 zero = {0u, 0u, 0u, 0u};
    vec16* dst = a.recv_x + static_cast<size_t>(row) * a.row_vecs;
    for (int v = lane; v < a.row_vecs; v += kWave) __builtin_nontemporal_store(zero, dst + v);
    return;
  }
  const int K = a.num_topk;

  // Payload loads first: they do not depend on the routing data.
  const vec16* src = a.x + static_cast<size_t>(token) * a.row_vecs;
  const int v0 = batch * (kBatchVecs * kWave) + lane;
  vec16 buf[kBatchVecs];
#pragma unroll
  for (int u = 0; u < kBatchVecs; ++u) {
    const int v = v0 + u * kWave;
    if (v < a.row_vecs) buf[u] = src[v];
  }

  // Lane k < K resolves slot k of the token.
  int slot = -1;
  int64_t expert = -1;
  if (lane < K) {
    const size_t i = static_cast<size_t>(token) * K + lane;
    const int rel = a.slot_rel[i];
    expert = a.topk_idx[i];
    if (rel >= 0 && expert >= 0 && expert < static_cast<int64_t>(a.num_experts)) {
      slot = a.expert_offsets[expert] + rel;
      // Beyond the capacity, or negative (tables that are not a finished layout's): dropped, never
      // written.  One unsigned comparison: capacity_rows is not negative.
      if (static_cast<unsigned>(slot) >= static_cast<unsigned>(a.capacity_rows)) slot = -1;
    }
    if (batch == 0) {
      a.slot_map[i] = slot;
      if (slot >= 0) {
        a.recv_src_map[slot] = token;
        if (a.recv_topk_idx != nullptr) a.recv_topk_idx[slot] = expert;
        if (a.recv_topk_weights != nullptr)
          a.recv_topk_weights[slot] = a.topk_weights != nullptr ? a.topk_weights[i] : 1.0f;
      }
    }
  }

  if (batch == 0 && a.recv_scales != nullptr) {
    for (int j = lane; j < a.num_scales; j += kWave) {
      const float s = a.x_scales[static_cast<size_t>(token) * a.xs_token_stride +
                                 static_cast<size_t>(j) * a.xs_hidden_stride];
      for (int k = 0; k < K; ++k) {
        const int row = wave_read(slot, k);
        if (row >= 0)
          a.recv_scales[static_cast<size_t>(row) * a.rs_token_stride + static_cast<size_t>(j) * a.rs_hidden_stride] = s;
      }
    }
  }

#pragma unroll
  for (int k = 0; k < kMaxTopk; ++k) {
    if (k < K) {
      const int row = wave_read(slot, k);
      if (row >= 0) {
        vec16* dst = a.recv_x + static_cast<size_t>(row) * a.row_vecs;
#pragma unroll
        for (int u = 0; u < kBatchVecs; ++u) {
          const int v = v0 + u * kWave;
          if (v < a.row_vecs) {
            if (kStreamStores)
              __builtin_nontemporal_store(buf[u], dst + v);
            else
              dst[v] = buf[u];
          }
        }
      }
    }
  }
}

// The prefetch workgroups of the destination-order kernel (of every die and round, also those
// without a tile) share out the pad rows' side data, one item per thread.
__device__ __forceinline__ void pad_markers_from_prefetch_workgroup(const PermuteArgs& a, const int prefetch_ys,
                                                                    const int rounds) {
  const long long wg = (static_cast<long long>(blockIdx.z) * prefetch_ys + blockIdx.y) * gridDim.x + blockIdx.x;
  write_pad_markers(a, wg * blockDim.x + static_cast<int>(threadIdx.x),
                    static_cast<long long>(rounds) * prefetch_ys * gridDim.x * blockDim.x);
}

// The same copy in destination order.  A tile is the layout kernel's 256 tokens; its
// routes arrive sorted by (expert, position in segment), so consecutive workgroups write
// consecutive rows of recv_x: a tile leaves ~256*K/E adjacent rows per expert, which the
// memory controllers take far better than rows scattered one by one.  Sources are then
// read once per route, K times per token; that only pays because tile j goes to
// accelerator die j % 8 (workgroup b is dispatched to die b % 8: read back from the XCC_ID
// register, every workgroup of a 3-D grid sat on die (linear id) % 8) and a tile's 256 rows
// fit that die's 4 MiB L2, so the repeats never leave the die.  A workgroup copies
// kPushWaves * kVecs KiB of one route's row; part 0 also writes the row's side data.
// Launched as a 3-D grid (x = part of the row * 8 + die, y = entry of the tile's list, z = round
// of eight tiles) so that no index needs a division: a wave moves only 1 KiB, which leaves it
// a budget of about a hundred vector instructions before instruction issue, not HBM, sets the pace.
// kPads: expert_alignment > 1 (pad markers compiled in); kZeroPads: the pad rows' payload is zeroed too (pad
// entries compiled in; callers that leave the pad payload alone get a kernel without them); kScales:
// scale factors travel.
// kRowWide: one workgroup of ceil(row / 1 KiB) waves per route instead of two-wave workgroups that
// each take kVecs KiB-per-wave parts of it: no idle lanes on rows that are not a multiple of the
// part size (kVecs is 1 then and there is one part).
template <int kVecs, bool kPads, bool kZeroPads, bool kScales, bool kRowWide>
__global__ __launch_bounds__(kRowWide ? static_cast<int>(kRowWideBytesMax / sizeof(vec16)) : kPushThreads) void ep_permute_tiles_kernel(const PermuteArgs args,
                                                                                         const int num_tiles,
                                                                                         const int pad_items_per_tile) {
  static_assert(!kRowWide || kVecs == 1, "a row-wide workgroup moves one vector per lane");
  const PermuteArgs a = fixed::apply(args);
  constexpr int prefetch_ys = kPrefetchGroups;
  const int lane = lane_id();
  const int wave = static_cast<int>(threadIdx.x) >> 6;
  const int die = static_cast<int>(blockIdx.x) & (kDies - 1);
  const int part = static_cast<int>(blockIdx.x) >> 3;
  const int tile = static_cast<int>(blockIdx.z) * kDies + die;
  // Everything that is not a route copy returns before the copy's code: dies without a tile in the
  // last round first, then the tile's prefetch workgroups; the pad entries share the exit of entries
  // past the end of the tile's list.  All of it is marked unlikely, so that a route copy runs from
  // the kernel's entry to its stores without a taken branch: a wave lives for about a hundred
  // instructions, and with the pad entries' test and code laid out in its way the same copy took 168
  // to 172 instead of 162 us.
  if (__builtin_expect(tile >= num_tiles, 0)) {  // dies without a tile in the last round
    if (kPads && static_cast<int>(blockIdx.y) < prefetch_ys)
      pad_markers_from_prefetch_workgroup(a, prefetch_ys, (num_tiles + kDies - 1) / kDies);
    return;
  }
  if (__builtin_expect(static_cast<int>(blockIdx.y) < prefetch_ys, 0)) {
    if (kPads) pad_markers_from_prefetch_workgroup(a, prefetch_ys, (num_tiles + kDies - 1) / kDies);
    // The tile's first workgroups pull its source rows into the die's L2 as one linear burst:
    // when the rows come from HBM (not from the memory-side cache) this keeps their reads from
    // being sprinkled over the whole tile, where they would break up the runs of writes
    // (measured at 8192 x 14 KiB rows: 182 us against 208 us; a few us lost when the rows are cached).
    const int v0 = kRowWide ? static_cast<int>(threadIdx.x) : (part * kPushWaves + wave) * (kWave * kVecs) + lane;
    constexpr int rows_per_y = kTileTokens / prefetch_ys;
    const int row0 = tile * kTileTokens + static_cast<int>(blockIdx.y) * rows_per_y;
    // Rows past the last token are clamped to it, so that all loads are issued back to back under
    // one condition and the workgroup lives for one memory round trip, not eight.
    uint32_t fold = 0;
    const int last_row = a.num_tokens - 1;
#pragma unroll
    for (int u = 0; u < kVecs; ++u) {
      const int v = v0 + u * kWave;
      if (v < a.row_vecs) {
        vec16 q[rows_per_y];
#pragma unroll
        for (int i = 0; i < rows_per_y; ++i) {
          const int row = row0 + i < last_row ? row0 + i : last_row;
          q[i] = a.x[static_cast<size_t>(row) * a.row_vecs + v];
        }
#pragma unroll
        for (int i = 0; i < rows_per_y; ++i) fold ^= q[i][0] ^ q[i][1] ^ q[i][2] ^ q[i][3];
      }
    }
    if (fold == 0x9e3779b9u && a.capacity_rows < 0) a.slot_map[0] = -1;  // never true: keeps the loads alive
    return;
  }
  const int entry = static_cast<int>(blockIdx.y) - prefetch_ys;
  const int K = a.num_topk;
  const int tokens_left = a.num_tokens - tile * kTileTokens;
  const int routes = (tokens_left < kTileTokens ? tokens_left : kTileTokens) * K;
  if (__builtin_expect(entry >= routes, 0)) {
    if (kZeroPads && entry >= kTileTokens * K) {
      // Pad entries (only launched when pad rows are zeroed): the possible pad rows are shared out
      // over the tiles in row order, tile j taking items [j * pad_items_per_tile, ...), and follow
      // the tile's routes in its list.  Every workgroup zeroes one whole row; consecutive workgroups
      // of a die take consecutive rows, so the fill is made of runs like the copy's own and joins its
      // write stream instead of trailing it.
      const int parts = static_cast<int>(gridDim.x) >> 3;
      const int index = (entry - kTileTokens * K) * parts + part;
      if (index >= pad_items_per_tile) return;
      const int item = tile * pad_items_per_tile + index;  // below num_tiles * per_tile < items + num_tiles: fits int
      const int row = pad_row_of_item(a, item);
      if (row < 0) return;
      const vec16 zero = {0u, 0u, 0u, 0u};
      vec16* dst = a.recv_x + static_cast<size_t>(row) * a.row_vecs;
      for (int v = static_cast<int>(threadIdx.x); v < a.row_vecs; v += static_cast<int>(blockDim.x))
        __builtin_nontemporal_store(zero, dst + v);
    }
    return;
  }
  const int first_flat = tile * kTileTokens * K;
  // The routing tables are only read here: through the constant address space their (wave-uniform)
  // loads are scalar loads whatever else the kernel stores.
  typedef int route_entry __attribute__((ext_vector_type(4)));
  const route_entry r =
      as_constant(reinterpret_cast<const route_entry*>(a.route_order))[static_cast<size_t>(first_flat) + entry];
  const int flat = __builtin_amdgcn_readfirstlane(r[0]);
  const int expert = __builtin_amdgcn_readfirstlane(r[1]);
  const int rel = __builtin_amdgcn_readfirstlane(r[2]);
  const int token = __builtin_amdgcn_readfirstlane(r[3]);
  // A table that is not this launch's (wrong shape, stale memory) must not send accesses astray.
  if (__builtin_expect(flat < first_flat || flat >= first_flat + routes || token < 0 || token >= a.num_tokens, 0)) return;
  const bool routed = expert >= 0 && expert < a.num_experts && rel >= 0;

  const int v0 = kRowWide ? static_cast<int>(threadIdx.x) : (part * kPushWaves + wave) * (kWave * kVecs) + lane;
  // The two-wave workgroups address the source and destination rows through buffer descriptors one
  // row long (empty when there is nothing to copy): lanes past the row's end and whole non-routes are
  // dropped by the bounds check instead of being branched around (8192 x 14 KiB rows: 166 -> 164.7 us).
  // Row-wide workgroups keep plain guarded accesses: with descriptors they lost 3 % (8192 x 7 KiB rows:
  // 88 -> 90.4 us; 16384 x 8 KiB rows: 179.5 -> 185.7 us).
  const int row_bytes = a.row_vecs * static_cast<int>(sizeof(vec16));
  vec16 buf[kVecs];
  if constexpr (kRowWide) {
#pragma unroll
    for (int u = 0; u < kVecs; ++u) {
      const int v = v0 + u * kWave;
      if (routed && v < a.row_vecs) buf[u] = a.x[static_cast<size_t>(token) * a.row_vecs + v];
    }
  } else {
    const __amdgpu_buffer_rsrc_t source_row = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<vec16*>(a.x + static_cast<size_t>(token) * a.row_vecs), 0, routed ? row_bytes : 0, kRawBufferFormat);
#pragma unroll
    for (int u = 0; u < kVecs; ++u)
      buf[u] = __builtin_amdgcn_raw_buffer_load_b128(source_row, (v0 + u * kWave) * static_cast<int>(sizeof(vec16)), 0, 0);
  }

  int slot = -1;
  if (routed) {
    slot = as_constant(a.expert_offsets)[expert] + rel;
    // One unsigned comparison drops rows beyond the capacity and negative ones alike; written as two
    // signed tests the same check made this kernel 3 % slower.
    if (static_cast<unsigned>(slot) >= static_cast<unsigned>(a.capacity_rows)) slot = -1;
  }
  if (part == 0 && wave == 0) {
    if (lane == 0) {
      a.slot_map[flat] = slot;
      if (slot >= 0) {
        a.recv_src_map[slot] = token;
        if (a.recv_topk_idx != nullptr) a.recv_topk_idx[slot] = expert;
        if (a.recv_topk_weights != nullptr)
          a.recv_topk_weights[slot] = a.topk_weights != nullptr ? a.topk_weights[flat] : 1.0f;
      }
    }
    if (kScales && slot >= 0)
      for (int j = lane; j < a.num_scales; j += kWave)
        a.recv_scales[static_cast<size_t>(slot) * a.rs_token_stride + static_cast<size_t>(j) * a.rs_hidden_stride] =
            a.x_scales[static_cast<size_t>(token) * a.xs_token_stride + static_cast<size_t>(j) * a.xs_hidden_stride];
  }
  if constexpr (kRowWide) {
    if (slot >= 0) {
#pragma unroll
      for (int u = 0; u < kVecs; ++u) {
        const int v = v0 + u * kWave;
        if (v < a.row_vecs)
          __builtin_nontemporal_store(buf[u], a.recv_x + static_cast<size_t>(slot) * a.row_vecs + v);
      }
    }
  } else {
    const __amdgpu_buffer_rsrc_t destination_row = __builtin_amdgcn_make_buffer_rsrc(
        a.recv_x + static_cast<size_t>(slot >= 0 ? slot : 0) * a.row_vecs, 0, slot >= 0 ? row_bytes : 0, kRawBufferFormat);
#pragma unroll
    for (int u = 0; u < kVecs; ++u)
      __builtin_amdgcn_raw_buffer_store_b128(buf[u], destination_row, (v0 + u * kWave) * static_cast<int>(sizeof(vec16)), 0,
                                             kCachePolicyStreaming);
  }
}

template <int kVecs, bool kRowWide>
hipError_t launch_permute_tiles(const PermuteArgs& a, const dim3 grid, const int threads, const int tiles,
                                const int pad_items_per_tile, hipStream_t stream) {
  const bool pads = a.expert_alignment > 1, scales = a.recv_scales != nullptr;
  const bool zero = pads && pad_items_per_tile > 0;
#define MI_EP_LAUNCH_TILES(P, Z, S)                                                                                  \
  hipLaunchKernelGGL((ep_permute_tiles_kernel<kVecs, P, Z, S, kRowWide>), grid, dim3(threads), 0, stream, a, tiles, \
                     pad_items_per_tile)
  if (zero && scales)
    MI_EP_LAUNCH_TILES(true, true, true);
  else if (zero)
    MI_EP_LAUNCH_TILES(true, true, false);
  else if (pads && scales)
    MI_EP_LAUNCH_TILES(true, false, true);
  else if (pads)
    MI_EP_LAUNCH_TILES(true, false, false);
  else if (scales)
    MI_EP_LAUNCH_TILES(false, false, true);
  else
    MI_EP_LAUNCH_TILES(false, false, false);
#undef MI_EP_LAUNCH_TILES
  return hipGetLastError();
}

// Dispatch de-duplicated by destination rank (the reference's own format: payload role of
// dispatch_impl, example080 .cu:241-256, then the copy epilogue without expansion,
// example081 .cu:22-60).  Same wave-per-(token, KiB) shape as ep_permute_kernel; a token's
// destinations are the first slot of each distinct rank, whose position inside the rank's rows
// the layout kernel has already fixed (rank_slot_idx).
__global__ __launch_bounds__(kPushThreads) void ep_permute_ranks_kernel(const RankPermuteArgs args,
                                                                       const int batches_per_row) {
  const RankPermuteArgs a = fixed::apply(args);
  const int lane = lane_id();
  const int wave = static_cast<int>(threadIdx.x) >> 6;
  const long long unit = static_cast<long long>(blockIdx.x) * kPushWaves + wave;
  const int token = static_cast<int>(unit / batches_per_row);
  const int batch = static_cast<int>(unit - static_cast<long long>(token) * batches_per_row);
  if (unit == 0 && lane < a.num_ranks) {  // inclusive rows per rank, for callers that size by it
    int run = 0;
    for (int r = 0; r <= lane; ++r) run += a.num_tokens_per_rank[r];
    a.psum_rank_tokens[lane] = run;
  }
  if (token >= a.num_tokens) return;
  const int K = a.num_topk;

  const vec16* src = a.x + static_cast<size_t>(token) * a.row_vecs;
  const int v = batch * kWave + lane;
  vec16 buf = {0u, 0u, 0u, 0u};
  if (v < a.row_vecs) buf = src[v];

  // First row of every rank: an exclusive scan of the layout's per-rank counts (at most 8 of them).
  int rank_base[kMaxRanks];
  {
    int run = 0;
#pragma unroll
    for (int r = 0; r < kMaxRanks; ++r) {
      rank_base[r] = run;
      if (r < a.num_ranks) run += a.num_tokens_per_rank[r];  // wave-uniform addresses: scalar loads
    }
  }
  // Lane k < K resolves slot k: its rank, and on the first slot of a rank the row it opens.
  const size_t i = static_cast<size_t>(token) * K + (lane < K ? lane : 0);
  int64_t expert = -1;
  int rank = -1, own_row = -1;
  bool opens = false;
  if (lane < K) {
    expert = a.topk_idx[i];
    if (expert >= 0 && expert < static_cast<int64_t>(a.num_experts)) {
      rank = static_cast<int>(expert) / a.experts_per_rank;
      const int slot = a.rank_slot_idx[i];
      opens = slot >= 0;
      if (opens) {
        own_row = rank_base[rank] + (slot - a.rank_slot_base);
        if (static_cast<unsigned>(own_row) >= static_cast<unsigned>(a.capacity_rows)) own_row = -1;  // dropped
      }
    }
  }

  if (batch == 0) {
    // The row that carries each route: the one its rank's first slot opened.
    int route_row = -1;
    for (int j = 0; j < K; ++j) {
      const int rank_j = wave_read(rank, j);
      const int row_j = wave_read(own_row, j);
      const bool opens_j = wave_read(static_cast<int>(opens), j) != 0;
      if (opens_j && rank >= 0 && rank == rank_j) route_row = row_j;
    }
    if (lane < K) {
      a.rank_row_map[i] = route_row;
      if (a.combine_map != nullptr) a.combine_map[i] = own_row;
    }
    const int stride = 2 + K;
    for (int j = 0; j < K; ++j) {
      const int row = wave_read(own_row, j);
      if (row < 0) continue;
      const int rank_j = wave_read(rank, j);
      if (lane < K) {
        const bool local = rank == rank_j;
        const size_t o = static_cast<size_t>(row) * K + lane;
        if (a.recv_topk_idx != nullptr)
          a.recv_topk_idx[o] =
              local ? expert - (a.local_expert_ids ? static_cast<int64_t>(rank_j) * a.experts_per_rank : 0) : -1;
        if (a.recv_topk_weights != nullptr)
          a.recv_topk_weights[o] = local ? (a.topk_weights != nullptr ? a.topk_weights[i] : 1.0f) : 0.0f;
        if (a.recv_src_metadata != nullptr)
          a.recv_src_metadata[static_cast<size_t>(row) * stride + 2 + lane] =
              (local && a.expand_slot_map != nullptr) ? a.expand_slot_map[i] : -1;
      }
      if (lane == 0 && a.recv_src_metadata != nullptr) {
        a.recv_src_metadata[static_cast<size_t>(row) * stride + 0] = a.source_token_base + token;
        a.recv_src_metadata[static_cast<size_t>(row) * stride + 1] = rank_j;
      }
      if (a.recv_scales != nullptr)
        for (int s = lane; s < a.num_scales; s += kWave)
          a.recv_scales[static_cast<size_t>(row) * a.rs_token_stride + static_cast<size_t>(s) * a.rs_hidden_stride] =
              a.x_scales[static_cast<size_t>(token) * a.xs_token_stride + static_cast<size_t>(s) * a.xs_hidden_stride];
    }
  }

#pragma unroll
  for (int j = 0; j < kMaxTopk; ++j) {
    if (j < K) {
      const int row = wave_read(own_row, j);
      if (row >= 0 && v < a.row_vecs)
        __builtin_nontemporal_store(buf, a.recv_x + static_cast<size_t>(row) * a.row_vecs + v);
    }
  }
}

// combined_topk_weights[t,k] / combined_topk_idx[t,k] = the weight / expert id that travelled with
// route (t,k) in the per-rank format (0 / -1 for non-routes).
__global__ __launch_bounds__(256) void ep_gather_rank_weights_kernel(const float* __restrict__ recv_topk_weights,
                                                                    const int64_t* __restrict__ recv_topk_idx,
                                                                    const int* __restrict__ rank_row_map,
                                                                    const int total, const int num_topk,
                                                                    const int num_rows,
                                                                    float* __restrict__ out_weights,
                                                                    int64_t* __restrict__ out_idx) {
  const int i = static_cast<int>(blockIdx.x * blockDim.x + threadIdx.x);
  if (i >= total) return;
  const int row = rank_row_map[i];
  const int k = i % num_topk;
  const bool live = row >= 0 && row < num_rows;
  if (out_weights != nullptr)
    out_weights[i] = live ? recv_topk_weights[static_cast<size_t>(row) * num_topk + k] : 0.0f;
  if (out_idx != nullptr) out_idx[i] = live ? recv_topk_idx[static_cast<size_t>(row) * num_topk + k] : -1;
}

// Pull-mode dispatch: one wave per (destination row, batch).  Destination rows are
// written in order (a linear stream); every source row is read once per route, which
// the caches absorb only in part -- the push kernel above is the fast path, this one
// serves callers that hold nothing but a source map.
template <int kBatchVecs>
__global__ __launch_bounds__(kPermuteThreads) void ep_gather_rows_kernel(
    const vec16* __restrict__ x, const float* __restrict__ x_scales, const int* __restrict__ recv_src_map,
    const int num_rows, const int num_tokens, const int row_vecs, const int num_scales,
    vec16* __restrict__ recv_x, float* __restrict__ recv_scales, const int batches_per_row) {
  const int lane = lane_id();
  const int wave = static_cast<int>(threadIdx.x) >> 6;
  const long long unit = static_cast<long long>(blockIdx.x) * kPermuteWaves + wave;
  const int row = static_cast<int>(unit / batches_per_row);
  const int batch = static_cast<int>(unit - static_cast<long long>(row) * batches_per_row);
  if (row >= num_rows) return;
  const int token = recv_src_map[row];
  const bool live = token >= 0 && token < num_tokens;
  const vec16* src = x + static_cast<size_t>(live ? token : 0) * row_vecs;
  vec16* dst = recv_x + static_cast<size_t>(row) * row_vecs;
  const int v0 = batch * (kBatchVecs * kWave) + lane;
  const vec16 zero = {0u, 0u, 0u, 0u};
  vec16 buf[kBatchVecs];
#pragma unroll
  for (int u = 0; u < kBatchVecs; ++u) {
    const int v = v0 + u * kWave;
    buf[u] = (live && v < row_vecs) ? src[v] : zero;
  }
#pragma unroll
  for (int u = 0; u < kBatchVecs; ++u) {
    const int v = v0 + u * kWave;
    if (v < row_vecs) __builtin_nontemporal_store(buf[u], dst + v);
  }
  if (batch == 0 && recv_scales != nullptr)
    for (int j = lane; j < num_scales; j += kWave)
      recv_scales[static_cast<size_t>(row) * num_scales + j] =
          live ? x_scales[static_cast<size_t>(token) * num_scales + j] : 0.0f;
}

// The same pull with arrival counters: one workgroup per destination row; when the whole row
// (pads included) is in place, ready_counters[row / rows_per_counter] is bumped once, with
// release semantics, so that a consumer that sees a block's counter reach its row count may
// read the block (the per-128-row barrier of the reference's pull dispatch,
// example056 .cu:181-202).
__global__ __launch_bounds__(kPermuteThreads) void ep_gather_rows_ready_kernel(
    const vec16* __restrict__ x, const float* __restrict__ x_scales, const int* __restrict__ recv_src_map,
    const int num_tokens, const int row_vecs, const int num_scales, vec16* __restrict__ recv_x,
    float* __restrict__ recv_scales, int* __restrict__ ready_counters, const int rows_per_counter) {
  const int row = static_cast<int>(blockIdx.x);
  const int tid = static_cast<int>(threadIdx.x);
  const int token = recv_src_map[row];
  const bool live = token >= 0 && token < num_tokens;
  const vec16* src = x + static_cast<size_t>(live ? token : 0) * row_vecs;
  vec16* dst = recv_x + static_cast<size_t>(row) * row_vecs;
  const vec16 zero = {0u, 0u, 0u, 0u};
  for (int v = tid; v < row_vecs; v += kPermuteThreads)
    __builtin_nontemporal_store(live ? src[v] : zero, dst + v);
  if (recv_scales != nullptr)
    for (int j = tid; j < num_scales; j += kPermuteThreads)
      recv_scales[static_cast<size_t>(row) * num_scales + j] =
          live ? x_scales[static_cast<size_t>(token) * num_scales + j] : 0.0f;
  __threadfence();  // every thread's stores are visible device-wide before the barrier
  __syncthreads();
  if (tid == 0)
    __hip_atomic_fetch_add(&ready_counters[row / rows_per_counter], 1, __ATOMIC_RELEASE,
                           __HIP_MEMORY_SCOPE_AGENT);
}

__global__ __launch_bounds__(256) void ep_pull_indices_kernel(const int* __restrict__ recv_src_map,
                                                             const int num_rows,
                                                             const int tokens_per_source_rank,
                                                             int2* __restrict__ pull_indices) {
  const int row = static_cast<int>(blockIdx.x * blockDim.x + threadIdx.x);
  if (row >= num_rows) return;
  const int token = recv_src_map[row];
  int2 out = {-1, -1};
  if (token >= 0) {
    out.x = token / tokens_per_source_rank;
    out.y = token - out.x * tokens_per_source_rank;
  }
  pull_indices[row] = out;
}

__global__ __launch_bounds__(256) void ep_copy_yardstick_kernel(vec16* __restrict__ dst,
                                                               const vec16* __restrict__ src,
                                                               size_t vecs) {
  constexpr int kPerThread = 4;
  const size_t tile = static_cast<size_t>(blockDim.x) * kPerThread;
  const size_t stride = static_cast<size_t>(gridDim.x) * tile;
  for (size_t base = static_cast<size_t>(blockIdx.x) * tile; base < vecs; base += stride) {
    vec16 buf[kPerThread];
#pragma unroll
    for (int u = 0; u < kPerThread; ++u) {
      const size_t v = base + static_cast<size_t>(u) * blockDim.x + threadIdx.x;
      if (v < vecs) buf[u] = __builtin_nontemporal_load(src + v);
    }
#pragma unroll
    for (int u = 0; u < kPerThread; ++u) {
      const size_t v = base + static_cast<size_t>(u) * blockDim.x + threadIdx.x;
      if (v < vecs) __builtin_nontemporal_store(buf[u], dst + v);
    }
  }
}

// Read-only stream: one pass, 4 KiB per workgroup, nothing written (the fold below can
// only equal the magic value by accident of the data, and the store exists so that the
// loads are not dead code).
__global__ __launch_bounds__(256) void ep_read_yardstick_kernel(const vec16* __restrict__ src, size_t vecs,
                                                               uint32_t* sink) {
  constexpr int kPerThread = 4;
  const size_t base = static_cast<size_t>(blockIdx.x) * 256 * kPerThread;
  vec16 buf[kPerThread];
#pragma unroll
  for (int u = 0; u < kPerThread; ++u) {
    const size_t v = base + static_cast<size_t>(u) * 256 + threadIdx.x;
    buf[u] = v < vecs ? __builtin_nontemporal_load(src + v) : vec16{0u, 0u, 0u, 0u};
  }
  uint32_t fold = 0;
#pragma unroll
  for (int u = 0; u < kPerThread; ++u) fold ^= buf[u][0] ^ buf[u][1] ^ buf[u][2] ^ buf[u][3];
  if (fold == 0x9e3779b9u) *sink = fold;
}

// Write-only stream: a fill, 4 KiB per workgroup.
__global__ __launch_bounds__(256) void ep_write_yardstick_kernel(vec16* __restrict__ dst, size_t vecs) {
  const size_t v = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  const vec16 value = {0x01010101u, 0x02020202u, 0x03030303u, 0x04040404u};
  if (v < vecs) dst[v] = value;
}

}  // namespace

hipError_t device_traits(hipStream_t stream, DeviceTraits* out) {
  // Properties of the hardware, read once per device ordinal and never changed afterwards.
  constexpr int kMaxDevices = 64;
  static std::atomic<int> ready[kMaxDevices];
  static DeviceTraits cached[kMaxDevices];
  int dev = 0;
  hipError_t e = stream != nullptr ? hipStreamGetDevice(stream, &dev) : hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  if (ready[dev].load(std::memory_order_acquire) == 0) {
    DeviceTraits t{};
    if (hipDeviceGetAttribute(&t.compute_units, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        t.compute_units <= 0)
      t.compute_units = 256;
    // Unknown values (an attribute this runtime does not report) switch the destination order off.
    if (hipDeviceGetAttribute(&t.dies, hipDeviceAttributeNumberOfXccs, dev) != hipSuccess) t.dies = 0;
    if (hipDeviceGetAttribute(&t.l2_bytes, hipDeviceAttributeL2CacheSize, dev) != hipSuccess) t.l2_bytes = 0;
    (void)hipGetLastError();
    cached[dev] = t;  // racing first calls store the same values
    ready[dev].store(1, std::memory_order_release);
  }
  *out = cached[dev];
  return hipSuccess;
}

// Destination order pays when every die has work in (nearly) every round, a tile's rows fit L2,
// rows are long enough for a workgroup to have something to move and a tile leaves an expert a
// run of several adjacent rows.  Measured against the token-order kernel, whole copy, 8192 tokens,
// 256 experts, top-8: rows of 4 / 5 / 6 / 7 / 8 / 10 / 12 / 14 KiB: -9 / -8 / -10 / -10 / -13 / -6 / -9 /
// -11 % (2 KiB rows: +11 %; 16 KiB rows, whose tile no longer fits: -4 %); within five points of that
// at 4096 tokens and at 16384 tokens with 128 experts, where 16 KiB rows gain nothing.
bool destination_order_pays(const PermuteArgs& a, const DeviceTraits& dev) {
  // The die mapping and the L2 budget are built into the kernel: any other device takes the token order.
  if (dev.dies != kDies || dev.l2_bytes < kDieL2BytesMin) return false;
  const int tiles = (a.num_tokens + kTileTokens - 1) / kTileTokens;
  const int rounds = (tiles + kDies - 1) / kDies;
  if (tiles * 8 < rounds * kDies * 7) return false;  // more than 1/8 of the die-rounds idle
  const size_t row_bytes = static_cast<size_t>(a.row_vecs) * sizeof(vec16);
  if (kTileTokens * row_bytes > kTileSourceBytesMax) return false;
  if (row_bytes < kRowBytesMin) return false;
  return kTileTokens * a.num_topk >= kRunRowsMin * a.num_experts;  // expected rows per (tile, expert)
}

hipError_t launch_permute(const PermuteArgs& args, int schedule, hipStream_t stream) {
  const PermuteArgs a = fixed::apply(args);
  const long long pad_items = a.expert_alignment > 1 ? static_cast<long long>(a.num_experts) * (a.expert_alignment - 1) : 0;
  if (a.num_tokens == 0 && pad_items == 0) return hipSuccess;
  bool by_destination = a.num_tokens > 0 && a.route_order != nullptr && schedule == kPermuteByDestination;
  if (a.num_tokens > 0 && a.route_order != nullptr && schedule == kPermuteAuto) {
    DeviceTraits dev{};
    const hipError_t e = device_traits(stream, &dev);
    if (e != hipSuccess) return e;
    by_destination = destination_order_pays(a, dev);
  }
  if (by_destination) {
    const int tiles = (a.num_tokens + kTileTokens - 1) / kTileTokens;
    const int rounds = (tiles + kDies - 1) / kDies;
    // Long rows: 2 KiB per workgroup, seven workgroups on a 14 KiB row.  Rows up to 12 KiB do better
    // with one workgroup of ceil(row / 1 KiB) waves each (measured at 8192 tokens, 5 / 6 / 7 / 8 / 10 /
    // 12 KiB rows: 63 / 75 / 88 / 93 / 122 / 140 us against 66 / 81 / 95 / 96 / 126 / 143 us; 14 KiB
    // rows: 170 against 166 us).
    const bool row_wide = static_cast<size_t>(a.row_vecs) * sizeof(vec16) <= kRowWideBytesMax;
    const int per_workgroup = row_wide ? static_cast<int>(kRowWideBytesMax / sizeof(vec16)) : kPushWaves * kWave;
    const int parts = (a.row_vecs + per_workgroup - 1) / per_workgroup;
    const int prefetch_ys = kPrefetchGroups;
    // Zeroed pads: extra entries behind every tile's routes, one possible pad row per workgroup.
    int ys = kTileTokens * a.num_topk + prefetch_ys;
    int pad_items_per_tile = 0;
    if (pad_items > 0 && a.zero_pad_payload) {
      pad_items_per_tile = static_cast<int>((pad_items + tiles - 1) / tiles);
      ys += (pad_items_per_tile + parts - 1) / parts;
    }
    // A grid that does not fit the launch limits (over 16 million tokens, or millions of pad rows to
    // zero per tile) is left to the token-order kernel below: the outputs are the same.
    if (rounds <= 65535 && ys <= 65535 && parts * kDies <= 65535) {
      const dim3 grid(static_cast<unsigned>(parts * kDies), static_cast<unsigned>(ys), static_cast<unsigned>(rounds));
      if (row_wide)
        return launch_permute_tiles<1, true>(a, grid, (a.row_vecs + kWave - 1) / kWave * kWave, tiles, pad_items_per_tile, stream);
      return launch_permute_tiles<1, false>(a, grid, kPushThreads, tiles, pad_items_per_tile, stream);
    }
  }
  const int batches = (a.row_vecs + kWave - 1) / kWave;
  long long units = static_cast<long long>(a.num_tokens) * batches;
  if (pad_items > 0) {
    units += (pad_items + kWave - 1) / kWave;             // side data of the pad rows, one item per lane
    if (a.zero_pad_payload) units += pad_items;            // their payload, one unit per possible pad row
  }
  const long long blocks = (units + kPushWaves - 1) / kPushWaves;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL((ep_permute_kernel<1, true>), dim3(static_cast<unsigned>(blocks)), dim3(kPushThreads), 0,
                     stream, a, batches);
  return hipGetLastError();
}

hipError_t launch_permute_ranks(const RankPermuteArgs& args, hipStream_t stream) {
  const RankPermuteArgs a = fixed::apply(args);
  const int batches = (a.row_vecs + kWave - 1) / kWave;
  // At least one unit, so that the per-rank row totals are written for an empty batch too.
  const long long units = a.num_tokens > 0 ? static_cast<long long>(a.num_tokens) * batches : 1;
  const long long blocks = (units + kPushWaves - 1) / kPushWaves;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(ep_permute_ranks_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kPushThreads), 0, stream,
                     a, batches);
  return hipGetLastError();
}

hipError_t launch_gather_rank_weights(const float* recv_topk_weights, const int64_t* recv_topk_idx,
                                      const int* rank_row_map, int num_tokens, int num_topk, int num_rows,
                                      float* combined_topk_weights, int64_t* combined_topk_idx,
                                      hipStream_t stream) {
  const long long total = static_cast<long long>(num_tokens) * num_topk;
  if (total == 0) return hipSuccess;
  hipLaunchKernelGGL(ep_gather_rank_weights_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                     stream, recv_topk_weights, recv_topk_idx, rank_row_map, static_cast<int>(total), num_topk,
                     num_rows, combined_topk_weights, combined_topk_idx);
  return hipGetLastError();
}

hipError_t launch_gather_rows(const vec16* x, const float* x_scales, const int* recv_src_map, int num_rows,
                              int num_tokens, int row_vecs, int num_scales, vec16* recv_x,
                              float* recv_scales, int* ready_counters, int rows_per_counter,
                              hipStream_t stream) {
  if (num_rows == 0) return hipSuccess;
  if (ready_counters != nullptr) {
    hipLaunchKernelGGL(ep_gather_rows_ready_kernel, dim3(static_cast<unsigned>(num_rows)),
                       dim3(kPermuteThreads), 0, stream, x, x_scales, recv_src_map, num_tokens, row_vecs,
                       num_scales, recv_x, recv_scales, ready_counters, rows_per_counter);
    return hipGetLastError();
  }
  const int batch_vecs = row_vecs > kWave ? 2 : 1;
  const int per_batch = batch_vecs * kWave;
  const int batches = (row_vecs + per_batch - 1) / per_batch;
  const long long units = static_cast<long long>(num_rows) * batches;
  const long long blocks = (units + kPermuteWaves - 1) / kPermuteWaves;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  if (batch_vecs == 2)
    hipLaunchKernelGGL((ep_gather_rows_kernel<2>), dim3(static_cast<unsigned>(blocks)), dim3(kPermuteThreads), 0,
                       stream, x, x_scales, recv_src_map, num_rows, num_tokens, row_vecs, num_scales, recv_x,
                       recv_scales, batches);
  else
    hipLaunchKernelGGL((ep_gather_rows_kernel<1>), dim3(static_cast<unsigned>(blocks)), dim3(kPermuteThreads), 0,
                       stream, x, x_scales, recv_src_map, num_rows, num_tokens, row_vecs, num_scales, recv_x,
                       recv_scales, batches);
  return hipGetLastError();
}

hipError_t launch_pull_indices(const int* recv_src_map, int num_rows, int tokens_per_source_rank,
                               int* pull_indices, hipStream_t stream) {
  if (num_rows == 0) return hipSuccess;
  hipLaunchKernelGGL(ep_pull_indices_kernel, dim3((num_rows + 255) / 256), dim3(256), 0, stream, recv_src_map,
                     num_rows, tokens_per_source_rank, reinterpret_cast<int2*>(pull_indices));
  return hipGetLastError();
}

hipError_t launch_copy_yardstick(vec16* dst, const vec16* src, size_t vecs, hipStream_t stream) {
  if (vecs == 0) return hipSuccess;
  size_t blocks = (vecs + 1023) / 1024;
  if (blocks > 8192) blocks = 8192;
  hipLaunchKernelGGL(ep_copy_yardstick_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                     dst, src, vecs);
  return hipGetLastError();
}

hipError_t launch_read_yardstick(const vec16* src, size_t vecs, uint32_t* sink, hipStream_t stream) {
  if (vecs == 0) return hipSuccess;
  const size_t blocks = (vecs + 1023) / 1024;
  if (blocks > 0x7fffffffULL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(ep_read_yardstick_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, src,
                     vecs, sink);
  return hipGetLastError();
}

hipError_t launch_write_yardstick(vec16* dst, size_t vecs, hipStream_t stream) {
  if (vecs == 0) return hipSuccess;
  const size_t blocks = (vecs + 255) / 256;
  if (blocks > 0x7fffffffULL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(ep_write_yardstick_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, dst,
                     vecs);
  return hipGetLastError();
}

}  // namespace mi_ep
