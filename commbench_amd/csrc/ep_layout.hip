// Layout kernels for gfx950.
//
// ep_layout_fused_kernel: one pass over topk_idx that yields per-expert counts,
// de-duplicated per-rank counts, is_token_in_rank, aligned exclusive expert
// offsets, inclusive per-partition rows, per-channel inclusive prefixes and the
// deterministic position of every route inside its expert segment.  It replaces
// the reference's layout kernel (example042 .cu:48-86), the notify role of
// dispatch_impl (example080 .cu:78-240), the deterministic prologue
// (example078 .cu:27-43) and the channel half of notify_dispatch
// (example047 .cu:132-143).
//
// Shape of the computation (wave64):
//   * a tile is 256 tokens = 256*K routes, owned by one 1024-thread workgroup;
//     one fetch-add per tile on the workspace's turn word returns the launch's
//     generation and an arrival number, and the last arrival resets the word.
//     Large grids take the arrival number as their tile, so that every tile's
//     predecessors have already started and the look-back below cannot wait on a
//     workgroup that is not resident; small grids (a tile per eight compute
//     units at most) take workgroup b = tile b and need the fetch-add's answer
//     only when they publish;
//   * the workgroup is 16 waves; each walks its share of the tile's 4*K chunks
//     of 64 routes in (token, slot) order;
//     lanes holding the same expert find each other with log2(E) ballots, the
//     lowest such lane bumps the wave's private LDS counter once, and every lane
//     derives its rank among equals with a popcount -- no LDS atomics, so routing
//     skew costs nothing;
//   * columns (E experts followed by R ranks) are scanned across tiles in a single
//     pass over 64-bit status words {flag:2 | generation:30 | value:32}; the
//     generation tag makes the words of earlier launches invalid without any
//     clearing pass.  Small grids (the last tile's predecessors amount to at most
//     kGatherLimitWords words) publish two 16-bit column totals per word and every
//     tile fetches all its predecessors' rows at once, as one contiguous run read
//     with 16-byte loads by the whole workgroup and summed with LDS adds; larger
//     grids publish one column per word and walk back column by column (decoupled
//     look-back: aggregates until a tile's inclusive prefix is met);
//   * the last tile knows every column total and emits counts and the aligned
//     offsets.
//
// ep_layout_counts_kernel: the workspace-free variant behind the reference's
// DeepepDispatchLayout::compute signature (counts and flags only).
#include "ep_device.h"

namespace mi_ep {
namespace {

constexpr uint32_t kFlagAggregate = 1;
constexpr uint32_t kFlagPrefix = 2;
constexpr uint32_t kGenMask = 0x3fffffffu;
constexpr int kLookbackWindow = 32;
constexpr int kTimedOutCode = -110;  // MI_EP_ETIMEDOUT of the C ABI
constexpr int kCountsThreads = 1024;  // the counts-only kernel: one token per thread, 16 waves

__device__ __forceinline__ uint64_t pack_status(uint32_t flag, uint32_t gen, uint32_t value) {
  return (static_cast<uint64_t>(flag) << 62) | (static_cast<uint64_t>(gen & kGenMask) << 32) |
         static_cast<uint64_t>(value);
}
__device__ __forceinline__ uint32_t pack_pair(int first, int second) {
  return (static_cast<uint32_t>(first) & 0xffffu) | (static_cast<uint32_t>(second) << 16);
}
__device__ __forceinline__ void publish(uint64_t* p, uint64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t peek(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Lanes of the wave that hold the same valid expert as this lane (including it).
// Executed by all lanes; the result is meaningful only where `valid`.
__device__ __forceinline__ uint64_t match_expert(bool valid, int e, int expert_bits) {
  uint64_t mask = __ballot(valid);
  for (int b = 0; b < expert_bits; ++b) {
    const bool bit = ((e >> b) & 1) != 0;
    const uint64_t with_bit = __ballot(valid && bit);
    mask &= bit ? with_bit : ~with_bit;
  }
  return mask;
}

// The arguments with top-k, the expert count and the rank count replaced by compile-time constants
// (0: left as given).
template <int kTopk, int kExperts, int kRanks>
__device__ __forceinline__ LayoutArgs with_shapes(LayoutArgs a) {
  if constexpr (kTopk != 0) {
    a.num_topk = kTopk;
    a.inv_topk = ((1u << 19) + kTopk - 1) / kTopk;
  }
  if constexpr (kExperts != 0) {
    a.num_experts = kExperts;
    int bits = 1;
    while ((1 << bits) < kExperts) ++bits;
    a.expert_bits = bits;
  }
  if constexpr (kRanks != 0) a.num_ranks = kRanks;
  if constexpr (kExperts != 0 && kRanks != 0) {
    a.experts_per_rank = kExperts / kRanks;
    a.inv_experts_per_rank = ((1u << 22) + kExperts / kRanks - 1) / (kExperts / kRanks);
  }
  return a;
}

__device__ __forceinline__ void store_token_flags(uint8_t* is_token_in_rank, int token,
                                                  int num_ranks, uint64_t flags) {
  uint8_t* dst = is_token_in_rank + static_cast<size_t>(token) * num_ranks;
  if (num_ranks == 8 && (reinterpret_cast<uintptr_t>(is_token_in_rank) & 7u) == 0) {
    *reinterpret_cast<uint64_t*>(dst) = flags;
  } else if (num_ranks == 4 && (reinterpret_cast<uintptr_t>(is_token_in_rank) & 3u) == 0) {
    *reinterpret_cast<uint32_t*>(dst) = static_cast<uint32_t>(flags);
  } else {
    for (int r = 0; r < num_ranks; ++r) dst[r] = static_cast<uint8_t>((flags >> (8 * r)) & 1u);
  }
}

// kTopk / kExperts / kRanks: that shape as a constant (0: taken from the arguments).  The launcher
// picks an instantiation for the shapes it knows; the chunk loops, the ballots of match_expert and
// the multiply-shift divisions then unroll and fold (32 tiles, top-8 over 256 experts on 8 ranks:
// 9.3 us with run-time shapes, 8.7 with the expert count fixed, 8.2 with all three).
template <int kTopk, int kExperts, int kRanks>
__global__ __launch_bounds__(kLayoutThreads) void ep_layout_fused_kernel(const LayoutArgs args) {
  const LayoutArgs a = with_shapes<kTopk, kExperts, kRanks>(fixed::apply(args));
  extern __shared__ int smem[];
  const int E = a.num_experts, R = a.num_ranks, K = a.num_topk, T = a.num_tokens;
  const int cols = E + R;
  int* col_total = smem;                    // [cols] this tile's total per column
  int* col_excl = col_total + cols;         // [cols] sum over earlier tiles
  int* wave_sums = col_excl + cols;         // [kLayoutWaves]
  int* misc = wave_sums + kLayoutWaves;     // [4] tile, generation, wait limit
  int* rank_wave = misc + 4;                // [kTileTokens / kWave][kMaxRanks] flagged tokens per wave
  int* order_sums = rank_wave + (kTileTokens / kWave) * kMaxRanks;  // [kLayoutWaves] scan of the tile's counts
  int* masked_wave = order_sums + kLayoutWaves;                      // [kLayoutWaves] non-routes per wave
  int* offs = masked_wave + kLayoutWaves;   // [E + 2] per-expert bases: of the tile's route order, then of the segments
  uint64_t* tok_flags = reinterpret_cast<uint64_t*>(offs + E + 2 + (E & 1));  // [kTileTokens], byte r = rank r
  uint16_t* hist = reinterpret_cast<uint16_t*>(tok_flags + kTileTokens);  // [kLayoutWaves][E] wave-private

  const int tid = static_cast<int>(threadIdx.x);
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  uint64_t* status = reinterpret_cast<uint64_t*>(a.ws + 1);
  // Small grids pack two columns into a status word: experts first, then ranks.
  const int expert_words = (E + 1) >> 1;
  const int row_words = expert_words + ((R + 1) >> 1);

  // ---- routes: the tile's 256*K routes are 4*K chunks of 64 in (token, slot)
  // order; wave w owns chunks [w * per_wave, (w + 1) * per_wave).
  const int flat_end = T * K;
  const int num_chunks = (kTileTokens / kWave) * K;
  const int per_wave = (num_chunks + kLayoutWaves - 1) / kLayoutWaves;  // <= kChunksPerWave
  int64_t raw[kChunksPerWave];
  auto load_routes = [&](const int of_tile) {
#pragma unroll
    for (int c = 0; c < kChunksPerWave; ++c) {
      raw[c] = -1;
      const int chunk = wave * per_wave + c;
      if (c < per_wave && chunk < num_chunks) {
        const int g = of_tile * (kTileTokens * K) + chunk * kWave + lane;
        if (g < flat_end) {
          raw[c] = a.topk_idx[g];
          if (a.copied_topk_idx != nullptr) a.copied_topk_idx[g] = raw[c];
        }
      }
    }
  };

  // One fetch-add per tile on the workspace's turn word: its high half is the launch's generation,
  // its low half counts arrivals; the last arrival hands the workspace to the next launch.  The
  // arrival number is also the tile unless tiles are static; then nothing needs the fetch-add's
  // answer before the aggregates are published, so it travels while the routes are fetched and
  // ranked, and thread 0 hands the generation out just before the barrier that ends the ranking.
  uint64_t turn = 0;
  uint32_t limit = 0;
  if (tid == 0) {
    turn = __hip_atomic_fetch_add(&a.ws->turn, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    limit = a.ws->wait_limit;
  }
  auto hand_out = [&]() {
    if (tid == 0) {
      const uint32_t ticket = static_cast<uint32_t>(turn);
      const uint32_t generation = static_cast<uint32_t>(turn >> 32) & kGenMask;
      misc[0] = static_cast<int>(ticket);
      misc[1] = static_cast<int>(generation);
      misc[2] = static_cast<int>(limit != 0 ? limit : kDefaultWaitLimit);
      if (ticket == static_cast<uint32_t>(a.num_tiles) - 1u)
        __hip_atomic_store(&a.ws->turn, static_cast<uint64_t>((generation + 1u) & kGenMask) << 32,
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  };
  if (a.static_tiles)
    load_routes(static_cast<int>(blockIdx.x));
  else
    hand_out();
  {
    uint32_t* hist_words = reinterpret_cast<uint32_t*>(hist);
    for (int i = tid; i < (kLayoutWaves * E + 1) / 2; i += kLayoutThreads) hist_words[i] = 0;
  }
  if (tid < kTileTokens) tok_flags[tid] = 0;
  if (a.gather_rows)  // the gathered look-back adds into these
    for (int i = tid; i < cols; i += kLayoutThreads) col_excl[i] = 0;
  __syncthreads();

  const int tile = a.static_tiles ? static_cast<int>(blockIdx.x) : misc[0];
  if (tile >= a.num_tiles) return;  // stale ticket: never with an initialised workspace
  const int t0 = tile * kTileTokens;
  const int flat0 = t0 * K;
  uint16_t* my_hist = hist + wave * E;
  if (!a.static_tiles) load_routes(tile);

  int my_e[kChunksPerWave];
  int my_pos[kChunksPerWave];  // rank among the wave's earlier routes to the same expert (among its non-routes if masked)
  int masked_seen = 0;
#pragma unroll
  for (int c = 0; c < kChunksPerWave; ++c) {
    my_e[c] = -1;
    my_pos[c] = 0;
    const int chunk = wave * per_wave + c;
    if (c < per_wave && chunk < num_chunks) {  // wave-uniform
      const int local = chunk * kWave + lane;  // < 256 * K <= 2048
      const int64_t e64 = raw[c];
      const bool valid = e64 >= 0 && e64 < static_cast<int64_t>(E);
      const int e = valid ? static_cast<int>(e64) : 0;
      const uint64_t same = match_expert(valid, e, a.expert_bits);
      const bool masked = !valid && flat0 + local < flat_end;
      const uint64_t masked_lanes = __ballot(masked);
      if (masked) my_pos[c] = masked_seen + __popcll(masked_lanes & lanes_below(lane));
      masked_seen += __popcll(masked_lanes);
      int old = 0, below = 0;
      if (valid) {
        below = __popcll(same & lanes_below(lane));
        old = my_hist[e];
        my_e[c] = e;
        my_pos[c] = old + below;
        // local / K and e / experts_per_rank by multiply-shift (exact on these ranges)
        const int token_local = static_cast<int>((static_cast<uint32_t>(local) * a.inv_topk) >> 19);
        const int rank = static_cast<int>((static_cast<uint32_t>(e) * a.inv_experts_per_rank) >> 22);
        reinterpret_cast<uint8_t*>(tok_flags + token_local)[rank] = 1;
      }
      __builtin_amdgcn_wave_barrier();
      if (valid && below == 0) my_hist[e] = static_cast<uint16_t>(old + __popcll(same));
      __builtin_amdgcn_wave_barrier();
    }
  }
  if (lane == 0) masked_wave[wave] = masked_seen;
  if (a.static_tiles) hand_out();
  __syncthreads();
  const uint32_t gen = static_cast<uint32_t>(misc[1]);
  const uint32_t wait_limit = static_cast<uint32_t>(misc[2]);

  // ---- every column's aggregate is published as early as possible: the status words need a
  // microsecond or two to become visible to the other tiles, and a look-back that polls before
  // its predecessors' words have landed pays a whole extra round trip.  Everything that does not
  // need the look-back's result runs between the publication and the first poll.
  // Expert columns (thread e < E): wave bases, tile total, aggregate out.
  int my_col_total = 0;  // thread e < E: this tile's routes to expert e
  for (int col = tid; col < E; col += kLayoutThreads) {
    // All reads before the first write: as one read-modify-write chain the sixteen LDS round trips
    // would run one after the other.
    int v[kLayoutWaves];
#pragma unroll
    for (int w = 0; w < kLayoutWaves; ++w) v[w] = hist[w * E + col];
    int total = 0;
#pragma unroll
    for (int w = 0; w < kLayoutWaves; ++w) {
      hist[w * E + col] = static_cast<uint16_t>(total);  // becomes the wave's base inside the tile
      total += v[w];
    }
    col_total[col] = total;
    my_col_total = total;
    if (a.gather_rows) {
      // Two columns per word (a tile holds at most 256 * 8 routes, so 16 bits each): the even
      // lane takes its neighbour's total and publishes for both.
      const int neighbour = __builtin_amdgcn_update_dpp(0, total, 0x101, 0xf, 0xf, false);  // row_shl:1
      if ((col & 1) == 0)
        publish(status + static_cast<size_t>(tile) * row_words + (col >> 1),
                pack_status(kFlagAggregate, gen, pack_pair(total, col + 1 < E ? neighbour : 0)));
    } else {
      publish(status + static_cast<size_t>(tile) * cols + col,
              pack_status(tile == 0 ? kFlagPrefix : kFlagAggregate, gen, static_cast<uint32_t>(total)));
    }
  }
  // Exclusive scan of the tile's per-expert counts (one expert per thread): where each expert's
  // routes start in the tile's route order.  The cross-wave half follows the next barrier.
  int order_incl = my_col_total;
  if (a.route_order != nullptr) {
    order_incl = wave_inclusive_scan(my_col_total);
    if (lane == kWave - 1) order_sums[wave] = order_incl;
  }
  // Rank hits, de-duplicated per token: one token per thread of waves 4..7 (the waves next to the
  // ones that hold the expert columns of up to 256 experts).  below_packed, byte r: flagged tokens
  // of rank r in this wave before this token, kept for the slot table after the look-back.  The
  // token's ids for that table are fetched here and folded into four bits per slot further down,
  // so that little state stays in registers across the look-back.
  const int ftid = tid - kTileTokens;           // token of the tile, on the flag threads
  const bool flag_thread = ftid >= 0 && ftid < kTileTokens;
  const int fwave = ftid >> 6;                  // 0..3 on the flag threads
  uint64_t my_flags = 0, below_packed = 0;
  int64_t my_ids[kMaxTopk];
#pragma unroll
  for (int k = 0; k < kMaxTopk; ++k) my_ids[k] = -1;
  if (flag_thread) {  // whole waves
    if (a.rank_slot_idx != nullptr && t0 + ftid < T) {
#pragma unroll
      for (int k = 0; k < kMaxTopk; ++k)
        if (k < K) my_ids[k] = a.topk_idx[static_cast<size_t>(t0 + ftid) * K + k];
    }
    my_flags = tok_flags[ftid];
#pragma unroll
    for (int r = 0; r < kMaxRanks; ++r) {
      const uint64_t hit = __ballot(r < R && ((my_flags >> (8 * r)) & 1u) != 0);
      below_packed |= static_cast<uint64_t>(__popcll(hit & lanes_below(lane))) << (8 * r);
      if (lane == 0) rank_wave[fwave * kMaxRanks + r] = __popcll(hit);
    }
  }
  __syncthreads();

  // Rank columns (thread r < R): the tile's total out.
  if (tid < R) {
    int total = 0;
#pragma unroll
    for (int w = 0; w < kTileTokens / kWave; ++w) total += rank_wave[w * kMaxRanks + tid];
    col_total[E + tid] = total;
    if (a.gather_rows) {
      const int neighbour = __builtin_amdgcn_update_dpp(0, total, 0x101, 0xf, 0xf, false);  // row_shl:1
      if ((tid & 1) == 0)
        publish(status + static_cast<size_t>(tile) * row_words + expert_words + (tid >> 1),
                pack_status(kFlagAggregate, gen, pack_pair(total, tid + 1 < R ? neighbour : 0)));
    } else {
      publish(status + static_cast<size_t>(tile) * cols + E + tid,
              pack_status(tile == 0 ? kFlagPrefix : kFlagAggregate, gen, static_cast<uint32_t>(total)));
    }
    if (a.tile_rank_counts != nullptr) a.tile_rank_counts[static_cast<size_t>(tile) * R + tid] = total;
  }
  // In the shadow of the publication: the flags go out and the cross-wave half of the route-order
  // scan is folded in.
  if (flag_thread && t0 + ftid < T) store_token_flags(a.is_token_in_rank, t0 + ftid, R, my_flags);
  int masked_base = 0;  // where this wave's non-routes start in the tile's route order
  if (a.route_order != nullptr) {
    // Unconditional reads, selected afterwards, so that they are issued together.
    int sums[kLayoutWaves], masked[kLayoutWaves];
#pragma unroll
    for (int w = 0; w < kLayoutWaves; ++w) {
      sums[w] = order_sums[w];
      masked[w] = masked_wave[w];
    }
    int base = order_incl - my_col_total;
#pragma unroll
    for (int w = 0; w < kLayoutWaves; ++w) {
      base += (w < wave) ? sums[w] : 0;
      masked_base += sums[w] + ((w < wave) ? masked[w] : 0);  // every route of the tile comes first
    }
    if (tid < E) offs[tid] = base;
  }
  __syncthreads();

  // Each route's place inside the tile (needs the wave bases and the scan, not the look-back).
  int in_tile[kChunksPerWave], order_pos[kChunksPerWave];
#pragma unroll
  for (int c = 0; c < kChunksPerWave; ++c) {
    const int e = my_e[c];
    in_tile[c] = (e >= 0) ? my_hist[e] + my_pos[c] : 0;
    order_pos[c] = (a.route_order == nullptr) ? 0 : (e >= 0) ? offs[e] + in_tile[c] : masked_base + my_pos[c];
  }

  // Slot k of the token opens a row of rank r when it is the first slot that reaches r: nibble k
  // of first_ranks holds 8 | r then, 0 otherwise.
  uint32_t first_ranks = 0;
  if (flag_thread && a.rank_slot_idx != nullptr) {
    uint32_t seen = 0;
#pragma unroll
    for (int k = 0; k < kMaxTopk; ++k) {
      const int64_t e64 = my_ids[k];
      if (k < K && e64 >= 0 && e64 < static_cast<int64_t>(E)) {
        const uint32_t rank = (static_cast<uint32_t>(e64) * a.inv_experts_per_rank) >> 22;
        if (((seen >> rank) & 1u) == 0) {
          seen |= 1u << rank;
          first_ranks |= (8u | rank) << (4 * k);
        }
      }
    }
  }

  // ---- small grids: every predecessor's row gathered at once ---------------------
  // The rows of tiles 0 .. tile-1 are one contiguous run of tile * row_words status words.  The
  // whole workgroup fetches it, two words (four columns) per lane and load, and adds what it finds
  // to the columns' sums in LDS: a tile with 31 predecessors issues two loads per wave where a
  // column-per-thread walk issues 31, and a device-scope load costs by the instruction, not by
  // the byte.
  if (a.gather_rows) {
    const int words = tile * row_words;
    const __amdgpu_buffer_rsrc_t rows = __builtin_amdgcn_make_buffer_rsrc(status, 0, (words + 1) * 8, kRawBufferFormat);
    auto fold = [&](const uint32_t lo, const uint32_t hi, const int word) -> bool {
      if ((hi & kGenMask) != gen || (hi >> 30) == 0) return false;
      const int w = word % row_words;
      const int col = w < expert_words ? 2 * w : E + 2 * (w - expert_words);
      // A column that does not exist (odd E or R) was published as zero.
      if ((lo & 0xffffu) != 0) atomicAdd(&col_excl[col], static_cast<int>(lo & 0xffffu));
      if ((lo >> 16) != 0) atomicAdd(&col_excl[col + 1], static_cast<int>(lo >> 16));
      return true;
    };
    for (int first = 0; first < words; first += kGatherWords) {
      vec16 got[kGatherDepth];
#pragma unroll
      for (int d = 0; d < kGatherDepth; ++d) {
        const int word = first + 2 * (d * kLayoutThreads + tid);
        got[d] = vec16{0u, 0u, 0u, 0u};
        if (word < words) got[d] = __builtin_amdgcn_raw_buffer_load_b128(rows, word * 8, 0, kCachePolicyDeviceScope);
      }
#pragma unroll
      for (int d = 0; d < kGatherDepth; ++d) {
        const int word = first + 2 * (d * kLayoutThreads + tid);
        bool need_0 = word < words, need_1 = word + 1 < words;
        uint32_t spins = 0;
        vec16 v = got[d];
        while (true) {
          if (need_0 && fold(v.x, v.y, word)) need_0 = false;
          if (need_1 && fold(v.z, v.w, word + 1)) need_1 = false;
          if (!need_0 && !need_1) break;
          if (++spins >= wait_limit) {
            __hip_atomic_store(&a.ws->timed_out, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (a.timeout_report != nullptr)
              __hip_atomic_store(a.timeout_report, kTimedOutCode, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
          }
          __builtin_amdgcn_s_sleep(2);
          v = __builtin_amdgcn_raw_buffer_load_b128(rows, word * 8, 0, kCachePolicyDeviceScope);
        }
      }
    }
  }

  // ---- larger grids: the decoupled look-back of every column ----------------------
  for (int col = tid; col < cols && !a.gather_rows; col += kLayoutThreads) {
    const int total = col_total[col];
    uint64_t* mine = status + static_cast<size_t>(tile) * cols + col;
    int excl = 0;
    if (tile != 0) {
      // Fold predecessors in, nearest first, a window of independent loads at a
      // time so that one memory round trip covers kLookbackWindow tiles.  "Tile -1"
      // is an empty prefix, which ends the walk at the front of the grid.
      int next = tile - 1;
      uint32_t spins = 0;
      bool found_prefix = false;
      while (!found_prefix) {
        // Only rows that exist are fetched: every row costs about 0.1 us (33 uncached 64-byte
        // sectors per row and tile), far more than the branch around its load.
        uint64_t s[kLookbackWindow];
#pragma unroll
        for (int i = 0; i < kLookbackWindow; ++i) {
          const int j = next - i;
          s[i] = (j >= 0) ? peek(status + static_cast<size_t>(j) * cols + col)
                          : pack_status(kFlagPrefix, gen, 0u);
        }
        bool stalled = false;
#pragma unroll
        for (int i = 0; i < kLookbackWindow; ++i) {
          if (!found_prefix && !stalled) {
            const bool ready = (static_cast<uint32_t>(s[i] >> 32) & kGenMask) == gen && (s[i] >> 62) != 0;
            if (ready) {
              excl += static_cast<int>(static_cast<uint32_t>(s[i]));
              found_prefix = (s[i] >> 62) == kFlagPrefix;
              --next;
              spins = 0;
            } else {
              stalled = true;
            }
          }
        }
        if (stalled) {
          if (++spins >= wait_limit) {
            __hip_atomic_store(&a.ws->timed_out, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (a.timeout_report != nullptr)
              __hip_atomic_store(a.timeout_report, kTimedOutCode, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
          }
          __builtin_amdgcn_s_sleep(2);
        }
      }
      publish(mine, pack_status(kFlagPrefix, gen, static_cast<uint32_t>(excl + total)));
    }
    col_excl[col] = excl;
  }
  __syncthreads();

  // ---- position of every route inside its expert segment, and the tile's routes in
  // destination order: by (expert, position in segment), then the non-routes in (token, slot)
  // order.  Entry = {flat route index, expert, position, token}.
  if (a.slot_rel != nullptr || a.route_order != nullptr) {
    int4* order = reinterpret_cast<int4*>(a.route_order) + static_cast<size_t>(tile) * (kTileTokens * K);
#pragma unroll
    for (int c = 0; c < kChunksPerWave; ++c) {
      const int chunk = wave * per_wave + c;
      if (c < per_wave && chunk < num_chunks) {
        const int local = chunk * kWave + lane;
        const int g = flat0 + local;
        if (g < flat_end) {
          const int e = my_e[c];
          const int rel = (e >= 0) ? col_excl[e] + in_tile[c] : -1;
          if (a.slot_rel != nullptr) a.slot_rel[g] = rel;
          if (a.route_order != nullptr) {
            const int token = t0 + static_cast<int>((static_cast<uint32_t>(local) * a.inv_topk) >> 19);
            order[order_pos[c]] = make_int4(g, e, rel, token);
          }
        }
      }
    }
  }

  // ---- the deterministic prologue's table: per destination rank, tokens take slots in
  // token order; the first slot of a token that reaches the rank carries the slot number
  if (a.rank_slot_idx != nullptr && flag_thread && t0 + ftid < T) {
    int position[kMaxRanks];
#pragma unroll
    for (int r = 0; r < kMaxRanks; ++r) {
      int base = col_excl[E + (r < R ? r : 0)];
#pragma unroll
      for (int w = 0; w < kTileTokens / kWave - 1; ++w) {
        const int before = rank_wave[w * kMaxRanks + r];  // read by every wave, counted by the later ones
        base += (w < fwave) ? before : 0;
      }
      position[r] = a.rank_slot_base + base + static_cast<int>((below_packed >> (8 * r)) & 0xffu);
    }
#pragma unroll
    for (int k = 0; k < kMaxTopk; ++k) {
      if (k < K) {
        const uint32_t nibble = (first_ranks >> (4 * k)) & 0xfu;
        int out = -1;
#pragma unroll
        for (int r = 0; r < kMaxRanks; ++r) out = (nibble == (8u | r)) ? position[r] : out;
        a.rank_slot_idx[static_cast<size_t>(t0 + ftid) * K + k] = out;
      }
    }
  }

  // ---- per-channel and per-source-chunk inclusive prefixes: the tile holding a range's end
  // writes it.  Ranges are the reference's get_channel_task_range (example047 .cu:73-79): range c
  // of C covers [min(per * c, T), min(per * c + per, T)) with per = ceil(T / C).  The channel matrix
  // is [rank, channel]; the rank prefix matrix takes the tokens as R such chunks, one per source rank,
  // and is [source, rank] (rank_prefix_matrix_copy, example047 .cu:128-143,352-360).
  if (a.channel_prefix_matrix != nullptr || a.rank_prefix_matrix != nullptr) {
    // Tokens among the tile's first n that are flagged for rank r: whole waves from the per-wave
    // counts, the rest from the flag words.
    auto flagged_before = [&](const int r, const int n) -> int {
      if (n >= kTileTokens) return col_total[E + r];
      int cnt = 0;
      for (int w = 0; w < (n >> 6); ++w) cnt += rank_wave[w * kMaxRanks + r];
      for (int tl = n & ~(kWave - 1); tl < n; ++tl) cnt += static_cast<int>((tok_flags[tl] >> (8 * r)) & 1u);
      return cnt;
    };
    const int C = a.channel_prefix_matrix != nullptr ? a.num_channels : 0;
    const int chunks = a.rank_prefix_matrix != nullptr ? R : 0;
    for (int idx = tid; idx < (C + chunks) * R; idx += kLayoutThreads) {
      const int c_all = idx / R, r = idx - c_all * R;
      const bool channel = c_all < C;
      const int c = channel ? c_all : c_all - C;
      const int ranges = channel ? C : R;
      const int per_range = (T + ranges - 1) / ranges;
      const long long s64 = static_cast<long long>(per_range) * c;
      const int start = s64 < T ? static_cast<int>(s64) : T;
      const int end = (T - start < per_range) ? T : start + per_range;
      if (end > t0 && end <= t0 + kTileTokens) {
        const int value = col_excl[E + r] + flagged_before(r, end - t0);
        if (channel)
          a.channel_prefix_matrix[r * C + c] = value;
        else
          a.rank_prefix_matrix[c * R + r] = value;
      }
    }
  }

  // ---- the last tile owns the grand totals ----------------------------------
  if (tile == a.num_tiles - 1) {
    for (int col = tid; col < cols; col += kLayoutThreads) {
      const int cnt = col_excl[col] + col_total[col];
      if (col < E) {
        a.num_tokens_per_expert[col] = cnt;
        // One adder per launch and expert; launches that share the array may overlap, hence atomic.
        if (a.cumulative_expert_stats != nullptr && cnt != 0) atomicAdd(&a.cumulative_expert_stats[col], cnt);
      } else {
        a.num_tokens_per_rank[col - E] = cnt;
      }
    }
    if (a.expert_offsets != nullptr) {
      // Block-wide exclusive scan of the aligned counts, one expert per thread
      // (kMaxExperts <= kLayoutThreads), so the scan order is the expert order.
      const int align = a.expert_alignment;
      int local = 0;
      if (tid < E) {
        const int cnt = col_excl[tid] + col_total[tid];
        local = (cnt + align - 1) / align * align;
      }
      const int incl = wave_inclusive_scan(local);
      if (lane == kWave - 1) wave_sums[wave] = incl;
      __syncthreads();
      int base = incl - local;
      int grand = 0;
#pragma unroll
      for (int w = 0; w < kLayoutWaves; ++w) {
        const int sum = wave_sums[w];
        base += (w < wave) ? sum : 0;
        grand += sum;
      }
      if (tid < E) {
        a.expert_offsets[tid] = base;
        // The thread of a rank's last expert holds the rank's inclusive row count.
        const int rank_end = static_cast<int>((static_cast<uint32_t>(tid + 1) * a.inv_experts_per_rank) >> 22);
        if (a.psum_rank_rows != nullptr && rank_end * a.experts_per_rank == tid + 1)
          a.psum_rank_rows[rank_end - 1] = base + local;
      }
      if (tid == 0) a.expert_offsets[E] = grand;
    }
  }
}

// Counts and flags only, up to 1024 tokens: one workgroup, one token per thread, one launch and
// one barrier.  What bounds a call this small is its chain of latencies, so everything hangs off
// the first load: a thread fetches its token's ids, the wave zeroes and fills its private row of
// counters (equal experts found with ballots, the lowest lane of a group adds the group's size: no
// atomics, no barrier before them), the token's flags go out from registers, and after the only
// barrier thread e adds up column e of the waves' rows and stores the total.
__global__ __launch_bounds__(kCountsThreads) void ep_layout_counts_small_kernel(
    const int64_t* __restrict__ topk_idx, int* num_tokens_per_rank, int* num_tokens_per_expert,
    uint8_t* is_token_in_rank, const int T, const int K, const int R, const int E,
    const uint32_t inv_experts_per_rank, const int expert_bits) {
  extern __shared__ int smem[];
  const int tid = static_cast<int>(threadIdx.x);
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int waves = static_cast<int>(blockDim.x) >> 6;
  int* rank_wave = smem;                                                          // [waves][kMaxRanks]
  uint16_t* hist = reinterpret_cast<uint16_t*>(smem + waves * kMaxRanks);         // [waves][E]: a wave holds at most 64 * 8 routes
  uint16_t* my_hist = hist + wave * E;

  int64_t ids[kMaxTopk];
#pragma unroll
  for (int k = 0; k < kMaxTopk; ++k)
    ids[k] = (k < K && tid < T) ? topk_idx[static_cast<size_t>(tid) * K + k] : -1;
  for (int i = lane; i < E; i += kWave) my_hist[i] = 0;
  __builtin_amdgcn_wave_barrier();

  uint64_t flags = 0;
#pragma unroll
  for (int k = 0; k < kMaxTopk; ++k) {
    if (k < K) {
      const bool valid = ids[k] >= 0 && ids[k] < static_cast<int64_t>(E);
      const int e = valid ? static_cast<int>(ids[k]) : 0;
      const uint64_t same = match_expert(valid, e, expert_bits);
      if (valid) {
        // One writer per counter and instruction: the lowest lane of every group of equal experts.
        if ((same & lanes_below(lane)) == 0) my_hist[e] = static_cast<uint16_t>(my_hist[e] + __popcll(same));
        flags |= 1ull << (8 * ((static_cast<uint32_t>(e) * inv_experts_per_rank) >> 22));
      }
    }
  }
  if (tid < T) store_token_flags(is_token_in_rank, tid, R, flags);
#pragma unroll
  for (int r = 0; r < kMaxRanks; ++r) {
    const uint64_t hit = __ballot(r < R && ((flags >> (8 * r)) & 1u) != 0);
    if (lane == 0) rank_wave[wave * kMaxRanks + r] = __popcll(hit);
  }
  __syncthreads();
  for (int e = tid; e < E; e += static_cast<int>(blockDim.x)) {
    int total = 0;
    for (int w = 0; w < waves; ++w) total += hist[w * E + e];
    num_tokens_per_expert[e] = total;
  }
  if (tid < R) {
    int total = 0;
    for (int w = 0; w < waves; ++w) total += rank_wave[w * kMaxRanks + tid];
    num_tokens_per_rank[tid] = total;
  }
}

// Counts and flags only, more than 1024 tokens.  One token per thread, 1024 tokens per workgroup
// pass; totals are accumulated with global atomics into zeroed outputs.
__global__ __launch_bounds__(kCountsThreads) void ep_layout_counts_kernel(
    const int64_t* __restrict__ topk_idx, int* num_tokens_per_rank, int* num_tokens_per_expert,
    uint8_t* is_token_in_rank, int T, int K, int R, int E, int experts_per_rank, int expert_bits,
    int num_tiles) {
  extern __shared__ int smem[];
  int* hist = smem;                // [E]
  int* rank_cnt = hist + E;        // [kMaxRanks]
  uint64_t* tok_flags = reinterpret_cast<uint64_t*>(rank_cnt + kMaxRanks + (E & 1));  // [kCountsThreads]
  const int tid = static_cast<int>(threadIdx.x);
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;

  for (int i = tid; i < E; i += kCountsThreads) hist[i] = 0;
  if (tid < kMaxRanks) rank_cnt[tid] = 0;
  const int flat_end = T * K;
  for (int tile = static_cast<int>(blockIdx.x); tile < num_tiles; tile += static_cast<int>(gridDim.x)) {
    tok_flags[tid] = 0;
    __syncthreads();
    const int t0 = tile * kCountsThreads;
    const int flat0 = t0 * K;
    int64_t raw[kMaxTopk];  // every chunk's load is in flight before the first ballot
#pragma unroll
    for (int c = 0; c < kMaxTopk; ++c) {
      const int g = flat0 + (wave * K + c) * kWave + lane;
      raw[c] = (c < K && g < flat_end) ? topk_idx[g] : -1;
    }
#pragma unroll
    for (int c = 0; c < kMaxTopk; ++c) {
      if (c < K) {
        const int local = (wave * K + c) * kWave + lane;
        const int64_t e64 = raw[c];
        const bool valid = e64 >= 0 && e64 < static_cast<int64_t>(E);
        const int e = valid ? static_cast<int>(e64) : 0;
        const uint64_t same = match_expert(valid, e, expert_bits);
        if (valid) {
          if ((same & lanes_below(lane)) == 0) atomicAdd(&hist[e], __popcll(same));
          reinterpret_cast<uint8_t*>(tok_flags + local / K)[e / experts_per_rank] = 1;
        }
      }
    }
    __syncthreads();
    const int t = t0 + tid;
    const uint64_t f = tok_flags[tid];
    if (t < T) store_token_flags(is_token_in_rank, t, R, f);
    for (int r = 0; r < R; ++r) {
      const uint64_t hit = __ballot(((f >> (8 * r)) & 1u) != 0);
      if (lane == 0 && hit != 0) atomicAdd(&rank_cnt[r], __popcll(hit));
    }
    __syncthreads();
  }
  __syncthreads();
  for (int i = tid; i < E; i += kCountsThreads)
    if (hist[i] != 0) atomicAdd(&num_tokens_per_expert[i], hist[i]);
  if (tid < R && rank_cnt[tid] != 0) atomicAdd(&num_tokens_per_rank[tid], rank_cnt[tid]);
}

__global__ void ep_fill_u32_kernel(uint32_t* dst, size_t count, uint32_t value) {
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += stride)
    dst[i] = value;
}

__global__ void ep_zero_counts_kernel(int* a, int na, int* b, int nb) {
  const int i = static_cast<int>(blockIdx.x * blockDim.x + threadIdx.x);
  if (i < na) a[i] = 0;
  if (i < nb) b[i] = 0;
}

}  // namespace

hipError_t launch_fill_u32(uint32_t* dst, size_t count, uint32_t value, hipStream_t stream) {
  if (count == 0) return hipSuccess;
  const int threads = 256;
  size_t blocks = (count + threads - 1) / threads;
  if (blocks > 2048) blocks = 2048;
  hipLaunchKernelGGL(ep_fill_u32_kernel, dim3(static_cast<unsigned>(blocks)), dim3(threads), 0, stream,
                     dst, count, value);
  return hipGetLastError();
}

hipError_t launch_layout_fused(const LayoutArgs& args, hipStream_t stream) {
  const LayoutArgs a = fixed::apply(args);
  static_assert(kMaxExperts <= kLayoutThreads, "the offset scan takes one expert per thread");
  const int E = a.num_experts;
  const int cols = E + a.num_ranks;
  const size_t lds = sizeof(int) * (2 * static_cast<size_t>(cols) + kLayoutWaves + 4 +
                                    (kTileTokens / kWave) * kMaxRanks + 2 * kLayoutWaves + E + 2 + (E & 1)) +
                     sizeof(uint64_t) * kTileTokens + sizeof(uint16_t) * (static_cast<size_t>(kLayoutWaves) * E + 2);
  // Shapes with an instantiation of their own: top-8 over 256 or 128 experts on 8 ranks; everything
  // else takes the kernel that reads its shapes from the arguments.
  const bool top8_on_8 = a.num_topk == 8 && a.num_ranks == 8;
  if (top8_on_8 && a.num_experts == 256)
    hipLaunchKernelGGL((ep_layout_fused_kernel<8, 256, 8>), dim3(a.num_tiles), dim3(kLayoutThreads), lds, stream, a);
  else if (top8_on_8 && a.num_experts == 128)
    hipLaunchKernelGGL((ep_layout_fused_kernel<8, 128, 8>), dim3(a.num_tiles), dim3(kLayoutThreads), lds, stream, a);
  else
    hipLaunchKernelGGL((ep_layout_fused_kernel<0, 0, 0>), dim3(a.num_tiles), dim3(kLayoutThreads), lds, stream, a);
  return hipGetLastError();
}

hipError_t launch_layout_counts(const int64_t* topk_idx, int* num_tokens_per_rank,
                                int* num_tokens_per_expert, uint8_t* is_token_in_rank,
                                int num_tokens, int num_topk, int num_ranks, int num_experts,
                                hipStream_t stream) {
  int expert_bits = 1;
  while ((1 << expert_bits) < num_experts) ++expert_bits;
  const int experts_per_rank = num_experts / num_ranks;
  if (num_tokens <= kCountsThreads) {
    // One workgroup sees everything and stores the totals itself: one launch instead of zero +
    // accumulate, which is what matters at these sizes (no tokens: one wave stores the zeros).
    const int waves = num_tokens > 0 ? (num_tokens + kWave - 1) / kWave : 1;
    const size_t lds = static_cast<size_t>(waves) * (sizeof(int) * kMaxRanks + sizeof(uint16_t) * num_experts);
    const uint32_t inv_experts_per_rank = ((1u << 22) + experts_per_rank - 1) / experts_per_rank;
    hipLaunchKernelGGL(ep_layout_counts_small_kernel, dim3(1), dim3(waves * kWave), lds, stream, topk_idx,
                       num_tokens_per_rank, num_tokens_per_expert, is_token_in_rank, num_tokens, num_topk,
                       num_ranks, num_experts, inv_experts_per_rank, expert_bits);
    return hipGetLastError();
  }
  const int num_tiles = (num_tokens + kCountsThreads - 1) / kCountsThreads;
  const int n = num_experts > num_ranks ? num_experts : num_ranks;
  hipLaunchKernelGGL(ep_zero_counts_kernel, dim3((n + 255) / 256), dim3(256), 0, stream,
                     num_tokens_per_expert, num_experts, num_tokens_per_rank, num_ranks);
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  const int grid = num_tiles < 1024 ? num_tiles : 1024;
  const size_t lds = sizeof(int) * (num_experts + kMaxRanks + (num_experts & 1)) +
                     sizeof(uint64_t) * kCountsThreads;
  hipLaunchKernelGGL(ep_layout_counts_kernel, dim3(grid), dim3(kCountsThreads), lds, stream, topk_idx,
                     num_tokens_per_rank, num_tokens_per_expert, is_token_in_rank, num_tokens, num_topk,
                     num_ranks, num_experts, experts_per_rank, expert_bits, num_tiles);
  return hipGetLastError();
}

}  // namespace mi_ep
