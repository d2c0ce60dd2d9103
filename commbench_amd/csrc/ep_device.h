// Shared device helpers and launcher declarations for the gfx950 dispatch core.
// Wave64 only: every kernel here assumes 64-lane wavefronts.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi_ep {

// 16 bytes as a native vector, so that non-temporal builtins accept it.
typedef uint32_t vec16 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
// Raw buffer descriptor word 3 for 32-bit elements on this architecture, and the cache-policy
// operand of buffer instructions (bit 1: streaming hint "nt"; bit 4: device scope "sc1").
constexpr int kRawBufferFormat = 0x00020000;
constexpr int kCachePolicyStreaming = 2;
constexpr int kCachePolicyDeviceScope = 16;
constexpr int kMaxRanks = 8;
constexpr int kMaxTopk = 8;
constexpr int kMaxExperts = 1024;

// ---- layout ---------------------------------------------------------------
constexpr int kLayoutThreads = 1024;
constexpr int kLayoutWaves = kLayoutThreads / kWave;
constexpr int kTileTokens = 256;
// A tile's 256 * K routes are 4 * K chunks of 64, shared out over the 16 waves.
constexpr int kChunksPerWave = ((kTileTokens / kWave) * kMaxTopk + kLayoutWaves - 1) / kLayoutWaves;

// Header of the fused layout kernel's workspace; the look-back status words follow.
// `turn` packs {generation:32 | ticket:32}: one fetch-add hands a tile both its
// index and the launch's generation; the tile that draws the last ticket stores
// {generation + 1, 0}, which is safe because every ticket of the launch is out.
struct alignas(256) LayoutWorkspace {
  uint64_t turn;
  uint32_t timed_out;   // sticky: a bounded wait expired
  uint32_t wait_limit;  // unsuccessful polls before a wait gives up; 0 = kDefaultWaitLimit
};
// Polls are spaced by s_sleep, roughly a microsecond apart: a few seconds before a launch gives up.
constexpr uint32_t kDefaultWaitLimit = 1u << 22;
// Small grids gather their predecessors' status rows whole: 16-byte loads, two in flight per lane
// (four cost 0.7 us more at 32 tiles), so that a workgroup takes in kGatherWords status words per
// round trip.  The rule is that the last tile's predecessors take at most two rounds.
constexpr int kGatherDepth = 2;
constexpr int kGatherWords = 2 * kGatherDepth * kLayoutThreads;
constexpr int kGatherLimitWords = 2 * kGatherWords;

struct LayoutArgs {
  const int64_t* topk_idx;
  int* num_tokens_per_rank;
  int* num_tokens_per_expert;
  uint8_t* is_token_in_rank;
  int* expert_offsets;
  int* psum_rank_rows;
  int* channel_prefix_matrix;
  int* rank_prefix_matrix;  // [R][R] or null: [source chunk][rank], inclusive over source chunks
  int* slot_rel;
  int* rank_slot_idx;
  int* route_order;  // [num_tiles * kTileTokens * K][4] or null
  int* tile_rank_counts;         // [num_tiles][R] or null: tokens of the tile flagged for each rank
  int64_t* copied_topk_idx;      // [T][K] or null: verbatim copy of topk_idx
  int* cumulative_expert_stats;  // [E] or null: += num_tokens_per_expert
  LayoutWorkspace* ws;
  int* timeout_report;  // null, or a device word that receives MI_EP_ETIMEDOUT when a bounded wait expires
  int num_tokens;
  int num_topk;
  int num_ranks;
  int num_experts;
  int experts_per_rank;
  int expert_alignment;
  int num_channels;
  int num_tiles;
  int static_tiles;  // 1: workgroup b takes tile b (every workgroup is resident at once); 0: tiles by ticket
  int gather_rows;   // 1: two columns per status word, every predecessor's row fetched at once (small grids)
  int rank_slot_base;
  int expert_bits;  // ceil(log2(num_experts)), at least 1
  uint32_t inv_topk;              // ceil(2^19 / num_topk): n / num_topk == (n * inv) >> 19 for n < 2048
  uint32_t inv_experts_per_rank;  // ceil(2^22 / experts_per_rank): exact for e < 1024
};

hipError_t launch_layout_fused(const LayoutArgs& a, hipStream_t stream);
hipError_t launch_layout_counts(const int64_t* topk_idx, int* num_tokens_per_rank,
                                int* num_tokens_per_expert, uint8_t* is_token_in_rank,
                                int num_tokens, int num_topk, int num_ranks, int num_experts,
                                hipStream_t stream);
hipError_t launch_fill_u32(uint32_t* dst, size_t count, uint32_t value, hipStream_t stream);

// ---- permute ----------------------------------------------------------------
struct PermuteArgs {
  const vec16* x;
  const float* x_scales;
  const int64_t* topk_idx;
  const float* topk_weights;
  const int* expert_offsets;
  const int* slot_rel;
  const int* route_order;  // the layout kernel's per-tile destination order, or null
  const int* num_tokens_per_expert;
  vec16* recv_x;
  float* recv_scales;
  int* recv_src_map;
  int64_t* recv_topk_idx;
  float* recv_topk_weights;
  int* slot_map;
  int num_tokens;
  int num_topk;
  int num_experts;
  int row_vecs;  // 16-byte vectors per row
  int num_scales;
  int capacity_rows;
  // Scale factors are addressed as [row * token_stride + j * hidden_stride], in 4-byte elements
  // (sf_token_stride / sf_hidden_stride of the reference's dispatch, example080 .cu:40).
  long long xs_token_stride, xs_hidden_stride;
  long long rs_token_stride, rs_hidden_stride;
  int expert_alignment;  // > 1: segments are padded; the copy kernels also write the pad rows
  int zero_pad_payload;  // pad rows get zero payload and scales (their map entries are always written)
};

// Which copy kernel serves mi_ep_dispatch: chosen by shape, or forced (tests, measurements).
constexpr int kPermuteAuto = 0;
constexpr int kPermuteByToken = 1;        // wave per (token, 1 KiB): source read once, rows scattered
constexpr int kPermuteByDestination = 2;  // needs route_order: rows written in destination order
hipError_t launch_permute(const PermuteArgs& a, int schedule, hipStream_t stream);
// What the destination-order copy assumes of the device, read once per device ordinal.
struct DeviceTraits {
  int compute_units;  // 256 on the part these kernels are tuned for
  int dies;           // accelerator dies (XCCs) that take workgroups round-robin
  int l2_bytes;       // L2 of one die
};
// Traits of the device `stream` belongs to (of the current device for the null stream).
hipError_t device_traits(hipStream_t stream, DeviceTraits* out);
// The shape rule behind kPermuteAuto (reads num_tokens, num_topk, num_experts, row_vecs only).
bool destination_order_pays(const PermuteArgs& a, const DeviceTraits& dev);
hipError_t launch_gather_rows(const vec16* x, const float* x_scales, const int* recv_src_map, int num_rows,
                              int num_tokens, int row_vecs, int num_scales, vec16* recv_x,
                              float* recv_scales, int* ready_counters, int rows_per_counter,
                              hipStream_t stream);
hipError_t launch_pull_indices(const int* recv_src_map, int num_rows, int tokens_per_source_rank,
                               int* pull_indices, hipStream_t stream);

// Dispatch de-duplicated by destination rank: one row per (token, rank that owns one of its experts).
struct RankPermuteArgs {
  const vec16* x;
  const float* x_scales;
  const int64_t* topk_idx;
  const float* topk_weights;
  const int* rank_slot_idx;        // from the layout kernel: rank_slot_base + slot on first-of-rank slots
  const int* num_tokens_per_rank;  // from the layout kernel
  const int* expand_slot_map;      // rows of the expanded buffer, or null
  vec16* recv_x;
  float* recv_scales;
  int64_t* recv_topk_idx;     // [rows, K]
  float* recv_topk_weights;   // [rows, K]
  int* recv_src_metadata;     // [rows, 2 + K]
  int* rank_row_map;          // [T, K]
  int* combine_map;           // [T, K] or null: each received row once
  int* psum_rank_tokens;      // [R]
  int num_tokens;
  int num_topk;
  int num_ranks;
  int num_experts;
  int experts_per_rank;
  int row_vecs;
  int num_scales;
  int capacity_rows;
  int rank_slot_base;
  int source_token_base;
  int local_expert_ids;
  // scale factors as [row * token_stride + j * hidden_stride], in 4-byte elements
  long long xs_token_stride, xs_hidden_stride;
  long long rs_token_stride, rs_hidden_stride;
};
hipError_t launch_permute_ranks(const RankPermuteArgs& a, hipStream_t stream);
hipError_t launch_gather_rank_weights(const float* recv_topk_weights, const int64_t* recv_topk_idx,
                                      const int* rank_row_map, int num_tokens, int num_topk, int num_rows,
                                      float* combined_topk_weights, int64_t* combined_topk_idx,
                                      hipStream_t stream);

// ---- combine ----------------------------------------------------------------
struct CombineArgs {
  const vec16* y;
  const int* slot_map;
  const float* topk_weights;
  const vec16* bias_0;
  const vec16* bias_1;
  const float* recv_topk_weights;
  const int64_t* recv_topk_idx;
  vec16* combined_x;
  float* combined_topk_weights;
  int64_t* combined_topk_idx;
  int num_tokens;
  int num_topk;
  int num_rows;  // rows of y; map entries at or beyond it are treated as non-routes
  int row_vecs;  // 16-byte vectors (8 bf16) per row
  int stream_output;  // 1: combined_x goes straight to HBM whatever its size
};

hipError_t launch_combine(const CombineArgs& a, hipStream_t stream);

hipError_t launch_copy_yardstick(vec16* dst, const vec16* src, size_t vecs, hipStream_t stream);
hipError_t launch_read_yardstick(const vec16* src, size_t vecs, uint32_t* sink, hipStream_t stream);
hipError_t launch_write_yardstick(vec16* dst, size_t vecs, hipStream_t stream);

// ---- shapes fixed at build time: the plug-in point for run-time compilation ---------------
// The reference compiles its dispatch and combine kernels per shape: top-k, experts, ranks and the
// hidden size are template parameters filled in by a just-in-time build of one overlaid header
// (example080 .cu:17-30; its harness, build_and_run.py:154-172,678).  The shipped library takes
// every shape at run time; the same sources built with any of the macros below fold that shape
// into the kernels as a constant and refuse calls with another (MI_EP_EINVAL).  0 = not fixed.
#ifndef MI_EP_FIXED_TOPK
#define MI_EP_FIXED_TOPK 0
#endif
#ifndef MI_EP_FIXED_EXPERTS
#define MI_EP_FIXED_EXPERTS 0
#endif
#ifndef MI_EP_FIXED_RANKS
#define MI_EP_FIXED_RANKS 0
#endif
#ifndef MI_EP_FIXED_ROW_BYTES  // bytes of a dispatch payload row
#define MI_EP_FIXED_ROW_BYTES 0
#endif
#ifndef MI_EP_FIXED_HIDDEN  // bf16 elements of a combine row
#define MI_EP_FIXED_HIDDEN 0
#endif
namespace fixed {
constexpr int kTopk = MI_EP_FIXED_TOPK, kExperts = MI_EP_FIXED_EXPERTS, kRanks = MI_EP_FIXED_RANKS;
constexpr int kRowBytes = MI_EP_FIXED_ROW_BYTES, kHidden = MI_EP_FIXED_HIDDEN;
static_assert(kTopk >= 0 && kTopk <= kMaxTopk && kRanks >= 0 && kRanks <= kMaxRanks && kExperts >= 0 &&
                  kExperts <= kMaxExperts && kRowBytes % 16 == 0 && kHidden % 8 == 0,
              "fixed shapes out of range");
static_assert(kRanks == 0 || kExperts % kRanks == 0, "fixed experts must be divisible by fixed ranks");

constexpr bool accepts(int fixed_value, long long given) { return fixed_value == 0 || given == fixed_value; }

// The arguments with every fixed shape replaced by its constant (the identity in the shipped
// library): kernels start from this copy, so that the compiler sees the constants.
__host__ __device__ inline LayoutArgs apply(LayoutArgs a) {
  if (kTopk != 0) {
    a.num_topk = kTopk;
    a.inv_topk = ((1u << 19) + kTopk - 1) / (kTopk != 0 ? kTopk : 1);
  }
  if (kRanks != 0) a.num_ranks = kRanks;
  if (kExperts != 0) {
    a.num_experts = kExperts;
    int bits = 1;
    while ((1 << bits) < kExperts) ++bits;
    a.expert_bits = bits;
  }
  if (kExperts != 0 && kRanks != 0) {
    constexpr int per_rank = kRanks != 0 ? kExperts / kRanks : 1;
    a.experts_per_rank = per_rank;
    a.inv_experts_per_rank = ((1u << 22) + per_rank - 1) / (per_rank != 0 ? per_rank : 1);
  }
  return a;
}
__host__ __device__ inline PermuteArgs apply(PermuteArgs a) {
  if (kTopk != 0) a.num_topk = kTopk;
  if (kExperts != 0) a.num_experts = kExperts;
  if (kRowBytes != 0) a.row_vecs = kRowBytes / 16;
  return a;
}
__host__ __device__ inline RankPermuteArgs apply(RankPermuteArgs a) {
  if (kTopk != 0) a.num_topk = kTopk;
  if (kExperts != 0) a.num_experts = kExperts;
  if (kRanks != 0) a.num_ranks = kRanks;
  if (kExperts != 0 && kRanks != 0) a.experts_per_rank = kExperts / (kRanks != 0 ? kRanks : 1);
  if (kRowBytes != 0) a.row_vecs = kRowBytes / 16;
  return a;
}
__host__ __device__ inline CombineArgs apply(CombineArgs a) {
  if (kTopk != 0) a.num_topk = kTopk;
  if (kHidden != 0) a.row_vecs = kHidden / 8;
  return a;
}
}  // namespace fixed

// ---- device helpers -------------------------------------------------------
#ifdef __HIPCC__
__device__ __forceinline__ int lane_id() { return static_cast<int>(threadIdx.x) & (kWave - 1); }

__device__ __forceinline__ uint64_t lanes_below(int lane) { return (1ull << lane) - 1ull; }

// Inclusive prefix sum over the 64 lanes of a wave with data-parallel-primitive moves (no LDS
// round trips as a shuffle would take): shifts by 1, 2, 4, 8 inside each row of 16 lanes (lanes
// without a source add the 0 given as the old value), then the last lane of row 0 / 2 into rows 1 / 3
// and lane 31 into rows 2 and 3.
__device__ __forceinline__ int wave_inclusive_scan(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
  return v;
}

// Value of `v` in lane `src` (wave-uniform src), as a scalar.
__device__ __forceinline__ int wave_read(int v, int src) {
  return __builtin_amdgcn_readlane(v, src);
}
__device__ __forceinline__ float wave_read(float v, int src) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src));
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// fp32 -> bf16 bits, round to nearest even, NaN kept quiet.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  uint32_t rounded = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
  uint32_t nan = (u >> 16) | 0x0040u;
  return ((u & 0x7fffffffu) > 0x7f800000u) ? nan : rounded;
}
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return (f32_to_bf16_bits(lo) & 0xffffu) | (f32_to_bf16_bits(hi) << 16);
}
#endif

}  // namespace mi_ep
