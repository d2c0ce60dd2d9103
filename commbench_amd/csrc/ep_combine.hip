// Combine kernel for gfx950.
//
// Each wavefront owns (token, batch): kBatchVecs * 64 consecutive 16-byte vectors
// (8 bf16 each) of the token's output row.  It issues the loads of that column
// range from all of the token's up-to-K rows before any arithmetic, accumulates
// in fp32 registers in ascending slot order with one fused multiply-add per row,
// adds the two optional bias rows and rounds to bf16 once.  No MFMA: there is no
// contraction here, only a K-way gather-reduce bound by HBM.
// Replaces combine_impl + combine_reduce_epilogue_impl (example082 .cu:28-67,
// example083 .cu:23-53); the reduce buffer of the reference is skipped because
// the rows already live in this GPU's HBM.
#include "ep_device.h"

namespace mi_ep {
namespace {

constexpr int kCombineThreads = 256;
constexpr int kCombineWaves = kCombineThreads / kWave;

template <int kTopk, int kBatchVecs>
__global__ __launch_bounds__(kCombineThreads) void ep_combine_kernel(const CombineArgs a,
                                                                     const int batches_per_row) {
  const int lane = lane_id();
  const int wave = static_cast<int>(threadIdx.x) >> 6;
  const long long unit = static_cast<long long>(blockIdx.x) * kCombineWaves + wave;
  const int token = static_cast<int>(unit / batches_per_row);
  const int batch = static_cast<int>(unit - static_cast<long long>(token) * batches_per_row);
  if (token >= a.num_tokens) return;

  int slot = -1;
  float weight = 1.0f;
  if (lane < kTopk) {
    const size_t i = static_cast<size_t>(token) * kTopk + lane;
    slot = a.slot_map[i];
    if (a.topk_weights != nullptr) weight = a.topk_weights[i];
    if (batch == 0 && a.combined_topk_weights != nullptr)
      a.combined_topk_weights[i] = slot >= 0 ? a.recv_topk_weights[slot] : 0.0f;
  }
  const uint64_t routed = __ballot(slot >= 0);
  const int v0 = batch * (kBatchVecs * kWave) + lane;

  float acc[kBatchVecs][8];
#pragma unroll
  for (int u = 0; u < kBatchVecs; ++u)
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[u][i] = 0.0f;

  if (routed != 0) {
    // Non-routes load the token's first routed row again (a cache hit) so that
    // every load can be issued before the first multiply-add.
    const int fallback = wave_read(slot, __builtin_ctzll(routed));
    vec16 buf[kTopk][kBatchVecs];
#pragma unroll
    for (int k = 0; k < kTopk; ++k) {
      const int row = wave_read(slot, k);
      const vec16* src = a.y + static_cast<size_t>(row >= 0 ? row : fallback) * a.row_vecs;
#pragma unroll
      for (int u = 0; u < kBatchVecs; ++u) {
        const int v = v0 + u * kWave;
        if (v < a.row_vecs) buf[k][u] = __builtin_nontemporal_load(src + v);
      }
    }
#pragma unroll
    for (int k = 0; k < kTopk; ++k) {
      const int row = wave_read(slot, k);
      const float w = wave_read(weight, k);
      if (row >= 0) {
#pragma unroll
        for (int u = 0; u < kBatchVecs; ++u) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const uint32_t pair = buf[k][u][i];
            acc[u][2 * i] = __builtin_fmaf(w, bf16_lo(pair), acc[u][2 * i]);
            acc[u][2 * i + 1] = __builtin_fmaf(w, bf16_hi(pair), acc[u][2 * i + 1]);
          }
        }
      }
    }
  }

#pragma unroll
  for (int u = 0; u < kBatchVecs; ++u) {
    const int v = v0 + u * kWave;
    if (v < a.row_vecs) {
      const size_t o = static_cast<size_t>(token) * a.row_vecs + v;
      if (a.bias_0 != nullptr) {
        const vec16 b = a.bias_0[o];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          acc[u][2 * i] = acc[u][2 * i] + bf16_lo(b[i]);
          acc[u][2 * i + 1] = acc[u][2 * i + 1] + bf16_hi(b[i]);
        }
      }
      if (a.bias_1 != nullptr) {
        const vec16 b = a.bias_1[o];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          acc[u][2 * i] = acc[u][2 * i] + bf16_lo(b[i]);
          acc[u][2 * i + 1] = acc[u][2 * i + 1] + bf16_hi(b[i]);
        }
      }
      vec16 out;
#pragma unroll
      for (int i = 0; i < 4; ++i) out[i] = pack_bf16(acc[u][2 * i], acc[u][2 * i + 1]);
      a.combined_x[o] = out;
    }
  }
}

template <int kTopk, int kBatchVecs>
hipError_t launch_combine_kb(const CombineArgs& a, hipStream_t stream) {
  const int per_batch = kBatchVecs * kWave;
  const int batches = (a.row_vecs + per_batch - 1) / per_batch;
  const long long units = static_cast<long long>(a.num_tokens) * batches;
  const long long blocks = (units + kCombineWaves - 1) / kCombineWaves;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL((ep_combine_kernel<kTopk, kBatchVecs>), dim3(static_cast<unsigned>(blocks)),
                     dim3(kCombineThreads), 0, stream, a, batches);
  return hipGetLastError();
}

template <int kTopk>
hipError_t launch_combine_k(const CombineArgs& a, hipStream_t stream) {
  return launch_combine_kb<kTopk, 1>(a, stream);
}

}  // namespace

hipError_t launch_combine(const CombineArgs& a, hipStream_t stream) {
  if (a.num_tokens == 0) return hipSuccess;
  switch (a.num_topk) {
    case 1: return launch_combine_k<1>(a, stream);
    case 2: return launch_combine_k<2>(a, stream);
    case 3: return launch_combine_k<3>(a, stream);
    case 4: return launch_combine_k<4>(a, stream);
    case 5: return launch_combine_k<5>(a, stream);
    case 6: return launch_combine_k<6>(a, stream);
    case 7: return launch_combine_k<7>(a, stream);
    case 8: return launch_combine_k<8>(a, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace mi_ep
