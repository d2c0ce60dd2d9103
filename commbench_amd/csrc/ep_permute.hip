// Permute (dispatch payload) kernels for gfx950.
//
// ep_permute_kernel: each wavefront owns (token, batch): one batch is up to
// kBatchVecs * 64 consecutive 16-byte vectors of the token's row.  The wave reads
// its batch once into registers and stores it to every row the token was routed
// to, so the source is read once and every destination row is written once.
// Every access of a wave is 1 KiB contiguous.  The first batch of a token also
// carries the per-row side data: block scales, gate weight, owning expert,
// source token, and the absolute slot map.
// Replaces the payload role of dispatch_impl (example080 .cu:241-256) and the
// expand-mode copy epilogue (example081 .cu:22-60); one partition of this GPU's
// HBM stands where the reference has a peer GPU's receive buffer.
#include "ep_device.h"

namespace mi_ep {
namespace {

constexpr int kPermuteThreads = 256;
constexpr int kPermuteWaves = kPermuteThreads / kWave;

template <int kBatchVecs, bool kStreamStores>
__global__ __launch_bounds__(kPermuteThreads) void ep_permute_kernel(const PermuteArgs a,
                                                                     const int batches_per_row) {
  const int lane = lane_id();
  const int wave = static_cast<int>(threadIdx.x) >> 6;
  const long long unit = static_cast<long long>(blockIdx.x) * kPermuteWaves + wave;
  const int token = static_cast<int>(unit / batches_per_row);
  const int batch = static_cast<int>(unit - static_cast<long long>(token) * batches_per_row);
  if (token >= a.num_tokens) return;
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
      if (slot >= a.capacity_rows) slot = -1;
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
      const float s = a.x_scales[static_cast<size_t>(token) * a.num_scales + j];
      for (int k = 0; k < K; ++k) {
        const int row = wave_read(slot, k);
        if (row >= 0) a.recv_scales[static_cast<size_t>(row) * a.num_scales + j] = s;
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

// Zero-fills the rows that expert_alignment > 1 leaves between a segment's last
// route and the next segment.  One workgroup per expert.
__global__ __launch_bounds__(kPermuteThreads) void ep_pad_rows_kernel(const PermuteArgs a) {
  const int e = static_cast<int>(blockIdx.x);
  const int begin = a.expert_offsets[e] + a.num_tokens_per_expert[e];
  int end = a.expert_offsets[e + 1];
  if (end > a.capacity_rows) end = a.capacity_rows;
  const int tid = static_cast<int>(threadIdx.x);
  const vec16 zero = {0u, 0u, 0u, 0u};
  for (int row = begin; row < end; ++row) {
    vec16* dst = a.recv_x + static_cast<size_t>(row) * a.row_vecs;
    for (int v = tid; v < a.row_vecs; v += kPermuteThreads) dst[v] = zero;
    if (a.recv_scales != nullptr)
      for (int j = tid; j < a.num_scales; j += kPermuteThreads)
        a.recv_scales[static_cast<size_t>(row) * a.num_scales + j] = 0.0f;
    if (tid == 0) {
      a.recv_src_map[row] = -1;
      if (a.recv_topk_idx != nullptr) a.recv_topk_idx[row] = -1;
      if (a.recv_topk_weights != nullptr) a.recv_topk_weights[row] = 0.0f;
    }
  }
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

template <int kBatchVecs>
hipError_t launch_permute_batch(const PermuteArgs& a, hipStream_t stream) {
  const int per_batch = kBatchVecs * kWave;
  const int batches = (a.row_vecs + per_batch - 1) / per_batch;
  const long long units = static_cast<long long>(a.num_tokens) * batches;
  const long long blocks = (units + kPermuteWaves - 1) / kPermuteWaves;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL((ep_permute_kernel<kBatchVecs, true>), dim3(static_cast<unsigned>(blocks)),
                     dim3(kPermuteThreads), 0, stream, a, batches);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_permute(const PermuteArgs& a, hipStream_t stream) {
  if (a.num_tokens == 0) return hipSuccess;
  // Short rows fit one single-vector batch; long rows use two vectors per lane so
  // that a wave keeps 2 KiB of loads in flight.
  if (a.row_vecs <= kWave) return launch_permute_batch<1>(a, stream);
  return launch_permute_batch<2>(a, stream);
}

hipError_t launch_pad_rows(const PermuteArgs& a, hipStream_t stream) {
  hipLaunchKernelGGL(ep_pad_rows_kernel, dim3(a.num_experts), dim3(kPermuteThreads), 0, stream, a);
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

}  // namespace mi_ep
