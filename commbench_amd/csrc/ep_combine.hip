// Combine kernels for gfx950.
//
// The unit of work is (token, batch): kBatchVecs * 64 consecutive 16-byte vectors
// (8 bf16 each) of the token's output row, owned by one wavefront.  The wave
// issues the loads of that column range from all of the token's up-to-K rows
// before any arithmetic, accumulates in fp32 registers in ascending slot order
// with one fused multiply-add per row, adds the two optional bias rows and rounds
// to bf16 once.  No MFMA: there is no contraction here, only a K-way
// gather-reduce bound by HBM.
//
// Two schedules share that unit:
//   ep_combine_kernel         one unit per wave, result stored straight to HBM;
//   ep_combine_staged_kernel  one persistent 16-wave workgroup per CU walks groups
//                             of tokens; a group's output rows are staged in LDS
//                             (up to 160 KiB) and then written as one contiguous
//                             burst.  Keeping the 1/9
//                             of the traffic that is writes out of the read stream
//                             for most of the time is worth ~6 % on large shapes
//                             (HBM read/write turnarounds).
// Replaces combine_impl + combine_reduce_epilogue_impl (example082 .cu:28-67,
// example083 .cu:23-53); the reduce buffer of the reference is skipped because
// the rows already live in this GPU's HBM.
#include <atomic>

#include "ep_device.h"

namespace mi_ep {
namespace {

constexpr int kCombineThreads = 512;
constexpr int kCombineWaves = kCombineThreads / kWave;
constexpr int kStagedThreads = 1024;
constexpr int kStagedWaves = kStagedThreads / kWave;
constexpr int kStageBytes = 160 * 1024;  // all of the CU's LDS: one workgroup per CU
// What one step may keep in the memory-side cache (256 MB on this part; not reported by the
// runtime): the output written through into it plus an input of the output's size, which the next
// step re-reads, have to fit.
constexpr long long kMemorySideCacheBudget = 240ll * 1024 * 1024;

// Computes one unit; out[u] holds the packed bf16 of vector v0 + u * 64 (valid
// where that index is inside the row).
template <int kTopk, int kBatchVecs>
__device__ __forceinline__ void combine_unit(const CombineArgs& a, const int token, const int batch,
                                             const int lane, vec16 (&out)[kBatchVecs]) {
  int slot = -1;
  float weight = 1.0f;
  if (lane < kTopk) {
    const size_t i = static_cast<size_t>(token) * kTopk + lane;
    slot = a.slot_map[i];
    if (slot >= a.num_rows) slot = -1;
    if (a.topk_weights != nullptr) weight = a.topk_weights[i];
    if (batch == 0 && a.combined_topk_weights != nullptr)
      a.combined_topk_weights[i] = slot >= 0 ? a.recv_topk_weights[slot] : 0.0f;
    if (batch == 0 && a.combined_topk_idx != nullptr)
      a.combined_topk_idx[i] = slot >= 0 ? a.recv_topk_idx[slot] : -1;
  }
  const uint64_t routed = __ballot(slot >= 0);
  const int v0 = batch * (kBatchVecs * kWave) + lane;

  float acc[kBatchVecs][8];
#pragma unroll
  for (int u = 0; u < kBatchVecs; ++u)
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[u][i] = 0.0f;

  if (routed != 0) {
    // Every load is issued before the first multiply-add, as straight-line code: each row is read
    // through a buffer descriptor of its own, one row long for a route and empty for a non-route, so
    // that lanes past the row's end and the loads of non-routes are dropped by the bounds check (they
    // return zeros without a memory request) instead of being branched around.
    vec16 buf[kTopk][kBatchVecs];
    const int row_bytes = a.row_vecs * static_cast<int>(sizeof(vec16));
#pragma unroll
    for (int k = 0; k < kTopk; ++k) {
      const int row = wave_read(slot, k);
      const __amdgpu_buffer_rsrc_t row_k = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<vec16*>(a.y + static_cast<size_t>(row >= 0 ? row : 0) * a.row_vecs), 0,
          row >= 0 ? row_bytes : 0, kRawBufferFormat);
#pragma unroll
      for (int u = 0; u < kBatchVecs; ++u)
        buf[k][u] = __builtin_amdgcn_raw_buffer_load_b128(row_k, (v0 + u * kWave) * static_cast<int>(sizeof(vec16)), 0,
                                                          kCachePolicyStreaming);
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
#pragma unroll
      for (int i = 0; i < 4; ++i) out[u][i] = pack_bf16(acc[u][2 * i], acc[u][2 * i + 1]);
    }
  }
}

template <int kTopk, int kBatchVecs>
__global__ __launch_bounds__(kCombineThreads) void ep_combine_kernel(const CombineArgs args,
                                                                     const int batches_per_row) {
  const CombineArgs a = fixed::apply(args);
  const int lane = lane_id();
  const int wave = static_cast<int>(threadIdx.x) >> 6;
  const long long unit = static_cast<long long>(blockIdx.x) * kCombineWaves + wave;
  const int token = static_cast<int>(unit / batches_per_row);
  const int batch = static_cast<int>(unit - static_cast<long long>(token) * batches_per_row);
  if (token >= a.num_tokens) return;
  vec16 out[kBatchVecs];
  combine_unit<kTopk, kBatchVecs>(a, token, batch, lane, out);
  const int v0 = batch * (kBatchVecs * kWave) + lane;
#pragma unroll
  for (int u = 0; u < kBatchVecs; ++u) {
    const int v = v0 + u * kWave;
    if (v < a.row_vecs)
      __builtin_nontemporal_store(out[u], a.combined_x + static_cast<size_t>(token) * a.row_vecs + v);
  }
}

// Persistent schedule.  A group is `group_tokens` consecutive tokens of one workgroup; its units
// (token, KiB batch), numbered row by row, are staged before one burst writes them out: units below
// `lds_units` in LDS (1 KiB slot per unit), the following 16 * kRegUnits in registers of the wave
// that computed them (unit lds_units + 16 r + w is register r of wave w).  The register tail makes
// groups longer than the LDS alone allows; it is used where that turns two bursts into one.
//
// The burst's stores come in two kinds.  Written through at device scope ("sc1", no streaming hint)
// they are taken up by the 256 MB memory-side cache and reach HBM later, largely while the next,
// latency-bound kernel leaves it idle: the kernel no longer pays for turning the memory bus around
// in the middle of its reads (8192 x 14 KiB rows: 174 -> 164 us, whole step 346 -> 338 us).  That
// holds while the output and an input of its size that the next step re-reads both fit that cache;
// beyond, the dirty lines fall out during the next kernel's writes and cost it more than was gained
// (176 MB of output all written through: this kernel -12 us, the following copy +32 us), so only
// groups of tokens below `through_tokens` are written through and the rest is streamed ("nt"): with the
// share that still fits, 16384 x 8 KiB rows gain 10 us of 388 and 12288 x 14 KiB rows 9 us of 520.
template <int kTopk, int kRegUnits>
__global__ __launch_bounds__(kStagedThreads) void ep_combine_staged_kernel(const CombineArgs args,
                                                                          const int group_tokens,
                                                                          const int lds_units,
                                                                          const int through_tokens) {
  const CombineArgs a = fixed::apply(args);
  extern __shared__ vec16 stage[];  // [lds_units][64]
  const int lane = lane_id();
  const int wave = static_cast<int>(threadIdx.x) >> 6;
  const int batches = (a.row_vecs + kWave - 1) / kWave;
  const int groups = (a.num_tokens + group_tokens - 1) / group_tokens;

  // Group g is tokens [g * group_tokens, ...).  In every phase the grid covers one
  // contiguous run of groups, so the bursts of a phase tile a contiguous span.
  for (int g = static_cast<int>(blockIdx.x); g < groups; g += static_cast<int>(gridDim.x)) {
    const int g0 = g * group_tokens;
    const int gn = a.num_tokens - g0 < group_tokens ? a.num_tokens - g0 : group_tokens;
    const int units = gn * batches;
    const int in_lds = units < lds_units ? units : lds_units;
    {
      // unit u = wave, wave + 16, ...: (local, batch) stepped along instead of divided out
      int local = wave / batches, batch = wave - local * batches;
      for (int u = wave; u < in_lds; u += kStagedWaves) {
        vec16 out[1];
        combine_unit<kTopk, 1>(a, g0 + local, batch, lane, out);
        stage[u * kWave + lane] = out[0];
        batch += kStagedWaves;
        while (batch >= batches) {
          batch -= batches;
          ++local;
        }
      }
    }
    vec16 keep[kRegUnits > 0 ? kRegUnits : 1];
#pragma unroll
    for (int r = 0; r < kRegUnits; ++r) {
      const int u = lds_units + r * kStagedWaves + wave;
      if (u < units) {  // wave-uniform
        const int local = u / batches;
        vec16 out[1];
        combine_unit<kTopk, 1>(a, g0 + local, u - local * batches, lane, out);
        keep[r] = out[0];
      }
    }
    __syncthreads();
    // The group's rows are contiguous in combined_x: one burst, first what the LDS holds (every
    // thread takes 16-byte pieces in order), then each wave's own registers.
    vec16* dst = a.combined_x + static_cast<size_t>(g0) * a.row_vecs;
    // A buffer descriptor over the group's rows: the store's cache policy is an operand of the buffer
    // form of the instruction (and stores beyond the descriptor's end would be dropped).
    const __amdgpu_buffer_rsrc_t group_rows =
        __builtin_amdgcn_make_buffer_rsrc(dst, 0, gn * a.row_vecs * static_cast<int>(sizeof(vec16)), kRawBufferFormat);
    auto store = [&](const vec16 value, const int vec_index) {
      const int offset = vec_index * static_cast<int>(sizeof(vec16));
      if (g0 < through_tokens)
        __builtin_amdgcn_raw_buffer_store_b128(value, group_rows, offset, 0, kCachePolicyDeviceScope);
      else
        __builtin_amdgcn_raw_buffer_store_b128(value, group_rows, offset, 0, kCachePolicyStreaming);
    };
    {
      int local = wave / batches, batch = wave - local * batches;
      for (int u = wave; u < in_lds; u += kStagedWaves) {
        const int v = batch * kWave + lane;
        if (v < a.row_vecs) store(stage[u * kWave + lane], local * a.row_vecs + v);
        batch += kStagedWaves;
        while (batch >= batches) {
          batch -= batches;
          ++local;
        }
      }
    }
#pragma unroll
    for (int r = 0; r < kRegUnits; ++r) {
      const int u = lds_units + r * kStagedWaves + wave;
      if (u < units) {
        const int local = u / batches;
        const int v = (u - local * batches) * kWave + lane;
        if (v < a.row_vecs) store(keep[r], local * a.row_vecs + v);
      }
    }
    __syncthreads();
  }
}

constexpr int kStagedRegUnits = 4;  // units per wave kept in registers when that makes one burst do

template <int kTopk>
hipError_t launch_combine_k(const CombineArgs& a, hipStream_t stream) {
  const long long row_bytes = static_cast<long long>(a.row_vecs) * 16;
  DeviceTraits dev{};
  int ordinal = 0;
  hipError_t err = device_traits(stream, &dev);
  if (err == hipSuccess) err = stream != nullptr ? hipStreamGetDevice(stream, &ordinal) : hipGetDevice(&ordinal);
  if (err != hipSuccess) return err;
  const int cus = dev.compute_units;
  // Large shapes: persistent staged schedule.  It needs enough tokens per CU for
  // its phases to be long, and rows that fit the staging area.
  if (a.num_tokens >= 16 * cus && row_bytes >= 2048 && row_bytes <= kStageBytes) {
    // Phases of equal length on every CU: split a CU's share of the tokens into the fewest groups
    // that fit the staging area, with the register tail only if it makes a single burst possible.
    const int batches = (a.row_vecs + kWave - 1) / kWave;
    const int tokens_per_wg = (a.num_tokens + cus - 1) / cus;
    const int lds_capacity = static_cast<int>(kStageBytes / (kWave * sizeof(vec16)));  // units of 1 KiB
    const int rows_lds = lds_capacity / batches;
    const int rows_reg = (lds_capacity + kStagedRegUnits * kStagedWaves) / batches;
    const int phases_lds = (tokens_per_wg + rows_lds - 1) / rows_lds;
    const int phases_reg = (tokens_per_wg + rows_reg - 1) / rows_reg;
    // Measured: going from two bursts to one is worth 1-3 us (4096 x 14 KiB rows: 85 -> 82 us);
    // three to two gains nothing at 8192 rows and four to three loses 3 us at 16384 x 8 KiB, where
    // the unrolled tail's registers and code cost more than the boundary it saves.
    const bool with_registers = phases_reg == 1 && phases_lds > 1;
    const int phases = with_registers ? phases_reg : phases_lds;
    const int group_tokens = (tokens_per_wg + phases - 1) / phases;
    const int group_units = group_tokens * batches;
    const int lds_units = group_units < lds_capacity ? group_units : lds_capacity;
    const int groups = (a.num_tokens + group_tokens - 1) / group_tokens;
    const int grid = groups < cus ? groups : cus;
    const size_t lds = static_cast<size_t>(lds_units) * kWave * sizeof(vec16);
    // The kernel's LDS ceiling is raised once per device (a function attribute lives with the
    // device's copy of the code object); the flags only ever go from 0 to 1.
    constexpr int kMaxDevices = 64;
    static std::atomic<int> lds_limit_raised[2][kMaxDevices];
    if (ordinal < 0 || ordinal >= kMaxDevices) return hipErrorInvalidDevice;
    const void* kernel = with_registers
                             ? reinterpret_cast<const void*>(&ep_combine_staged_kernel<kTopk, kStagedRegUnits>)
                             : reinterpret_cast<const void*>(&ep_combine_staged_kernel<kTopk, 0>);
    std::atomic<int>& raised = lds_limit_raised[with_registers ? 1 : 0][ordinal];
    if (raised.load(std::memory_order_acquire) == 0) {
      const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kStageBytes);
      if (e != hipSuccess) return e;
      raised.store(1, std::memory_order_release);
    }
    // Rows written through: all of them while twice the output fits the budget, else the first
    // whole phases that leave room for an input of the output's size (a phase in which some
    // workgroups write through and others stream costs more than it saves: 16384 x 14 KiB rows with
    // 16 MiB written through, +11 us), none from an output of the budget's size on.
    const long long out_bytes = static_cast<long long>(a.num_tokens) * row_bytes;
    long long through_bytes = kMemorySideCacheBudget - out_bytes;
    if (through_bytes > out_bytes) through_bytes = out_bytes;
    if (through_bytes < 0 || a.stream_output) through_bytes = 0;
    const long long phase_tokens = static_cast<long long>(grid) * group_tokens;
    const int through_tokens = through_bytes == out_bytes
                                   ? a.num_tokens
                                   : static_cast<int>(through_bytes / row_bytes / phase_tokens * phase_tokens);
    if (with_registers)
      hipLaunchKernelGGL((ep_combine_staged_kernel<kTopk, kStagedRegUnits>), dim3(grid), dim3(kStagedThreads), lds,
                         stream, a, group_tokens, lds_units, through_tokens);
    else
      hipLaunchKernelGGL((ep_combine_staged_kernel<kTopk, 0>), dim3(grid), dim3(kStagedThreads), lds, stream, a,
                         group_tokens, lds_units, through_tokens);
    return hipGetLastError();
  }
  // Everything else: one unit per wave; two vectors per lane once rows are long.
  const int batch_vecs = a.row_vecs > kWave ? 2 : 1;
  const int per_batch = batch_vecs * kWave;
  const int batches = (a.row_vecs + per_batch - 1) / per_batch;
  const long long units = static_cast<long long>(a.num_tokens) * batches;
  const long long blocks = (units + kCombineWaves - 1) / kCombineWaves;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  if (batch_vecs == 2)
    hipLaunchKernelGGL((ep_combine_kernel<kTopk, 2>), dim3(static_cast<unsigned>(blocks)),
                       dim3(kCombineThreads), 0, stream, a, batches);
  else
    hipLaunchKernelGGL((ep_combine_kernel<kTopk, 1>), dim3(static_cast<unsigned>(blocks)),
                       dim3(kCombineThreads), 0, stream, a, batches);
  return hipGetLastError();
}

// A library built for one top-k carries that instantiation only.
template <int kFixedTopk>
hipError_t launch_combine_for(const CombineArgs& a, hipStream_t stream) {
  if constexpr (kFixedTopk != 0) {
    return launch_combine_k<kFixedTopk>(a, stream);
  } else {
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
}

}  // namespace

hipError_t launch_combine(const CombineArgs& args, hipStream_t stream) {
  const CombineArgs a = fixed::apply(args);
  if (a.num_tokens == 0) return hipSuccess;
  return launch_combine_for<fixed::kTopk>(a, stream);
}

}  // namespace mi_ep
