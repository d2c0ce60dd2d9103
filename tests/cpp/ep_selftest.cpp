// Self-checking executable in the reference's own style: a correctness phase against the CPU
// checker, then a benchmark phase, then exactly one JSON object on stdout; exit code 0 <=> PASS
// (datasets/readme.md:127-167 of the reference).  It drives the C++ surface of include/mi_ep.hpp
// the way the reference's main() drives its classes
// (datasets/example042_deepep_dispatch_layout/nv/empty_deepep_dispatch_layout.cu:391-427):
// the same 13 correctness cases and 7 benchmark cases, 20 warm-up + 100 timed launches between two
// events, Mtokens/s = tokens / microsecond.  Added beyond the reference: the fused layout on the
// same cases, the notify example's channel-prefix cases (example047 .cu:599-610) and one
// dispatch -> combine round trip.
//
// Test code: links the CPU checker (oracle/libep_oracle.so) as well as libmi_ep.so.
#include <algorithm>
#include <chrono>
#include <cstring>
#include <iomanip>
#include <iostream>
#include <string>
#include <vector>

#include "mi_ep.hpp"

extern "C" {
int ep_oracle_layout(const int64_t*, int, int, int, int, int*, int*, uint8_t*);
int ep_oracle_expert_offsets(const int*, int, int, int, int*, int*);
int ep_oracle_slot_maps(const int64_t*, int, int, int, const int*, int*, int*, int*, int*, int*);
int ep_oracle_channel_prefix(const uint8_t*, int, int, int, int*);
void ep_oracle_rank_prefix(const int*, int, int*);
int ep_oracle_permute(const void*, int, const float*, int, const int64_t*, const float*, int, const int*,
                      const int*, int, void*, float*, int64_t*, float*, int);
int ep_oracle_permute_ranks(const void*, int, const float*, int, const int64_t*, const float*, int, int, int, int, int,
                            int, const int*, int, void*, float*, int64_t*, float*, int*, int*, int*);
int ep_oracle_combine(const uint16_t*, const int*, const float*, const uint16_t*, const uint16_t*, int, int,
                      int, uint16_t*, int);
uint16_t ep_oracle_f32_to_bf16(float);
}

namespace {

using mi_ep::TopkIdx;

enum Pattern { kSpread = 0, kRankSweep = 1, kSameRank = 2 };
const char* pattern_name(int p) { return p == kRankSweep ? "rank_sweep" : p == kSameRank ? "same_rank" : "spread"; }

struct Case { int tokens, topk, ranks, experts, pattern; };

// The reference's closed-form routing tables (example042 .cu:178-206).
std::vector<TopkIdx> make_topk(const Case& c) {
  std::vector<TopkIdx> idx(static_cast<size_t>(c.tokens) * c.topk);
  const int per_rank = c.experts / c.ranks;
  for (int t = 0; t < c.tokens; ++t)
    for (int k = 0; k < c.topk; ++k) {
      int e;
      switch (c.pattern) {
        case kRankSweep: e = ((t + k) % c.ranks) * per_rank + (5 * t + 3 * k) % per_rank; break;
        case kSameRank: e = ((3 * t + c.topk) % c.ranks) * per_rank + (t + 7 * k) % per_rank; break;
        default: e = (17 * t + 31 * k + c.ranks) % c.experts; break;
      }
      idx[static_cast<size_t>(t) * c.topk + k] = e;
    }
  return idx;
}

template <class T>
struct DeviceArray {
  T* p = nullptr;
  size_t n = 0;
  explicit DeviceArray(size_t count) : n(count) { MI_EP_HIP_CHECK(hipMalloc(&p, std::max<size_t>(count, 1) * sizeof(T))); }
  ~DeviceArray() { (void)hipFree(p); }
  void upload(const std::vector<T>& h) { MI_EP_HIP_CHECK(hipMemcpy(p, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice)); }
  std::vector<T> download(size_t count) const {
    std::vector<T> h(count);
    MI_EP_HIP_CHECK(hipMemcpy(h.data(), p, count * sizeof(T), hipMemcpyDeviceToHost));
    return h;
  }
  void fill_bytes(int v) { MI_EP_HIP_CHECK(hipMemset(p, v, std::max<size_t>(n, 1) * sizeof(T))); }
};

struct HostLayout {
  std::vector<int> per_rank, per_expert, offsets, psum, slot_rel, slot_map, src_map, src_k;
  std::vector<uint8_t> flags;
};

HostLayout host_layout(const Case& c, const std::vector<TopkIdx>& idx, int align) {
  HostLayout h;
  h.per_rank.resize(c.ranks);
  h.per_expert.resize(c.experts);
  h.flags.resize(static_cast<size_t>(c.tokens) * c.ranks);
  ep_oracle_layout(idx.data(), c.tokens, c.topk, c.ranks, c.experts, h.per_rank.data(), h.per_expert.data(), h.flags.data());
  h.offsets.resize(c.experts + 1);
  h.psum.resize(c.ranks);
  ep_oracle_expert_offsets(h.per_expert.data(), c.experts, c.ranks, align, h.offsets.data(), h.psum.data());
  const size_t tk = static_cast<size_t>(c.tokens) * c.topk;
  h.slot_rel.resize(tk);
  h.slot_map.resize(tk);
  h.src_map.resize(h.offsets.back());
  h.src_k.resize(h.offsets.back());
  std::vector<int> fill(c.experts);
  ep_oracle_slot_maps(idx.data(), c.tokens, c.topk, c.experts, h.offsets.data(), h.slot_rel.data(), h.slot_map.data(),
                      h.src_map.data(), h.src_k.data(), fill.data());
  return h;
}

// Counts + flags through DeepepDispatchLayout, as the reference's runCorrectnessCase (:236-295).
bool check_counts_surface(const Case& c) {
  const std::vector<TopkIdx> idx = make_topk(c);
  const HostLayout ref = host_layout(c, idx, 1);
  DeviceArray<TopkIdx> d_idx(idx.size());
  DeviceArray<int> d_rank(c.ranks), d_expert(c.experts);
  DeviceArray<bool> d_flags(static_cast<size_t>(c.tokens) * c.ranks);
  d_idx.upload(idx);
  d_rank.fill_bytes(0);
  d_expert.fill_bytes(0);
  d_flags.fill_bytes(0);
  mi_ep::DeepepDispatchLayout layout(c.tokens, c.topk, c.ranks, c.experts);
  layout.compute(d_idx.p, d_rank.p, d_expert.p, d_flags.p);
  layout.compute(d_idx.p, d_rank.p, d_expert.p, d_flags.p);  // relaunch without re-zeroing (:313-329)
  MI_EP_HIP_CHECK(hipDeviceSynchronize());
  bool ok = d_rank.download(c.ranks) == ref.per_rank && d_expert.download(c.experts) == ref.per_expert;
  std::vector<uint8_t> got(ref.flags.size());
  MI_EP_HIP_CHECK(hipMemcpy(got.data(), d_flags.p, got.size(), hipMemcpyDeviceToHost));
  for (size_t i = 0; i < got.size(); ++i) ok = ok && ((got[i] != 0) == (ref.flags[i] != 0));
  return ok;
}

// Fused layout through ExpertParallelBuffer: everything the counts surface gives plus offsets,
// partition rows, channel prefixes and per-route positions, bit-exact.
bool check_fused_surface(const Case& c, int align, int channels) {
  const std::vector<TopkIdx> idx = make_topk(c);
  const HostLayout ref = host_layout(c, idx, align);
  DeviceArray<TopkIdx> d_idx(idx.size());
  d_idx.upload(idx);
  mi_ep::ExpertParallelBuffer buf(c.tokens, c.topk, c.experts, c.ranks, align, channels);
  const mi_ep::DispatchHandle& h = buf.get_dispatch_layout(d_idx.p, c.tokens);
  buf.check_status();
  auto pull = [](const int* p, size_t n) {
    std::vector<int> v(n);
    MI_EP_HIP_CHECK(hipMemcpy(v.data(), p, n * sizeof(int), hipMemcpyDeviceToHost));
    return v;
  };
  bool ok = pull(h.num_tokens_per_rank, c.ranks) == ref.per_rank && pull(h.num_tokens_per_expert, c.experts) == ref.per_expert &&
            pull(h.expert_offsets, c.experts + 1) == ref.offsets && pull(h.psum_rank_rows, c.ranks) == ref.psum &&
            pull(h.slot_rel, ref.slot_rel.size()) == ref.slot_rel;
  std::vector<uint8_t> flags(ref.flags.size());
  MI_EP_HIP_CHECK(hipMemcpy(flags.data(), h.is_token_in_rank, flags.size(), hipMemcpyDeviceToHost));
  ok = ok && flags == ref.flags;
  if (channels > 0) {
    std::vector<int> want(static_cast<size_t>(c.ranks) * channels);
    ep_oracle_channel_prefix(ref.flags.data(), c.tokens, c.ranks, channels, want.data());
    ok = ok && pull(h.channel_prefix_matrix, want.size()) == want;
  }
  return ok;
}

// The notify example's inputs (example047 .cu:189-193,437-447): the batches of all R source ranks,
// `tokens` each, laid end to end (two destinations per token, one expert per rank), so that the R
// source chunks of the launch are exactly the R ranks' batches; C = min(16, max(4, 2R)).  One launch
// must give the harness's expected rank prefix matrix (.cu:352-360) and the per-channel prefix of
// the whole batch (.cu:386-428).
bool check_notify_case(int tokens, int ranks) {
  const int total = tokens * ranks;
  Case c{total, std::min(2, ranks), ranks, ranks, kSpread};
  std::vector<TopkIdx> idx(static_cast<size_t>(total) * c.topk);
  std::vector<int> counts(static_cast<size_t>(ranks) * ranks, 0);
  for (int src = 0; src < ranks; ++src) {
    const int stride = ranks > 1 ? src % (ranks - 1) + 1 : 0;
    for (int t = 0; t < tokens; ++t)
      for (int s = 0; s < c.topk; ++s) {
        const int dst = (t + src + s * stride) % ranks;
        idx[(static_cast<size_t>(src) * tokens + t) * c.topk + s] = dst;
        ++counts[static_cast<size_t>(src) * ranks + dst];  // distinct per token: stride is in [1, R)
      }
  }
  const int channels = std::min(16, std::max(4, 2 * ranks));
  const HostLayout ref = host_layout(c, idx, 1);
  std::vector<int> want(static_cast<size_t>(ranks) * channels), want_rank(counts.size());
  ep_oracle_channel_prefix(ref.flags.data(), total, ranks, channels, want.data());
  ep_oracle_rank_prefix(counts.data(), ranks, want_rank.data());
  DeviceArray<TopkIdx> d_idx(idx.size());
  d_idx.upload(idx);
  mi_ep::ExpertParallelBuffer buf(total, c.topk, ranks, ranks, 1, channels);
  const mi_ep::DispatchHandle& h = buf.get_dispatch_layout(d_idx.p, total);
  buf.check_status();
  std::vector<int> got(want.size()), got_rank(want_rank.size());
  MI_EP_HIP_CHECK(hipMemcpy(got.data(), h.channel_prefix_matrix, got.size() * sizeof(int), hipMemcpyDeviceToHost));
  MI_EP_HIP_CHECK(hipMemcpy(got_rank.data(), h.rank_prefix_matrix, got_rank.size() * sizeof(int), hipMemcpyDeviceToHost));
  return got == want && got_rank == want_rank;
}

// Dispatch -> identity experts -> weighted combine on a small bf16 case, against the checker.
bool check_round_trip() {
  Case c{517, 8, 8, 64, kRankSweep};
  const int hidden = 1032, row_bytes = hidden * 2;
  std::vector<TopkIdx> idx = make_topk(c);
  for (size_t i = 0; i < idx.size(); i += 13) idx[i] = -1;  // masked slots
  std::vector<float> w(idx.size());
  for (size_t i = 0; i < w.size(); ++i) w[i] = 0.03125f * static_cast<float>(1 + (i * 7) % 11);
  std::vector<uint16_t> x(static_cast<size_t>(c.tokens) * hidden);
  for (size_t i = 0; i < x.size(); ++i) x[i] = ep_oracle_f32_to_bf16(static_cast<float>(static_cast<int>((i * 2654435761u) >> 20 & 1023) - 512) / 64.0f);
  const HostLayout ref = host_layout(c, idx, 1);
  const int rows = ref.offsets.back();
  std::vector<uint16_t> want_recv(static_cast<size_t>(rows) * hidden), want_out(x.size());
  std::vector<int64_t> want_idx(rows);
  std::vector<float> want_w(rows);
  ep_oracle_permute(x.data(), row_bytes, nullptr, 0, idx.data(), w.data(), c.topk, ref.src_map.data(), ref.src_k.data(),
                    rows, want_recv.data(), nullptr, want_idx.data(), want_w.data(), 1);
  ep_oracle_combine(want_recv.data(), ref.slot_map.data(), w.data(), nullptr, nullptr, c.tokens, c.topk, hidden,
                    want_out.data(), 1);

  DeviceArray<TopkIdx> d_idx(idx.size());
  DeviceArray<float> d_w(w.size());
  DeviceArray<uint16_t> d_x(x.size()), d_out(x.size());
  d_idx.upload(idx);
  d_w.upload(w);
  d_x.upload(x);
  mi_ep::ExpertParallelBuffer buf(c.tokens, c.topk, c.experts, c.ranks);
  DeviceArray<uint16_t> d_recv(static_cast<size_t>(buf.capacity_rows()) * hidden);
  const mi_ep::DispatchHandle& h = buf.dispatch(d_x.p, nullptr, d_idx.p, d_w.p, c.tokens, row_bytes, 0, d_recv.p, nullptr);
  buf.combine(d_recv.p, buf.capacity_rows(), d_w.p, nullptr, nullptr, hidden, d_out.p);
  buf.check_status();
  bool ok = d_recv.download(want_recv.size()) == want_recv;
  std::vector<int> got_map(ref.slot_map.size()), got_src(rows);
  MI_EP_HIP_CHECK(hipMemcpy(got_map.data(), h.slot_map, got_map.size() * sizeof(int), hipMemcpyDeviceToHost));
  MI_EP_HIP_CHECK(hipMemcpy(got_src.data(), h.recv_src_map, got_src.size() * sizeof(int), hipMemcpyDeviceToHost));
  ok = ok && got_map == ref.slot_map && got_src == ref.src_map;
  ok = ok && d_out.download(want_out.size()) == want_out;  // same fma chain: bit-exact
  return ok;
}

// The reference's own receive format (one row per token and destination rank) and its combine.
bool check_rank_format() {
  Case c{517, 8, 8, 64, kRankSweep};
  const int hidden = 264, row_bytes = hidden * 2, stride = 2 + c.topk, base = 3 * 1024;
  std::vector<TopkIdx> idx = make_topk(c);
  for (size_t i = 0; i < idx.size(); i += 11) idx[i] = -1;
  std::vector<float> w(idx.size());
  for (size_t i = 0; i < w.size(); ++i) w[i] = 0.0625f * static_cast<float>(1 + (i * 5) % 13);
  std::vector<uint16_t> x(static_cast<size_t>(c.tokens) * hidden);
  for (size_t i = 0; i < x.size(); ++i) x[i] = ep_oracle_f32_to_bf16(static_cast<float>(static_cast<int>((i * 2246822519u) >> 21 & 511) - 256) / 32.0f);
  mi_ep::ExpertParallelBuffer buf(c.tokens, c.topk, c.experts, c.ranks);
  const int cap = buf.rank_capacity_rows();
  std::vector<uint16_t> want_recv(static_cast<size_t>(cap) * hidden), want_out(x.size());
  std::vector<int64_t> want_idx(static_cast<size_t>(cap) * c.topk);
  std::vector<float> want_w(static_cast<size_t>(cap) * c.topk);
  std::vector<int> want_meta(static_cast<size_t>(cap) * stride), want_map(idx.size()), want_psum(c.ranks);
  ep_oracle_permute_ranks(x.data(), row_bytes, nullptr, 0, idx.data(), w.data(), c.tokens, c.topk, c.ranks, c.experts,
                          base, 1, nullptr, cap, want_recv.data(), nullptr, want_idx.data(), want_w.data(),
                          want_meta.data(), want_map.data(), want_psum.data());
  const int rows = want_psum.back();

  DeviceArray<TopkIdx> d_idx(idx.size());
  DeviceArray<float> d_w(w.size()), d_recv_w(want_w.size());
  DeviceArray<uint16_t> d_x(x.size()), d_out(x.size()), d_recv(want_recv.size());
  DeviceArray<int64_t> d_recv_idx(want_idx.size());
  DeviceArray<int> d_meta(want_meta.size());
  d_idx.upload(idx);
  d_w.upload(w);
  d_x.upload(x);
  const mi_ep::DispatchHandle& h = buf.dispatch_ranks(d_x.p, nullptr, d_idx.p, d_w.p, c.tokens, row_bytes, 0, base, true,
                                                      d_recv.p, nullptr, d_recv_idx.p, d_recv_w.p, d_meta.p);
  buf.combine_ranks(d_recv.p, cap, nullptr, nullptr, hidden, d_out.p);
  buf.check_status();
  auto head = [](auto v, size_t n) { v.resize(n); return v; };
  bool ok = head(d_recv.download(want_recv.size()), static_cast<size_t>(rows) * hidden) == head(want_recv, static_cast<size_t>(rows) * hidden);
  ok = ok && head(d_recv_idx.download(want_idx.size()), static_cast<size_t>(rows) * c.topk) == head(want_idx, static_cast<size_t>(rows) * c.topk);
  ok = ok && head(d_recv_w.download(want_w.size()), static_cast<size_t>(rows) * c.topk) == head(want_w, static_cast<size_t>(rows) * c.topk);
  ok = ok && head(d_meta.download(want_meta.size()), static_cast<size_t>(rows) * stride) == head(want_meta, static_cast<size_t>(rows) * stride);
  std::vector<int> got_map(want_map.size()), got_combine(want_map.size()), got_psum(c.ranks);
  MI_EP_HIP_CHECK(hipMemcpy(got_map.data(), h.rank_row_map, got_map.size() * sizeof(int), hipMemcpyDeviceToHost));
  MI_EP_HIP_CHECK(hipMemcpy(got_combine.data(), h.rank_combine_map, got_combine.size() * sizeof(int), hipMemcpyDeviceToHost));
  MI_EP_HIP_CHECK(hipMemcpy(got_psum.data(), h.psum_rank_tokens, got_psum.size() * sizeof(int), hipMemcpyDeviceToHost));
  ok = ok && got_map == want_map && got_psum == want_psum;
  // the ordered sum over the rows the checker says each token sent out
  ep_oracle_combine(want_recv.data(), got_combine.data(), nullptr, nullptr, nullptr, c.tokens, c.topk, hidden,
                    want_out.data(), 1);
  ok = ok && d_out.download(want_out.size()) == want_out;
  // each received row exactly once in the combine map
  std::vector<int> seen(rows, 0);
  for (int r : got_combine)
    if (r >= 0 && r < rows) ++seen[r];
  for (int n : seen) ok = ok && n == 1;
  return ok;
}

struct MetricRow {
  std::string surface;
  Case c;
  double latency_us = 0.0, mtokens_per_s = 0.0;
  int hidden = 0;             // payload rows only
  double data_bytes = 0.0;    // the reference harness's own data-size formula for the row
  double hbm_bytes = 0.0;     // minimum traffic of the call: every input read once, every output written once
  bool host_pointers = false; // timed through a host-pointer entry point (transfers and allocation included)
};

constexpr double kPeakHbmGBps = 8000.0;  // published HBM bandwidth of the part the kernels are written for

// Minimum traffic of the layout calls: the routing table in, flags and counters out
// (the fused form also writes the offsets, per-route positions and its destination-order table).
double layout_bytes(const Case& c, bool fused) {
  const double t = c.tokens, k = c.topk;
  double b = t * k * 8 + t * c.ranks + (c.ranks + c.experts) * 4.0;
  if (fused) b += (c.experts + 1) * 4.0 + t * k * 4 + t * k * 16;
  return b;
}

template <class Launch>
MetricRow time_launches(const std::string& surface, const Case& c, Launch launch) {
  const int warmup_iters = 20, bench_iters = 100;
  for (int i = 0; i < warmup_iters; ++i) launch();
  MI_EP_HIP_CHECK(hipDeviceSynchronize());
  hipEvent_t start, stop;
  MI_EP_HIP_CHECK(hipEventCreate(&start));
  MI_EP_HIP_CHECK(hipEventCreate(&stop));
  MI_EP_HIP_CHECK(hipEventRecord(start));
  for (int i = 0; i < bench_iters; ++i) launch();
  MI_EP_HIP_CHECK(hipEventRecord(stop));
  MI_EP_HIP_CHECK(hipEventSynchronize(stop));
  float ms = 0.0f;
  MI_EP_HIP_CHECK(hipEventElapsedTime(&ms, start, stop));
  MI_EP_HIP_CHECK(hipEventDestroy(start));
  MI_EP_HIP_CHECK(hipEventDestroy(stop));
  MetricRow row{surface, c};
  row.latency_us = static_cast<double>(ms) * 1000.0 / bench_iters;
  row.mtokens_per_s = row.latency_us > 0.0 ? c.tokens / row.latency_us : 0.0;
  return row;
}

// What one launch costs when the kernel does nothing: one wave that returns at once, timed like
// every other row (20 + 100 back-to-back launches between two events).  No layout call at a small
// batch can be faster than this.
__global__ void ep_selftest_empty_kernel() {}

void benchmark_launch_floor(std::vector<MetricRow>* rows) {
  MetricRow row = time_launches("launch_floor", Case{0, 1, 1, 1, kSpread},
                                [] { hipLaunchKernelGGL(ep_selftest_empty_kernel, dim3(1), dim3(64), 0, nullptr); });
  MI_EP_HIP_CHECK(hipGetLastError());
  rows->push_back(row);
}

void benchmark_case(const Case& c, std::vector<MetricRow>* rows) {
  const std::vector<TopkIdx> idx = make_topk(c);
  DeviceArray<TopkIdx> d_idx(idx.size());
  DeviceArray<int> d_rank(c.ranks), d_expert(c.experts);
  DeviceArray<bool> d_flags(static_cast<size_t>(c.tokens) * c.ranks);
  d_idx.upload(idx);
  mi_ep::DeepepDispatchLayout layout(c.tokens, c.topk, c.ranks, c.experts);
  MetricRow counts = time_launches("get_dispatch_layout", c, [&] { layout.compute(d_idx.p, d_rank.p, d_expert.p, d_flags.p); });
  counts.hbm_bytes = layout_bytes(c, false);
  rows->push_back(counts);
  mi_ep::ExpertParallelBuffer buf(c.tokens, c.topk, c.experts, c.ranks);
  MetricRow fused = time_launches("fused_layout", c, [&] { buf.get_dispatch_layout(d_idx.p, c.tokens); });
  fused.hbm_bytes = layout_bytes(c, true);
  rows->push_back(fused);
  buf.check_status();
}

// The same layout through the host-pointer twin: what a caller that keeps its data in host vectors
// pays (allocation, transfers and a synchronisation per call), as the reference's harness does around
// its kernel (example042 .cu:243-293).
void benchmark_host_case(const Case& c, std::vector<MetricRow>* rows) {
  const std::vector<TopkIdx> idx = make_topk(c);
  std::vector<int> rank(c.ranks), expert(c.experts);
  std::vector<unsigned char> flags(static_cast<size_t>(c.tokens) * c.ranks);
  const int iters = 10;
  const auto t0 = std::chrono::steady_clock::now();
  for (int i = 0; i < iters; ++i)
    MI_EP_CHECK(mi_ep_host_get_dispatch_layout(idx.data(), rank.data(), nullptr, expert.data(),
                                               reinterpret_cast<bool*>(flags.data()), c.tokens, c.topk, c.ranks,
                                               c.experts));
  const double us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count() / iters;
  MetricRow row{"host_get_dispatch_layout", c};
  row.latency_us = us;
  row.mtokens_per_s = us > 0.0 ? c.tokens / us : 0.0;
  row.hbm_bytes = layout_bytes(c, false);
  row.host_pointers = true;
  rows->push_back(row);
}

// Dispatch (fused layout + permute) and combine at one shape, timed the same way.  data_bytes
// follows the reference harnesses: index bytes for dispatch
// (example080 build_and_run.py:761-765: T*K*8 + T*K*4 + workgroups*R*4, the last term taken as
// tiles*R*4 here) and payload bytes for combine (example082 build_and_run.py:778-782:
// n*H*2 + T*H*2 + T*K*4).
void benchmark_payload_case(const Case& c, int hidden, std::vector<MetricRow>* rows) {
  const std::vector<TopkIdx> idx = make_topk(c);
  std::vector<float> w(idx.size(), 1.0f / c.topk);
  DeviceArray<TopkIdx> d_idx(idx.size());
  DeviceArray<float> d_w(w.size());
  DeviceArray<uint16_t> d_x(static_cast<size_t>(c.tokens) * hidden), d_out(static_cast<size_t>(c.tokens) * hidden);
  d_idx.upload(idx);
  d_w.upload(w);
  d_x.fill_bytes(0x3c);
  mi_ep::ExpertParallelBuffer buf(c.tokens, c.topk, c.experts, c.ranks);
  DeviceArray<uint16_t> d_recv(static_cast<size_t>(buf.capacity_rows()) * hidden);
  d_recv.fill_bytes(0x3c);
  const double n = static_cast<double>(c.tokens) * c.topk;  // no masked slots in these patterns
  MetricRow d = time_launches("dispatch", c, [&] {
    buf.dispatch(d_x.p, nullptr, d_idx.p, d_w.p, c.tokens, hidden * 2, 0, d_recv.p, nullptr);
  });
  d.hidden = hidden;
  d.data_bytes = n * 8 + n * 4 + ((c.tokens + 255) / 256) * c.ranks * 4.0;
  d.hbm_bytes = layout_bytes(c, true) + static_cast<double>(c.tokens) * hidden * 2 + n * hidden * 2 + n * 8 + n * 4 + n * 4;
  rows->push_back(d);
  MetricRow m = time_launches("combine", c, [&] { buf.combine(d_recv.p, buf.capacity_rows(), d_w.p, nullptr, nullptr, hidden, d_out.p); });
  m.hidden = hidden;
  m.data_bytes = n * hidden * 2 + static_cast<double>(c.tokens) * hidden * 2 + n * 4;
  m.hbm_bytes = n * hidden * 2 + static_cast<double>(c.tokens) * hidden * 2 + n * 4 + n * 4;
  rows->push_back(m);
  buf.check_status();
}

void print_json(bool pass, const std::vector<MetricRow>& rows) {
  std::cout << std::fixed << std::setprecision(3);
  std::cout << "{\n  \"Correctness\": \"" << (pass ? "PASS" : "FAIL") << "\",\n";
  std::cout << "  \"data_size_unit\": \"tokens\",\n  \"throughput_unit\": \"Mtokens/s\",\n  \"latency_unit\": \"us\",\n";
  std::cout << "  \"metrics\": [\n";
  for (size_t i = 0; i < rows.size(); ++i) {
    const MetricRow& r = rows[i];
    std::cout << "    {\"surface\": \"" << r.surface << "\", \"data_size\": " << r.c.tokens << ", \"num_topk\": " << r.c.topk
              << ", \"num_ranks\": " << r.c.ranks << ", \"num_experts\": " << r.c.experts << ", \"pattern\": \""
              << pattern_name(r.c.pattern) << "\", \"throughput_avg\": " << r.mtokens_per_s
              << ", \"latency_avg\": " << r.latency_us;
    {
      const double gbps = r.latency_us > 0.0 ? r.hbm_bytes / r.latency_us / 1e3 : 0.0;
      std::cout << ", \"hbm_bytes\": " << r.hbm_bytes << ", \"hbm_gbps\": " << gbps << ", \"roofline_frac\": "
                << std::setprecision(5) << gbps / kPeakHbmGBps << std::setprecision(3)
                << ", \"host_pointers\": " << (r.host_pointers ? "true" : "false");
    }
    if (r.hidden > 0)
      std::cout << ", \"hidden\": " << r.hidden << ", \"data_bytes\": " << r.data_bytes
                << ", \"gbytes_per_s\": " << (r.latency_us > 0.0 ? r.data_bytes / r.latency_us / 1e3 : 0.0);
    std::cout << "}" << (i + 1 != rows.size() ? "," : "") << "\n";
  }
  std::cout << "  ]\n}\n";
}

}  // namespace

int main(int argc, char** argv) {
  const bool skip_bench = argc > 1 && std::string(argv[1]) == "--skip-perf-test";
  int device_count = 0;
  if (hipGetDeviceCount(&device_count) != hipSuccess || device_count <= 0) {
    std::cout << "{\"Correctness\": \"SKIP\", \"reason\": \"no HIP device available\"}\n";
    return 0;
  }
  MI_EP_HIP_CHECK(hipSetDevice(0));

  std::vector<Case> cases = {{257, 1, 1, 4, kSpread}};
  for (int r : {2, 4, 8}) {
    cases.push_back({257, 1, r, 4 * r, kSpread});
    cases.push_back({1024, 2, r, 4 * r, kSpread});
    cases.push_back({4096, 4, r, 4 * r, kRankSweep});
    cases.push_back({4096, 8, r, 4 * r, kSameRank});
  }
  bool pass = true;
  for (const Case& c : cases) {
    const bool a = check_counts_surface(c);
    const bool b = check_fused_surface(c, 1, 2 * c.ranks) && check_fused_surface(c, 128, 0);
    if (!a || !b)
      std::cerr << "FAIL layout case T=" << c.tokens << " K=" << c.topk << " R=" << c.ranks << " E=" << c.experts << " "
                << pattern_name(c.pattern) << " counts=" << a << " fused=" << b << "\n";
    pass = pass && a && b;
  }
  for (int r : {2, 4, 8})
    for (int t : {7, 4096, 4097}) {
      const bool ok = check_notify_case(t, r);
      if (!ok) std::cerr << "FAIL notify case T=" << t << " R=" << r << "\n";
      pass = pass && ok;
    }
  {
    const bool ok = check_round_trip();
    if (!ok) std::cerr << "FAIL dispatch/combine round trip\n";
    pass = pass && ok;
  }
  {
    const bool ok = check_rank_format();
    if (!ok) std::cerr << "FAIL per-rank dispatch format\n";
    pass = pass && ok;
  }

  std::vector<MetricRow> rows;
  if (!skip_bench) {
    benchmark_launch_floor(&rows);
    for (int tokens : {1024, 4096, 16384, 65536}) benchmark_case({tokens, 2, 8, 32, kSpread}, &rows);
    benchmark_case({65536, 4, 8, 32, kRankSweep}, &rows);
    benchmark_case({65536, 8, 8, 32, kSameRank}, &rows);
    benchmark_case({65536, 2, 4, 32, kSpread}, &rows);
    benchmark_host_case({4096, 2, 8, 32, kSpread}, &rows);
    // The JIT examples' default shape (example080 build_and_run.py:542-548) and the large shape.
    benchmark_payload_case({512, 2, 8, 64, kSpread}, 256, &rows);
    benchmark_payload_case({8192, 8, 8, 256, kSpread}, 7168, &rows);
  }
  print_json(pass, rows);
  return pass ? 0 : 1;
}
