#!/usr/bin/env python3
"""Benchmark of the dispatch-layout + permute + combine path on one MI355X.

One step = one pass of the three kernels over one batch of synthetic input that already sits
in HBM: fused layout -> permute into the expert-contiguous buffer -> weighted combine of fresh
bf16 expert outputs.  Inputs come from the same seeded generators the parity tests use
(commbench_amd/workloads.py).  Prints one JSON line (see the keys below).  The CPU checker is
timed on the same workload and inputs as a reported baseline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config target|c2|c3|c4|c5] [--jit]
                    [--sustained-steps N --sustained-window M]
"""
import argparse
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_HBM_GBPS = 8000.0      # MI355X published HBM3E bandwidth
ZERO_PAD_PAYLOAD = 1        # MI_EP_DISPATCH_ZERO_PAD_PAYLOAD
STREAM_OUTPUT = 1           # MI_EP_COMBINE_STREAM_OUTPUT


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="target")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--rotate-x", type=int, default=1,
                    help="number of distinct source buffers cycled through by consecutive steps "
                         "(3 or more keeps the source out of the 256 MB memory-side cache)")
    ap.add_argument("--no-cold-source", action="store_true",
                    help="skip the extra pass with the source rows cycling through three buffers")
    ap.add_argument("--no-host-path", action="store_true",
                    help="skip the PCIe-inclusive pass through the host-pointer entry points")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the short runs of the other configurations reported under other_configs")
    ap.add_argument("--other-configs", default="all",
                    help="comma-separated names of the other configurations to run (e.g. 'target/ranks,target@128'); "
                         "default: all of them")
    ap.add_argument("--no-yardsticks", action="store_true",
                    help="skip the linear copy / read / write streams measured beside the roofline")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--jit", action="store_true",
                    help="run on a library compiled at run time with this configuration's shapes as constants "
                         "(commbench_amd.jit); implies --no-other-configs, whose shapes such a library refuses")
    ap.add_argument("--sustained-steps", type=int, default=3000,
                    help="back-to-back steps of each sustained-load leg, timed in windows of "
                         "--sustained-window steps (0 skips the legs)")
    ap.add_argument("--sustained-window", type=int, default=100)
    ap.add_argument("--schedule-sweep", action="store_true",
                    help="instead of the benchmark: time the dispatch copy under both schedules over a grid of row "
                         "sizes and token counts (the table the automatic choice is derived from) and print it as JSON")
    return ap.parse_args()


_EXPERT_OUTPUTS = {}   # config name -> the longest generated y so far (shorter ones are prefixes of it)


def fill_expert_outputs(cfg, y):
    """Fills y ([rows, hidden] bf16 on the GPU) with wl.make_expert_outputs(cfg, rows), generated in
    blocks of rows so that the float32 staging stays small (same generator, same stream).  Variants
    of one configuration reuse what was generated before."""
    from commbench_amd import workloads as wl
    rows = y.shape[0]
    have = _EXPERT_OUTPUTS.get(cfg.name)
    if have is not None and have.shape[0] >= rows:
        y.copy_(have[:rows])
        return
    rng = wl.rng_for(cfg, 2)
    for i in range(0, rows, 8192):
        n = min(8192, rows - i)
        y[i:i + n].copy_(wl.bf16_normal(rng, n, cfg.hidden))
    _EXPERT_OUTPUTS[cfg.name] = y.clone()


class Workload:
    """Device buffers and raw C-ABI calls of one configuration (nothing allocates in a step)."""

    def __init__(self, cfg, dev, rotate_x=1, expert_alignment=1, dispatch_flags=0):
        import torch
        from commbench_amd import _lib, workloads as wl

        self.cfg, self.torch, self.lib, self._lib = cfg, torch, _lib.load(), _lib
        T, K, E, R, H = cfg.num_tokens, cfg.num_topk, cfg.num_experts, cfg.num_ranks, cfg.hidden
        topk_np, w_np = wl.make_routing(cfg)
        self.topk_np, self.w_np = topk_np, w_np
        self.num_routes = int((topk_np >= 0).sum())
        self.topk = torch.from_numpy(topk_np).to(dev)
        self.w = torch.from_numpy(w_np).to(dev)
        x_cpu, scales_cpu = wl.make_payload(cfg)          # the tests' generator: seeded PCG64, N(0,1) as bf16
        self.x_cpu, self.scales_cpu = x_cpu, scales_cpu
        self.x = x_cpu.to(dev).contiguous()
        self.scales = None if scales_cpu is None else scales_cpu.to(dev).contiguous()
        self.x_ring = [self.x] + [self.x.clone() for _ in range(max(0, rotate_x - 1))]
        self.step_index = 0
        self.align = expert_alignment
        self.dispatch_flags = dispatch_flags
        cap = T * K + E * (expert_alignment - 1)
        self.cap = cap
        self.recv_x = torch.empty((cap, H), dtype=self.x.dtype, device=dev)
        self.recv_scales = (torch.empty((cap, cfg.num_scales), dtype=torch.float32, device=dev)
                            if self.scales is not None else None)
        # Expert outputs: a buffer of their own, so combine reads from HBM, not from lines the
        # permute just wrote.
        self.y = torch.empty((cap, H), dtype=torch.bfloat16, device=dev)
        fill_expert_outputs(cfg, self.y)
        i32 = dict(dtype=torch.int32, device=dev)
        self.per_rank = torch.empty(R, **i32)
        self.per_expert = torch.empty(E, **i32)
        self.in_rank = torch.empty((T, R), dtype=torch.bool, device=dev)
        self.off = torch.empty(E + 1, **i32)
        self.psum = torch.empty(R, **i32)
        self.rank_prefix = torch.empty((R, R), **i32)
        self.slot_rel = torch.empty((T, K), **i32)
        self.slot_map = torch.empty((T, K), **i32)
        self.route_order = torch.empty((self.lib.mi_ep_route_order_bytes(T, K) // 16, 4), **i32)
        self.src_map = torch.empty(cap, **i32)
        self.recv_idx = torch.empty(cap, dtype=torch.int64, device=dev)
        self.recv_w = torch.empty(cap, dtype=torch.float32, device=dev)
        self.out = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
        self.out_ring = [self.out]
        self.combine_flags = 0
        ws_bytes = self.lib.mi_ep_workspace_bytes(T, K, E, R)
        self.ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        self.stream = torch.cuda.current_stream().cuda_stream
        _lib.check(self.lib.mi_ep_workspace_init(self.ws.data_ptr(), ws_bytes, self.stream), "ws init")
        self.bytes = wl.algorithmic_bytes(T, H, E, K, R, self.num_routes,
                                          1 if cfg.payload == "fp8" else 2, cfg.num_scales)
        # Bytes of the zero-filled pad rows (alignment > 1, payload not kept): extra writes on top of
        # the algorithmic count.
        counts = wl.np.bincount(topk_np[topk_np >= 0].ravel(), minlength=E)
        pad_rows = int(((counts + expert_alignment - 1) // expert_alignment * expert_alignment - counts).sum())
        zeroed = expert_alignment > 1 and bool(dispatch_flags & ZERO_PAD_PAYLOAD)
        self.pad_rows = pad_rows
        self.padded_bytes = pad_rows * (cfg.row_bytes + cfg.num_scales * 4) if zeroed else 0

    def layout(self):
        c = self.cfg
        self._lib.check(self.lib.mi_ep_dispatch_layout(
            self.topk.data_ptr(), c.num_tokens, c.num_topk, c.num_ranks, c.num_experts, self.align, 0,
            self.per_rank.data_ptr(), self.per_expert.data_ptr(), self.in_rank.data_ptr(),
            self.off.data_ptr(), self.psum.data_ptr(), None, self.rank_prefix.data_ptr(), self.slot_rel.data_ptr(),
            None, 0, self.route_order.data_ptr(), None, None, None, self.ws.data_ptr(), self.ws.numel(),
            self.stream),
            "layout")

    def dispatch(self):
        c = self.cfg
        x = self.x_ring[self.step_index % len(self.x_ring)]
        self.step_index += 1
        self._lib.check(self.lib.mi_ep_dispatch(
            x.data_ptr(), None if self.scales is None else self.scales.data_ptr(),
            self.topk.data_ptr(), self.w.data_ptr(), self.off.data_ptr(), self.slot_rel.data_ptr(),
            self.route_order.data_ptr(), self.per_expert.data_ptr(), c.num_tokens, c.num_topk,
            c.num_experts, self.align, c.row_bytes, c.num_scales, self.recv_x.data_ptr(),
            None if self.recv_scales is None else self.recv_scales.data_ptr(),
            self.src_map.data_ptr(), self.recv_idx.data_ptr(), self.recv_w.data_ptr(),
            self.slot_map.data_ptr(), self.cap, self.dispatch_flags, self.stream), "dispatch")

    def combine(self):
        c = self.cfg
        out = self.out_ring[self.step_index % len(self.out_ring)]
        self._lib.check(self.lib.mi_ep_combine(
            self.y.data_ptr(), self.cap, self.slot_map.data_ptr(), self.w.data_ptr(), None, None, None, None,
            c.num_tokens, c.num_topk, c.hidden, out.data_ptr(), None, None, self.combine_flags, self.stream), "combine")

    def step(self):
        self.layout()
        self.dispatch()
        self.combine()


class RankWorkload:
    """The same step in the reference's own receive format: one row per (token, destination rank),
    K expert ids / gate weights and the source metadata per row; combine is the plain ordered sum of
    a token's rows (mi_ep_dispatch_ranks, then mi_ep_combine over combine_map)."""

    def __init__(self, cfg, dev):
        import torch
        from commbench_amd import _lib, workloads as wl

        self.cfg, self.lib, self._lib = cfg, _lib.load(), _lib
        T, K, E, R, H = cfg.num_tokens, cfg.num_topk, cfg.num_experts, cfg.num_ranks, cfg.hidden
        topk_np, w_np = wl.make_routing(cfg)
        valid = topk_np >= 0
        ranks = wl.np.where(valid, topk_np // (E // R), -1)
        self.num_rows = int(sum(len(set(r[r >= 0].tolist())) for r in ranks))   # distinct ranks per token
        self.topk = torch.from_numpy(topk_np).to(dev)
        self.w = torch.from_numpy(w_np).to(dev)
        x_cpu, _ = wl.make_payload(cfg)
        self.x = x_cpu.to(dev).contiguous()
        cap = T * min(K, R)
        self.cap = cap
        i32 = dict(dtype=torch.int32, device=dev)
        self.per_rank, self.per_expert = torch.empty(R, **i32), torch.empty(E, **i32)
        self.in_rank = torch.empty((T, R), dtype=torch.bool, device=dev)
        self.rank_slot_idx = torch.empty((T, K), **i32)
        self.recv_x = torch.empty((cap, H), dtype=self.x.dtype, device=dev)
        self.recv_idx = torch.empty((cap, K), dtype=torch.int64, device=dev)
        self.recv_w = torch.empty((cap, K), dtype=torch.float32, device=dev)
        self.meta = torch.empty((cap, 2 + K), **i32)
        self.row_map, self.combine_map = torch.empty((T, K), **i32), torch.empty((T, K), **i32)
        self.psum = torch.empty(R, **i32)
        self.y = torch.empty((cap, H), dtype=torch.bfloat16, device=dev)
        fill_expert_outputs(cfg, self.y)
        self.out = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
        ws_bytes = self.lib.mi_ep_workspace_bytes(T, K, E, R)
        self.ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        self.stream = torch.cuda.current_stream().cuda_stream
        _lib.check(self.lib.mi_ep_workspace_init(self.ws.data_ptr(), ws_bytes, self.stream), "ws init")
        n, row = self.num_rows, cfg.row_bytes
        layout = T * K * 8 + T * R + (R + E) * 4 + T * K * 4
        dispatch = T * row + n * row + T * K * 8 + T * K * 4 + T * K * 4 + n * (K * 8 + K * 4 + (2 + K) * 4) + 2 * T * K * 4
        combine = n * H * 2 + T * H * 2 + T * K * 4
        self.bytes = {"layout": layout, "dispatch": dispatch, "combine": combine, "total": layout + dispatch + combine}

    def layout(self):
        c = self.cfg
        self._lib.check(self.lib.mi_ep_dispatch_layout(
            self.topk.data_ptr(), c.num_tokens, c.num_topk, c.num_ranks, c.num_experts, 1, 0,
            self.per_rank.data_ptr(), self.per_expert.data_ptr(), self.in_rank.data_ptr(), None, None, None, None,
            None, self.rank_slot_idx.data_ptr(), 0, None, None, None, None, self.ws.data_ptr(), self.ws.numel(),
            self.stream), "layout")

    def dispatch(self):
        c = self.cfg
        self._lib.check(self.lib.mi_ep_dispatch_ranks(
            self.x.data_ptr(), None, self.topk.data_ptr(), self.w.data_ptr(), self.rank_slot_idx.data_ptr(), 0,
            self.per_rank.data_ptr(), None, c.num_tokens, c.num_topk, c.num_ranks, c.num_experts, c.row_bytes, 0,
            0, 0, self.recv_x.data_ptr(), None, self.recv_idx.data_ptr(), self.recv_w.data_ptr(),
            self.meta.data_ptr(), self.row_map.data_ptr(), self.combine_map.data_ptr(), self.psum.data_ptr(),
            self.cap, self.stream), "dispatch_ranks")

    def combine(self):
        c = self.cfg
        self._lib.check(self.lib.mi_ep_combine(
            self.y.data_ptr(), self.cap, self.combine_map.data_ptr(), None, None, None, None, None,
            c.num_tokens, c.num_topk, c.hidden, self.out.data_ptr(), None, None, 0, self.stream), "combine")

    def step(self):
        self.layout()
        self.dispatch()
        self.combine()


def host_path(cfg, wk, sample_tokens=2048):
    """The same step through the host-pointer entry points (numpy in, numpy out) on the first
    tokens of the same inputs: what a caller pays when the data lives in host memory.  Never `value`."""
    import numpy as np
    import torch
    from commbench_amd import ops
    n = min(sample_tokens, cfg.num_tokens)
    topk_np, w_np = wk.topk_np[:n], wk.w_np[:n]
    x = wk.x_cpu[:n].contiguous().view(torch.uint8).numpy().reshape(n, -1)
    scales = None if wk.scales_cpu is None else wk.scales_cpu[:n].contiguous().numpy()
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        d = ops.host_dispatch(x, scales, topk_np, w_np, cfg.num_experts, cfg.num_ranks)
        y = (d["recv_x"].view(np.uint16) if cfg.payload == "bf16"
             else np.zeros((d["recv_x"].shape[0], cfg.hidden), np.uint16))
        ops.host_combine(y, d["slot_map"], w_np)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    moved = x.nbytes + d["recv_x"].nbytes + y.nbytes + n * cfg.hidden * 2
    return {"tokens_per_s": n / best, "ms": best * 1e3, "sample_tokens": n, "pcie_bytes": int(moved),
            "note": "layout + dispatch + combine through mi_ep_host_*: pageable host arrays, device "
                    "buffers allocated per call, best of 3"}


def cpu_baseline(cfg, wk, seconds):
    """The CPU checker on the full workload with the benchmark's own inputs (same generators, same
    seeds), one thread and all the host cores this job may use; returns the cpu_baseline object."""
    import numpy as np
    import torch
    from oracle import ep_oracle

    T = cfg.num_tokens
    topk_np, w_np = wk.topk_np, wk.w_np
    x = wk.x_cpu.contiguous().view(torch.uint8).numpy().reshape(T, -1)
    scales = None if wk.scales_cpu is None else wk.scales_cpu.numpy()
    rows = wk.num_routes
    y = wk.y[:rows].cpu().view(torch.int16).numpy().view(np.uint16)
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    threads = max(1, min(threads, os.cpu_count() or 1, 16))

    def one_pass(nthreads):
        res = ep_oracle.full_path(topk_np, w_np, x, scales, cfg.num_experts, cfg.num_ranks, 1, nthreads)
        ep_oracle.combine(y, res["slot_map"], w_np, num_threads=nthreads)

    def rate(nthreads, budget):
        one_pass(nthreads)                           # warm
        n, t0 = 0, time.perf_counter()
        while True:
            one_pass(nthreads)
            n += 1
            dt = time.perf_counter() - t0
            if dt >= budget:
                return n * T / dt, n

    single, n1 = rate(1, seconds * 0.5)
    multi, nm = rate(threads, seconds * 0.5) if threads > 1 else (single, n1)
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"value": multi, "unit": "tokens/s", "cores": threads, "kind": "port",
            "single_thread_value": single, "threads": threads, "host_nproc": os.cpu_count(),
            "host_cpu_model": model,
            "sample": f"full workload, {T} tokens ({rows} routes), the benchmark's own inputs: layout + "
                      f"offsets + slot maps + permute + combine; {n1} passes on 1 thread and {nm} passes on "
                      f"{threads} OpenMP threads (~{seconds:.0f} s in all)"}


def source_fingerprint(path):
    """sha256 prefix of a C++/HIP source with comments removed and whitespace collapsed: it changes
    with the code, not with its commentary."""
    import re
    text = open(path, encoding="utf-8").read()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    return hashlib.sha256(" ".join(text.split()).encode()).hexdigest()[:16]


TRAFFIC_FILE = "profiles/hbm_traffic.json"


def profiled_record(workload_name):
    """What the committed counter and trace runs hold for a workload: {"traffic": {kernel: HBM bytes
    per launch}, "profiled_us": {kernel: average duration of the timed region's dispatches under
    rocprofv3}}; empty when the kernel sources have changed since they were taken (the file records
    their fingerprints).  Read from a committed file, not measured in this run."""
    path = os.path.join(ROOT, TRAFFIC_FILE)
    if not os.path.exists(path):
        return {}
    with open(path) as f:
        rec = json.load(f)
    for name, want in rec.get("source_sha16", {}).items():
        src = os.path.join(ROOT, "commbench_amd", "csrc", name)
        if not os.path.exists(src) or source_fingerprint(src) != want:
            return {}
    return {"traffic": rec.get(workload_name, {}), "profiled_us": rec.get("profiled_us", {}).get(workload_name, {})}


def time_steps(torch, wk, warmup, steps):
    for _ in range(warmup):
        wk.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        wk.step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def sustained_leg(torch, wk, total_steps, window):
    """`total_steps` steps back to back on the launch stream with one HIP event every `window`
    steps: the fraction of peak HBM bandwidth (algorithmic bytes of the whole step) of every
    window, so that a throughput that only holds for milliseconds shows."""
    windows = max(1, total_steps // window)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(windows + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(windows):
        for _ in range(window):
            wk.step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    us = [marks[i].elapsed_time(marks[i + 1]) * 1e3 / window for i in range(windows)]
    frac = [wk.bytes["total"] / (u * 1e-6) / 1e9 / PEAK_HBM_GBPS for u in us]
    ordered = sorted(frac)
    return {"steps": windows * window, "window_steps": window, "seconds": seconds,
            "us_per_step_median": sorted(us)[len(us) // 2], "us_per_step_max": max(us),
            "hbm_frac_first_window": frac[0], "hbm_frac_median_window": ordered[len(ordered) // 2],
            "hbm_frac_min_window": ordered[0], "hbm_frac_last_window": frac[-1],
            "min_window_index": frac.index(ordered[0])}


def kernel_medians(torch, wk, reps):
    marks = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(reps)]
    for ev in marks:
        ev[0].record()
        wk.layout()
        ev[1].record()
        wk.dispatch()
        ev[2].record()
        wk.combine()
        ev[3].record()
    torch.cuda.synchronize()
    return marks


def schedule_sweep():
    """Median duration of the dispatch copy inside the running step (layout, dispatch, combine back to
    back), forced to the token order and to the destination order, for rows of 2-16 KiB."""
    import torch
    from commbench_amd import ops, workloads as wl
    torch.cuda.set_device(0)

    def measure(cfg, flag):
        wk = Workload(cfg, "cuda:0", dispatch_flags=flag)
        for _ in range(60):
            wk.step()
        torch.cuda.synchronize()
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(40)]
        for a, b in ev:
            wk.layout()
            a.record()
            wk.dispatch()
            b.record()
            wk.combine()
        torch.cuda.synchronize()
        t = sorted(a.elapsed_time(b) * 1e3 for a, b in ev)
        return t[len(t) // 2]

    rows = []
    for T, E in ((8192, 256), (4096, 256), (16384, 128)):
        for row_bytes in (2048, 4096, 5120, 6144, 7168, 8192, 10240, 12288, 14336, 16384):
            cfg = wl.Config(f"sweep{T}_{row_bytes}", 40, T, row_bytes // 2, E, 8, 8)
            _EXPERT_OUTPUTS.clear()
            by_token = measure(cfg, ops.BY_TOKEN)
            by_destination = measure(cfg, ops.BY_DESTINATION)
            rows.append({"num_tokens": T, "num_experts": E, "row_bytes": row_bytes,
                         "by_token_us": round(by_token, 1), "by_destination_us": round(by_destination, 1),
                         "change_pct": round((by_destination / by_token - 1) * 100, 1),
                         "automatic": ops.dispatch_schedule_for(T, 8, E, row_bytes)})
            print(json.dumps(rows[-1]), file=sys.stderr, flush=True)
    print(json.dumps({"schedule_sweep": rows, "device_traits": ops.device_traits()}))


def main():
    args = parse_args()
    if args.schedule_sweep:
        schedule_sweep()
        return
    if args.gpus != 1:
        print(f"bench.py measures one GPU only: --gpus {args.gpus} is not supported "
              "(this path has no multi-GPU leg; partitions of one GPU's HBM stand for ranks)",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from commbench_amd import ops, workloads as wl

    cfg = wl.CONFIGS[args.config]
    dev = "cuda:0"
    torch.cuda.set_device(0)
    jit_shapes = None
    if args.jit:
        from commbench_amd import jit
        jit_shapes = dict(num_topk=cfg.num_topk, num_experts=cfg.num_experts, num_ranks=cfg.num_ranks,
                          row_bytes=cfg.row_bytes, hidden=cfg.hidden)
        jit.activate(**jit_shapes)
        args.no_other_configs = True
    wk = Workload(cfg, dev, args.rotate_x)
    T = cfg.num_tokens

    # Load before any measurement: the device idled while the inputs were generated on the CPU, and its
    # clocks take about 20 ms of work to settle.
    for _ in range(80):
        wk.step()
    torch.cuda.synchronize()

    # The same steps with the source rows cycling through three buffers, so that they come from
    # HBM instead of the 256 MB memory-side cache that keeps a single re-read source resident.
    # Then also with the combined output cycling through three buffers: the combine writes outputs
    # of up to 120 MiB (and part of larger ones) through into the memory-side cache, and an output buffer that is rewritten every
    # step would never have to leave it; three of them do.
    # That case is measured under both output policies of the combine: written through (the default)
    # and streamed straight to HBM (MI_EP_COMBINE_STREAM_OUTPUT).
    cold_ms_per_step = cold_both_ms_per_step = cold_both_streamed_ms_per_step = None
    cold_both_marks = sustained_hot = sustained_cold = sustained_cold_streamed = None
    if len(wk.x_ring) == 1 and not args.no_cold_source:
        ring = wk.x_ring
        wk.x_ring = [wk.x, wk.x.clone(), wk.x.clone()]

        def cold_pass():
            for _ in range(9):
                wk.step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                wk.step()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) * 1e3 / args.steps

        cold_ms_per_step = cold_pass()
        wk.out_ring = [wk.out, torch.empty_like(wk.out), torch.empty_like(wk.out)]
        cold_both_ms_per_step = cold_pass()
        cold_both_marks = kernel_medians(torch, wk, args.steps)
        if args.sustained_steps > 0:
            sustained_cold = sustained_leg(torch, wk, args.sustained_steps, args.sustained_window)
        wk.combine_flags = STREAM_OUTPUT
        cold_both_streamed_ms_per_step = cold_pass()
        if args.sustained_steps > 0:
            sustained_cold_streamed = sustained_leg(torch, wk, args.sustained_steps, args.sustained_window)
        wk.combine_flags = 0
        wk.x_ring = ring
        wk.out_ring = [wk.out]
        wk.step()
        torch.cuda.synchronize()
    if args.sustained_steps > 0:
        sustained_hot = sustained_leg(torch, wk, args.sustained_steps, args.sustained_window)

    # The same steps replayed as one HIP graph of the three kernels (no host launch gaps).
    graph_ms_per_step = None
    if not args.no_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            wk.stream = side.cuda_stream
            wk.step()
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                wk.stream = torch.cuda.current_stream().cuda_stream
                wk.step()
        wk.stream = torch.cuda.current_stream().cuda_stream
        for _ in range(30):      # the capture left the device idle: back to sustained clocks first
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # Per-kernel durations: the same steps again with HIP events on the launch stream
    # bracketing every kernel (kept out of the region above, where they would add gaps).
    torch.cuda.synchronize()
    marks = kernel_medians(torch, wk, args.steps)

    # Kernel symbols as rocprofv3 reports them; the combine schedule depends on the shape
    # (persistent LDS-staged kernel from 16 tokens per compute unit and 2 KiB rows upwards).
    traits = ops.device_traits()
    cus = traits["compute_units"]
    staged = T >= 16 * cus and 2048 <= cfg.hidden * 2 <= 160 * 1024
    schedule = ops.dispatch_schedule_for(T, cfg.num_topk, cfg.num_experts, cfg.row_bytes)
    names = ["ep_layout_fused_kernel",
             "ep_permute_tiles_kernel" if schedule == "destination" else "ep_permute_kernel",
             "ep_combine_staged_kernel" if staged else "ep_combine_kernel"]
    per_step = {n: sorted(ev[i].elapsed_time(ev[i + 1]) * 1e3 for ev in marks) for i, n in enumerate(names)}
    kernel_us = {n: sum(v) / len(v) for n, v in per_step.items()}
    kernel_us_stats = {n: {"avg": sum(v) / len(v), "median": v[len(v) // 2], "min": v[0]}
                       for n, v in per_step.items()}
    kernel_bytes = dict(zip(names, (wk.bytes["layout"], wk.bytes["dispatch"], wk.bytes["combine"])))
    # Wall clock of the event-bracketed steps, first record to last: what the four records per step
    # cost shows as the difference to the plain steps of the headline region further down.
    bracketed_step_us = marks[0][0].elapsed_time(marks[-1][3]) * 1e3 / len(marks)

    # Measured ceilings next to the nominal peak: 16-byte streaming copy, read-only and
    # write-only passes over the same 0.94-1 GiB buffers.
    copy_gbps = read_gbps = write_gbps = None
    if not args.no_yardsticks:
        lib, check = wk.lib, wk._lib.check
        src = wk.y.view(torch.uint8).reshape(-1)[: 1 << 30]
        dst = wk.recv_x.view(torch.uint8).reshape(-1)[: src.numel()]
        src = src[: dst.numel()]
        nbytes = src.numel() - src.numel() % 16
        sink = torch.zeros(1, dtype=torch.int32, device=dev)

        def timed(fn, moved_bytes, iters=10):
            for _ in range(3):
                fn()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return moved_bytes * iters / (e0.elapsed_time(e1) * 1e-3) / 1e9

        copy_gbps = timed(lambda: check(lib.mi_ep_copy_yardstick(dst.data_ptr(), src.data_ptr(), nbytes, wk.stream),
                                        "copy yardstick"), 2 * nbytes)
        read_gbps = timed(lambda: check(lib.mi_ep_read_yardstick(src.data_ptr(), nbytes, sink.data_ptr(), wk.stream),
                                        "read yardstick"), nbytes)
        write_gbps = timed(lambda: check(lib.mi_ep_write_yardstick(dst.data_ptr(), nbytes, wk.stream),
                                         "write yardstick"), nbytes)

    # The headline region comes last of the GPU measurements: after an idle period (the CPU-side
    # input generation above) the device's power management needs about 20 ms of load to reach its
    # sustained clocks (measured here: 389 -> 365 -> 356 us per step over the first 15 ms), and the
    # passes above provide that load.  W warm-up steps, a synchronisation, exactly K timed steps back
    # to back on one stream, a synchronisation.
    for _ in range(args.warmup):
        wk.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        wk.step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps

    # An interval between two event records holds a kernel and one record.  The cost of a record is
    # measured, not assumed: the bracketed steps took bracketed_step_us from the first record to the
    # last, i.e. len(marks) steps less the gap between one step's last record and the next step's
    # first, and the plain steps ms_per_step.  The roofline is taken on the intervals net of that
    # cost (they still hold the launch gap); kernel_us keeps the raw intervals.
    records = 4 * len(marks) - 1
    event_record_us = min(5.0, max(0.0, (bracketed_step_us - ms_per_step * 1e3) * len(marks) / records))
    kernel_us_net = {n: kernel_us[n] - event_record_us for n in names}
    # The roofline is taken on the RAW intervals (kernel + launch gap + one event record): they can
    # only overstate a kernel's duration, so the fraction is a lower bound that the profiler's own
    # durations (profiled_us, from the committed trace) must not fall below.  Both hot kernels are
    # reported; the line's headline kernel is the slower of the two in this run.
    profiled = profiled_record(cfg.name)
    hot = names[1:]
    dominant = max(hot, key=lambda n: kernel_us[n])
    gbps = lambda n, us: kernel_bytes[n] / (us * 1e-6) / 1e9

    def kernel_entry(n):
        entry = {"algorithmic_bytes": kernel_bytes[n], "us_raw": kernel_us[n], "us_net": kernel_us_net[n],
                 "frac_raw": gbps(n, kernel_us[n]) / PEAK_HBM_GBPS, "frac_net": gbps(n, kernel_us_net[n]) / PEAK_HBM_GBPS,
                 "traffic": profiled.get("traffic", {}).get(n), "profiled_us": profiled.get("profiled_us", {}).get(n)}
        if entry["profiled_us"]:
            entry["frac_profiled"] = gbps(n, entry["profiled_us"]) / PEAK_HBM_GBPS
        return entry

    roofline_kernels = {n: kernel_entry(n) for n in hot}
    achieved = gbps(dominant, kernel_us[dominant])
    # The same intervals with the source rows and the output cycling through three buffers each:
    # nothing counted stays in the memory-side cache from one step to the next.
    all_hbm = None
    if cold_both_marks is not None:
        cold_us = {n: sum(ev[i + 1].elapsed_time(ev[i + 2]) * 1e3 for ev in cold_both_marks) / len(cold_both_marks)
                   for i, n in enumerate(hot)}
        all_hbm = {n: {"us_raw": cold_us[n], "frac_raw": gbps(n, cold_us[n]) / PEAK_HBM_GBPS} for n in hot}

    result = {
        "metric": "dispatch+combine tokens/s and achieved HBM GB/s (% of peak), 1 MI355X",
        "value": T / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if cfg.payload == "bf16" else "u8",
        "data": "synthetic",
        "config": {
            "workload": f"{cfg.name}: layout + permute + combine, {T} tokens x {cfg.hidden} hidden "
                        f"{cfg.payload}, {cfg.num_experts} experts, top-{cfg.num_topk}, "
                        f"{cfg.num_ranks} HBM partitions, {cfg.routing} routing, "
                        f"{wk.num_routes} routes",
            "num_tokens": T, "hidden": cfg.hidden, "num_experts": cfg.num_experts,
            "num_topk": cfg.num_topk, "num_ranks": cfg.num_ranks, "payload": cfg.payload,
            "source_buffers": args.rotate_x,
            "library": "shipped (every shape a run-time argument)" if jit_shapes is None
                       else f"compiled at run time for {jit_shapes}",
            "inputs": "commbench_amd.workloads generators (PCG64 seeded 0xC0FFEE + config id): "
                      "make_routing, make_payload, make_expert_outputs",
        },
        "hbm_gbps_whole_step": wk.bytes["total"] / (ms_per_step * 1e-3) / 1e9,
        "hbm_frac_whole_step": wk.bytes["total"] / (ms_per_step * 1e-3) / 1e9 / PEAK_HBM_GBPS,
        "graph_replay_ms_per_step": graph_ms_per_step,
        "cold_source": None if cold_ms_per_step is None else {
            "ms_per_step": cold_ms_per_step,
            "tokens_per_s": T / (cold_ms_per_step * 1e-3),
            "hbm_frac_whole_step": wk.bytes["total"] / (cold_ms_per_step * 1e-3) / 1e9 / PEAK_HBM_GBPS,
            "note": "source rows cycled through 3 buffers so that they are read from HBM"},
        "cold_source_and_sink": None if cold_both_ms_per_step is None else {
            "ms_per_step": cold_both_ms_per_step,
            "tokens_per_s": T / (cold_both_ms_per_step * 1e-3),
            "hbm_frac_whole_step": wk.bytes["total"] / (cold_both_ms_per_step * 1e-3) / 1e9 / PEAK_HBM_GBPS,
            "streamed_output_ms_per_step": cold_both_streamed_ms_per_step,
            "streamed_output_hbm_frac_whole_step": wk.bytes["total"] / (cold_both_streamed_ms_per_step * 1e-3) / 1e9
                                                   / PEAK_HBM_GBPS,
            "note": "source rows and combined output each cycled through 3 buffers: every counted byte "
                    "crosses the HBM interface; once with the combine's output written through the "
                    "memory-side cache (default), once streamed to HBM (MI_EP_COMBINE_STREAM_OUTPUT)"},
        "algorithmic_bytes": wk.bytes,
        "device_traits": traits,
        "kernel_us": kernel_us,
        "kernel_us_stats": kernel_us_stats,
        "event_record_us": event_record_us,
        "kernel_us_net": kernel_us_net,
        "kernel_gbps": {n: kernel_bytes[n] / (kernel_us_net[n] * 1e-6) / 1e9 for n in names},
        "copy_yardstick_gbps": copy_gbps,
        "read_yardstick_gbps": read_gbps,
        "write_yardstick_gbps": write_gbps,
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": achieved,
                     "peak": PEAK_HBM_GBPS, "unit": "GB/s", "frac": achieved / PEAK_HBM_GBPS,
                     "duration_us": kernel_us[dominant],
                     "timing": "average raw HIP-event interval around the kernel over the timed steps: the kernel, "
                               "its launch gap and one event record (frac_net in `kernels` subtracts the measured "
                               "cost of a record, event_record_us; profiled_us / frac_profiled are the dispatches' "
                               "own durations under rocprofv3, from the committed trace)",
                     "traffic": roofline_kernels[dominant]["traffic"],
                     "traffic_source": TRAFFIC_FILE + " (two rocprofv3 --pmc runs, committed; not measured in this "
                                                      "run; null when the kernel sources have changed since)",
                     "kernels": roofline_kernels,
                     "cache_assisted": "in the timed region the single source buffer (re-read every step) and the "
                                       "combine's output (rewritten every step, written through) stay in the "
                                       "256 MB memory-side cache; all_bytes_cross_hbm repeats the intervals with "
                                       "both cycling through three buffers",
                     "all_bytes_cross_hbm": all_hbm},
    }
    if sustained_hot is not None:
        sustained = dict(sustained_hot)
        if sustained_cold is not None:
            sustained["cold_both"] = dict(sustained_cold, output_policy="written through (default)")
            sustained["cold_both_streamed"] = dict(sustained_cold_streamed,
                                                   output_policy="streamed (MI_EP_COMBINE_STREAM_OUTPUT)")
        sustained["note"] = ("steps back to back on one stream, one HIP event per window; fractions are "
                             "algorithmic bytes of the whole step against 8 TB/s; cold_both: source rows and "
                             "combined output each cycling through three buffers")
        result["sustained"] = sustained
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(cfg, wk, args.cpu_seconds)
    if not args.no_host_path:
        result["host_path"] = host_path(cfg, wk)
    if not args.no_other_configs:
        # Short runs of the other configurations, same step, for reference beside the headline.
        del wk
        torch.cuda.empty_cache()
        others = {}
        # "<name>@128": the same shape with expert segments padded to 128 rows, as the reference's
        # harness asks of dispatch (example080 build_and_run.py:718); the pad rows' map entries are
        # written, their payload is left alone, as in the reference's receive buffer.
        # "<name>@128/zero": the pad payload zero-filled as well; the fill is extra traffic
        # (padded_bytes) on top of the algorithmic count.
        # "<name>/ranks": the reference's per-rank receive format.
        variants = [("c2", 1, 0), ("c3", 1, 0), ("c4", 1, 0), ("c5", 1, 0), ("target", 1, 0),
                    (cfg.name + "@128", 128, 0), (cfg.name + "@128/zero", 128, ZERO_PAD_PAYLOAD),
                    (cfg.name + "/ranks", 1, 0)]
        wanted = None if args.other_configs == "all" else set(args.other_configs.split(","))
        if wanted is not None and not wanted <= {v[0] for v in variants}:
            sys.exit(f"--other-configs: unknown name(s) {sorted(wanted - {v[0] for v in variants})}")
        for name, align, flags in variants:
            if name == cfg.name or (wanted is not None and name not in wanted):
                continue
            ocfg = wl.CONFIGS[name.split("@")[0].split("/")[0]]
            ranks_format = name.endswith("/ranks")
            owk = RankWorkload(ocfg, dev) if ranks_format else Workload(ocfg, dev, expert_alignment=align,
                                                                         dispatch_flags=flags)
            us = time_steps(torch, owk, 60, 100) * 1e6      # 60 steps: past the clock ramp that follows idle
            omarks = kernel_medians(torch, owk, 30)
            median = lambda i: sorted(ev[i].elapsed_time(ev[i + 1]) * 1e3 for ev in omarks)[len(omarks) // 2]
            # cost of one event record, as for the headline: bracketed steps against plain steps
            bracketed_us = omarks[0][0].elapsed_time(omarks[-1][3]) * 1e3
            record_us = min(5.0, max(0.0, (bracketed_us - us * len(omarks)) / (4 * len(omarks) - 1)))
            entry = {"us_per_step": us, "tokens_per_s": ocfg.num_tokens / (us * 1e-6),
                     "kernel_us_median": {"layout": median(0), "dispatch": median(1), "combine": median(2)},
                     "event_record_us": record_us,
                     "kernel_us_median_net": {"layout": median(0) - record_us, "dispatch": median(1) - record_us,
                                              "combine": median(2) - record_us},
                     "algorithmic_bytes": owk.bytes["total"],
                     "hbm_gbps_whole_step": owk.bytes["total"] / (us * 1e-6) / 1e9,
                     "hbm_frac_whole_step": owk.bytes["total"] / (us * 1e-6) / 1e9 / PEAK_HBM_GBPS}
            if ranks_format:
                entry["num_rows"] = owk.num_rows
            else:
                entry["num_routes"] = owk.num_routes
                entry["dispatch_schedule"] = ops.dispatch_schedule_for(ocfg.num_tokens, ocfg.num_topk,
                                                                       ocfg.num_experts, ocfg.row_bytes)
                if align > 1:
                    entry["pad_rows"] = owk.pad_rows
                    entry["padded_bytes"] = owk.padded_bytes
                    entry["hbm_frac_with_pads"] = ((owk.bytes["total"] + owk.padded_bytes) / (us * 1e-6) / 1e9
                                                   / PEAK_HBM_GBPS)
            others[name] = entry
            del owk
            torch.cuda.empty_cache()
        result["other_configs"] = others
    print(json.dumps(result))


if __name__ == "__main__":
    main()
