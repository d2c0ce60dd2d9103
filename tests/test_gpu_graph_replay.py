"""The three calls captured in one HIP graph: every replay must equal the eager result, also after
the inputs changed in place and with eager work and synchronisations between replays (the layout
kernel's workspace hands itself over from launch to launch without any clearing node)."""
import numpy as np
import pytest
import torch

from commbench_amd import _lib, ops
from commbench_amd import workloads as wl

from . import gpu_util as gu

pytestmark = pytest.mark.gpu


@pytest.fixture(params=[gu.BY_TOKEN, gu.BY_DESTINATION], ids=["by_token", "by_destination"])
def schedule(request):
    """One of the two copy kernels, as the flag bit mi_ep_dispatch takes."""
    return request.param


def test_graph_replays_match_eager(oracle, schedule):
    T, K, E, R, H = 3000, 8, 64, 8, 1024
    print(f"schedule {schedule}", flush=True)
    rng = np.random.default_rng(12)
    lib = _lib.load()
    dev = gu.DEV
    topk = torch.empty((T, K), dtype=torch.int64, device=dev)
    w = torch.empty((T, K), dtype=torch.float32, device=dev)
    x = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    cap = T * K
    i32 = dict(dtype=torch.int32, device=dev)
    per_rank, per_expert = torch.empty(R, **i32), torch.empty(E, **i32)
    in_rank = torch.empty((T, R), dtype=torch.bool, device=dev)
    off, psum = torch.empty(E + 1, **i32), torch.empty(R, **i32)
    slot_rel, slot_map = torch.empty((T, K), **i32), torch.empty((T, K), **i32)
    route_order = torch.empty((lib.mi_ep_route_order_bytes(T, K) // 16, 4), **i32)
    src_map = torch.empty(cap, **i32)
    recv_idx = torch.empty(cap, dtype=torch.int64, device=dev)
    recv_w = torch.empty(cap, dtype=torch.float32, device=dev)
    recv_x = torch.empty((cap, H), dtype=torch.bfloat16, device=dev)
    out = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    ws_bytes = lib.mi_ep_workspace_bytes(T, K, E, R)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    _lib.check(lib.mi_ep_workspace_init(ws.data_ptr(), ws_bytes, torch.cuda.current_stream().cuda_stream), "init")

    def step(stream):
        _lib.check(lib.mi_ep_dispatch_layout(
            topk.data_ptr(), T, K, R, E, 1, 0, per_rank.data_ptr(), per_expert.data_ptr(),
            in_rank.data_ptr(), off.data_ptr(), psum.data_ptr(), None, None, slot_rel.data_ptr(), None, 0,
            route_order.data_ptr(), None, None, None, ws.data_ptr(), ws_bytes, stream), "layout")
        _lib.check(lib.mi_ep_dispatch(
            x.data_ptr(), None, topk.data_ptr(), w.data_ptr(), off.data_ptr(), slot_rel.data_ptr(),
            route_order.data_ptr(), per_expert.data_ptr(), T, K, E, 1, H * 2, 0, recv_x.data_ptr(), None, src_map.data_ptr(),
            recv_idx.data_ptr(), recv_w.data_ptr(), slot_map.data_ptr(), cap, schedule, stream), "dispatch")
        _lib.check(lib.mi_ep_combine(
            recv_x.data_ptr(), cap, slot_map.data_ptr(), w.data_ptr(), None, None, None, None, T, K, H,
            out.data_ptr(), None, None, 0, stream), "combine")

    def load_inputs(seed):
        r = np.random.default_rng(seed)
        t = wl.zipf_distinct_topk(r, T, E, K, 1.2)
        t[r.random((T, K)) < 0.05] = -1
        topk.copy_(torch.from_numpy(t))
        w.copy_(torch.from_numpy(wl.softmax_gates(r, T, K)))
        x.copy_(wl.bf16_normal(r, T, H))
        return t

    def snapshot():
        torch.cuda.synchronize()
        rows = int(off[-1].item())
        return (per_expert.cpu().numpy().copy(), slot_map.cpu().numpy().copy(),
                gu.bf16_bits(recv_x[:rows]).copy(), gu.bf16_bits(out).copy())

    load_inputs(0)
    step(torch.cuda.current_stream().cuda_stream)          # eager warm-up before capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()

    for seed in (1, 2, 3, 4):
        t_np = load_inputs(seed)
        step(torch.cuda.current_stream().cuda_stream)      # eager
        eager = snapshot()
        for buf in (per_expert, slot_map, recv_x, out):
            buf.view(torch.uint8).fill_(0x5A)               # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        replayed = snapshot()
        for a, b in zip(eager, replayed):
            np.testing.assert_array_equal(a, b)
        _, want_expert, _ = oracle.layout(t_np, R, E)
        np.testing.assert_array_equal(replayed[0], want_expert)
    _lib.check(lib.mi_ep_workspace_status(ws.data_ptr(), torch.cuda.current_stream().cuda_stream), "status")


def test_two_streams_with_their_own_workspaces(oracle):
    """Calls are stream-ordered and re-entrant: two buffers on two streams, interleaved launches,
    each stream under its own copy kernel (the choice travels in the call's flags) and wait limit."""
    E, R, K, H = 64, 8, 8, 512
    rng = np.random.default_rng(77)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    cases = []
    for i, T in enumerate((2500, 3100)):
        topk_np = wl.zipf_distinct_topk(rng, T, E, K, 1.2)
        w_np = wl.softmax_gates(rng, T, K)
        x_cpu = wl.bf16_normal(rng, T, H)
        cases.append(dict(T=T, topk_np=topk_np, w_np=w_np, x_cpu=x_cpu, buf=ops.Buffer(T, K, E, R, device=gu.DEV),
                          topk=torch.from_numpy(topk_np).to(gu.DEV), w=torch.from_numpy(w_np).to(gu.DEV),
                          x=x_cpu.to(gu.DEV)))
    cases[1]["buf"].set_wait_limit(1 << 20)   # a limit of its own, too: it lives in the buffer's workspace
    torch.cuda.synchronize()
    results = [None, None]
    for rep in range(3):
        for i, c in enumerate(cases):
            with torch.cuda.stream(streams[i]):
                recv_x, _, _, h = c["buf"].dispatch(c["x"], None, c["topk"], c["w"], schedule=gu.SCHEDULES[i])
                out = ops.combine(recv_x, h, c["w"])
                results[i] = (recv_x, h, out)
    torch.cuda.synchronize()
    for c, (recv_x, h, out) in zip(cases, results):
        ref = oracle.full_path(c["topk_np"], c["w_np"], gu.as_bytes(c["x_cpu"]), None, E, R)
        rows = int(ref["expert_offsets"][-1])
        np.testing.assert_array_equal(h.slot_map.cpu().numpy(), ref["slot_map"])
        np.testing.assert_array_equal(gu.as_bytes(recv_x)[:rows], ref["recv_x"])
        want = oracle.combine(ref["recv_x"].view(np.uint16), ref["slot_map"], c["w_np"], num_threads=8)
        np.testing.assert_array_equal(gu.bf16_bits(out), want)
        c["buf"].status()


def test_host_threads_with_their_own_streams(oracle):
    """Four host threads, each with its own stream and buffer, launch layout + permute + combine at
    the same time (ctypes releases the interpreter lock during the calls): the library keeps no
    mutable state of its own, so every thread must get exactly its own results."""
    import threading
    E, R, K, H = 32, 4, 4, 256
    rng = np.random.default_rng(91)
    cases = []
    for i, T in enumerate((900, 1300, 257, 2048)):
        topk_np = wl.uniform_distinct_topk(rng, T, E, K)
        w_np = wl.softmax_gates(rng, T, K)
        x_cpu = wl.bf16_normal(rng, T, H)
        cases.append(dict(T=T, topk_np=topk_np, w_np=w_np, x_cpu=x_cpu, buf=ops.Buffer(T, K, E, R, device=gu.DEV),
                          topk=torch.from_numpy(topk_np).to(gu.DEV), w=torch.from_numpy(w_np).to(gu.DEV),
                          x=x_cpu.to(gu.DEV), stream=torch.cuda.Stream(), schedule=gu.SCHEDULES[i % 2]))
    torch.cuda.synchronize()
    results, errors = [None] * len(cases), []

    def work(i):
        c = cases[i]
        try:
            with torch.cuda.stream(c["stream"]):
                for _ in range(10):
                    recv_x, _, _, h = c["buf"].dispatch(c["x"], None, c["topk"], c["w"], schedule=c["schedule"])
                    out = ops.combine(recv_x, h, c["w"])
                c["stream"].synchronize()
            results[i] = (recv_x, h, out)
        except Exception as exc:          # reported by the main thread
            errors.append((i, repr(exc)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(cases))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    torch.cuda.synchronize()
    for c, (recv_x, h, out) in zip(cases, results):
        ref = oracle.full_path(c["topk_np"], c["w_np"], gu.as_bytes(c["x_cpu"]), None, E, R)
        rows = int(ref["expert_offsets"][-1])
        np.testing.assert_array_equal(h.slot_map.cpu().numpy(), ref["slot_map"])
        np.testing.assert_array_equal(gu.as_bytes(recv_x)[:rows], ref["recv_x"])
        want = oracle.combine(ref["recv_x"].view(np.uint16), ref["slot_map"], c["w_np"], num_threads=8)
        np.testing.assert_array_equal(gu.bf16_bits(out), want)
        c["buf"].status()
