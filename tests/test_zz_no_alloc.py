"""GPU parity of the allocation-free layout entry point (mi_ep_dispatch_layout_static) against
mi_ep_dispatch_layout, through the C ABI: every output bit-exact, on calls in a row that share
the library's static scratch, the later ones with smaller inputs."""
import numpy as np
import pytest
import torch

from commbench_amd import _lib
from commbench_amd import workloads as wl

from . import gpu_util as gu

pytestmark = pytest.mark.gpu

STATUS_WORDS = 262144      # MI_EP_STATIC_LAYOUT_STATUS_WORDS
E2BIG = -7


class LayoutOutputs:
    """One set of output buffers for either entry point, pre-filled with a pattern."""

    def __init__(self, T, K, R, E, channels, lib):
        i32 = dict(dtype=torch.int32, device=gu.DEV)
        self.per_rank = torch.full((R,), -3, **i32)
        self.per_expert = torch.full((E,), -3, **i32)
        self.flags = gu.garbage_like(torch.empty((max(T, 1), R), dtype=torch.bool, device=gu.DEV)).view(torch.uint8)
        self.off = torch.full((E + 1,), -3, **i32)
        self.psum = torch.full((R,), -3, **i32)
        self.channel_prefix = torch.full((R, channels), -3, **i32)
        self.rank_prefix = torch.full((R, R), -3, **i32)
        self.slot_rel = torch.full((max(T, 1), K), -3, **i32)
        self.rank_slot_idx = torch.full((max(T, 1), K), -3, **i32)
        # entries past the last token are never written: same fill on both sides
        self.route_order = torch.full((max(lib.mi_ep_route_order_bytes(T, K) // 16, 1), 4), -3, **i32)
        self.tile_rank_counts = torch.full((max((T + 255) // 256, 1), R), -3, **i32)
        self.copied_topk_idx = torch.full((max(T, 1), K), -3, dtype=torch.int64, device=gu.DEV)
        self.stats = torch.full((E,), 1000, **i32)          # accumulated into, not overwritten

    def tensors(self):
        return [self.per_rank, self.per_expert, self.flags, self.off, self.psum, self.channel_prefix,
                self.rank_prefix, self.slot_rel, self.rank_slot_idx, self.route_order, self.tile_rank_counts,
                self.copied_topk_idx, self.stats]


def run_both(lib, topk_np, R, E, align, channels):
    T, K = topk_np.shape
    topk = torch.from_numpy(topk_np).to(gu.DEV)
    stream = torch.cuda.current_stream().cuda_stream
    want, got = LayoutOutputs(T, K, R, E, channels, lib), LayoutOutputs(T, K, R, E, channels, lib)
    ws_bytes = lib.mi_ep_workspace_bytes(max(T, 1), K, E, R)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=gu.DEV)
    _lib.check(lib.mi_ep_workspace_init(ws.data_ptr(), ws_bytes, stream), "workspace init")
    _lib.check(lib.mi_ep_dispatch_layout(
        topk.data_ptr(), T, K, R, E, align, channels, want.per_rank.data_ptr(), want.per_expert.data_ptr(),
        want.flags.data_ptr(), want.off.data_ptr(), want.psum.data_ptr(), want.channel_prefix.data_ptr(),
        want.rank_prefix.data_ptr(), want.slot_rel.data_ptr(), want.rank_slot_idx.data_ptr(), gu.RANK_SLOT_BASE,
        want.route_order.data_ptr(), want.tile_rank_counts.data_ptr(), want.copied_topk_idx.data_ptr(), want.stats.data_ptr(),
        ws.data_ptr(), ws_bytes, stream), "mi_ep_dispatch_layout")
    report = torch.zeros(1, dtype=torch.int32, device=gu.DEV)
    _lib.check(lib.mi_ep_dispatch_layout_static(
        topk.data_ptr(), T, K, R, E, align, channels, got.per_rank.data_ptr(), got.per_expert.data_ptr(),
        got.flags.data_ptr(), got.off.data_ptr(), got.psum.data_ptr(), got.channel_prefix.data_ptr(),
        got.rank_prefix.data_ptr(), got.slot_rel.data_ptr(), got.rank_slot_idx.data_ptr(), gu.RANK_SLOT_BASE,
        got.route_order.data_ptr(), got.tile_rank_counts.data_ptr(), got.copied_topk_idx.data_ptr(), got.stats.data_ptr(),
        report.data_ptr(), stream), "mi_ep_dispatch_layout_static")
    torch.cuda.synchronize()
    _lib.check(lib.mi_ep_workspace_status(ws.data_ptr(), stream), "workspace status")
    _lib.check(lib.mi_ep_workspace_status(_lib.STATIC_SCRATCH, stream), "static scratch status")
    assert int(report.item()) == 0
    for a, b in zip(want.tensors(), got.tensors()):
        assert torch.equal(a, b)
    return want


def test_static_layout_matches_the_workspace_entry_point_on_calls_in_a_row(oracle):
    lib = _lib.load()
    # (T, K, R, E, alignment, channels): large first, then smaller inputs on the same scratch,
    # with other column counts, so that status words of earlier calls lie under later ones.
    shapes = [(8192, 8, 8, 256, 128, 16), (1000, 8, 8, 256, 1, 16), (4097, 4, 4, 64, 16, 8),
              (300, 2, 2, 8, 1, 4), (8192, 8, 8, 256, 1, 16)]
    for n, (T, K, R, E, align, channels) in enumerate(shapes):
        print(f"call {n}: shape {(T, K, R, E)} alignment {align}", flush=True)
        rng = np.random.default_rng(100 + n)
        topk_np = wl.uniform_distinct_topk(rng, T, E, K)
        topk_np[rng.random((T, K)) < 0.05] = -1
        want = run_both(lib, topk_np, R, E, align, channels)
        # and the shared result is the checker's
        per_rank, per_expert, flags = oracle.layout(topk_np, R, E)
        off, _ = oracle.expert_offsets(per_expert, R, align)
        np.testing.assert_array_equal(want.per_rank.cpu().numpy(), per_rank)
        np.testing.assert_array_equal(want.per_expert.cpu().numpy(), per_expert)
        np.testing.assert_array_equal(want.off.cpu().numpy(), off)
        np.testing.assert_array_equal(want.flags.cpu().numpy()[:T], flags)


def test_static_layout_refuses_shapes_beyond_its_scratch():
    lib = _lib.load()
    K, R, E = 2, 8, 1024
    tiles = STATUS_WORDS // (E + R) + 1
    T = tiles * 256
    # nothing is launched, so no buffer is touched: null outputs are never reached
    one = torch.zeros(8, dtype=torch.int64, device=gu.DEV)
    rc = lib.mi_ep_dispatch_layout_static(one.data_ptr(), T, K, R, E, 1, 0, one.data_ptr(), one.data_ptr(),
                                          one.data_ptr(), None, None, None, None, None, None, 0, None, None, None,
                                          None, None, torch.cuda.current_stream().cuda_stream)
    assert rc == E2BIG
    assert "static scratch" in _lib.strerror(rc)
    torch.cuda.synchronize()
    assert int(one.sum().item()) == 0


def test_static_layout_reports_an_expired_wait_and_recovers(oracle):
    """Failure handling on the library's own scratch, forced from the host: with its wait limit set to
    one poll, launches over hundreds of tiles give up a wait of their scan; every launch still ends,
    the caller's report word and the scratch's status both say so, and after the scratch is
    initialised again the entry point gives the workspace entry's results."""
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    T, K, R, E = 65536, 8, 8, 256                    # 256 tiles x 264 columns: within the scratch
    topk_np = wl.uniform_distinct_topk(np.random.default_rng(3), T, E, K)
    topk = torch.from_numpy(topk_np).to(gu.DEV)
    out = LayoutOutputs(T, K, R, E, 4, lib)
    report = torch.zeros(1, dtype=torch.int32, device=gu.DEV)
    _lib.check(lib.mi_ep_workspace_set_wait_limit(_lib.STATIC_SCRATCH, 1, stream), "static wait limit")
    try:
        expired = False
        for _ in range(20):
            _lib.check(lib.mi_ep_dispatch_layout_static(
                topk.data_ptr(), T, K, R, E, 1, 4, out.per_rank.data_ptr(), out.per_expert.data_ptr(),
                out.flags.data_ptr(), out.off.data_ptr(), out.psum.data_ptr(), out.channel_prefix.data_ptr(),
                out.rank_prefix.data_ptr(), out.slot_rel.data_ptr(), None, 0, None, None, None, None,
                report.data_ptr(), stream), "mi_ep_dispatch_layout_static")
            torch.cuda.synchronize()
            if int(report.item()) != 0:
                expired = True
                break
        assert expired, "no wait expired with a one-poll limit over hundreds of tiles"
        assert int(report.item()) == -110
        assert lib.mi_ep_workspace_status(_lib.STATIC_SCRATCH, stream) == -110
    finally:
        _lib.check(lib.mi_ep_workspace_init(_lib.STATIC_SCRATCH, 0, stream), "static scratch re-init")
    assert lib.mi_ep_workspace_status(_lib.STATIC_SCRATCH, stream) == 0
    rng = np.random.default_rng(9)
    run_both(lib, wl.uniform_distinct_topk(rng, 5000, 64, 4), 8, 64, 1, 16)


def test_static_layout_replays_in_a_graph(oracle):
    """What the entry point is for: captured in a HIP graph (no allocation, no memset node, the scratch
    address resolved by an eager call beforehand), every replay must give the eager result for the
    inputs of the moment, with eager work and synchronisations between the replays."""
    lib = _lib.load()
    T, K, R, E = 5000, 8, 8, 256                      # 20 tiles: static tiles, gathered scan
    topk = torch.empty((T, K), dtype=torch.int64, device=gu.DEV)
    out = LayoutOutputs(T, K, R, E, 16, lib)
    report = torch.zeros(1, dtype=torch.int32, device=gu.DEV)

    def launch(stream):
        _lib.check(lib.mi_ep_dispatch_layout_static(
            topk.data_ptr(), T, K, R, E, 4, 16, out.per_rank.data_ptr(), out.per_expert.data_ptr(),
            out.flags.data_ptr(), out.off.data_ptr(), out.psum.data_ptr(), out.channel_prefix.data_ptr(),
            out.rank_prefix.data_ptr(), out.slot_rel.data_ptr(), out.rank_slot_idx.data_ptr(), gu.RANK_SLOT_BASE,
            out.route_order.data_ptr(), out.tile_rank_counts.data_ptr(), None, None, report.data_ptr(), stream),
            "mi_ep_dispatch_layout_static")

    def load_inputs(seed):
        rng = np.random.default_rng(seed)
        t = wl.zipf_distinct_topk(rng, T, E, K, 1.2)
        t[rng.random((T, K)) < 0.05] = -1
        topk.copy_(torch.from_numpy(t))
        return t

    load_inputs(0)
    launch(torch.cuda.current_stream().cuda_stream)          # eager: resolves the scratch's address
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for seed in (1, 2, 3):
        t_np = load_inputs(seed)
        for t in out.tensors()[:-2]:                         # eager work between the replays
            t.view(torch.uint8).fill_(0x5A)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert int(report.item()) == 0
        per_rank, per_expert, flags = oracle.layout(t_np, R, E)
        off, psum = oracle.expert_offsets(per_expert, R, 4)
        slot_rel, _, _, _ = oracle.slot_maps(t_np, E, off)
        np.testing.assert_array_equal(out.per_rank.cpu().numpy(), per_rank)
        np.testing.assert_array_equal(out.per_expert.cpu().numpy(), per_expert)
        np.testing.assert_array_equal(out.flags.cpu().numpy()[:T], flags)
        np.testing.assert_array_equal(out.off.cpu().numpy(), off)
        np.testing.assert_array_equal(out.psum.cpu().numpy(), psum)
        np.testing.assert_array_equal(out.slot_rel.cpu().numpy(), slot_rel)
        np.testing.assert_array_equal(out.channel_prefix.cpu().numpy(), oracle.channel_prefix(flags, 16))
        np.testing.assert_array_equal(out.rank_prefix.cpu().numpy(),
                                      oracle.rank_prefix(gu.source_chunk_counts(flags, R)))
        np.testing.assert_array_equal(out.rank_slot_idx.cpu().numpy(),
                                      oracle.rank_slots(t_np, R, E, gu.RANK_SLOT_BASE))
    assert lib.mi_ep_workspace_status(_lib.STATIC_SCRATCH, torch.cuda.current_stream().cuda_stream) == 0
