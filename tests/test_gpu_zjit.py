"""GPU parity of a library compiled at run time for fixed shapes (commbench_amd/jit.py): the mid-size
configuration through kernels that hold its shapes as constants, against the CPU checker."""
import numpy as np
import pytest
import torch

from commbench_amd import _lib, jit, ops
from commbench_amd import workloads as wl

from . import gpu_util as gu

pytestmark = pytest.mark.gpu


def test_fixed_shape_library_matches_the_checker_and_the_shipped_library(oracle):
    cfg = wl.CONFIGS["c3"]                                       # skewed routing, masked slots
    shapes = dict(num_topk=cfg.num_topk, num_experts=cfg.num_experts, num_ranks=cfg.num_ranks,
                  row_bytes=cfg.row_bytes, hidden=cfg.hidden)
    print(f"library for {shapes}: {jit.library_path(**shapes)}", flush=True)
    topk_np, w_np = wl.make_routing(cfg)
    x_cpu, _ = wl.make_payload(cfg)
    topk, w, x = torch.from_numpy(topk_np).to(gu.DEV), torch.from_numpy(w_np).to(gu.DEV), x_cpu.to(gu.DEV)

    def run():
        buf = ops.Buffer(cfg.num_tokens, cfg.num_topk, cfg.num_experts, cfg.num_ranks, device=gu.DEV)
        recv_x, _, src_map, h = buf.dispatch(x, None, topk, w, expert_alignment=16, num_channels=16, zero_pads=True)
        rows = h.num_recv_rows()
        out = ops.combine(recv_x[:rows].contiguous(), h, w)
        torch.cuda.synchronize()
        buf.status()
        return recv_x[:rows], src_map[:rows], h, out

    want_x, want_map, want_h, want_out = run()                   # the shipped library
    jit.activate(**shapes)
    try:
        got_x, got_map, got_h, got_out = run()
        # another shape is refused by this library
        with pytest.raises(_lib.MiEpError):
            ops.get_dispatch_layout(topk[:, :4].contiguous(), cfg.num_experts, cfg.num_ranks)
    finally:
        jit.deactivate()
    assert torch.equal(got_x, want_x) and torch.equal(got_map, want_map) and torch.equal(got_out, want_out)
    for name in ("num_tokens_per_rank", "num_tokens_per_expert", "is_token_in_rank", "expert_offsets", "psum_rank_rows",
                 "channel_prefix_matrix", "rank_prefix_matrix_", "slot_rel", "slot_map"):
        assert torch.equal(getattr(got_h, name), getattr(want_h, name)), name
    rows = got_x.shape[0]                                        # rows beyond the total are unspecified
    for name in ("recv_topk_idx", "recv_topk_weights"):
        assert torch.equal(getattr(got_h, name)[:rows], getattr(want_h, name)[:rows]), name
    ref = gu.check_layout_against_oracle(oracle, got_h, topk_np, cfg.num_ranks, cfg.num_experts, 16, 16)
    np.testing.assert_array_equal(got_h.slot_map.cpu().numpy(), ref["slot_map"])
    full = oracle.full_path(topk_np, w_np, gu.as_bytes(x_cpu), None, cfg.num_experts, cfg.num_ranks, 16)
    np.testing.assert_array_equal(gu.as_bytes(got_x), full["recv_x"])
    want_bits = oracle.combine(full["recv_x"].view(np.uint16), full["slot_map"], w_np, num_threads=8)
    assert gu.bf16_ulp_distance(gu.bf16_bits(got_out), want_bits).max() <= 2      # the bar; observed 0
