"""GPU parity (through the C ABI) of the side outputs the reference's signatures carry next to the
main results: per-tile rank counts, the copied routing table, running per-expert statistics, the
expert ids that travel back through combine, scale factors through strides in the per-rank format,
the host-pointer twin of the fused layout; and the whole path at the shape the headline number is
quoted on, against the checker."""
import numpy as np
import pytest
import torch

from commbench_amd import ops
from commbench_amd import workloads as wl

from . import gpu_util as gu
from .test_gpu_dispatch_combine import combine_and_check, dispatch_and_check

pytestmark = pytest.mark.gpu


def _routing(seed, T, K, E, mask=0.05):
    rng = np.random.default_rng(seed)
    topk = wl.zipf_distinct_topk(rng, T, E, K, 1.2)
    topk[rng.random((T, K)) < mask] = -1
    return rng, topk


@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (300, 3, 4, 12), (4097, 8, 8, 256), (70000, 2, 8, 32)],
                         ids=lambda s: "x".join(map(str, s)))
def test_layout_side_outputs(oracle, shape):
    """tile_rank_counts (example078 .cu:34-35), copied_topk_idx (example080 .cu:33) and
    cumulative_expert_stats accumulated over launches (example080 .cu:211-212)."""
    T, K, R, E = shape
    print(f"shape {shape}", flush=True)
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    stats = torch.full((E,), 11, dtype=torch.int32, device=gu.DEV)
    want_stats = np.full(E, 11, dtype=np.int32)
    for launch in range(3):
        _, topk_np = _routing(100 * launch + T, T, K, E)
        topk = torch.from_numpy(topk_np).to(gu.DEV)
        h = buf.dispatch_layout(topk, tile_rank_counts=True, copy_topk_idx=True, cumulative_expert_stats=stats)
        torch.cuda.synchronize()
        buf.status()
        per_rank, per_expert, flags = oracle.layout(topk_np, R, E)
        np.testing.assert_array_equal(h.num_tokens_per_expert.cpu().numpy(), per_expert)
        np.testing.assert_array_equal(h.tile_rank_counts.cpu().numpy(), oracle.tile_rank_counts(flags, gu.TILE_TOKENS))
        np.testing.assert_array_equal(h.tile_rank_counts.cpu().numpy().sum(axis=0), per_rank)
        np.testing.assert_array_equal(h.copied_topk_idx.cpu().numpy(), topk_np)
        oracle.accumulate_stats(per_expert, want_stats)
        np.testing.assert_array_equal(stats.cpu().numpy(), want_stats)


def test_combine_returns_travelled_expert_ids(oracle):
    """combined_topk_idx (example083 .cu:26): the ids that dispatch stored with the rows come back
    per (token, slot), -1 for masked slots, next to the weights."""
    rng, topk_np = _routing(5, 900, 8, 64, mask=0.1)
    T, K = topk_np.shape
    w_np = wl.softmax_gates(rng, T, K)
    x_cpu = wl.bf16_normal(rng, T, 256)
    recv_x, h, ref = dispatch_and_check(oracle, (64, 8), topk_np, w_np, x_cpu, None, align=16)
    out, out_w, out_i = ops.combine(recv_x, h, None, recv_topk_weights=h.recv_topk_weights,
                                    recv_topk_idx=h.recv_topk_idx)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out_i.cpu().numpy(), oracle.gather_idx(ref["recv_topk_idx"], ref["slot_map"]))
    np.testing.assert_array_equal(out_i.cpu().numpy(), np.where(topk_np >= 0, topk_np, -1))
    np.testing.assert_array_equal(out_w.cpu().numpy(), oracle.gather_weights(ref["recv_topk_weights"], ref["slot_map"]))
    only_ids = ops.combine(recv_x, h, None, recv_topk_idx=h.recv_topk_idx)
    assert len(only_ids) == 2 and torch.equal(only_ids[1], out_i) and torch.equal(only_ids[0], out)


@pytest.mark.parametrize("local_ids", [False, True])
def test_rank_format_scales_through_strides_and_echoed_side_data(oracle, local_ids):
    """Per-rank format with the scale factors in a padded column-major tensor on the way in and
    column-major on the way out (recv_sf_token_stride / recv_sf_hidden_stride, example081 .cu:31),
    then the weights and ids that travelled, gathered back per route."""
    rng, topk_np = _routing(9, 777, 8, 32)
    T, K, E, R, H = 777, 8, 32, 8, 1024
    w_np = wl.softmax_gates(rng, T, K)
    xq, scales_cpu = wl.quantize_fp8_blockwise(wl.bf16_normal(rng, T, H))
    S = scales_cpu.shape[1]
    padded = torch.full((S, T + 13), -7.0, dtype=torch.float32, device=gu.DEV)
    padded[:, :T] = scales_cpu.t().to(gu.DEV)
    scales_view = padded[:, :T].t()
    assert scales_view.stride() == (1, T + 13)
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    topk = torch.from_numpy(topk_np).to(gu.DEV)
    recv_x, recv_idx, recv_w, rh = ops.dispatch_ranks(buf, xq.to(gu.DEV), scales_view, topk,
                                                      torch.from_numpy(w_np).to(gu.DEV), local_expert_ids=local_ids,
                                                      column_major_recv_scales=True)
    torch.cuda.synchronize()
    buf.status()
    ref = oracle.permute_ranks(gu.as_bytes(xq), scales_cpu.numpy(), topk_np, w_np, R, E, 0, local_ids)
    rows = rh.num_recv_rows()
    assert rows == ref["recv_x"].shape[0]
    assert rh.recv_scales.stride()[0] == 1
    np.testing.assert_array_equal(gu.as_bytes(recv_x)[:rows], ref["recv_x"])
    np.testing.assert_array_equal(rh.recv_scales.cpu().numpy()[:rows].view(np.uint32), ref["recv_scales"].view(np.uint32))
    np.testing.assert_array_equal(recv_idx.cpu().numpy()[:rows], ref["recv_topk_idx"])
    assert bool((padded[:, T:] == -7.0).all())
    # what travelled comes back per route
    y = torch.zeros((recv_x.shape[0], 64), dtype=torch.bfloat16, device=gu.DEV)
    out, out_w, out_i = ops.combine_ranks(y, rh, recv_w, recv_topk_idx=recv_idx)
    torch.cuda.synchronize()
    want_w, want_i = oracle.gather_rank_side(ref["recv_topk_weights"], ref["recv_topk_idx"], ref["rank_row_map"])
    np.testing.assert_array_equal(out_w.cpu().numpy().view(np.uint32), want_w.view(np.uint32))
    np.testing.assert_array_equal(out_i.cpu().numpy(), want_i)
    np.testing.assert_array_equal(out_w.cpu().numpy(), np.where(topk_np >= 0, w_np, 0).astype(np.float32))
    if not local_ids:
        np.testing.assert_array_equal(out_i.cpu().numpy(), np.where(topk_np >= 0, topk_np, -1))


@pytest.mark.parametrize("shape", [(257, 3, 4, 12), (4096, 8, 8, 256)], ids=lambda s: "x".join(map(str, s)))
def test_host_twin_of_the_fused_layout(oracle, shape):
    T, K, R, E = shape
    _, topk_np = _routing(T, T, K, E)
    stats = np.full(E, 5, dtype=np.int32)
    out = ops.host_dispatch_layout(topk_np, E, R, expert_alignment=16, num_channels=2 * R,
                                   rank_slot_base=gu.RANK_SLOT_BASE, cumulative_expert_stats=stats)
    per_rank, per_expert, flags = oracle.layout(topk_np, R, E)
    off, psum = oracle.expert_offsets(per_expert, R, 16)
    slot_rel, _, _, _ = oracle.slot_maps(topk_np, E, off)
    np.testing.assert_array_equal(out["num_tokens_per_rank"], per_rank)
    np.testing.assert_array_equal(out["num_tokens_per_expert"], per_expert)
    np.testing.assert_array_equal(out["is_token_in_rank"].view(np.uint8), flags)
    np.testing.assert_array_equal(out["expert_offsets"], off)
    np.testing.assert_array_equal(out["psum_rank_rows"], psum)
    np.testing.assert_array_equal(out["slot_rel"], slot_rel)
    np.testing.assert_array_equal(out["channel_prefix_matrix"], oracle.channel_prefix(flags, 2 * R))
    np.testing.assert_array_equal(out["rank_prefix_matrix"], oracle.rank_prefix(gu.source_chunk_counts(flags, R)))
    np.testing.assert_array_equal(out["rank_slot_idx"], oracle.rank_slots(topk_np, R, E, gu.RANK_SLOT_BASE))
    want_order = oracle.route_order(topk_np, E, gu.TILE_TOKENS, fill=0)
    np.testing.assert_array_equal(out["route_order"], want_order)
    np.testing.assert_array_equal(out["tile_rank_counts"], oracle.tile_rank_counts(flags, gu.TILE_TOKENS))
    np.testing.assert_array_equal(out["copied_topk_idx"], topk_np)
    np.testing.assert_array_equal(stats, 5 + per_expert)


def test_headline_shape_against_the_checker(oracle):
    """8192 x 7168 bf16, 256 experts, top-8 with the benchmark's own inputs: every output of layout
    and permute bit-exact under both copy kernels, combine within the tolerance."""
    cfg = wl.CONFIGS["target"]
    topk_np, w_np = wl.make_routing(cfg)
    x_cpu, _ = wl.make_payload(cfg)
    recv_x, h, ref = dispatch_and_check(oracle, (cfg.num_experts, cfg.num_ranks), topk_np, w_np, x_cpu, None)
    rows = int(ref["expert_offsets"][-1])
    assert rows == cfg.num_tokens * cfg.num_topk
    del recv_x
    y = wl.make_expert_outputs(cfg, rows).to(gu.DEV)
    combine_and_check(oracle, y, h.slot_map, w_np, ref["slot_map"])


def test_device_traits_match_the_part_the_copy_kernel_is_tuned_for():
    traits = ops.device_traits()
    print(f"traits {traits}", flush=True)
    assert traits["compute_units"] > 0
    # On the part these kernels target (8 dies, 4 MiB L2 each) long rows take the destination order;
    # anything else must fall back to the token order by itself.
    want = "destination" if traits["dies"] == 8 and traits["l2_bytes"] >= (4 << 20) else "token"
    assert ops.dispatch_schedule_for(8192, 8, 256, 14336) == want
    assert ops.dispatch_schedule_for(8192, 8, 256, 2048) == "token"


@pytest.mark.parametrize("zero_pads", [True, False])
def test_many_pad_rows_under_both_copy_kernels(oracle, zero_pads):
    """More pad rows than routes (256 experts padded to 128 rows, two routes per token): the pad
    rounds of the destination-order kernel and the pad units of the token-order kernel must write
    every pad row's markers, zero its payload and scales only when asked, and touch nothing else."""
    rng = np.random.default_rng(17)
    T, K, E, R, H, align = 2048, 2, 256, 8, 128, 128
    topk_np = wl.uniform_distinct_topk(rng, T, E, K)
    topk_np[rng.random((T, K)) < 0.05] = -1
    xq, scales_cpu = wl.quantize_fp8_blockwise(wl.bf16_normal(rng, T, H))
    ref = oracle.full_path(topk_np, None, gu.as_bytes(xq), scales_cpu.numpy(), E, R, align)
    rows = int(ref["expert_offsets"][-1])
    real = ref["recv_src_map"] >= 0
    assert (~real).sum() > real.sum()
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    topk = torch.from_numpy(topk_np).to(gu.DEV)
    h = buf.dispatch_layout(topk, align)
    cap = rows + 3                                                   # rows beyond the total stay untouched
    lib = ops._lib.load()
    x_dev, scales_dev = xq.to(gu.DEV), scales_cpu.to(gu.DEV)
    for schedule in gu.SCHEDULES:
        print(f"schedule {schedule} zero_pads {zero_pads}", flush=True)
        recv_x = gu.garbage_like(torch.empty((cap, H), dtype=torch.uint8, device=gu.DEV))
        recv_scales = torch.full((cap, 1), -3.0, dtype=torch.float32, device=gu.DEV)
        src_map = torch.full((cap,), 77, dtype=torch.int32, device=gu.DEV)
        recv_idx = torch.full((cap,), 77, dtype=torch.int64, device=gu.DEV)
        recv_w = torch.full((cap,), 77.0, dtype=torch.float32, device=gu.DEV)
        slot_map = torch.empty((T, K), dtype=torch.int32, device=gu.DEV)
        flags = (ops.ZERO_PAD_PAYLOAD if zero_pads else 0) | ops._SCHEDULE_FLAGS[schedule]
        ops._lib.check(lib.mi_ep_dispatch(
            x_dev.data_ptr(), scales_dev.data_ptr(), topk.data_ptr(), None,
            h.expert_offsets.data_ptr(), h.slot_rel.data_ptr(), h.route_order.data_ptr(),
            h.num_tokens_per_expert.data_ptr(), T, K, E, align, H, 1, recv_x.data_ptr(), recv_scales.data_ptr(),
            src_map.data_ptr(), recv_idx.data_ptr(), recv_w.data_ptr(), slot_map.data_ptr(), cap, flags,
            torch.cuda.current_stream().cuda_stream), "mi_ep_dispatch")
        torch.cuda.synchronize()
        np.testing.assert_array_equal(src_map.cpu().numpy()[:rows], ref["recv_src_map"])
        np.testing.assert_array_equal(recv_idx.cpu().numpy()[:rows], ref["recv_topk_idx"])
        np.testing.assert_array_equal(recv_w.cpu().numpy()[:rows], np.where(real, 1.0, 0.0).astype(np.float32))
        got_x, got_s = recv_x.cpu().numpy(), recv_scales.cpu().numpy()
        np.testing.assert_array_equal(got_x[:rows][real], ref["recv_x"][real])
        np.testing.assert_array_equal(got_s[:rows][real], ref["recv_scales"][real])
        if zero_pads:
            assert not got_x[:rows][~real].any() and not got_s[:rows][~real].any()
        else:
            assert (got_x[:rows][~real] == 0xA5).all() and (got_s[:rows][~real] == -3.0).all()
        assert (got_x[rows:] == 0xA5).all() and (src_map.cpu().numpy()[rows:] == 77).all()
