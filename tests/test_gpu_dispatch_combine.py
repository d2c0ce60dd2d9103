"""GPU parity of permute and combine (through the C ABI) against the CPU checker.

Bars: maps, side data and permuted payload bit-exact; combine within 2 bf16 ulp of the
fp32-accumulated host result (the kernel uses the same fused multiply-add chain, so the tests
also report whether it was bit-exact).
"""
import numpy as np
import pytest
import torch

from commbench_amd import ops
from commbench_amd import workloads as wl

from . import gpu_util as gu

pytestmark = pytest.mark.gpu

COMBINE_ULP_TOLERANCE = 2


def dispatch_and_check(oracle, cfg_or_shape, topk_np, w_np, x_cpu, scales_cpu, align=1):
    """Runs layout + permute on the GPU under both copy schedules (by token, by destination),
    compares everything with the checker each time, returns the last run and the checker's."""
    from commbench_amd import _lib
    T, K = topk_np.shape
    E, R = cfg_or_shape
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    topk = torch.from_numpy(topk_np).to(gu.DEV)
    w = torch.from_numpy(w_np).to(gu.DEV) if w_np is not None else None
    x = x_cpu.to(gu.DEV)
    scales = scales_cpu.to(gu.DEV) if scales_cpu is not None else None
    ref = oracle.full_path(topk_np, w_np, gu.as_bytes(x_cpu),
                           None if scales_cpu is None else scales_cpu.numpy(), E, R, align)
    rows = int(ref["expert_offsets"][-1])
    for schedule in gu.SCHEDULES:
        print(f"schedule {schedule}", flush=True)
        recv_x, recv_scales, recv_src_map, h = buf.dispatch(x, scales, topk, w, expert_alignment=align,
                                                            schedule=schedule, zero_pads=True)
        torch.cuda.synchronize()
        buf.status()
        assert h.num_recv_rows() == rows
        np.testing.assert_array_equal(h.slot_map.cpu().numpy(), ref["slot_map"])
        np.testing.assert_array_equal(recv_src_map.cpu().numpy()[:rows], ref["recv_src_map"])
        np.testing.assert_array_equal(h.recv_topk_idx.cpu().numpy()[:rows], ref["recv_topk_idx"])
        np.testing.assert_array_equal(gu.as_bytes(recv_x)[:rows], ref["recv_x"])
        if scales_cpu is not None:
            np.testing.assert_array_equal(recv_scales.cpu().numpy()[:rows].view(np.uint32),
                                          ref["recv_scales"].view(np.uint32))
        if w_np is not None:
            np.testing.assert_array_equal(h.recv_topk_weights.cpu().numpy()[:rows].view(np.uint32),
                                          ref["recv_topk_weights"].view(np.uint32))
    return recv_x, h, ref


def combine_and_check(oracle, y_gpu, slot_map_gpu, w_np, ref_slot_map, biases=(None, None)):
    w = torch.from_numpy(w_np).to(gu.DEV) if w_np is not None else None
    b_gpu = tuple(None if b is None else b.to(gu.DEV) for b in biases)
    out = ops.combine(y_gpu, slot_map_gpu, w, bias=b_gpu)
    torch.cuda.synchronize()
    want = oracle.combine(gu.bf16_bits(y_gpu), ref_slot_map, w_np,
                          *[None if b is None else gu.bf16_bits(b) for b in biases], num_threads=8)
    got = gu.bf16_bits(out)
    dist = gu.bf16_ulp_distance(got, want)
    assert dist.max() <= COMBINE_ULP_TOLERANCE, f"max distance {dist.max()} bf16 ulp"
    return got, want, int(dist.max())


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c5"])
def test_bf16_configs_dispatch_then_combine(oracle, name):
    cfg = wl.CONFIGS[name]
    print(f"config {name}", flush=True)
    topk_np, w_np = wl.make_routing(cfg)
    x_cpu, _ = wl.make_payload(cfg)
    recv_x, h, ref = dispatch_and_check(oracle, (cfg.num_experts, cfg.num_ranks), topk_np, w_np, x_cpu, None)
    rows = int(ref["expert_offsets"][-1])
    if cfg.expert_scale_denom > 0:
        # expert e multiplies its rows by 1 + e / denom (fp32 multiply, one rounding to bf16)
        e_of_row = h.recv_topk_idx[:rows].to(torch.float32)
        scale = 1.0 + e_of_row / cfg.expert_scale_denom
        y = (recv_x[:rows].to(torch.float32) * scale[:, None]).to(torch.bfloat16)
        want_y = oracle.scale_rows_by_expert(ref["recv_x"].view(np.uint16), ref["expert_offsets"],
                                             cfg.expert_scale_denom, num_threads=8)
        np.testing.assert_array_equal(gu.bf16_bits(y), want_y)
    else:
        y = recv_x[:rows]                         # identity experts
    got, want, worst = combine_and_check(oracle, y.contiguous(), h.slot_map, w_np, ref["slot_map"])
    print(f"{name}: combine max distance {worst} ulp, bit-exact={bool((got == want).all())}", flush=True)
    if cfg.expert_scale_denom == 0 and cfg.mask_prob == 0:
        # identity experts + gates summing to 1: the round trip returns x to within 2 ulp
        xb = gu.bf16_bits(x_cpu)
        assert gu.bf16_ulp_distance(got, xb).max() <= 2


def test_fp8_config_with_scales(oracle):
    cfg = wl.CONFIGS["c4"]
    topk_np, w_np = wl.make_routing(cfg)
    q_cpu, scales_cpu = wl.make_payload(cfg)
    assert q_cpu.dtype == torch.float8_e4m3fn and scales_cpu.shape == (cfg.num_tokens, 56)
    _, h, ref = dispatch_and_check(oracle, (cfg.num_experts, cfg.num_ranks), topk_np, w_np, q_cpu, scales_cpu)
    rows = int(ref["expert_offsets"][-1])
    y = wl.make_expert_outputs(cfg, rows).to(gu.DEV)          # combine consumes fresh bf16 outputs
    combine_and_check(oracle, y, h.slot_map, w_np, ref["slot_map"])


@pytest.mark.parametrize("align", [2, 128])
def test_alignment_pads_are_zero_rows(oracle, align):
    rng = np.random.default_rng(align)
    T, K, E, R, H = 777, 8, 64, 8, 512
    topk_np = wl.zipf_distinct_topk(rng, T, E, K, 1.2)
    topk_np[rng.random((T, K)) < 0.05] = -1
    w_np = wl.softmax_gates(rng, T, K)
    x_cpu = wl.bf16_normal(rng, T, H)
    recv_x, h, ref = dispatch_and_check(oracle, (E, R), topk_np, w_np, x_cpu, None, align=align)
    off = ref["expert_offsets"]
    assert (off % align == 0).all()
    pads = ref["recv_src_map"] < 0
    assert pads.any() and not gu.as_bytes(recv_x)[:off[-1]][pads].any()


def test_huge_alignment_beyond_the_destination_order_grid(oracle):
    """An alignment so large that the zeroed pad rows of a tile no longer fit the destination-order
    kernel's grid (65535 list entries per tile): the call must fall back to the token-order kernel by
    itself, with the same outputs, under either schedule flag."""
    rng = np.random.default_rng(41)
    T, K, E, R, H, align = 300, 2, 8, 2, 8, 40000                 # 16-byte rows, 320 000 possible pad rows
    topk_np = wl.uniform_distinct_topk(rng, T, E, K)
    w_np = wl.softmax_gates(rng, T, K)
    x_cpu = wl.bf16_normal(rng, T, H)
    recv_x, h, ref = dispatch_and_check(oracle, (E, R), topk_np, w_np, x_cpu, None, align=align)
    assert int(ref["expert_offsets"][-1]) == E * align and (ref["recv_src_map"] < 0).sum() == E * align - T * K


@pytest.mark.parametrize("schedule", gu.SCHEDULES)
def test_scale_factors_through_strides(oracle, schedule):
    """Scale factors in a column-major, padded tensor on the way in and column-major on the way out
    (the reference addresses them through token and hidden strides, example080 .cu:40)."""
    from commbench_amd import _lib
    rng = np.random.default_rng(40)
    T, K, E, R, H, align = 777, 8, 32, 8, 1024, 16
    topk_np = wl.uniform_distinct_topk(rng, T, E, K)
    topk_np[rng.random((T, K)) < 0.05] = -1
    xq, scales_cpu = wl.quantize_fp8_blockwise(wl.bf16_normal(rng, T, H))
    S = scales_cpu.shape[1]
    padded = torch.full((S, T + 19), -7.0, dtype=torch.float32, device=gu.DEV)   # [S, T padded], column-major view
    padded[:, :T] = scales_cpu.t().to(gu.DEV)
    scales_view = padded[:, :T].t()
    assert not scales_view.is_contiguous() and scales_view.stride() == (1, T + 19)
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    recv_x, recv_scales, _, h = buf.dispatch(xq.to(gu.DEV), scales_view, torch.from_numpy(topk_np).to(gu.DEV),
                                             None, expert_alignment=align, column_major_recv_scales=True,
                                             schedule=schedule, zero_pads=True)
    torch.cuda.synchronize()
    ref = oracle.full_path(topk_np, None, gu.as_bytes(xq), scales_cpu.numpy(), E, R, align)
    rows = int(ref["expert_offsets"][-1])
    assert recv_scales.stride()[0] == 1                                    # column-major as asked
    np.testing.assert_array_equal(gu.as_bytes(recv_x)[:rows], ref["recv_x"])
    np.testing.assert_array_equal(recv_scales.cpu().numpy()[:rows].view(np.uint32), ref["recv_scales"].view(np.uint32))
    assert (padded[:, T:] == -7.0).all()                                   # the padding was not touched


def test_pad_payload_is_left_alone_unless_asked_for_zeros(oracle):
    """By default the pad rows keep what the buffer held (the reference's receive buffer is not
    cleared either); their map entries and every real row are written as usual.  With zero_pads the
    pad rows are zero rows."""
    rng = np.random.default_rng(6)
    T, K, E, R, H, align = 600, 4, 32, 4, 128, 16
    topk_np = wl.uniform_distinct_topk(rng, T, E, K)
    x_cpu = wl.bf16_normal(rng, T, H)
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    h = buf.dispatch_layout(torch.from_numpy(topk_np).to(gu.DEV), align)
    # same layout handle, once with zero-filled pads and once with the pad payload left alone
    filled = buf.dispatch(x_cpu.to(gu.DEV), None, torch.from_numpy(topk_np).to(gu.DEV), None, align, handle=h,
                          zero_pads=True)
    kept = buf.dispatch(x_cpu.to(gu.DEV), None, torch.from_numpy(topk_np).to(gu.DEV), None, align, handle=h)
    torch.cuda.synchronize()
    ref = oracle.full_path(topk_np, None, gu.as_bytes(x_cpu), None, E, R, align)
    rows = int(ref["expert_offsets"][-1])
    real = ref["recv_src_map"] >= 0
    assert (~real).any()
    for recv_x, _, src_map, hh in (filled, kept):
        np.testing.assert_array_equal(src_map.cpu().numpy()[:rows], ref["recv_src_map"])
        np.testing.assert_array_equal(hh.recv_topk_idx.cpu().numpy()[:rows], ref["recv_topk_idx"])
        np.testing.assert_array_equal(gu.as_bytes(recv_x)[:rows][real], ref["recv_x"][real])
    assert not gu.as_bytes(filled[0])[:rows][~real].any()


@pytest.mark.parametrize("shape", [
    # T, K, E, R, row_bytes, num_scales
    (1, 1, 1, 1, 16, 0), (5, 3, 6, 2, 48, 1), (300, 8, 32, 4, 1024, 8), (300, 8, 32, 4, 1040, 0),
    (129, 2, 8, 8, 2064, 70), (64, 7, 1024, 8, 14336, 0)], ids=lambda s: "x".join(map(str, s)))
def test_permute_ragged_shapes(oracle, shape):
    T, K, E, R, row_bytes, S = shape
    print(f"shape {shape}", flush=True)
    rng = np.random.default_rng(sum(shape))
    topk_np = rng.integers(-1, E, size=(T, K)).astype(np.int64)
    w_np = rng.standard_normal((T, K)).astype(np.float32)
    x_cpu = torch.from_numpy(rng.integers(0, 256, size=(T, row_bytes), dtype=np.uint8))
    scales_cpu = torch.from_numpy(rng.standard_normal((T, S)).astype(np.float32)) if S else None
    dispatch_and_check(oracle, (E, R), topk_np, w_np, x_cpu, scales_cpu, align=1)


@pytest.mark.parametrize("seed", range(12))
def test_permute_random_shapes(oracle, seed):
    """Shapes drawn at random (tile remainders, tile counts that do not divide by eight, masked and
    out-of-range ids, duplicates, alignment pads, scales), both copy kernels, bit-exact."""
    rng = np.random.default_rng(1000 + seed)
    T = int(rng.integers(1, 6000))
    K = int(rng.integers(1, 9))
    R = int(rng.choice([1, 2, 4, 8]))
    E = R * int(rng.integers(1, 1024 // R + 1 if seed % 3 == 0 else 17))
    row_bytes = 16 * int(rng.integers(1, 80))
    S = int(rng.integers(0, 9))
    align = int(rng.choice([1, 1, 3, 16, 128]))
    print(f"seed {seed}: T={T} K={K} R={R} E={E} row_bytes={row_bytes} S={S} align={align}", flush=True)
    topk_np = rng.integers(-2, E + 2, size=(T, K)).astype(np.int64)
    w_np = rng.standard_normal((T, K)).astype(np.float32)
    x_cpu = torch.from_numpy(rng.integers(0, 256, size=(T, row_bytes), dtype=np.uint8))
    scales_cpu = torch.from_numpy(rng.standard_normal((T, S)).astype(np.float32)) if S else None
    dispatch_and_check(oracle, (E, R), topk_np, w_np, x_cpu, scales_cpu, align=align)


@pytest.mark.parametrize("shape", [
    # T, K, E, R, row_bytes, num_scales, alignment: rows on both sides of every workgroup shape of the
    # destination-order kernel (one workgroup of up to twelve waves per row; 2 KiB parts above 12 KiB)
    (700, 8, 32, 8, 5136, 3, 1), (700, 8, 32, 8, 12288, 0, 16), (520, 8, 32, 8, 12304, 5, 1),
    (520, 4, 16, 4, 14352, 0, 128), (300, 8, 16, 8, 20000, 2, 3), (900, 8, 64, 8, 4096, 32, 128)],
    ids=lambda s: "x".join(map(str, s)))
def test_permute_row_sizes_around_the_workgroup_shapes(oracle, shape):
    T, K, E, R, row_bytes, S, align = shape
    print(f"shape {shape}", flush=True)
    rng = np.random.default_rng(sum(shape))
    topk_np = rng.integers(-1, E, size=(T, K)).astype(np.int64)
    w_np = rng.standard_normal((T, K)).astype(np.float32)
    x_cpu = torch.from_numpy(rng.integers(0, 256, size=(T, row_bytes), dtype=np.uint8))
    scales_cpu = torch.from_numpy(rng.standard_normal((T, S)).astype(np.float32)) if S else None
    dispatch_and_check(oracle, (E, R), topk_np, w_np, x_cpu, scales_cpu, align=align)


def test_capacity_limits_writes(oracle):
    """Rows at or beyond capacity_rows are dropped: never written, slot_map = -1."""
    rng = np.random.default_rng(3)
    T, K, E, R, H = 200, 4, 16, 4, 64
    topk_np = wl.uniform_distinct_topk(rng, T, E, K)
    x = wl.bf16_normal(rng, T, H).to(gu.DEV)
    topk = torch.from_numpy(topk_np).to(gu.DEV)
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    cap = 500
    recv_x, _, src_map, h = buf.dispatch(x, None, topk, None, capacity_rows=cap)
    torch.cuda.synchronize()
    ref = oracle.full_path(topk_np, None, gu.as_bytes(x), None, E, R)
    want_slots = np.where(ref["slot_map"] < cap, ref["slot_map"], -1)
    np.testing.assert_array_equal(h.slot_map.cpu().numpy(), want_slots)
    np.testing.assert_array_equal(gu.as_bytes(recv_x), ref["recv_x"][:cap])
    np.testing.assert_array_equal(src_map.cpu().numpy(), ref["recv_src_map"][:cap])


@pytest.mark.parametrize("K", [1, 2, 3, 4, 5, 6, 7, 8])
def test_combine_every_topk_with_biases(oracle, K):
    rng = np.random.default_rng(K)
    T, E, R, H = 333, 32, 4, 1096            # 137 vectors per row: ragged last batch
    topk_np = wl.uniform_distinct_topk(rng, T, E, K)
    topk_np[rng.random((T, K)) < 0.15] = -1
    w_np = wl.softmax_gates(rng, T, K)
    _, per_expert, _ = oracle.layout(topk_np, R, E)
    off, _ = oracle.expert_offsets(per_expert, R, 1)
    _, slot_map, _, _ = oracle.slot_maps(topk_np, E, off)
    y = wl.bf16_normal(rng, int(off[-1]) + 3, H).to(gu.DEV)
    b0, b1 = wl.bf16_normal(rng, T, H), wl.bf16_normal(rng, T, H)
    sm = torch.from_numpy(slot_map).to(gu.DEV)
    for weights, biases in ((w_np, (None, None)), (None, (None, None)), (w_np, (b0, None)), (w_np, (b0, b1))):
        got, want, worst = combine_and_check(oracle, y, sm, weights, slot_map, biases)
        assert worst == 0, "same fma chain on both sides: expected bit-exact"


@pytest.mark.parametrize("shape", [(4099, 3, 1032), (6000, 8, 2048), (4096, 1, 1024), (9001, 5, 1280),
                                   (4099, 2, 5000), (5000, 8, 4232), (4100, 4, 7168)],
                         ids=lambda s: "x".join(map(str, s)))
def test_combine_large_token_counts_use_the_staged_schedule(oracle, shape):
    """>= 16 tokens per compute unit and rows >= 2 KiB take the persistent LDS-staged schedule:
    ragged token ranges, ragged last vectors, masks, weights on/off and both biases.  The last three
    shapes need more staging than the LDS holds for a single burst (170, 180 and 238 KiB per
    workgroup): the first two put the rest in registers, the third takes two bursts."""
    T, K, H = shape
    print(f"shape {shape}", flush=True)
    rng = np.random.default_rng(T + K)
    E, R = 64, 8
    topk_np = wl.uniform_distinct_topk(rng, T, E, K)
    topk_np[rng.random((T, K)) < 0.1] = -1
    topk_np[5] = -1                                   # a token with no routes at all
    w_np = wl.softmax_gates(rng, T, K)
    _, per_expert, _ = oracle.layout(topk_np, R, E)
    off, _ = oracle.expert_offsets(per_expert, R, 1)
    _, slot_map, _, _ = oracle.slot_maps(topk_np, E, off)
    y = wl.bf16_normal(rng, int(off[-1]), H).to(gu.DEV)
    b0, b1 = wl.bf16_normal(rng, T, H), wl.bf16_normal(rng, T, H)
    sm = torch.from_numpy(slot_map).to(gu.DEV)
    for weights, biases in ((w_np, (None, None)), (None, (b0, b1))):
        got, want, worst = combine_and_check(oracle, y, sm, weights, slot_map, biases)
        assert worst == 0


def test_combine_integer_payload_is_exact(oracle):
    rng = np.random.default_rng(21)
    T, K, E, R, H = 500, 8, 64, 8, 256
    topk_np = wl.uniform_distinct_topk(rng, T, E, K)
    _, per_expert, _ = oracle.layout(topk_np, R, E)
    off, _ = oracle.expert_offsets(per_expert, R, 1)
    _, slot_map, _, _ = oracle.slot_maps(topk_np, E, off)
    y_int = rng.integers(-15, 16, size=(int(off[-1]), H))
    y = torch.from_numpy(y_int.astype(np.float32)).to(torch.bfloat16).to(gu.DEV)
    out = ops.combine(y, torch.from_numpy(slot_map).to(gu.DEV), None)
    want = y_int[slot_map.reshape(-1)].reshape(T, K, H).sum(axis=1)
    np.testing.assert_array_equal(out.to(torch.float32).cpu().numpy(), want)


def test_combine_returns_travelled_weights(oracle):
    """The reference's harness expects combined_topk_weights == topk_weights
    (example082 build_and_run.py:764-765); masked slots come back as 0."""
    rng = np.random.default_rng(8)
    T, K, E, R, H = 257, 8, 64, 8, 128
    topk_np = wl.uniform_distinct_topk(rng, T, E, K)
    topk_np[rng.random((T, K)) < 0.1] = -1
    w_np = wl.softmax_gates(rng, T, K)
    x_cpu = wl.bf16_normal(rng, T, H)
    recv_x, h, ref = dispatch_and_check(oracle, (E, R), topk_np, w_np, x_cpu, None)
    rows = int(ref["expert_offsets"][-1])
    out, out_w = ops.combine(recv_x[:rows].contiguous(), h, None, recv_topk_weights=h.recv_topk_weights)
    want_w = np.where(topk_np >= 0, w_np, 0).astype(np.float32)
    np.testing.assert_array_equal(out_w.cpu().numpy().view(np.uint32), want_w.view(np.uint32))
    np.testing.assert_array_equal(out_w.cpu().numpy(), oracle.gather_weights(ref["recv_topk_weights"], ref["slot_map"]))


def test_full_size_properties_without_the_checker():
    """Target shape (8192 x 7168 bf16, 256 experts, top-8): properties that need no CPU pass.
    K = 8 distinct experts, gates = 1/8 exactly: permute then combine returns x bit-for-bit
    (eight equal fma steps of x/8 are exact in fp32), every row is written exactly once."""
    cfg = wl.CONFIGS["target"]
    T, K, E, R, H = cfg.num_tokens, cfg.num_topk, cfg.num_experts, cfg.num_ranks, cfg.hidden
    topk_np, _ = wl.make_routing(cfg)
    gen = torch.Generator(device=gu.DEV).manual_seed(1)
    x = torch.randn((T, H), device=gu.DEV, generator=gen, dtype=torch.float32).to(torch.bfloat16)
    topk = torch.from_numpy(topk_np).to(gu.DEV)
    w = torch.full((T, K), 0.125, dtype=torch.float32, device=gu.DEV)
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    recv_x, _, src_map, h = buf.dispatch(x, None, topk, w)
    torch.cuda.synchronize()
    assert h.num_recv_rows() == T * K
    sm = h.slot_map.reshape(-1).to(torch.int64)
    assert torch.equal(torch.sort(sm).values, torch.arange(T * K, device=gu.DEV))   # a permutation
    assert torch.equal(src_map.to(torch.int64)[sm], torch.arange(T * K, device=gu.DEV) // K)
    assert torch.equal(recv_x.view(torch.int16)[sm[::K]], x.view(torch.int16))     # slot 0 rows
    seg = h.recv_topk_idx[:T * K]
    assert torch.equal(seg, torch.sort(seg).values)                                 # expert-contiguous
    assert torch.equal(torch.bincount(seg, minlength=E).to(torch.int32), h.num_tokens_per_expert)
    out = ops.combine(recv_x, h, w)
    assert torch.equal(out.view(torch.int16), x.view(torch.int16))


@pytest.mark.parametrize("payload", ["bf16", "fp8"])
def test_cached_pull_dispatch_and_pull_indices(oracle, payload):
    """Pull-mode dispatch with the map of an earlier dispatch must reproduce that dispatch
    (fresh payload, same routing), pads zero; pull indices in the ThunderKittens example's format."""
    rng = np.random.default_rng(31)
    T, K, E, R, H, align = 1500, 8, 64, 8, 2048, 128
    topk_np = wl.zipf_distinct_topk(rng, T, E, K, 1.2)
    topk_np[rng.random((T, K)) < 0.05] = -1
    x_cpu = wl.bf16_normal(rng, T, H)
    scales_cpu = None
    if payload == "fp8":
        x_cpu, scales_cpu = wl.quantize_fp8_blockwise(x_cpu)
    recv_x, h, ref = dispatch_and_check(oracle, (E, R), topk_np, None, x_cpu, scales_cpu, align=align)
    rows = int(ref["expert_offsets"][-1])
    x2 = wl.bf16_normal(rng, T, H)
    s2 = None
    if payload == "fp8":
        x2, s2 = wl.quantize_fp8_blockwise(x2)
    got_x, got_s = ops.dispatch_cached(x2.to(gu.DEV), None if s2 is None else s2.to(gu.DEV),
                                       h.recv_src_map, num_rows=rows)
    want_x, want_s = oracle.gather_rows(gu.as_bytes(x2), None if s2 is None else s2.numpy(), ref["recv_src_map"])
    np.testing.assert_array_equal(gu.as_bytes(got_x), want_x)
    if s2 is not None:
        np.testing.assert_array_equal(got_s.cpu().numpy().view(np.uint32), want_s.view(np.uint32))
    # the same pull with arrival counters: same rows, every 128-row block counted in full
    ready = torch.zeros((rows + 127) // 128, dtype=torch.int32, device=gu.DEV)
    got_x2, got_s2 = ops.dispatch_cached(x2.to(gu.DEV), None if s2 is None else s2.to(gu.DEV),
                                         h.recv_src_map, num_rows=rows, ready_counters=ready)
    np.testing.assert_array_equal(gu.as_bytes(got_x2), want_x)
    if s2 is not None:
        np.testing.assert_array_equal(got_s2.cpu().numpy().view(np.uint32), want_s.view(np.uint32))
    want_ready = np.minimum(128, rows - 128 * np.arange(ready.numel())).astype(np.int32)
    np.testing.assert_array_equal(ready.cpu().numpy(), want_ready)
    # and with the first payload it is the first dispatch again
    again, _ = ops.dispatch_cached(x_cpu.to(gu.DEV), None if scales_cpu is None else scales_cpu.to(gu.DEV),
                                   h.recv_src_map, num_rows=rows)
    np.testing.assert_array_equal(gu.as_bytes(again), ref["recv_x"])
    pulls = ops.pull_indices(h.recv_src_map, T // 4, num_rows=rows)
    np.testing.assert_array_equal(pulls.cpu().numpy(), oracle.pull_indices(ref["recv_src_map"], T // 4))


@pytest.mark.parametrize("shape", [(4096, 8), (4097, 8), (7, 2), (1000, 4), (333, 8), (5, 8)],
                         ids=lambda s: "x".join(map(str, s)))
def test_rank_prefix_matrix_from_channel_prefix(oracle, shape):
    """The launch's rank_prefix_matrix[src, dst] is the notify example's (example047 .cu:352-360) for
    R contiguous source chunks of ceil(T / R) tokens (its get_channel_task_range, .cu:73-79), ragged
    and empty chunks included; with one channel per source chunk it is also the transposed channel
    matrix of the same launch."""
    T, R = shape
    print(f"shape {shape}", flush=True)
    rng = np.random.default_rng(5 + T)
    K, E = 4, 4 * R
    topk_np = wl.uniform_distinct_topk(rng, T, E, K)
    topk_np[rng.random((T, K)) < 0.3] = -1
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    h = buf.dispatch_layout(torch.from_numpy(topk_np).to(gu.DEV), num_channels=R)
    torch.cuda.synchronize()
    _, _, flags = oracle.layout(topk_np, R, E)
    counts = gu.source_chunk_counts(flags, R)
    np.testing.assert_array_equal(h.rank_prefix_matrix().cpu().numpy(), oracle.rank_prefix(counts))
    np.testing.assert_array_equal(h.rank_prefix_matrix().cpu().numpy(), h.channel_prefix_matrix.t().cpu().numpy())
    assert (h.rank_prefix_matrix()[-1].cpu().numpy() == h.num_tokens_per_rank.cpu().numpy()).all()


def test_combine_ignores_map_entries_beyond_the_rows_it_was_given(oracle):
    """Memory safety: a map entry at or beyond y's row count is treated as a non-route, never read."""
    rng = np.random.default_rng(41)
    T, K, E, R, H = 600, 4, 16, 4, 256
    topk_np = wl.uniform_distinct_topk(rng, T, E, K)
    w_np = wl.softmax_gates(rng, T, K)
    _, per_expert, _ = oracle.layout(topk_np, R, E)
    off, _ = oracle.expert_offsets(per_expert, R, 1)
    _, slot_map, _, _ = oracle.slot_maps(topk_np, E, off)
    rows_given = int(off[-1]) // 2
    y = wl.bf16_normal(rng, rows_given, H).to(gu.DEV)
    out = ops.combine(y, torch.from_numpy(slot_map).to(gu.DEV), torch.from_numpy(w_np).to(gu.DEV))
    torch.cuda.synchronize()
    clipped = np.where(slot_map < rows_given, slot_map, -1).astype(np.int32)
    want = oracle.combine(gu.bf16_bits(y), clipped, w_np)
    np.testing.assert_array_equal(gu.bf16_bits(out), want)


@pytest.mark.parametrize("kind", ["one_expert", "two_experts_alternating", "last_expert_only"])
def test_extreme_skew_round_trip(oracle, kind):
    """Every route on one or two experts (with duplicates inside each token): one giant segment,
    every lane of every wave in the same ballot group."""
    T, K, E, R, H = 3000, 8, 64, 8, 512
    if kind == "one_expert":
        topk_np = np.full((T, K), 5, dtype=np.int64)
    elif kind == "two_experts_alternating":
        topk_np = np.tile(np.array([7, 40] * (K // 2), dtype=np.int64), (T, 1))
    else:
        topk_np = np.full((T, K), -1, dtype=np.int64)
        topk_np[:, K - 1] = E - 1
    rng = np.random.default_rng(9)
    w_np = wl.softmax_gates(rng, T, K)
    x_cpu = wl.bf16_normal(rng, T, H)
    recv_x, h, ref = dispatch_and_check(oracle, (E, R), topk_np, w_np, x_cpu, None, align=128)
    rows = int(ref["expert_offsets"][-1])
    got, want, worst = combine_and_check(oracle, recv_x[:rows].contiguous(), h.slot_map, w_np, ref["slot_map"])
    assert worst == 0


def test_combine_denormals_infinities_and_nans(oracle):
    """Special values go through the same arithmetic on both sides: fp32 denormals are kept, an
    infinity times a zero weight is NaN, NaNs stay NaNs (quiet bit set), signed zeros survive."""
    rng = np.random.default_rng(23)
    T, K, E, R, H = 400, 4, 16, 4, 64
    topk_np = wl.uniform_distinct_topk(rng, T, E, K)
    _, per_expert, _ = oracle.layout(topk_np, R, E)
    off, _ = oracle.expert_offsets(per_expert, R, 1)
    _, slot_map, _, _ = oracle.slot_maps(topk_np, E, off)
    rows = int(off[-1])
    specials = np.array([0x0000, 0x8000, 0x0001, 0x8001, 0x007F, 0x0080, 0x7F7F, 0xFF7F, 0x7F80, 0xFF80,
                         0x7FC0, 0x7F81, 0x3F80, 0xBF80], dtype=np.uint16)
    y_bits = specials[rng.integers(0, specials.size, size=(rows, H))]
    y = torch.from_numpy(y_bits.view(np.int16)).view(torch.bfloat16).to(gu.DEV)
    w_np = rng.choice(np.array([0.0, -0.0, 0.5, 1.0, 2.0 ** -20, -3.0], dtype=np.float32), size=(T, K))
    out = ops.combine(y, torch.from_numpy(slot_map).to(gu.DEV), torch.from_numpy(w_np).to(gu.DEV))
    torch.cuda.synchronize()
    want = oracle.combine(y_bits, slot_map, w_np)
    got = gu.bf16_bits(out)
    is_nan = lambda b: ((b & 0x7F80) == 0x7F80) & ((b & 0x007F) != 0)
    np.testing.assert_array_equal(is_nan(got), is_nan(want))
    keep = ~is_nan(want)
    np.testing.assert_array_equal(got[keep], want[keep])
    assert is_nan(want).any() and ((want & 0x7F80) == 0).any()      # the case really has both
