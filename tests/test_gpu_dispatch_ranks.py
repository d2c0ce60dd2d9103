"""GPU parity of the per-rank dispatch format (one row per token and destination rank) and its
combine, through the C ABI, against the CPU checker: bit-exact maps, ids, weights, metadata and
payload; combine within 2 bf16 ulp."""
import numpy as np
import pytest
import torch

from commbench_amd import ops
from commbench_amd import workloads as wl

from . import gpu_util as gu

pytestmark = pytest.mark.gpu


def run_and_check(oracle, topk_np, w_np, x_cpu, scales_cpu, E, R, local_ids=False, expand=False,
                  rank_idx=0, max_tokens=None):
    T, K = topk_np.shape
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    topk = torch.from_numpy(topk_np).to(gu.DEV)
    w = None if w_np is None else torch.from_numpy(w_np).to(gu.DEV)
    x = x_cpu.to(gu.DEV)
    scales = None if scales_cpu is None else scales_cpu.to(gu.DEV)
    recv_x, recv_idx, recv_w, h = ops.dispatch_ranks(buf, x, scales, topk, w, max_tokens, rank_idx,
                                                     local_ids, expand)
    torch.cuda.synchronize()
    buf.status()
    base = rank_idx * (T if max_tokens is None else max_tokens)
    expand_map = None
    if expand:
        _, per_expert, _ = oracle.layout(topk_np, R, E)
        off, _ = oracle.expert_offsets(per_expert, R, 1)
        _, expand_map, _, _ = oracle.slot_maps(topk_np, E, off)
        np.testing.assert_array_equal(h.layout.slot_map.cpu().numpy(), expand_map)
    ref = oracle.permute_ranks(gu.as_bytes(x_cpu), None if scales_cpu is None else scales_cpu.numpy(), topk_np,
                               w_np, R, E, base, local_ids, expand_map)
    rows = int(ref["psum_rank_tokens"][-1])
    assert h.num_recv_rows() == rows
    np.testing.assert_array_equal(h.psum_rank_tokens.cpu().numpy(), ref["psum_rank_tokens"])
    np.testing.assert_array_equal(h.rank_row_map.cpu().numpy(), ref["rank_row_map"])
    first = oracle.rank_slots(topk_np, R, E, 0) >= 0
    np.testing.assert_array_equal(h.combine_map.cpu().numpy(), np.where(first, ref["rank_row_map"], -1))
    np.testing.assert_array_equal(gu.as_bytes(recv_x)[:rows], ref["recv_x"])
    np.testing.assert_array_equal(recv_idx.cpu().numpy()[:rows], ref["recv_topk_idx"])
    np.testing.assert_array_equal(recv_w.cpu().numpy()[:rows].view(np.uint32), ref["recv_topk_weights"].view(np.uint32))
    np.testing.assert_array_equal(h.recv_src_metadata.cpu().numpy()[:rows], ref["recv_src_metadata"])
    if scales_cpu is not None:
        np.testing.assert_array_equal(h.recv_scales.cpu().numpy()[:rows].view(np.uint32),
                                      ref["recv_scales"].view(np.uint32))
    return recv_x, recv_idx, recv_w, h, ref


@pytest.mark.parametrize("local_ids", [False, True])
@pytest.mark.parametrize("shape", [(1, 1, 1, 1, 16), (64, 8, 4, 16, 256), (300, 8, 8, 64, 1032), (257, 3, 2, 10, 72),
                                   (4099, 8, 8, 256, 512)], ids=lambda s: "x".join(map(str, s)))
def test_dispatch_ranks_ragged_shapes(oracle, shape, local_ids):
    T, K, R, E, H = shape
    print(f"shape {shape} local_ids {local_ids}", flush=True)
    rng = np.random.default_rng(T * 3 + K)
    topk_np = rng.integers(-2, E + 1, size=(T, K)).astype(np.int64)      # masks, out of range, duplicates
    w_np = rng.random((T, K), dtype=np.float32)
    x_cpu = wl.bf16_normal(rng, T, H)
    run_and_check(oracle, topk_np, w_np, x_cpu, None, E, R, local_ids, expand=(T % 2 == 0), rank_idx=3,
                  max_tokens=T + 5)


def test_dispatch_ranks_reference_harness_shape_then_combine(oracle):
    """The JIT examples' default shape (512 x 256, top-2 of 64 experts, 8 ranks) with the
    reference harness's checks (example080 bar.py:728-748, example082 bar.py:757-765)."""
    rng = np.random.default_rng(82)
    T, H, K, E, R = 512, 256, 2, 64, 8
    topk_np = wl.uniform_distinct_topk(rng, T, E, K)
    w_np = wl.softmax_gates(rng, T, K)
    x_cpu = wl.bf16_normal(rng, T, H)
    recv_x, recv_idx, recv_w, h, ref = run_and_check(oracle, topk_np, w_np, x_cpu, None, E, R)
    rows = h.num_recv_rows()
    meta = h.recv_src_metadata[:rows]
    order = torch.sort(meta[:, 0], stable=True).indices
    # every received row is its source token's row
    assert torch.equal(recv_x[:rows][order], x_cpu.to(gu.DEV)[meta[:, 0][order].long()])
    # combine: "expert outputs" = the received rows themselves, so a token gets (number of ranks) * x
    out, out_w = ops.combine_ranks(recv_x, h, recv_w)
    torch.cuda.synchronize()
    want = oracle.combine(gu.bf16_bits(recv_x), np.where(oracle.rank_slots(topk_np, R, E, 0) >= 0,
                                                         ref["rank_row_map"], -1))
    assert gu.bf16_ulp_distance(gu.bf16_bits(out), want).max() <= 2
    ranks_per_token = torch.from_numpy((oracle.rank_slots(topk_np, R, E, 0) >= 0).sum(axis=1)).to(gu.DEV)
    exact = (x_cpu.to(gu.DEV).float() * ranks_per_token[:, None]).to(torch.bfloat16)
    assert torch.equal(out.view(torch.int16), exact.view(torch.int16))       # 1x or 2x: exact in bf16
    assert torch.equal(out_w, torch.from_numpy(w_np).to(gu.DEV))             # weights come back unchanged


def test_dispatch_ranks_fp8_rows_with_scales(oracle):
    rng = np.random.default_rng(11)
    T, K, E, R, H = 700, 8, 64, 8, 1024
    topk_np = wl.zipf_distinct_topk(rng, T, E, K, 1.2)
    topk_np[rng.random((T, K)) < 0.05] = -1
    xq, scales = wl.quantize_fp8_blockwise(wl.bf16_normal(rng, T, H))
    run_and_check(oracle, topk_np, None, xq, scales, E, R)


def test_dispatch_ranks_same_rank_pattern(oracle):
    """The reference's same_rank routing (example042 .cu:195-198): all eight slots of a token on
    one rank, every expert twice: one row per token, all eight ids local."""
    T, K, R, E = 4096, 8, 8, 32
    topk_np = wl.reference_pattern_topk(T, K, R, E, "same_rank")
    rng = np.random.default_rng(1)
    _, recv_idx, _, h, ref = run_and_check(oracle, topk_np, wl.softmax_gates(rng, T, K),
                                           wl.bf16_normal(rng, T, 128), None, E, R, local_ids=True)
    assert h.num_recv_rows() == T
    assert int(recv_idx[:T].min()) >= 0 and int(recv_idx[:T].max()) < E // R


def test_dispatch_ranks_zero_tokens(oracle):
    buf = ops.Buffer(16, 2, 8, 2, device=gu.DEV)
    topk = torch.zeros((0, 2), dtype=torch.int64, device=gu.DEV)
    x = torch.zeros((0, 64), dtype=torch.bfloat16, device=gu.DEV)
    _, _, _, h = ops.dispatch_ranks(buf, x, None, topk, None)
    assert h.psum_rank_tokens.cpu().tolist() == [0, 0]


def test_dispatch_ranks_at_a_benchmark_shape(oracle):
    """4096 tokens x 7168 bf16, 256 experts, top-8, 8 ranks (the c2 shape): about 5.25 rows per
    token, compared whole with the checker, then combined back."""
    cfg = wl.CONFIGS["c2"]
    topk_np, w_np = wl.make_routing(cfg)
    rng = np.random.default_rng(2)
    x_cpu = wl.bf16_normal(rng, cfg.num_tokens, cfg.hidden)
    recv_x, _, recv_w, h, ref = run_and_check(oracle, topk_np, w_np, x_cpu, None, cfg.num_experts, cfg.num_ranks,
                                              local_ids=True, expand=True)
    rows = h.num_recv_rows()
    assert 5.0 * cfg.num_tokens < rows < 5.5 * cfg.num_tokens
    out, out_w = ops.combine_ranks(recv_x, h, recv_w)
    torch.cuda.synchronize()
    first = oracle.rank_slots(topk_np, cfg.num_ranks, cfg.num_experts, 0) >= 0
    want = oracle.combine(ref["recv_x"].view(np.uint16), np.where(first, ref["rank_row_map"], -1), num_threads=8)
    assert gu.bf16_ulp_distance(gu.bf16_bits(out), want).max() <= 2
    np.testing.assert_array_equal(out_w.cpu().numpy(), w_np)
