"""The host-pointer twins against the CPU checker: numpy in, numpy out, same bars as the device calls."""
import numpy as np
import pytest

from commbench_amd import ops
from commbench_amd import workloads as wl

from . import gpu_util as gu

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", wl.REFERENCE_LAYOUT_CASES[:5], ids=lambda c: "-".join(map(str, c)))
def test_host_layout_reference_cases(oracle, case):
    T, K, R, E, pattern = case
    print(f"case {case}", flush=True)
    topk = wl.reference_pattern_topk(T, K, R, E, pattern)
    per_rank, per_expert, flags = ops.host_get_dispatch_layout(topk, E, R)
    w_rank, w_expert, w_flags = oracle.layout(topk, R, E)
    np.testing.assert_array_equal(per_rank, w_rank)
    np.testing.assert_array_equal(per_expert, w_expert)
    np.testing.assert_array_equal(flags.view(np.uint8), w_flags)


@pytest.mark.parametrize("shape", [(128, 2, 8, 2, 256, 1), (1000, 8, 64, 8, 1024, 128), (3, 1, 4, 1, 8, 2)],
                         ids=lambda s: "x".join(map(str, s)))
def test_host_dispatch_then_combine(oracle, shape):
    T, K, E, R, H, align = shape
    print(f"shape {shape}", flush=True)
    rng = np.random.default_rng(T + H)
    topk = wl.uniform_distinct_topk(rng, T, E, K)
    topk[rng.random((T, K)) < 0.1] = -1
    w = wl.softmax_gates(rng, T, K)
    x = wl.bf16_normal(rng, T, H)
    x_bits = gu.bf16_bits(x)
    got = ops.host_dispatch(x_bits, None, topk, w, E, R, expert_alignment=align)
    ref = oracle.full_path(topk, w, x_bits.view(np.uint8), None, E, R, align)
    for key in ("num_tokens_per_rank", "num_tokens_per_expert", "expert_offsets", "slot_map", "recv_src_map",
                "recv_topk_idx"):
        np.testing.assert_array_equal(got[key], ref[key], err_msg=key)
    np.testing.assert_array_equal(got["is_token_in_rank"].view(np.uint8), ref["is_token_in_rank"])
    np.testing.assert_array_equal(got["recv_x"].view(np.uint8), ref["recv_x"])
    np.testing.assert_array_equal(got["recv_topk_weights"].view(np.uint32), ref["recv_topk_weights"].view(np.uint32))
    bias = gu.bf16_bits(wl.bf16_normal(rng, T, H))
    out = ops.host_combine(got["recv_x"], got["slot_map"], w, bias, None)
    want = oracle.combine(got["recv_x"], ref["slot_map"], w, bias, None)
    np.testing.assert_array_equal(out, want)         # same fused multiply-add chain, one rounding: bit-exact


def test_host_dispatch_fp8_rows_with_scales(oracle):
    rng = np.random.default_rng(9)
    T, K, E, R, H = 300, 4, 16, 4, 512
    topk = wl.uniform_distinct_topk(rng, T, E, K)
    xq, scales = wl.quantize_fp8_blockwise(wl.bf16_normal(rng, T, H))
    x_bytes = gu.as_bytes(xq)
    got = ops.host_dispatch(x_bytes, scales.numpy(), topk, None, E, R)
    ref = oracle.full_path(topk, None, x_bytes, scales.numpy(), E, R, 1)
    np.testing.assert_array_equal(got["recv_x"], ref["recv_x"])
    np.testing.assert_array_equal(got["recv_scales"].view(np.uint32), ref["recv_scales"].view(np.uint32))
    np.testing.assert_array_equal(got["slot_map"], ref["slot_map"])


@pytest.mark.parametrize("local_ids", [False, True])
def test_host_dispatch_ranks_then_the_plain_sum(oracle, local_ids):
    """The per-rank receive format through host arrays: every output against the checker, then the
    reference's combine of that format (ordered sum over combine_map) on the rows it produced."""
    rng = np.random.default_rng(31)
    T, K, E, R, H = 700, 8, 32, 8, 256
    topk = rng.integers(-1, E, size=(T, K)).astype(np.int64)     # masks and duplicates included
    w = wl.softmax_gates(rng, T, K)
    x_bits = gu.bf16_bits(wl.bf16_normal(rng, T, H))
    scales = rng.standard_normal((T, 3)).astype(np.float32)
    got = ops.host_dispatch_ranks(x_bits, scales, topk, w, E, R, source_token_base=5 * T, local_expert_ids=local_ids)
    ref = oracle.permute_ranks(x_bits.view(np.uint8), scales, topk, w, R, E, 5 * T, local_ids, None)
    np.testing.assert_array_equal(got["psum_rank_tokens"], ref["psum_rank_tokens"])
    np.testing.assert_array_equal(got["num_tokens_per_rank"], oracle.layout(topk, R, E)[0])
    np.testing.assert_array_equal(got["rank_row_map"], ref["rank_row_map"])
    first = oracle.rank_slots(topk, R, E, 0) >= 0
    np.testing.assert_array_equal(got["combine_map"], np.where(first, ref["rank_row_map"], -1))
    np.testing.assert_array_equal(got["recv_x"].view(np.uint8), ref["recv_x"])
    np.testing.assert_array_equal(got["recv_scales"].view(np.uint32), ref["recv_scales"].view(np.uint32))
    np.testing.assert_array_equal(got["recv_topk_idx"], ref["recv_topk_idx"])
    np.testing.assert_array_equal(got["recv_topk_weights"].view(np.uint32), ref["recv_topk_weights"].view(np.uint32))
    np.testing.assert_array_equal(got["recv_src_metadata"], ref["recv_src_metadata"])
    out = ops.host_combine(got["recv_x"], got["combine_map"], None)
    want = oracle.combine(got["recv_x"], got["combine_map"], None)
    np.testing.assert_array_equal(out, want)         # an ordered sum in fp32, one rounding: bit-exact


def test_host_dispatch_cached_pulls_rows_by_the_source_map(oracle):
    rng = np.random.default_rng(32)
    T, H, rows = 333, 264, 900
    x_bits = gu.bf16_bits(wl.bf16_normal(rng, T, H))
    scales = rng.standard_normal((T, 2)).astype(np.float32)
    src_map = rng.integers(-1, T, size=rows).astype(np.int32)
    recv_x, recv_scales = ops.host_dispatch_cached(x_bits, scales, src_map)
    want_x, want_scales = oracle.gather_rows(x_bits.view(np.uint8), scales, src_map)
    np.testing.assert_array_equal(recv_x.view(np.uint8), want_x)
    np.testing.assert_array_equal(recv_scales.view(np.uint32), want_scales.view(np.uint32))
