"""Pins the pull-mode (cached) dispatch and the pull-index format of the CPU checker.

Known answers come from the closed form of the ThunderKittens MoE example's own generator
(example056_thunderkitten_moe_dispatch_gemm_easy/nv/empty_thunderkitten_moe_dispatch_gemm.cu:521-564):
token i selects experts (i + j) mod E, j < K; the rows of expert e are the tokens with
(e - i) mod E < K in ascending order, each expert padded to a fixed row count with {-1, -1}.
Also the equivalence between the notify example's rank prefix matrix and per-channel prefixes.
"""
import numpy as np
import pytest

from commbench_amd import workloads as wl


def tk_reference_pull_indices(total_tokens, world, E, K, padded_per_expert, rank):
    """Restated from the formulas in the example's comments, with numpy set arithmetic."""
    per_dev = total_tokens // world
    nepd = E // world
    out = np.full((nepd * padded_per_expert, 2), -1, dtype=np.int32)
    i = np.arange(total_tokens)
    for local_e in range(nepd):
        e = rank * nepd + local_e
        toks = i[((e - i % E) % E) < K]
        base = local_e * padded_per_expert
        out[base:base + toks.size, 0] = toks // per_dev
        out[base:base + toks.size, 1] = toks % per_dev
    return out


@pytest.mark.parametrize("world,E,K,T", [(8, 256, 8, 4096), (4, 64, 4, 1024), (2, 16, 8, 256)])
def test_pull_indices_match_the_thunderkittens_generator(oracle, world, E, K, T):
    i = np.arange(T)[:, None]
    topk = ((i + np.arange(K)[None, :]) % E).astype(np.int64)
    per_expert_true = T * K // E                       # balanced by construction
    align = 128
    padded = -(-per_expert_true // align) * align
    _, per_expert, _ = oracle.layout(topk, world, E)
    assert (per_expert == per_expert_true).all()
    off, psum = oracle.expert_offsets(per_expert, world, align)
    _, _, src_map, _ = oracle.slot_maps(topk, E, off)
    got = oracle.pull_indices(src_map, T // world)
    nepd = E // world
    for rank in range(world):
        rows = slice(rank * nepd * padded, (rank + 1) * nepd * padded)
        np.testing.assert_array_equal(got[rows], tk_reference_pull_indices(T, world, E, K, padded, rank))
        assert psum[rank] == (rank + 1) * nepd * padded


def test_gather_rows_is_a_gather_with_zero_pads(oracle):
    rng = np.random.default_rng(2)
    T, row_bytes, S = 50, 32, 3
    x = rng.integers(1, 256, size=(T, row_bytes), dtype=np.uint8)
    scales = rng.standard_normal((T, S)).astype(np.float32)
    src_map = rng.integers(-1, T, size=200).astype(np.int32)
    src_map[7] = T + 5                                  # out of range counts as a pad
    recv_x, recv_scales = oracle.gather_rows(x, scales, src_map)
    live = (src_map >= 0) & (src_map < T)
    np.testing.assert_array_equal(recv_x[live], x[src_map[live]])
    np.testing.assert_array_equal(recv_scales[live], scales[src_map[live]])
    assert not recv_x[~live].any() and not recv_scales[~live].any()


def test_cached_dispatch_equals_the_first_dispatch(oracle):
    rng = np.random.default_rng(3)
    T, K, E, R = 120, 4, 16, 4
    topk = wl.uniform_distinct_topk(rng, T, E, K)
    topk[rng.random((T, K)) < 0.1] = -1
    x = rng.integers(0, 256, size=(T, 48), dtype=np.uint8)
    res = oracle.full_path(topk, None, x, None, E, R, expert_alignment=8)
    again, _ = oracle.gather_rows(x, None, res["recv_src_map"])
    np.testing.assert_array_equal(again, res["recv_x"])


@pytest.mark.parametrize("R", [2, 4, 8])
def test_rank_prefix_matrix_is_the_channel_prefix_with_one_channel_per_source(oracle, R):
    """With the tokens split into R equal contiguous source chunks (the one-GPU stand-in for R source
    ranks), rank_prefix_matrix[src, dst] of the notify example (example047 .cu:352-360) is
    channel_prefix_matrix[dst, src] computed with num_channels = R."""
    rng = np.random.default_rng(R)
    T = 40 * R
    flags = (rng.random((T, R)) < 0.4).astype(np.uint8)
    counts = flags.reshape(R, T // R, R).sum(axis=1).astype(np.int32)      # [src, dst]
    np.testing.assert_array_equal(oracle.rank_prefix(counts), oracle.channel_prefix(flags, R).T)
