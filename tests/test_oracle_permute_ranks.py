"""Pins the CPU checker's rank-deduplicated dispatch (one row per token and destination rank).

A numpy restatement built from boolean masks and fancy indexing, the checks of the reference's
own harness (example080 build_and_run.py:728-748: rows sorted by source token id carry the
token's bytes, ids and weights; per-rank counts match), and one case by hand.
"""
import numpy as np
import pytest

from commbench_amd import workloads as wl


def np_permute_ranks(x, topk, w, R, E, base, local_ids, expand):
    T, K = topk.shape
    P = E // R
    valid = (topk >= 0) & (topk < E)
    rank = np.where(valid, topk // P, -1)
    rows_x, rows_idx, rows_w, rows_meta, counts = [], [], [], [], []
    row_map = np.full((T, K), -1, dtype=np.int32)
    start = 0
    for r in range(R):
        on_r = rank == r                                   # [T, K]
        tokens = np.nonzero(on_r.any(axis=1))[0]           # token order
        counts.append(len(tokens))
        rows_x.append(x[tokens])
        rows_idx.append(np.where(on_r[tokens], topk[tokens] - (r * P if local_ids else 0), -1))
        rows_w.append(np.where(on_r[tokens], w[tokens], 0).astype(np.float32))
        meta = np.full((len(tokens), 2 + K), -1, dtype=np.int32)
        meta[:, 0] = base + tokens
        meta[:, 1] = r
        if expand is not None:
            meta[:, 2:] = np.where(on_r[tokens], expand[tokens], -1)
        rows_meta.append(meta)
        row_of_token = np.full(T, -1, dtype=np.int32)
        row_of_token[tokens] = start + np.arange(len(tokens))
        row_map = np.where(on_r, row_of_token[:, None], row_map)
        start += len(tokens)
    return dict(recv_x=np.concatenate(rows_x), recv_topk_idx=np.concatenate(rows_idx),
                recv_topk_weights=np.concatenate(rows_w), recv_src_metadata=np.concatenate(rows_meta),
                rank_row_map=row_map, psum_rank_tokens=np.cumsum(counts).astype(np.int32))


@pytest.mark.parametrize("local_ids", [False, True])
@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (64, 8, 4, 16), (300, 8, 8, 64), (257, 3, 2, 10), (500, 4, 8, 1024)],
                         ids=lambda s: "x".join(map(str, s)))
def test_permute_ranks_vs_numpy(oracle, shape, local_ids):
    T, K, R, E = shape
    rng = np.random.default_rng(T * 7 + K)
    topk = rng.integers(-2, E + 1, size=(T, K)).astype(np.int64)      # masks, out of range, duplicates
    w = rng.random((T, K), dtype=np.float32)
    x = rng.integers(0, 256, size=(T, 48), dtype=np.uint8)
    _, per_expert, _ = oracle.layout(topk, R, E)
    off, _ = oracle.expert_offsets(per_expert, R, 1)
    _, expand, _, _ = oracle.slot_maps(topk, E, off)
    got = oracle.permute_ranks(x, None, topk, w, R, E, source_token_base=3 * 4096,
                               local_expert_ids=local_ids, expand_slot_map=expand)
    want = np_permute_ranks(x, topk, w, R, E, 3 * 4096, local_ids, expand)
    for key, value in want.items():
        np.testing.assert_array_equal(got[key], value, err_msg=key)
    # the layout function's counts and flags describe the same rows
    per_rank, _, flags = oracle.layout(topk, R, E)
    np.testing.assert_array_equal(np.diff(np.concatenate([[0], got["psum_rank_tokens"]])), per_rank)
    meta = got["recv_src_metadata"]
    for r in range(R):
        tokens = meta[meta[:, 1] == r, 0] - 3 * 4096
        np.testing.assert_array_equal(tokens, np.nonzero(flags[:, r])[0])


def test_reference_harness_checks(oracle):
    """The reference's asserts after dispatch (example080 build_and_run.py:728-748), on the JIT
    examples' default shape: 512 tokens x 256 hidden, top-2 of 64 experts, 8 ranks."""
    rng = np.random.default_rng(80)
    T, H, K, E, R = 512, 256, 2, 64, 8
    topk = wl.uniform_distinct_topk(rng, T, E, K)
    w = wl.softmax_gates(rng, T, K)
    x = rng.integers(0, 1 << 16, size=(T, H), dtype=np.uint16)
    got = oracle.permute_ranks(x.view(np.uint8), None, topk, w, R, E)
    psum = np.concatenate([[0], got["psum_rank_tokens"]])
    P = E // R
    for r in range(R):
        rows = slice(psum[r], psum[r + 1])
        order = np.argsort(got["recv_src_metadata"][rows, 0], kind="stable")
        src = got["recv_src_metadata"][rows, 0][order]
        ref_tokens = np.nonzero(((topk // P) == r).any(axis=1))[0]
        np.testing.assert_array_equal(src, ref_tokens)
        np.testing.assert_array_equal(got["recv_x"][rows][order].view(np.uint16), x[ref_tokens])
        ref_idx = np.where(topk[ref_tokens] // P == r, topk[ref_tokens], -1)
        np.testing.assert_array_equal(got["recv_topk_idx"][rows][order], ref_idx)
        np.testing.assert_array_equal(np.where(ref_idx >= 0, got["recv_topk_weights"][rows][order], 0),
                                      np.where(ref_idx >= 0, w[ref_tokens], 0))
        assert psum[r + 1] - psum[r] == len(ref_tokens)


def test_by_hand(oracle):
    # 3 tokens, top-3, 2 ranks x 2 experts.  Token 0 -> experts 0, 3, 1 (ranks 0, 1, 0);
    # token 1 -> masked, 2, 2 (rank 1 twice); token 2 -> 1, masked, masked (rank 0).
    topk = np.array([[0, 3, 1], [-1, 2, 2], [1, -1, -1]], dtype=np.int64)
    w = np.arange(9, dtype=np.float32).reshape(3, 3) + 1
    x = np.array([[10] * 16, [20] * 16, [30] * 16], dtype=np.uint8)
    got = oracle.permute_ranks(x, None, topk, w, 2, 4, source_token_base=100, local_expert_ids=True)
    np.testing.assert_array_equal(got["psum_rank_tokens"], [2, 4])
    np.testing.assert_array_equal(got["recv_x"][:, 0], [10, 30, 10, 20])       # rank 0: t0, t2; rank 1: t0, t1
    np.testing.assert_array_equal(got["recv_topk_idx"], [[0, -1, 1], [1, -1, -1], [-1, 1, -1], [-1, 0, 0]])
    np.testing.assert_array_equal(got["recv_topk_weights"], [[1, 0, 3], [7, 0, 0], [0, 2, 0], [0, 5, 6]])
    np.testing.assert_array_equal(got["recv_src_metadata"][:, :2], [[100, 0], [102, 0], [100, 1], [101, 1]])
    np.testing.assert_array_equal(got["rank_row_map"], [[0, 2, 0], [-1, 3, 3], [1, -1, -1]])


def test_capacity_drops_rows(oracle):
    topk = np.array([[0, 1], [1, 0], [0, 1]], dtype=np.int64)                   # 2 ranks x 1 expert
    x = np.arange(3 * 16, dtype=np.uint8).reshape(3, 16)
    got = oracle.permute_ranks(x, None, topk, None, 2, 2, capacity_rows=4)
    np.testing.assert_array_equal(got["psum_rank_tokens"], [3, 6])
    np.testing.assert_array_equal(got["rank_row_map"], [[0, 3], [-1, 1], [2, -1]])   # rows 4 and 5 dropped
    assert got["recv_x"].shape[0] == 4
