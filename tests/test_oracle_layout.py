"""Pins the CPU checker's layout, offsets, slot maps and prefix matrices.

Expected values here never come from the checker's own loops: they are hand-derived closed forms
of the reference's routing patterns (example042 .cu:178-206, cases :401-410), numpy library
routines (bincount, unique, cumsum, stable argsort) and invariants.
"""
import numpy as np
import pytest

from commbench_amd import workloads as wl


# ---- independent restatements with numpy library routines --------------------------

def np_layout(topk, R, E):
    T, K = topk.shape
    P = E // R
    valid = (topk >= 0) & (topk < E)
    per_expert = np.bincount(topk[valid], minlength=E).astype(np.int32)
    tok = np.broadcast_to(np.arange(T)[:, None], (T, K))[valid]
    pairs = np.unique(tok * R + topk[valid] // P)          # distinct (token, rank) pairs
    flags = np.zeros(T * R, dtype=np.uint8)
    flags[pairs] = 1
    flags = flags.reshape(T, R)
    return flags.sum(axis=0).astype(np.int32), per_expert, flags


def closed_form_counts(T, K, R, E, pattern):
    """Hand-derived per-expert and per-rank counts of the reference's correctness cases."""
    P = E // R
    e = np.arange(E)
    r, l = e // P, e % P
    if pattern == "spread" and K == 1:
        # e(t) = (17 t + R) mod E walks all E residues with period E (17 is coprime to E = 4R);
        # expert e is first hit at t0 = 17^-1 (e - R) mod E and then every E tokens.
        inv17 = pow(17, -1, E) if E > 1 else 0
        t0 = (inv17 * (e - R)) % E
        per_expert = np.where(t0 < T, (T - 1 - t0) // E + 1, 0)
        per_rank = per_expert.reshape(R, P).sum(axis=1)     # K = 1: one rank per token
    elif pattern == "spread" and K == 2:
        assert T % E == 0
        per_expert = np.full(E, T * K // E)                  # each slot is uniform over a period
        # slot 1 lands one expert below slot 0 (31 = -1 mod 4R... only mod E | 32): ranks differ
        # for P consecutive-pair boundaries: 1 token in 4 touches two ranks.
        per_rank = np.full(R, T // R + T // (4 * R))
    elif pattern == "rank_sweep":
        # rank = (t + k) mod R, local = (t - k) mod 4, K = 4, P = 4, T a multiple of 8.
        if R == 2:
            per_expert = np.where(r % 2 == l % 2, T, 0)
            per_rank = np.full(R, T)
        elif R == 4:
            per_expert = np.where((r + l) % 2 == 0, T // 2, 0)
            per_rank = np.full(R, T)
        else:
            per_expert = np.where((r - l) % 2 == 0, T // 4, 0)
            per_rank = np.full(R, T // 2)
    elif pattern == "same_rank":
        # K = 8 over P = 4 local experts: each local expert twice per token; rank uniform in t.
        per_expert = np.full(E, 2 * T // R)
        per_rank = np.full(R, T // R)
    else:
        raise AssertionError
    return per_rank.astype(np.int32), per_expert.astype(np.int32)


@pytest.mark.parametrize("case", wl.REFERENCE_LAYOUT_CASES, ids=lambda c: "-".join(map(str, c)))
def test_reference_cases_closed_form(oracle, case):
    T, K, R, E, pattern = case
    topk = wl.reference_pattern_topk(T, K, R, E, pattern)
    per_rank, per_expert, flags = oracle.layout(topk, R, E)
    exp_rank, exp_expert = closed_form_counts(T, K, R, E, pattern)
    np.testing.assert_array_equal(per_expert, exp_expert)
    np.testing.assert_array_equal(per_rank, exp_rank)
    np_rank, np_expert, np_flags = np_layout(topk, R, E)
    np.testing.assert_array_equal(flags, np_flags)
    np.testing.assert_array_equal(per_rank, np_rank)
    np.testing.assert_array_equal(per_expert, np_expert)
    assert per_expert.sum() == T * K                       # no masked slots in these cases
    np.testing.assert_array_equal(flags.sum(axis=0), per_rank)


def test_reference_case_sums():
    """Totals quoted for the reference's cases: sum over ranks of the per-rank count."""
    from oracle import ep_oracle
    want = {(257, 1): 257, (1024, 2): 1280, (4096, 8): 4096}
    for T, K, R, E, pattern in wl.REFERENCE_LAYOUT_CASES:
        per_rank, _, _ = ep_oracle.layout(wl.reference_pattern_topk(T, K, R, E, pattern), R, E)
        if (T, K) == (4096, 4):
            assert per_rank.sum() == (8192 if R == 2 else 16384)
        else:
            assert per_rank.sum() == want[(T, K)]


def test_first_case_by_hand(oracle):
    # (257, 1, 1, 4, spread): e = (t + 1) mod 4 for t = 0..256.
    per_rank, per_expert, flags = oracle.layout(wl.reference_pattern_topk(257, 1, 1, 4, "spread"), 1, 4)
    assert per_expert.tolist() == [64, 65, 64, 64]
    assert per_rank.tolist() == [257]
    assert flags.all()


def test_spread_k2_r2_by_hand(oracle):
    # R=2, E=8: e0 = (t+2) mod 8, e1 = (t+1) mod 8; rank 0 is touched for t mod 8 in {6,7,0,1,2}.
    per_rank, _, flags = oracle.layout(wl.reference_pattern_topk(1024, 2, 2, 8, "spread"), 2, 8)
    assert per_rank.tolist() == [640, 640]
    assert flags[:8, 0].tolist() == [1, 1, 1, 0, 0, 0, 1, 1]
    assert flags[:8, 1].tolist() == [0, 0, 1, 1, 1, 1, 1, 0]


@pytest.mark.parametrize("seed", range(6))
def test_random_with_masks_and_duplicates(oracle, seed):
    rng = np.random.default_rng(seed)
    R = int(rng.choice([1, 2, 4, 8]))
    E = R * int(rng.choice([1, 3, 4, 32]))
    T = int(rng.integers(0, 700))
    K = int(rng.integers(1, 9))
    topk = rng.integers(-2, E + 2, size=(T, K)).astype(np.int64)   # masked, out-of-range, duplicates
    per_rank, per_expert, flags = oracle.layout(topk, R, E)
    np_rank, np_expert, np_flags = np_layout(topk, R, E)
    np.testing.assert_array_equal(per_rank, np_rank)
    np.testing.assert_array_equal(per_expert, np_expert)
    np.testing.assert_array_equal(flags, np_flags)


def test_brute_force_tiny(oracle):
    """Every routing table of 2 tokens x 2 slots over 3 values {-1, 0, 1}, E = 2, R = 2."""
    import itertools
    for cells in itertools.product([-1, 0, 1], repeat=4):
        topk = np.array(cells, dtype=np.int64).reshape(2, 2)
        per_rank, per_expert, flags = oracle.layout(topk, 2, 2)
        for e in (0, 1):
            assert per_expert[e] == sum(c == e for c in cells)
            for t in (0, 1):
                assert flags[t, e] == int(e in topk[t])
            assert per_rank[e] == int(e in topk[0]) + int(e in topk[1])


def test_layout_rejects_bad_shapes(oracle):
    topk = np.zeros((4, 2), dtype=np.int64)
    with pytest.raises(ValueError):
        oracle.layout(topk, 3, 8)        # 8 % 3 != 0
    with pytest.raises(ValueError):
        oracle.layout(topk, 9, 18)       # more than 8 ranks


# ---- offsets -------------------------------------------------------------------------

@pytest.mark.parametrize("align", [1, 2, 16, 128])
def test_expert_offsets_vs_cumsum(oracle, align):
    rng = np.random.default_rng(align)
    R, E = 8, 64
    cnt = rng.integers(0, 300, size=E).astype(np.int32)
    cnt[rng.integers(0, E, size=8)] = 0
    off, psum = oracle.expert_offsets(cnt, R, align)
    padded = -(-cnt // align) * align
    np.testing.assert_array_equal(off, np.concatenate([[0], np.cumsum(padded)]))
    np.testing.assert_array_equal(psum, np.cumsum(padded.reshape(R, E // R).sum(axis=1)))
    assert off[0] == 0 and off[-1] == padded.sum()
    if align == 1:
        assert off[-1] == cnt.sum()


# ---- slot maps: the source map is a stable sort of the routes by expert ------------------

def np_slot_maps(topk, E, off):
    T, K = topk.shape
    flat = topk.reshape(-1)
    valid = (flat >= 0) & (flat < E)
    routes = np.nonzero(valid)[0]                               # (t, k) ascending
    order = routes[np.argsort(flat[routes], kind="stable")]     # by expert, ties by (t, k)
    experts = flat[order]
    seg_start = np.concatenate([[0], np.cumsum(np.bincount(experts, minlength=E))])[:-1]
    rel = np.arange(order.size) - seg_start[experts]
    rows = off[experts] + rel
    slot_map = np.full(T * K, -1, dtype=np.int32)
    slot_map[order] = rows
    slot_rel = np.full(T * K, -1, dtype=np.int32)
    slot_rel[order] = rel
    src_map = np.full(off[E], -1, dtype=np.int32)
    src_map[rows] = order // K
    src_k = np.full(off[E], -1, dtype=np.int32)
    src_k[rows] = order % K
    return slot_rel.reshape(T, K), slot_map.reshape(T, K), src_map, src_k


@pytest.mark.parametrize("align", [1, 8])
@pytest.mark.parametrize("kind", ["uniform", "zipf_masked", "same_rank_duplicates"])
def test_slot_maps_are_a_stable_sort(oracle, kind, align):
    R, E, K, T = 4, 32, 8, 333
    rng = np.random.default_rng(7)
    if kind == "uniform":
        topk = wl.uniform_distinct_topk(rng, T, E, K)
    elif kind == "zipf_masked":
        topk = wl.zipf_distinct_topk(rng, T, E, K, 1.2)
        topk[rng.random((T, K)) < 0.1] = -1
    else:
        topk = wl.reference_pattern_topk(T, K, R, 4 * R, "same_rank")
        E = 4 * R
    _, per_expert, _ = oracle.layout(topk, R, E)
    off, _ = oracle.expert_offsets(per_expert, R, align)
    got = oracle.slot_maps(topk, E, off)
    want = np_slot_maps(topk, E, off)
    for g, w in zip(got, want):
        np.testing.assert_array_equal(g, w)
    slot_rel, slot_map, src_map, src_k = got
    # Permutation properties: rows are hit once, segments are sorted by (token, slot).
    rows = slot_map[slot_map >= 0]
    assert np.unique(rows).size == rows.size == per_expert.sum()
    for e in range(E):
        seg = src_map[off[e]:off[e] + per_expert[e]].astype(np.int64) * K + \
            src_k[off[e]:off[e] + per_expert[e]]
        assert np.all(np.diff(seg) > 0)
        assert np.all(src_map[off[e] + per_expert[e]:off[e + 1]] == -1)


# ---- channel / rank prefix matrices (example047 .cu:349-430) ---------------------------------

def notify_closed_form(T, R, C):
    """Source rank 0 marks destinations t mod R and (t+1) mod R (R >= 2).  A token range [0, n)
    holds floor-based counts of each residue; channel c ends at min((c+1) * ceil(T/C), T)."""
    tpc = -(-T // C)
    out = np.zeros((R, C), dtype=np.int32)
    for c in range(C):
        n = min(min(tpc * c, T) + tpc, T)
        for r in range(R):
            def residue_count(res):
                return (n - res + R - 1) // R if n > res else 0
            if R == 1:
                out[r, c] = n
            else:
                # flagged when t = r (slot 0) or t = r - 1 (slot 1) mod R; distinct for R >= 2
                out[r, c] = residue_count(r) + residue_count((r - 1) % R)
    return out


@pytest.mark.parametrize("T", [7, 4096, 4097])
@pytest.mark.parametrize("R", [2, 4, 8])
def test_channel_prefix_reference_cases(oracle, T, R):
    C = wl.reference_notify_channels(R)
    flags = wl.reference_notify_flags(T, R, 0)
    got = oracle.channel_prefix(flags, C)
    np.testing.assert_array_equal(got, notify_closed_form(T, R, C))
    # Textbook form: cumulative sum of per-tile counts.
    tpc = -(-T // C)
    bounds = [min(min(tpc * c, T) + tpc, T) for c in range(C)]
    want = np.stack([flags[:b].sum(axis=0) for b in bounds], axis=1)
    np.testing.assert_array_equal(got, want)
    assert np.all(got[:, -1] == flags.sum(axis=0))


def test_rank_prefix_vs_cumsum(oracle):
    rng = np.random.default_rng(3)
    for R in (1, 2, 4, 8):
        counts = rng.integers(0, 5000, size=(R, R)).astype(np.int32)
        np.testing.assert_array_equal(oracle.rank_prefix(counts), np.cumsum(counts, axis=0))


# ---- the deterministic prologue's own table (example078 .cu:36-40) ---------------------------

def np_rank_slots(topk, R, E, base):
    """Library restatement: exclusive cumsum of the rank flags gives each token's slot per rank;
    the first slot of the token on that rank carries it."""
    T, K = topk.shape
    P = E // R
    valid = (topk >= 0) & (topk < E)
    rank = np.where(valid, topk // P, -1)
    flags = np.zeros((T, R), dtype=np.int64)
    for r in range(R):
        flags[:, r] = (rank == r).any(axis=1)
    slot_of_token = np.cumsum(flags, axis=0) - flags                   # exclusive, per rank
    out = np.full((T, K), -1, dtype=np.int32)
    for k in range(K):
        first = valid[:, k] & ~(rank[:, :k] == rank[:, k:k + 1]).any(axis=1)
        rows = np.nonzero(first)[0]
        out[rows, k] = base + slot_of_token[rows, rank[rows, k]]
    return out


@pytest.mark.parametrize("case", wl.REFERENCE_LAYOUT_CASES[::2] + [(300, 8, 8, 64, "masked")],
                         ids=lambda c: "-".join(map(str, c)))
def test_rank_slots(oracle, case):
    T, K, R, E, pattern = case
    if pattern == "masked":
        rng = np.random.default_rng(4)
        topk = rng.integers(-2, E + 1, size=(T, K)).astype(np.int64)
    else:
        topk = wl.reference_pattern_topk(T, K, R, E, pattern)
    base = 7 * 4096
    got = oracle.rank_slots(topk, R, E, base)
    np.testing.assert_array_equal(got, np_rank_slots(topk, R, E, base))
    per_rank, _, flags = oracle.layout(topk, R, E)
    P = E // R
    for r in range(R):
        on_r = (got >= 0) & (np.where((topk >= 0) & (topk < E), topk // P, -1) == r)
        vals = got[on_r] - base
        assert np.array_equal(vals, np.arange(per_rank[r]))             # token order, no gaps
        assert np.array_equal(on_r.any(axis=1), flags[:, r].astype(bool))
        assert on_r.sum(axis=1).max(initial=0) <= 1                      # one slot per (token, rank)


def test_rank_slots_same_rank_case_by_hand(oracle):
    # same_rank, K = 8: all eight slots of token t go to rank (3t + 8) mod R; only slot 0 carries it.
    topk = wl.reference_pattern_topk(64, 8, 4, 16, "same_rank")
    got = oracle.rank_slots(topk, 4, 16, 0)
    assert (got[:, 1:] == -1).all()
    # rank of token t is 3t mod 4: tokens 0, 4, 8, ... share rank 0 and take slots 0, 1, 2, ...
    assert got[0, 0] == 0 and got[4, 0] == 1 and got[8, 0] == 2
    assert got[1, 0] == 0 and got[5, 0] == 1                              # rank 3


# ---- per-tile destination order of the routes -------------------------------------------------

def np_route_order(topk, E, tile):
    """Library restatement: inside a tile, routes by (expert, flat index) with numpy's lexsort,
    then the non-routes by flat index; the position column comes from the slot maps."""
    T, K = topk.shape
    flat = topk.reshape(-1)
    valid = (flat >= 0) & (flat < E)
    counts = np.bincount(flat[valid], minlength=E)
    off = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    tiles = (T + tile - 1) // tile
    out = np.full((tiles * tile * K, 4), -7, dtype=np.int32)
    # position inside the expert's segment = rank of the route among the expert's routes
    order = np.argsort(np.where(valid, flat, E), kind="stable")
    rel = np.full(T * K, -1, dtype=np.int64)
    rel[order[:valid.sum()]] = np.arange(valid.sum()) - off[flat[order[:valid.sum()]]]
    for j in range(tiles):
        g = np.arange(j * tile * K, min((j + 1) * tile, T) * K)
        v = valid[g]
        routed = g[v][np.lexsort((g[v], flat[g[v]]))]
        masked = g[~v]
        base = j * tile * K
        out[base:base + len(routed)] = np.stack(
            [routed, flat[routed], rel[routed], routed // K], axis=1)
        out[base + len(routed):base + len(g)] = np.stack(
            [masked, -np.ones_like(masked), -np.ones_like(masked), masked // K], axis=1)
    return out


@pytest.mark.parametrize("shape", [(1, 1, 1, 4), (7, 2, 4, 4), (256, 8, 64, 256), (257, 3, 5, 256),
                                   (1000, 8, 256, 256), (3000, 6, 1024, 256), (700, 4, 16, 64)],
                         ids=lambda s: "x".join(map(str, s)))
def test_route_order_vs_lexsort(oracle, shape):
    T, K, E, tile = shape
    rng = np.random.default_rng(T + K)
    topk = rng.integers(-2, E + 2, size=(T, K)).astype(np.int64)       # masks, out of range, duplicates
    got = oracle.route_order(topk, E, tile)
    np.testing.assert_array_equal(got, np_route_order(topk, E, tile))
    # every flat index exactly once; positions agree with the slot maps
    written = got[got[:, 0] != -7]
    assert np.array_equal(np.sort(written[:, 0]), np.arange(T * K))
    _, per_expert, _ = oracle.layout(topk, 1, E)
    off, _ = oracle.expert_offsets(per_expert, 1, 1)
    slot_rel, _, _, _ = oracle.slot_maps(topk, E, off)
    assert np.array_equal(written[:, 2], slot_rel.reshape(-1)[written[:, 0]])
    # destination rows of a tile's routes ascend: that is what the copy kernel relies on
    for j in range((T + tile - 1) // tile):
        part = got[j * tile * K:(j + 1) * tile * K]
        part = part[(part[:, 0] != -7) & (part[:, 1] >= 0)]
        dst = off[part[:, 1]].astype(np.int64) + part[:, 2]
        assert (np.diff(dst) > 0).all()


def test_route_order_by_hand(oracle):
    # 3 tokens x 2 slots, tile of 2 tokens, 3 experts.
    topk = np.array([[2, 0], [-1, 2], [0, 0]], dtype=np.int64)
    got = oracle.route_order(topk, 3, tile_tokens=2)
    want = np.array([
        [1, 0, 0, 0],      # tile 0: expert 0 <- route (0,1), first in its segment
        [0, 2, 0, 0],      #         expert 2 <- route (0,0)
        [3, 2, 1, 1],      #         expert 2 <- route (1,1), second in the segment
        [2, -1, -1, 1],    #         the masked slot (1,0)
        [4, 0, 1, 2],      # tile 1: expert 0 <- route (2,0), after tile 0's one
        [5, 0, 2, 2],      #         expert 0 <- route (2,1)
        [-7, -7, -7, -7], [-7, -7, -7, -7]], dtype=np.int32)
    np.testing.assert_array_equal(got, want)
