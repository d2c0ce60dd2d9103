"""GPU parity of the layout kernels (through the C ABI) against the CPU checker: bit-exact."""
import numpy as np
import pytest
import torch

from commbench_amd import ops
from commbench_amd import workloads as wl

from . import gpu_util as gu

pytestmark = pytest.mark.gpu


# ---- the reference's own correctness cases, on its own operator surface ---------------------

@pytest.mark.parametrize("case", wl.REFERENCE_LAYOUT_CASES, ids=lambda c: "-".join(map(str, c)))
def test_get_dispatch_layout_reference_cases(oracle, case):
    T, K, R, E, pattern = case
    print(f"case {case}", flush=True)
    topk_np = wl.reference_pattern_topk(T, K, R, E, pattern)
    topk = torch.from_numpy(topk_np).to(gu.DEV)
    per_rank, per_expert, flags = ops.get_dispatch_layout(topk, E, R)
    torch.cuda.synchronize()
    w_rank, w_expert, w_flags = oracle.layout(topk_np, R, E)
    np.testing.assert_array_equal(per_rank.cpu().numpy(), w_rank)
    np.testing.assert_array_equal(per_expert.cpu().numpy(), w_expert)
    np.testing.assert_array_equal(flags.cpu().numpy().view(np.uint8), w_flags)


@pytest.mark.parametrize("shape", [
    (1, 1, 1, 1), (1, 8, 8, 1024), (63, 3, 1, 5), (64, 8, 8, 8), (65, 2, 2, 6), (1000, 7, 4, 1024),
    (1024, 8, 8, 256), (1025, 8, 8, 256), (5000, 5, 8, 1024)], ids=lambda s: "x".join(map(str, s)))
def test_get_dispatch_layout_ragged_shapes(oracle, shape):
    """Both forms of the counts-only layout (one workgroup up to 1024 tokens, many beyond) on ragged
    token counts, every expert count's edge, masked, duplicated and out-of-range ids."""
    T, K, R, E = shape
    print(f"shape {shape}", flush=True)
    rng = np.random.default_rng(T * 7 + E)
    topk_np = rng.integers(-2, E + 2, size=(T, K)).astype(np.int64)
    per_rank, per_expert, flags = ops.get_dispatch_layout(torch.from_numpy(topk_np).to(gu.DEV), E, R)
    torch.cuda.synchronize()
    w_rank, w_expert, w_flags = oracle.layout(topk_np, R, E)
    np.testing.assert_array_equal(per_rank.cpu().numpy(), w_rank)
    np.testing.assert_array_equal(per_expert.cpu().numpy(), w_expert)
    np.testing.assert_array_equal(flags.cpu().numpy().view(np.uint8), w_flags)


def test_get_dispatch_layout_without_tokens():
    per_rank, per_expert, flags = ops.get_dispatch_layout(torch.zeros((0, 4), dtype=torch.int64, device=gu.DEV), 64, 8)
    torch.cuda.synchronize()
    assert not per_rank.cpu().numpy().any() and not per_expert.cpu().numpy().any() and flags.shape == (0, 8)


def test_get_dispatch_layout_overwrites_its_outputs(oracle):
    """The reference's benchmark relaunches without re-zeroing (example042 .cu:313-329)."""
    from commbench_amd import _lib
    T, K, R, E = 1000, 4, 4, 64
    topk_np = wl.uniform_distinct_topk(np.random.default_rng(0), T, E, K)
    topk = torch.from_numpy(topk_np).to(gu.DEV)
    per_rank = torch.full((R,), 12345, dtype=torch.int32, device=gu.DEV)
    per_expert = torch.full((E,), -777, dtype=torch.int32, device=gu.DEV)
    flags = gu.garbage_like(torch.empty((T, R), dtype=torch.bool, device=gu.DEV)).view(torch.uint8)
    lib = _lib.load()
    for _ in range(3):
        _lib.check(lib.mi_ep_get_dispatch_layout(topk.data_ptr(), per_rank.data_ptr(), None,
                                                 per_expert.data_ptr(), flags.data_ptr(), T, K, R, E,
                                                 torch.cuda.current_stream().cuda_stream), "layout")
    torch.cuda.synchronize()
    w_rank, w_expert, w_flags = oracle.layout(topk_np, R, E)
    np.testing.assert_array_equal(per_rank.cpu().numpy(), w_rank)
    np.testing.assert_array_equal(per_expert.cpu().numpy(), w_expert)
    np.testing.assert_array_equal(flags.cpu().numpy().reshape(T, R), w_flags)


# ---- fused single-pass layout --------------------------------------------------------------

@pytest.mark.parametrize("case", wl.REFERENCE_LAYOUT_CASES, ids=lambda c: "-".join(map(str, c)))
def test_fused_layout_reference_cases(oracle, case):
    T, K, R, E, pattern = case
    print(f"case {case}", flush=True)
    topk_np = wl.reference_pattern_topk(T, K, R, E, pattern)
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    _, h = gu.run_fused_layout(buf, topk_np, expert_alignment=1, num_channels=2 * R)
    gu.check_layout_against_oracle(oracle, h, topk_np, R, E, 1, 2 * R)


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c4", "c5"])
def test_fused_layout_configs(oracle, name):
    cfg = wl.CONFIGS[name]
    print(f"config {name}", flush=True)
    topk_np, _ = wl.make_routing(cfg)
    buf = ops.Buffer(cfg.num_tokens, cfg.num_topk, cfg.num_experts, cfg.num_ranks, device=gu.DEV)
    for align in (1, 128):
        _, h = gu.run_fused_layout(buf, topk_np, expert_alignment=align, num_channels=16)
        gu.check_layout_against_oracle(oracle, h, topk_np, cfg.num_ranks, cfg.num_experts, align, 16)


@pytest.mark.parametrize("shape", [
    (1, 1, 1, 1), (1, 8, 8, 8), (7, 2, 2, 4), (255, 3, 1, 5), (256, 8, 8, 1024), (257, 5, 4, 12),
    (513, 7, 2, 6), (3000, 6, 8, 1024), (65536, 2, 8, 32)], ids=lambda s: "x".join(map(str, s)))
def test_fused_layout_ragged_shapes(oracle, shape):
    T, K, R, E = shape
    print(f"shape {shape}", flush=True)
    rng = np.random.default_rng(T * 31 + K)
    topk_np = rng.integers(-1, E, size=(T, K)).astype(np.int64)     # masks and duplicates
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    _, h = gu.run_fused_layout(buf, topk_np, expert_alignment=3, num_channels=5)
    gu.check_layout_against_oracle(oracle, h, topk_np, R, E, 3, 5)


@pytest.mark.parametrize("shape", [
    (4096, 4, 8, 1024), (4097, 4, 8, 1024), (2304, 2, 8, 1024), (2000, 8, 3, 3), (8192, 8, 1, 1), (16384, 3, 7, 7)],
    ids=lambda s: "x".join(map(str, s)))
def test_fused_layout_gathered_and_walked_scans(oracle, shape):
    """Small grids fetch every predecessor's packed status row at once, larger ones walk back column
    by column: 1024 experts x 8 ranks change over between 16 and 17 tiles (4096 / 4097 tokens) and
    need one round of loads up to 8 predecessors (2304 tokens) and two beyond; odd expert and rank
    counts leave half a status word empty; a token whose slots all name one expert drives a column
    to the 2048 routes per tile that its 16 bits must hold."""
    T, K, R, E = shape
    print(f"shape {shape}", flush=True)
    rng = np.random.default_rng(T + E)
    topk_np = rng.integers(-1, E, size=(T, K)).astype(np.int64)
    if E <= 3:
        topk_np[: T // 2] = E - 1                        # whole tiles on one expert
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    for _ in range(2):
        _, h = gu.run_fused_layout(buf, topk_np, expert_alignment=2, num_channels=3)
    gu.check_layout_against_oracle(oracle, h, topk_np, R, E, 2, 3)


@pytest.mark.parametrize("shape", [(300000, 2, 8, 64), (131072, 8, 8, 256)], ids=lambda s: "x".join(map(str, s)))
def test_fused_layout_more_tiles_than_resident_workgroups(oracle, shape):
    """Over a thousand tiles: more workgroups than the device holds at once.  Tiles are handed out
    by ticket, so a tile only ever waits on tiles that have already started."""
    T, K, R, E = shape
    print(f"shape {shape}", flush=True)
    rng = np.random.default_rng(T)
    topk_np = wl.zipf_distinct_topk(rng, T, E, K, 1.2) if K == 8 else rng.integers(-1, E, size=(T, K)).astype(np.int64)
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    for _ in range(2):
        _, h = gu.run_fused_layout(buf, topk_np, expert_alignment=16, num_channels=16)
    gu.check_layout_against_oracle(oracle, h, topk_np, R, E, 16, 16)


def test_fused_layout_out_of_range_and_all_masked(oracle):
    T, K, R, E = 700, 4, 4, 16
    rng = np.random.default_rng(5)
    topk_np = rng.integers(-3, E + 3, size=(T, K)).astype(np.int64)
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    _, h = gu.run_fused_layout(buf, topk_np)
    gu.check_layout_against_oracle(oracle, h, topk_np, R, E)
    masked = np.full((T, K), -1, dtype=np.int64)
    _, h = gu.run_fused_layout(buf, masked)
    ref = gu.check_layout_against_oracle(oracle, h, masked, R, E)
    assert ref["off"][-1] == 0


def test_fused_layout_zero_tokens(oracle):
    buf = ops.Buffer(16, 2, 8, 2, device=gu.DEV)
    empty = np.zeros((0, 2), dtype=np.int64)
    _, h = gu.run_fused_layout(buf, empty, expert_alignment=4, num_channels=4)
    assert not h.num_tokens_per_expert.cpu().numpy().any()
    assert not h.expert_offsets.cpu().numpy().any()
    assert not h.channel_prefix_matrix.cpu().numpy().any()


def test_workspace_is_reusable_across_shapes_and_many_calls(oracle):
    """One workspace, alternating token counts: status words of earlier launches must never be
    mistaken for this launch's."""
    K, R, E = 8, 8, 64
    buf = ops.Buffer(5000, K, E, R, device=gu.DEV)
    rng = np.random.default_rng(17)
    for i, T in enumerate([5000, 300, 4097, 1, 5000, 2048, 300, 5000] * 3):
        topk_np = wl.uniform_distinct_topk(rng, T, E, K)
        _, h = gu.run_fused_layout(buf, topk_np)
        gu.check_layout_against_oracle(oracle, h, topk_np, R, E)


def test_workspace_alternates_between_gathered_and_walked_scans(oracle):
    """One workspace, 1024 experts: launches of up to 16 tiles pack two columns per status word, larger
    ones keep one; words left by the other form must never be taken for this launch's."""
    K, R, E = 4, 8, 1024
    buf = ops.Buffer(8192, K, E, R, device=gu.DEV)
    rng = np.random.default_rng(23)
    for T in [4096, 8192, 2304, 8192, 4096, 300, 8192, 4096]:
        topk_np = rng.integers(-1, E, size=(T, K)).astype(np.int64)
        _, h = gu.run_fused_layout(buf, topk_np, expert_alignment=4, num_channels=8)
        gu.check_layout_against_oracle(oracle, h, topk_np, R, E, 4, 8)


def notify_topk(T, R, src_rank):
    """Routing that reproduces the notify example's flags for one source rank (example047
    .cu:189-193,437-447) with one expert per rank: slot s of token t goes to routeDst(src_rank, t, s)."""
    t = np.arange(T)
    stride = (src_rank % (R - 1)) + 1
    return np.stack([(t + src_rank) % R, (t + src_rank + stride) % R], axis=1).astype(np.int64)


@pytest.mark.parametrize("T", [7, 4096, 4097])
@pytest.mark.parametrize("R", [2, 4, 8])
def test_channel_prefix_reference_notify_cases(oracle, T, R):
    """The reference's notify inputs (example047 .cu:599-610), every source rank's batch in turn: two
    destinations per token, C = min(16, max(4, 2R)) channels."""
    C = wl.reference_notify_channels(R)
    buf = ops.Buffer(T, 2, R, R, device=gu.DEV)
    for src in range(R):
        flags = wl.reference_notify_flags(T, R, src)
        _, h = gu.run_fused_layout(buf, notify_topk(T, R, src), num_channels=C)
        np.testing.assert_array_equal(h.is_token_in_rank.cpu().numpy().view(np.uint8), flags)
        np.testing.assert_array_equal(h.channel_prefix_matrix.cpu().numpy(), oracle.channel_prefix(flags, C))


@pytest.mark.parametrize("T", [7, 4096, 4097])
@pytest.mark.parametrize("R", [2, 4, 8])
def test_both_prefix_matrices_of_the_notify_cases_from_one_launch(oracle, T, R):
    """notify_dispatch's two outputs (example047 .cu:112-143) from one launch with the reference's
    channel count: the R source ranks' batches of T tokens laid end to end are R chunks of exactly
    ceil(R T / R) = T tokens, so rank_prefix_matrix must be the harness's expected_rank_prefix
    (.cu:352-360: counts[src, dst] summed over sources 0..src) and channel_prefix_matrix the
    per-channel prefix of the whole batch (.cu:386-428)."""
    C = wl.reference_notify_channels(R)
    flags = np.concatenate([wl.reference_notify_flags(T, R, src) for src in range(R)])
    topk_np = np.concatenate([notify_topk(T, R, src) for src in range(R)])
    buf = ops.Buffer(R * T, 2, R, R, device=gu.DEV)
    _, h = gu.run_fused_layout(buf, topk_np, num_channels=C)
    np.testing.assert_array_equal(h.is_token_in_rank.cpu().numpy().view(np.uint8), flags)
    counts = np.stack([wl.reference_notify_flags(T, R, src).sum(axis=0) for src in range(R)]).astype(np.int32)
    assert (counts.sum(axis=1) == 2 * T).all()                 # two distinct destinations per token
    got = h.rank_prefix_matrix().cpu().numpy()
    np.testing.assert_array_equal(got, oracle.rank_prefix(counts))
    np.testing.assert_array_equal(got[-1], h.num_tokens_per_rank.cpu().numpy())
    np.testing.assert_array_equal(h.channel_prefix_matrix.cpu().numpy(), oracle.channel_prefix(flags, C))


@pytest.mark.parametrize("shape", [(65536, 8, 8, 256), (262144, 2, 8, 8)], ids=["walked", "gathered"])
def test_expired_wait_terminates_and_is_reported(oracle, shape):
    """Failure handling without a hang: with the wait limit forced to one poll, a launch over many
    tiles gives up at least one wait of its scan (256 tiles walking back column by column; 1024 tiles
    of 16 columns gathering their predecessors' rows); it must still finish, the workspace must
    report it, and after re-initialisation the same workspace must work again."""
    from commbench_amd import _lib
    lib = _lib.load()
    T, K, R, E = shape
    print(f"shape {shape}", flush=True)
    topk_np = wl.uniform_distinct_topk(np.random.default_rng(3), T, E, K)
    topk = torch.from_numpy(topk_np).to(gu.DEV)
    buf = ops.Buffer(T, K, E, R, device=gu.DEV)
    try:
        buf.set_wait_limit(1)
        expired = False
        for _ in range(20):                       # every launch terminates; some wait will expire
            buf.dispatch_layout(topk)
            torch.cuda.synchronize()
            code = lib.mi_ep_workspace_status(buf.workspace.data_ptr(), torch.cuda.current_stream().cuda_stream)
            if code != 0:
                assert code == -110 and _lib.strerror(code) == "device-side wait timed out"
                expired = True
                break
        assert expired, "no wait expired with a one-poll limit over hundreds of tiles"
        with pytest.raises(_lib.MiEpError):
            buf.status()
    finally:
        buf.set_wait_limit(0)
    _lib.check(lib.mi_ep_workspace_init(buf.workspace.data_ptr(), buf.workspace.numel(),
                                        torch.cuda.current_stream().cuda_stream), "re-init")
    _, h = gu.run_fused_layout(buf, topk_np)
    gu.check_layout_against_oracle(oracle, h, topk_np, R, E)


@pytest.mark.parametrize("tokens", [3000, 20000], ids=["static_tiles", "tiles_by_arrival"])
def test_generation_counter_wraps_around(oracle, tokens):
    """The look-back's status words are told apart by a 30-bit generation in the workspace's turn
    word.  Starting two launches before the counter's end, five launches in a row (the last three
    after the wrap) must all see only their own words."""
    E, R, K = 64, 8, 4
    rng = np.random.default_rng(tokens)
    buf = ops.Buffer(tokens, K, E, R, device=gu.DEV)
    torch.cuda.synchronize()
    turn = buf.workspace[:8].view(torch.int64)
    turn[0] = (0x3FFFFFFF - 1) << 32          # {generation = 2^30 - 2, arrivals = 0}
    for launch in range(5):
        T = tokens - 17 * launch
        topk_np = wl.uniform_distinct_topk(rng, T, E, K)
        _, h = gu.run_fused_layout(buf, topk_np, expert_alignment=3, num_channels=8)
        gu.check_layout_against_oracle(oracle, h, topk_np, R, E, align=3, channels=8)
    assert int(turn[0].item()) >> 32 == 3       # 2^30 - 2 + 5 launches, modulo 2^30
