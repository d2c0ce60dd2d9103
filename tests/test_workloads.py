"""Seeded workload generators: determinism, distribution shape, byte budgets."""
import numpy as np

from commbench_amd import workloads as wl


def test_routing_is_seeded_and_distinct():
    for name in ("c1", "c2", "c3"):
        cfg = wl.CONFIGS[name]
        a_idx, a_w = wl.make_routing(cfg)
        b_idx, b_w = wl.make_routing(cfg)
        np.testing.assert_array_equal(a_idx, b_idx)
        np.testing.assert_array_equal(a_w, b_w)
        assert a_idx.shape == (cfg.num_tokens, cfg.num_topk) and a_idx.dtype == np.int64
        assert a_w.dtype == np.float32
        np.testing.assert_allclose(a_w.sum(axis=1), 1.0, rtol=1e-5)
        for row in a_idx[:512]:
            live = row[row >= 0]
            assert np.unique(live).size == live.size
        assert a_idx.max() < cfg.num_experts


def test_skewed_case_is_skewed_and_masked():
    cfg = wl.CONFIGS["c3"]
    idx, _ = wl.make_routing(cfg)
    masked = (idx < 0).mean()
    assert 0.04 < masked < 0.06
    counts = np.sort(np.bincount(idx[idx >= 0], minlength=cfg.num_experts))[::-1]
    assert counts[0] > 8 * np.median(counts)            # a few hot experts
    uni, _ = wl.make_routing(wl.CONFIGS["c2"])
    ucounts = np.bincount(uni.reshape(-1), minlength=256)
    assert ucounts.max() < 2 * ucounts.mean()


def test_byte_budgets_match_the_published_table():
    mb = 1e6
    c2 = wl.algorithmic_bytes(4096, 7168, 256, 8, 8, 4096 * 8, 2, 0)
    assert abs(c2["total"] / mb - 1058.1) < 0.1 and abs(c2["dispatch"] / mb - 529.0) < 0.1
    tgt = wl.algorithmic_bytes(8192, 7168, 256, 8, 8, 8192 * 8, 2, 0)
    assert abs(tgt["total"] / mb - 2116.1) < 0.1
    c4 = wl.algorithmic_bytes(8192, 7168, 256, 8, 8, 8192 * 8, 1, 56)
    assert abs(c4["total"] / mb - 1604.1) < 0.2 and abs(c4["dispatch"] / mb - 546.1) < 0.1
    c5 = wl.algorithmic_bytes(16384, 4096, 128, 8, 8, 16384 * 8, 2, 0)
    assert abs(c5["total"] / mb - 2420.3) < 0.1


def test_reference_patterns_match_their_formulas():
    t = wl.reference_pattern_topk(300, 4, 4, 16, "rank_sweep")
    assert t[7, 2] == ((7 + 2) % 4) * 4 + (35 + 6) % 4
    t = wl.reference_pattern_topk(300, 8, 8, 32, "same_rank")
    assert t[5, 3] == ((15 + 8) % 8) * 4 + (5 + 21) % 4
    t = wl.reference_pattern_topk(300, 2, 2, 8, "spread")
    assert t[9, 1] == (153 + 31 + 2) % 8
    assert len(wl.REFERENCE_LAYOUT_CASES) == 13
    f = wl.reference_notify_flags(10, 4, 0)
    assert f.sum() == 20 and f[3, 3] == 1 and f[3, 0] == 1


def test_expert_outputs_generated_in_blocks_equal_the_one_shot_generator():
    """bench.py fills its expert outputs block by block from the same generator stream."""
    import torch
    cfg = wl.CONFIGS["c1"]
    whole = wl.make_expert_outputs(cfg, 300)
    rng = wl.rng_for(cfg, 2)
    blocks = torch.cat([wl.bf16_normal(rng, n, cfg.hidden) for n in (128, 128, 44)])
    assert torch.equal(whole.view(torch.int16), blocks.view(torch.int16))
