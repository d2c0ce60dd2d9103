"""Pins the CPU checker's permute and combine.

permute: numpy fancy-index gather.  combine: exact rational arithmetic rounded to fp32 once per
fused multiply-add (python Fractions; no floating-point library in the loop), exact integer sums,
K = 1 copies and the closed forms of the identity-expert and scale-by-constant workloads.
"""
from fractions import Fraction

import numpy as np
import pytest
import torch

from commbench_amd import workloads as wl


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


# ---- exact arithmetic ------------------------------------------------------------------

def round_fraction_to_f32(x: Fraction) -> float:
    """Nearest float32 to an exact rational, ties to even (normals and subnormals; no overflow)."""
    if x == 0:
        return 0.0
    sign = -1 if x < 0 else 1
    ax = -x if x < 0 else x
    e = ax.numerator.bit_length() - ax.denominator.bit_length()
    if Fraction(2) ** e > ax:
        e -= 1
    e = max(e, -126)
    q = ax / (Fraction(2) ** (e - 23))            # significand in units of the last place
    m = q.numerator // q.denominator
    rem = q - m
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (m & 1)):
        m += 1
    return float(np.float32(sign * float(m) * 2.0 ** (e - 23)))


def exact_combine(y_bits, slot_map, w, b0=None, b1=None):
    T, K = slot_map.shape
    H = y_bits.shape[1]
    yf = bits_to_f32(y_bits)
    out = np.zeros((T, H), dtype=np.float32)
    for t in range(T):
        for h in range(H):
            acc = 0.0
            for k in range(K):
                row = slot_map[t, k]
                if row < 0:
                    continue
                wk = Fraction(float(w[t, k])) if w is not None else Fraction(1)
                acc = round_fraction_to_f32(wk * Fraction(float(yf[row, h])) + Fraction(acc))
            for b in (b0, b1):
                if b is not None:
                    acc = round_fraction_to_f32(Fraction(acc) + Fraction(float(bits_to_f32(b)[t, h])))
            out[t, h] = acc
    return out


def test_round_fraction_helper():
    assert round_fraction_to_f32(Fraction(1) + Fraction(1, 2 ** 24)) == 1.0               # tie -> even
    assert round_fraction_to_f32(Fraction(1) + Fraction(3, 2 ** 24)) == float(np.float32(1 + 2 ** -22))
    assert round_fraction_to_f32(Fraction(1, 3)) == float(np.float32(1.0) / np.float32(3.0))
    assert round_fraction_to_f32(Fraction(-5, 2 ** 149)) == float(np.float32(-5 * 2.0 ** -149))


def small_case(seed, T=12, K=4, E=8, R=2, H=16, mask=0.2):
    rng = np.random.default_rng(seed)
    topk = wl.uniform_distinct_topk(rng, T, E, K)
    topk[rng.random((T, K)) < mask] = -1
    w = wl.softmax_gates(rng, T, K)
    return rng, topk, w


@pytest.mark.parametrize("seed", range(4))
def test_combine_matches_exact_fma_chain(oracle, seed):
    rng, topk, w = small_case(seed)
    T, K = topk.shape
    E, R, H = 8, 2, 16
    _, per_expert, _ = oracle.layout(topk, R, E)
    off, _ = oracle.expert_offsets(per_expert, R, 1)
    _, slot_map, _, _ = oracle.slot_maps(topk, E, off)
    y = bf16_bits(wl.bf16_normal(rng, int(off[-1]) + 1, H))
    b0 = bf16_bits(wl.bf16_normal(rng, T, H))
    b1 = bf16_bits(wl.bf16_normal(rng, T, H))
    for weights, biases in ((w, (None, None)), (None, (None, None)), (w, (b0, None)), (w, (b0, b1))):
        got = oracle.combine(y, slot_map, weights, *biases)
        want_f32 = exact_combine(y, slot_map, weights, *biases)
        want = torch.from_numpy(want_f32).to(torch.bfloat16)
        np.testing.assert_array_equal(got, bf16_bits(want))


def test_combine_integer_payload_exact_sums(oracle):
    """Small integers are exact in bf16 and fp32: the plain sum must be the integer sum."""
    rng = np.random.default_rng(1)
    T, K, E, R, H = 64, 8, 16, 4, 40
    topk = wl.uniform_distinct_topk(rng, T, E, K)
    topk[rng.random((T, K)) < 0.1] = -1
    _, per_expert, _ = oracle.layout(topk, R, E)
    off, _ = oracle.expert_offsets(per_expert, R, 1)
    _, slot_map, _, _ = oracle.slot_maps(topk, E, off)
    y_int = rng.integers(-15, 16, size=(int(off[-1]), H))
    y = bf16_bits(torch.from_numpy(y_int.astype(np.float32)).to(torch.bfloat16))
    got = bits_to_f32(oracle.combine(y, slot_map, None))
    want = np.zeros((T, H))
    for t in range(T):
        for k in range(K):
            if slot_map[t, k] >= 0:
                want[t] += y_int[slot_map[t, k]]
    np.testing.assert_array_equal(got, want)          # |sum| <= 120 is exact in bf16


def test_combine_k1_unit_weight_is_a_copy(oracle):
    rng = np.random.default_rng(2)
    T, E, R, H = 50, 4, 2, 24
    topk = rng.integers(0, E, size=(T, 1)).astype(np.int64)
    _, per_expert, _ = oracle.layout(topk, R, E)
    off, _ = oracle.expert_offsets(per_expert, R, 1)
    _, slot_map, src_map, src_k = oracle.slot_maps(topk, E, off)
    x = wl.bf16_normal(rng, T, H)
    xb = bf16_bits(x)
    recv_x, _, _, _ = oracle.permute(xb.view(np.uint8), None, topk, None, src_map, src_k)
    got = oracle.combine(recv_x.view(np.uint16), slot_map, np.ones((T, 1), dtype=np.float32))
    np.testing.assert_array_equal(got, xb)


def test_combine_token_without_routes_is_zero(oracle):
    slot_map = np.full((3, 4), -1, dtype=np.int32)
    y = np.full((1, 8), 0x3F80, dtype=np.uint16)
    assert not oracle.combine(y, slot_map, None).any()


def test_identity_experts_closed_form(oracle):
    """Tiny config: identity experts, softmax gates: out[t] = bf16(sum_k fl(w_k * x[t] + ...)),
    within 2 bf16 ulp of x[t] because the gates sum to 1."""
    cfg = wl.CONFIGS["c1"]
    topk, w = wl.make_routing(cfg)
    x, _ = wl.make_payload(cfg)
    xb = bf16_bits(x)
    res = oracle.full_path(topk, w, xb.view(np.uint8), None, cfg.num_experts, cfg.num_ranks)
    out = oracle.combine(res["recv_x"].view(np.uint16), res["slot_map"], w)
    xf, of = bits_to_f32(xb), bits_to_f32(out)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(xf), 2.0 ** -126))) - 7)
    assert (np.abs(of - xf) <= 2 * ulp).all()
    assert (of == xf).mean() > 0.5


def test_scale_by_expert_closed_form(oracle):
    """Round trip with expert e scaling by 1 + e/128: out[t] ~= x[t] * sum_k w_k (1 + e_k/128)."""
    rng = np.random.default_rng(9)
    T, K, E, R, H = 40, 8, 128, 8, 32
    topk = wl.uniform_distinct_topk(rng, T, E, K)
    w = wl.softmax_gates(rng, T, K)
    x = wl.bf16_normal(rng, T, H)
    res = oracle.full_path(topk, w, bf16_bits(x).view(np.uint8), None, E, R)
    scaled = oracle.scale_rows_by_expert(res["recv_x"].view(np.uint16), res["expert_offsets"], 128.0)
    # per-row check of the scale step against torch arithmetic
    rows_e = res["recv_topk_idx"]
    want_rows = (res["recv_x"].view(np.uint16).astype(np.uint32) << 16).view(np.float32) * \
        (np.float32(1) + rows_e.astype(np.float32) / np.float32(128))[:, None]
    np.testing.assert_array_equal(
        scaled, bf16_bits(torch.from_numpy(want_rows.astype(np.float32)).to(torch.bfloat16)))
    out = bits_to_f32(oracle.combine(scaled, res["slot_map"], w))
    factor = (w.astype(np.float64) * (1 + topk / 128.0)).sum(axis=1)
    want = x.to(torch.float32).numpy().astype(np.float64) * factor[:, None]
    # each of the 8 rows carries one bf16 rounding (2^-9 relative) and the result one more
    np.testing.assert_allclose(out, want, rtol=2.0 ** -7, atol=1e-30)


# ---- permute -------------------------------------------------------------------------------

@pytest.mark.parametrize("align", [1, 16])
def test_permute_is_a_gather(oracle, align):
    rng = np.random.default_rng(4)
    T, K, E, R, row_bytes, S = 100, 8, 32, 8, 48, 3
    topk = wl.zipf_distinct_topk(rng, T, E, K, 1.2)
    topk[rng.random((T, K)) < 0.05] = -1
    w = wl.softmax_gates(rng, T, K)
    x = rng.integers(0, 256, size=(T, row_bytes), dtype=np.uint8)
    scales = rng.standard_normal((T, S)).astype(np.float32)
    _, per_expert, _ = oracle.layout(topk, R, E)
    off, _ = oracle.expert_offsets(per_expert, R, align)
    _, slot_map, src_map, src_k = oracle.slot_maps(topk, E, off)
    recv_x, recv_scales, recv_idx, recv_w = oracle.permute(x, scales, topk, w, src_map, src_k)
    live = src_map >= 0
    np.testing.assert_array_equal(recv_x[live], x[src_map[live]])
    np.testing.assert_array_equal(recv_scales[live], scales[src_map[live]])
    np.testing.assert_array_equal(recv_idx[live], topk[src_map[live], src_k[live]])
    np.testing.assert_array_equal(recv_w[live], w[src_map[live], src_k[live]])
    assert not recv_x[~live].any() and not recv_scales[~live].any()
    assert (recv_idx[~live] == -1).all() and (recv_w[~live] == 0).all()
    # every row of segment e belongs to expert e
    for e in range(E):
        seg = recv_idx[off[e]:off[e] + per_expert[e]]
        assert (seg == e).all()
    # inverse relation between the two maps
    t_idx, k_idx = np.nonzero(slot_map >= 0)
    np.testing.assert_array_equal(src_map[slot_map[t_idx, k_idx]], t_idx)
    np.testing.assert_array_equal(oracle.gather_weights(recv_w, slot_map),
                                  np.where(slot_map >= 0, w, 0).astype(np.float32))


def test_threaded_paths_agree(oracle):
    rng = np.random.default_rng(6)
    T, K, E, R, H = 300, 8, 64, 8, 256
    topk = wl.uniform_distinct_topk(rng, T, E, K)
    w = wl.softmax_gates(rng, T, K)
    x = bf16_bits(wl.bf16_normal(rng, T, H))
    a = oracle.full_path(topk, w, x.view(np.uint8), None, E, R, num_threads=1)
    b = oracle.full_path(topk, w, x.view(np.uint8), None, E, R, num_threads=4)
    np.testing.assert_array_equal(a["recv_x"], b["recv_x"])
    np.testing.assert_array_equal(oracle.combine(a["recv_x"].view(np.uint16), a["slot_map"], w, num_threads=1),
                                  oracle.combine(a["recv_x"].view(np.uint16), a["slot_map"], w, num_threads=4))
