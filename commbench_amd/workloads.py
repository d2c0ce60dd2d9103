"""Seeded synthetic workloads: routing tables, gate weights, bf16 / fp8 payloads.

Generator: numpy's PCG64 seeded with 0xC0FFEE + config id; the same arrays feed the HIP path, the
CPU checker and the benchmark.  Also the reference's closed-form routing patterns
(datasets/example042_deepep_dispatch_layout/nv/empty_deepep_dispatch_layout.cu:178-206,
datasets/example047_deepep_intranode_notify_dispatch/nv/empty_deepep_intranode_notify_dispatch.cu:189-193),
which its own correctness cases are built from.
"""
from dataclasses import dataclass
from typing import Optional

import numpy as np

SEED_BASE = 0xC0FFEE


@dataclass(frozen=True)
class Config:
    name: str
    config_id: int
    num_tokens: int
    hidden: int
    num_experts: int
    num_topk: int
    num_ranks: int
    routing: str = "uniform"      # "uniform" | "zipf"
    zipf_s: float = 1.2
    mask_prob: float = 0.0
    payload: str = "bf16"         # "bf16" | "fp8"
    expert_scale_denom: float = 0.0   # > 0: expert e multiplies its rows by 1 + e / denom

    @property
    def row_bytes(self) -> int:
        return self.hidden * (2 if self.payload == "bf16" else 1)

    @property
    def num_scales(self) -> int:
        return self.hidden // 128 if self.payload == "fp8" else 0


CONFIGS = {
    "c1": Config("c1", 1, 128, 256, 8, 2, 2),
    "c2": Config("c2", 2, 4096, 7168, 256, 8, 8),
    "c3": Config("c3", 3, 4096, 7168, 256, 8, 8, routing="zipf", mask_prob=0.05),
    "c4": Config("c4", 4, 8192, 7168, 256, 8, 8, payload="fp8"),
    "c5": Config("c5", 5, 16384, 4096, 128, 8, 8, expert_scale_denom=128.0),
    # The shape the throughput target is quoted on: 8192 x 7168 bf16, 256 experts, top-8.
    "target": Config("target", 6, 8192, 7168, 256, 8, 8),
}


def rng_for(cfg: Config, stream: int = 0) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64([SEED_BASE + cfg.config_id, stream]))


# ---- routing -----------------------------------------------------------------

def uniform_distinct_topk(rng: np.random.Generator, T: int, E: int, K: int) -> np.ndarray:
    """K distinct experts per token, uniform over K-subsets, in random order."""
    keys = rng.random((T, E), dtype=np.float32)
    return np.argsort(keys, axis=1, kind="stable")[:, :K].astype(np.int64)


def zipf_distinct_topk(rng: np.random.Generator, T: int, E: int, K: int, s: float) -> np.ndarray:
    """K draws without replacement from p(j) ~ (j+1)^-s over a seeded permutation of experts
    (Gumbel top-k, which is sequential renormalised sampling)."""
    perm = rng.permutation(E)
    logp = np.empty(E, dtype=np.float64)
    logp[perm] = -s * np.log(np.arange(1, E + 1, dtype=np.float64))
    gumbel = -np.log(-np.log(rng.random((T, E), dtype=np.float64)))
    keys = logp[None, :] + gumbel
    return np.argsort(-keys, axis=1, kind="stable")[:, :K].astype(np.int64)


def softmax_gates(rng: np.random.Generator, T: int, K: int) -> np.ndarray:
    """fp32 softmax over the K selected N(0,1) logits (= softmax over all experts renormalised
    over the selected ones)."""
    logits = rng.standard_normal((T, K), dtype=np.float32)
    z = np.exp(logits - logits.max(axis=1, keepdims=True), dtype=np.float32)
    return (z / z.sum(axis=1, keepdims=True, dtype=np.float32)).astype(np.float32)


def make_routing(cfg: Config):
    rng = rng_for(cfg, 0)
    T, E, K = cfg.num_tokens, cfg.num_experts, cfg.num_topk
    if cfg.routing == "zipf":
        topk_idx = zipf_distinct_topk(rng, T, E, K, cfg.zipf_s)
    else:
        topk_idx = uniform_distinct_topk(rng, T, E, K)
    if cfg.mask_prob > 0.0:
        topk_idx[rng.random((T, K)) < cfg.mask_prob] = -1
    topk_weights = softmax_gates(rng, T, K)
    return np.ascontiguousarray(topk_idx), np.ascontiguousarray(topk_weights)


# ---- the reference's closed-form patterns -----------------------------------------

def reference_pattern_topk(T: int, K: int, R: int, E: int, pattern: str) -> np.ndarray:
    """makeTopk of the reference's layout example (example042 .cu:178-206)."""
    P = E // R
    t = np.arange(T, dtype=np.int64)[:, None]
    k = np.arange(K, dtype=np.int64)[None, :]
    if pattern == "rank_sweep":
        e = ((t + k) % R) * P + (t * 5 + k * 3) % P
    elif pattern == "same_rank":
        e = ((t * 3 + K) % R) * P + (t + k * 7) % P
    elif pattern == "spread":
        e = (t * 17 + k * 31 + R) % E
    else:
        raise ValueError(pattern)
    return np.ascontiguousarray(e.astype(np.int64))


# (T, K, R, E, pattern): the reference's correctness cases (example042 .cu:401-410).
REFERENCE_LAYOUT_CASES = [(257, 1, 1, 4, "spread")] + [
    case for R in (2, 4, 8) for case in (
        (257, 1, R, 4 * R, "spread"), (1024, 2, R, 4 * R, "spread"),
        (4096, 4, R, 4 * R, "rank_sweep"), (4096, 8, R, 4 * R, "same_rank"))]

# The reference's benchmark cases (example042 .cu:419-424).
REFERENCE_LAYOUT_BENCH_CASES = [
    (1024, 2, 8, 32, "spread"), (4096, 2, 8, 32, "spread"), (16384, 2, 8, 32, "spread"),
    (65536, 2, 8, 32, "spread"), (65536, 4, 8, 32, "rank_sweep"), (65536, 8, 8, 32, "same_rank"),
    (65536, 2, 4, 32, "spread")]


def reference_notify_flags(T: int, R: int, src_rank: int = 0) -> np.ndarray:
    """is_token_in_rank built by the reference's notify example (example047 .cu:189-193,437-447):
    min(2, R) slots per token, destination routeDst(src_rank, token, slot)."""
    flags = np.zeros((T, R), dtype=np.uint8)
    t = np.arange(T)
    for slot in range(min(2, R)):
        if R == 1:
            dst = np.zeros(T, dtype=np.int64)
        else:
            stride = (src_rank % (R - 1)) + 1
            dst = (t + src_rank + slot * stride) % R
        flags[t, dst] = 1
    return flags


def reference_notify_channels(R: int) -> int:
    """C = min(16, max(4, 2R)) (example047 .cu:599-610)."""
    return min(16, max(4, 2 * R))


# ---- payloads ------------------------------------------------------------------

def bf16_normal(rng: np.random.Generator, rows: int, cols: int):
    """N(0,1) rounded to bf16 (round to nearest even); returns a torch.bfloat16 CPU tensor."""
    import torch
    f = rng.standard_normal((rows, cols), dtype=np.float32)
    return torch.from_numpy(f).to(torch.bfloat16)


def quantize_fp8_blockwise(x_bf16, block: int = 128):
    """Per token, per 128-column block: scale = amax / 448 in fp32 (1.0 for an all-zero block),
    q = e4m3fn(x / scale) with round to nearest even and saturation at +-448.
    Returns (q: torch.float8_e4m3fn [T,H], scales: torch.float32 [T,H/block])."""
    import torch
    T, H = x_bf16.shape
    xf = x_bf16.to(torch.float32).view(T, H // block, block)
    amax = xf.abs().amax(dim=2)
    scales = torch.where(amax > 0, amax / 448.0, torch.ones_like(amax))
    q = (xf / scales[:, :, None]).clamp_(-448.0, 448.0).to(torch.float8_e4m3fn)
    return q.view(T, H), scales.contiguous()


def make_payload(cfg: Config):
    """Returns (x, scales): x is torch.bfloat16 or torch.float8_e4m3fn [T,H] on the CPU; scales is
    float32 [T, H/128] for fp8 and None otherwise."""
    x = bf16_normal(rng_for(cfg, 1), cfg.num_tokens, cfg.hidden)
    if cfg.payload == "fp8":
        return quantize_fp8_blockwise(x)
    return x, None


def make_expert_outputs(cfg: Config, rows: int):
    """Fresh bf16 N(0,1) expert outputs [rows, hidden] (the combine input of the fp8 case)."""
    return bf16_normal(rng_for(cfg, 2), rows, cfg.hidden)


# ---- byte budgets -----------------------------------------------------------------

def algorithmic_bytes(T: int, H: int, E: int, K: int, R: int, N: int, payload_elt: int,
                      num_scales: int) -> dict:
    """Minimum traffic: every source row read once, every output row written once."""
    layout = T * K * 8 + T * R + (R + E) * 4 + (E + 1) * 4
    dispatch = (T * H * payload_elt + N * H * payload_elt + (T + N) * num_scales * 4
                + T * K * 8 + N * 4 + T * K * 4)
    combine = N * H * 2 + T * H * 2 + T * K * 4 + T * K * 4
    return {"layout": layout, "dispatch": dispatch, "combine": combine,
            "total": layout + dispatch + combine}
