"""numpy front end of the CPU checker (oracle/ep_oracle.c).

TEST INFRASTRUCTURE: imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg
of bench.py only.  The shipped package never imports it.
"""
import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_DIR, "libep_oracle.so")
_lib = None


def build() -> str:
    proc = subprocess.run(["make", "-C", _DIR, "-B", "libep_oracle.so"], capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("oracle build failed:\n" + proc.stdout + proc.stderr)
    return LIB_PATH


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        lib = ctypes.CDLL(LIB_PATH)
        lib.ep_oracle_bf16_to_f32.restype = ctypes.c_float
        lib.ep_oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        lib.ep_oracle_f32_to_bf16.restype = ctypes.c_uint16
        lib.ep_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        _lib = lib
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    x = _c(x, np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    _load().ep_oracle_f32_to_bf16_array(_p(x), _p(out), ctypes.c_int64(x.size))
    return out


def bf16_to_f32(x: np.ndarray) -> np.ndarray:
    x = _c(x, np.uint16)
    out = np.empty(x.shape, dtype=np.float32)
    _load().ep_oracle_bf16_to_f32_array(_p(x), _p(out), ctypes.c_int64(x.size))
    return out


def layout(topk_idx: np.ndarray, num_ranks: int, num_experts: int):
    topk_idx = _c(topk_idx, np.int64)
    T, K = topk_idx.shape
    per_rank = np.empty(num_ranks, dtype=np.int32)
    per_expert = np.empty(num_experts, dtype=np.int32)
    flags = np.empty((T, num_ranks), dtype=np.uint8)
    rc = _load().ep_oracle_layout(_p(topk_idx), T, K, num_ranks, num_experts, _p(per_rank),
                                  _p(per_expert), _p(flags))
    if rc != 0:
        raise ValueError(f"ep_oracle_layout: {rc}")
    return per_rank, per_expert, flags


def expert_offsets(per_expert: np.ndarray, num_ranks: int, expert_alignment: int = 1):
    per_expert = _c(per_expert, np.int32)
    E = per_expert.shape[0]
    off = np.empty(E + 1, dtype=np.int32)
    psum = np.empty(num_ranks, dtype=np.int32)
    rc = _load().ep_oracle_expert_offsets(_p(per_expert), E, num_ranks, expert_alignment, _p(off), _p(psum))
    if rc != 0:
        raise ValueError(f"ep_oracle_expert_offsets: {rc}")
    return off, psum


def slot_maps(topk_idx: np.ndarray, num_experts: int, off: np.ndarray):
    """Returns (slot_rel[T,K], slot_map[T,K], src_map[rows], src_k[rows])."""
    topk_idx = _c(topk_idx, np.int64)
    off = _c(off, np.int32)
    T, K = topk_idx.shape
    rows = int(off[num_experts])
    slot_rel = np.empty((T, K), dtype=np.int32)
    slot_map = np.empty((T, K), dtype=np.int32)
    src_map = np.empty(rows, dtype=np.int32)
    src_k = np.empty(rows, dtype=np.int32)
    fill = np.empty(num_experts, dtype=np.int32)
    _load().ep_oracle_slot_maps(_p(topk_idx), T, K, num_experts, _p(off), _p(slot_rel), _p(slot_map),
                                _p(src_map), _p(src_k), _p(fill))
    return slot_rel, slot_map, src_map, src_k


def rank_slots(topk_idx: np.ndarray, num_ranks: int, num_experts: int, base: int = 0) -> np.ndarray:
    topk_idx = _c(topk_idx, np.int64)
    T, K = topk_idx.shape
    out = np.empty((T, K), dtype=np.int32)
    rc = _load().ep_oracle_rank_slots(_p(topk_idx), T, K, num_ranks, num_experts, base, _p(out))
    if rc != 0:
        raise ValueError(f"ep_oracle_rank_slots: {rc}")
    return out


def route_order(topk_idx: np.ndarray, num_experts: int, tile_tokens: int = 256, fill: int = -7) -> np.ndarray:
    """int32[tiles * tile_tokens * K, 4]; entries past the last token's keep `fill`."""
    topk_idx = _c(topk_idx, np.int64)
    T, K = topk_idx.shape
    tiles = (T + tile_tokens - 1) // tile_tokens
    out = np.full((tiles * tile_tokens * K, 4), fill, dtype=np.int32)
    scratch = np.empty(2 * num_experts, dtype=np.int32)
    rc = _load().ep_oracle_route_order(_p(topk_idx), T, K, num_experts, tile_tokens, _p(out), _p(scratch))
    if rc != 0:
        raise ValueError(f"ep_oracle_route_order: {rc}")
    return out


def channel_prefix(flags: np.ndarray, num_channels: int) -> np.ndarray:
    flags = _c(flags, np.uint8)
    T, R = flags.shape
    out = np.empty((R, num_channels), dtype=np.int32)
    rc = _load().ep_oracle_channel_prefix(_p(flags), T, R, num_channels, _p(out))
    if rc != 0:
        raise ValueError(f"ep_oracle_channel_prefix: {rc}")
    return out


def rank_prefix(counts: np.ndarray) -> np.ndarray:
    counts = _c(counts, np.int32)
    out = np.empty_like(counts)
    _load().ep_oracle_rank_prefix(_p(counts), counts.shape[0], _p(out))
    return out


def permute(x_bytes: np.ndarray, scales, topk_idx, topk_weights, src_map, src_k, num_threads: int = 1):
    """x_bytes: uint8[T, row_bytes].  Returns (recv_x uint8[rows,row_bytes], recv_scales|None,
    recv_topk_idx int64[rows], recv_topk_weights float32[rows]|None)."""
    x_bytes = _c(x_bytes, np.uint8)
    topk_idx = _c(topk_idx, np.int64)
    src_map = _c(src_map, np.int32)
    src_k = _c(src_k, np.int32)
    T, row_bytes = x_bytes.shape
    K = topk_idx.shape[1]
    rows = src_map.shape[0]
    recv_x = np.empty((rows, row_bytes), dtype=np.uint8)
    num_scales = 0
    recv_scales = None
    if scales is not None:
        scales = _c(scales, np.float32)
        num_scales = scales.shape[1]
        recv_scales = np.empty((rows, num_scales), dtype=np.float32)
    recv_idx = np.empty(rows, dtype=np.int64)
    recv_w = None
    if topk_weights is not None:
        topk_weights = _c(topk_weights, np.float32)
        recv_w = np.empty(rows, dtype=np.float32)
    _load().ep_oracle_permute(_p(x_bytes), row_bytes, _p(scales), num_scales, _p(topk_idx),
                              _p(topk_weights), K, _p(src_map), _p(src_k), rows, _p(recv_x),
                              _p(recv_scales), _p(recv_idx), _p(recv_w), num_threads)
    return recv_x, recv_scales, recv_idx, recv_w


def permute_ranks(x_bytes: np.ndarray, scales, topk_idx, topk_weights, num_ranks: int, num_experts: int,
                  source_token_base: int = 0, local_expert_ids: bool = False, expand_slot_map=None,
                  capacity_rows=None):
    """Dispatch de-duplicated by destination rank; returns a dict (arrays trimmed to the row total)."""
    topk_idx = _c(topk_idx, np.int64)
    T, K = topk_idx.shape
    x_bytes = _c(x_bytes, np.uint8)
    row_bytes = x_bytes.shape[1]
    scales = None if scales is None else _c(scales, np.float32)
    S = 0 if scales is None else scales.shape[1]
    topk_weights = None if topk_weights is None else _c(topk_weights, np.float32)
    expand_slot_map = None if expand_slot_map is None else _c(expand_slot_map, np.int32)
    cap = T * min(K, num_ranks) if capacity_rows is None else capacity_rows
    out = dict(recv_x=np.zeros((cap, row_bytes), dtype=np.uint8),
               recv_scales=None if scales is None else np.zeros((cap, S), dtype=np.float32),
               recv_topk_idx=np.full((cap, K), -9, dtype=np.int64),
               recv_topk_weights=np.full((cap, K), -9.0, dtype=np.float32),
               recv_src_metadata=np.full((cap, 2 + K), -9, dtype=np.int32),
               rank_row_map=np.empty((T, K), dtype=np.int32),
               psum_rank_tokens=np.empty(num_ranks, dtype=np.int32))
    rc = _load().ep_oracle_permute_ranks(
        _p(x_bytes), row_bytes, _p(scales), S, _p(topk_idx), _p(topk_weights), T, K, num_ranks, num_experts,
        source_token_base, 1 if local_expert_ids else 0, _p(expand_slot_map), cap, _p(out["recv_x"]),
        _p(out["recv_scales"]), _p(out["recv_topk_idx"]), _p(out["recv_topk_weights"]),
        _p(out["recv_src_metadata"]), _p(out["rank_row_map"]), _p(out["psum_rank_tokens"]))
    if rc != 0:
        raise ValueError(f"ep_oracle_permute_ranks: {rc}")
    rows = min(int(out["psum_rank_tokens"][-1]), cap)
    for key in ("recv_x", "recv_scales", "recv_topk_idx", "recv_topk_weights", "recv_src_metadata"):
        if out[key] is not None:
            out[key] = out[key][:rows]
    return out


def gather_rows(x_bytes: np.ndarray, scales, src_map: np.ndarray):
    x_bytes = _c(x_bytes, np.uint8)
    src_map = _c(src_map, np.int32)
    T, row_bytes = x_bytes.shape
    rows = src_map.shape[0]
    recv_x = np.empty((rows, row_bytes), dtype=np.uint8)
    num_scales, recv_scales = 0, None
    if scales is not None:
        scales = _c(scales, np.float32)
        num_scales = scales.shape[1]
        recv_scales = np.empty((rows, num_scales), dtype=np.float32)
    _load().ep_oracle_gather_rows(_p(x_bytes), row_bytes, _p(scales), num_scales, _p(src_map), rows, T,
                                  _p(recv_x), _p(recv_scales))
    return recv_x, recv_scales


def pull_indices(src_map: np.ndarray, tokens_per_source_rank: int) -> np.ndarray:
    src_map = _c(src_map, np.int32)
    out = np.empty((src_map.shape[0], 2), dtype=np.int32)
    _load().ep_oracle_pull_indices(_p(src_map), src_map.shape[0], tokens_per_source_rank, _p(out))
    return out


def combine(y_bits: np.ndarray, slot_map: np.ndarray, topk_weights=None, bias_0=None, bias_1=None,
            num_threads: int = 1) -> np.ndarray:
    """y_bits: uint16[rows, H] bf16 bit patterns.  Returns uint16[T, H]."""
    y_bits = _c(y_bits, np.uint16)
    slot_map = _c(slot_map, np.int32)
    T, K = slot_map.shape
    H = y_bits.shape[1]
    if topk_weights is not None:
        topk_weights = _c(topk_weights, np.float32)
    if bias_0 is not None:
        bias_0 = _c(bias_0, np.uint16)
    if bias_1 is not None:
        bias_1 = _c(bias_1, np.uint16)
    out = np.empty((T, H), dtype=np.uint16)
    _load().ep_oracle_combine(_p(y_bits), _p(slot_map), _p(topk_weights), _p(bias_0), _p(bias_1),
                              T, K, H, _p(out), num_threads)
    return out


def gather_weights(recv_w: np.ndarray, slot_map: np.ndarray) -> np.ndarray:
    recv_w = _c(recv_w, np.float32)
    slot_map = _c(slot_map, np.int32)
    T, K = slot_map.shape
    out = np.empty((T, K), dtype=np.float32)
    _load().ep_oracle_gather_weights(_p(recv_w), _p(slot_map), T, K, _p(out))
    return out


def gather_idx(recv_idx: np.ndarray, slot_map: np.ndarray) -> np.ndarray:
    recv_idx = _c(recv_idx, np.int64)
    slot_map = _c(slot_map, np.int32)
    T, K = slot_map.shape
    out = np.empty((T, K), dtype=np.int64)
    _load().ep_oracle_gather_idx(_p(recv_idx), _p(slot_map), T, K, _p(out))
    return out


def gather_rank_side(recv_w, recv_idx, rank_row_map: np.ndarray):
    """(combined_topk_weights, combined_topk_idx) of the per-rank format; either input may be None."""
    rank_row_map = _c(rank_row_map, np.int32)
    T, K = rank_row_map.shape
    rows = 0
    out_w = out_i = None
    if recv_w is not None:
        recv_w = _c(recv_w, np.float32)
        rows = recv_w.shape[0]
        out_w = np.empty((T, K), dtype=np.float32)
    if recv_idx is not None:
        recv_idx = _c(recv_idx, np.int64)
        rows = recv_idx.shape[0]
        out_i = np.empty((T, K), dtype=np.int64)
    _load().ep_oracle_gather_rank_side(_p(recv_w), _p(recv_idx), _p(rank_row_map), T, K, rows, _p(out_w), _p(out_i))
    return out_w, out_i


def tile_rank_counts(flags: np.ndarray, tile_tokens: int = 256) -> np.ndarray:
    flags = _c(flags, np.uint8)
    T, R = flags.shape
    out = np.empty(((T + tile_tokens - 1) // tile_tokens, R), dtype=np.int32)
    rc = _load().ep_oracle_tile_rank_counts(_p(flags), T, R, tile_tokens, _p(out))
    if rc != 0:
        raise ValueError(f"ep_oracle_tile_rank_counts: {rc}")
    return out


def accumulate_stats(per_expert: np.ndarray, stats: np.ndarray) -> np.ndarray:
    """stats += per_expert, in place; returns stats."""
    per_expert = _c(per_expert, np.int32)
    assert stats.dtype == np.int32 and stats.flags.c_contiguous and stats.shape == per_expert.shape
    _load().ep_oracle_accumulate_stats(_p(per_expert), per_expert.shape[0], _p(stats))
    return stats


def scale_rows_by_expert(rows_bits: np.ndarray, off: np.ndarray, denom: float, num_threads: int = 1):
    rows_bits = _c(rows_bits, np.uint16)
    off = _c(off, np.int32)
    out = np.empty_like(rows_bits)
    _load().ep_oracle_scale_rows_by_expert(_p(rows_bits), _p(off), off.shape[0] - 1,
                                           rows_bits.shape[1], ctypes.c_float(denom), _p(out),
                                           num_threads)
    return out


def full_path(topk_idx, topk_weights, x_bytes, scales, num_experts, num_ranks,
              expert_alignment: int = 1, num_threads: int = 1):
    """Layout -> offsets -> slot maps -> permute, in one call.  Returns a dict."""
    per_rank, per_expert, flags = layout(topk_idx, num_ranks, num_experts)
    off, psum = expert_offsets(per_expert, num_ranks, expert_alignment)
    slot_rel, slot_map, src_map, src_k = slot_maps(topk_idx, num_experts, off)
    recv_x, recv_scales, recv_idx, recv_w = permute(x_bytes, scales, topk_idx, topk_weights,
                                                    src_map, src_k, num_threads)
    return dict(num_tokens_per_rank=per_rank, num_tokens_per_expert=per_expert,
                is_token_in_rank=flags, expert_offsets=off, psum_rank_rows=psum, slot_rel=slot_rel,
                slot_map=slot_map, recv_src_map=src_map, src_k=src_k, recv_x=recv_x,
                recv_scales=recv_scales, recv_topk_idx=recv_idx, recv_topk_weights=recv_w)
