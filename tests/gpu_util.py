"""Shared helpers of the GPU parity tests: run the HIP path through the C ABI on numpy inputs."""
import numpy as np
import torch

from commbench_amd import ops

DEV = "cuda:0"


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def as_bytes(t: torch.Tensor) -> np.ndarray:
    t = t.detach().cpu().contiguous()
    return t.view(torch.uint8).numpy().reshape(t.shape[0], -1)


def bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


def bf16_ulp_distance(a_bits: np.ndarray, b_bits: np.ndarray) -> np.ndarray:
    """Distance in representable bf16 values (sign-magnitude bits mapped to a monotone line)."""
    def line(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)
    return np.abs(line(a_bits) - line(b_bits))


def garbage_like(t: torch.Tensor) -> torch.Tensor:
    """Fills an output buffer with a recognisable non-zero pattern (kernels must overwrite)."""
    return t.view(torch.uint8).fill_(0xA5)


RANK_SLOT_BASE = 5 * 65536
SCHEDULES = ("token", "destination")                                   # both copy kernels (ops.Buffer.dispatch)
BY_TOKEN, BY_DESTINATION = 2, 4                                        # MI_EP_DISPATCH_BY_* flag bits
TILE_TOKENS = 256                                                     # tokens per route_order tile


def run_fused_layout(buf: ops.Buffer, topk_idx_np, expert_alignment=1, num_channels=0):
    topk = torch.from_numpy(topk_idx_np).to(DEV)
    h = buf.dispatch_layout(topk, expert_alignment, num_channels, rank_slot_base=RANK_SLOT_BASE)
    torch.cuda.synchronize()
    buf.status()
    return topk, h


def source_chunk_counts(flags: np.ndarray, num_ranks: int) -> np.ndarray:
    """int32[src, dst]: tokens of source chunk src flagged for rank dst, the tokens taken as num_ranks
    contiguous chunks of ceil(T / R) (the notify example's range rule, example047 .cu:73-79); input
    of oracle.rank_prefix."""
    T = flags.shape[0]
    per_chunk = -(-T // num_ranks) if T else 0
    counts = np.zeros((num_ranks, num_ranks), dtype=np.int32)
    for src in range(num_ranks):
        start = min(per_chunk * src, T)
        counts[src] = flags[start:min(start + per_chunk, T)].sum(axis=0)
    return counts


def check_layout_against_oracle(oracle, h, topk_np, R, E, align=1, channels=0):
    per_rank, per_expert, flags = oracle.layout(topk_np, R, E)
    off, psum = oracle.expert_offsets(per_expert, R, align)
    slot_rel, slot_map, src_map, src_k = oracle.slot_maps(topk_np, E, off)
    np.testing.assert_array_equal(h.num_tokens_per_rank.cpu().numpy(), per_rank)
    np.testing.assert_array_equal(h.num_tokens_per_expert.cpu().numpy(), per_expert)
    np.testing.assert_array_equal(h.is_token_in_rank.cpu().numpy().view(np.uint8), flags)
    np.testing.assert_array_equal(h.expert_offsets.cpu().numpy(), off)
    np.testing.assert_array_equal(h.psum_rank_rows.cpu().numpy(), psum)
    np.testing.assert_array_equal(h.slot_rel.cpu().numpy(), slot_rel)
    if h.rank_slot_idx is not None and topk_np.shape[0] > 0:
        np.testing.assert_array_equal(h.rank_slot_idx.cpu().numpy(),
                                      oracle.rank_slots(topk_np, R, E, RANK_SLOT_BASE))
    if h.route_order is not None and topk_np.shape[0] > 0:
        want = oracle.route_order(topk_np, E, TILE_TOKENS)
        got = h.route_order.cpu().numpy()
        assert got.shape == want.shape
        written = want[:, 0] != -7                       # entries past the last token are unspecified
        np.testing.assert_array_equal(got[written], want[written])
    if channels:
        np.testing.assert_array_equal(h.channel_prefix_matrix.cpu().numpy(),
                                      oracle.channel_prefix(flags, channels))
    np.testing.assert_array_equal(h.rank_prefix_matrix().cpu().numpy(),
                                  oracle.rank_prefix(source_chunk_counts(flags, R)))
    return dict(per_rank=per_rank, per_expert=per_expert, flags=flags, off=off, psum=psum,
                slot_rel=slot_rel, slot_map=slot_map, src_map=src_map, src_k=src_k)
