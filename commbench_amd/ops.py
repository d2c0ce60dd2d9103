"""Host-side operator surface over the C ABI (include/mi_ep.h).

Mirrors the DeepEP-style operators the reference drives
(datasets/example080_deepep_jit_dispatch_payload/nv/build_and_run.py:710-732,
datasets/example082_deepep_jit_combine/nv/build_and_run.py:751-765) for one GPU whose HBM is
split into `num_ranks` partitions:

    get_dispatch_layout(topk_idx, num_experts, num_ranks)
        -> (num_tokens_per_rank, num_tokens_per_expert, is_token_in_rank)
    dispatch(x, scales, topk_idx, topk_weights, ...)
        -> (recv_x, recv_scales, recv_src_map, handle)
    combine(y, slot_map | handle, topk_weights) -> combined_x
    dispatch_ranks(buffer, x, scales, topk_idx, topk_weights, ...)       the reference's own receive
        -> (recv_x, recv_topk_idx, recv_topk_weights, handle)            format: one row per token
    combine_ranks(y, handle, recv_topk_weights) -> combined_x[, weights]  and destination rank
    dispatch_cached / pull_indices                                        pull form from a source map
    host_get_dispatch_layout / host_dispatch_layout / host_dispatch / host_dispatch_ranks /
    host_dispatch_cached / host_combine                                   numpy in, numpy out

torch is used for device memory and streams only; all arithmetic runs in the HIP kernels of
libmi_ep.so.  Nothing here falls back to torch ops or to the CPU.
"""
from dataclasses import dataclass
from typing import Optional, Tuple, Union

import torch

from . import _lib

MAX_RANKS = 8
MAX_TOPK = 8
MAX_EXPERTS = 1024
ZERO_PAD_PAYLOAD = 1   # MI_EP_DISPATCH_ZERO_PAD_PAYLOAD
BY_TOKEN = 2           # MI_EP_DISPATCH_BY_TOKEN
BY_DESTINATION = 4     # MI_EP_DISPATCH_BY_DESTINATION
STREAM_OUTPUT = 1      # MI_EP_COMBINE_STREAM_OUTPUT
_SCHEDULE_FLAGS = {"auto": 0, "token": BY_TOKEN, "destination": BY_DESTINATION}


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _check_routing(topk_idx: torch.Tensor, num_experts: int, num_ranks: int) -> Tuple[int, int]:
    _require(topk_idx.is_cuda, "topk_idx must live on the GPU")
    _require(topk_idx.dtype == torch.int64 and topk_idx.dim() == 2 and topk_idx.is_contiguous(),
             "topk_idx must be a contiguous int64 [num_tokens, num_topk] tensor")
    # Same wording as the reference's constructor checks (example042 .cu:96-107).
    _require(0 < num_ranks <= MAX_RANKS, f"num_ranks must be in [1, {MAX_RANKS}]")
    _require(0 < topk_idx.shape[1] <= MAX_TOPK, f"num_topk must be in [1, {MAX_TOPK}]")
    _require(num_experts > 0 and num_experts % num_ranks == 0,
             "num_experts must be divisible by num_ranks")
    _require(num_experts <= MAX_EXPERTS, f"num_experts must be at most {MAX_EXPERTS}")
    return topk_idx.shape[0], topk_idx.shape[1]


def get_dispatch_layout(topk_idx: torch.Tensor, num_experts: int, num_ranks: int):
    """Counts and flags only; the reference's DeepepDispatchLayout::compute (example042 .cu:110-132)."""
    T, K = _check_routing(topk_idx, num_experts, num_ranks)
    dev = topk_idx.device
    per_rank = torch.empty(num_ranks, dtype=torch.int32, device=dev)
    per_expert = torch.empty(num_experts, dtype=torch.int32, device=dev)
    in_rank = torch.empty((T, num_ranks), dtype=torch.bool, device=dev)
    lib = _lib.load()
    _lib.check(lib.mi_ep_get_dispatch_layout(_ptr(topk_idx), _ptr(per_rank), None, _ptr(per_expert),
                                             _ptr(in_rank), T, K, num_ranks, num_experts, _stream()),
               "mi_ep_get_dispatch_layout")
    return per_rank, per_expert, in_rank


@dataclass
class DispatchHandle:
    """State carried from dispatch to combine (the reference's `handle`, example082 bar.py:744-755)."""
    num_tokens: int
    num_topk: int
    num_experts: int
    num_ranks: int
    expert_alignment: int
    num_tokens_per_rank: torch.Tensor      # int32[R]
    num_tokens_per_expert: torch.Tensor    # int32[E]
    is_token_in_rank: torch.Tensor         # bool[T, R]
    expert_offsets: torch.Tensor           # int32[E + 1], exclusive over aligned counts
    psum_rank_rows: torch.Tensor           # int32[R], inclusive rows per partition
    channel_prefix_matrix: Optional[torch.Tensor]  # int32[R, C]
    rank_prefix_matrix_: torch.Tensor      # int32[R, R], [source chunk, destination rank]
    slot_rel: torch.Tensor                 # int32[T, K]
    rank_slot_idx: Optional[torch.Tensor] = None   # int32[T, K], the prologue's dst_buffer_slot_idx
    route_order: Optional[torch.Tensor] = None     # int32[tiles * 256 * K, 4], routes in destination order
    tile_rank_counts: Optional[torch.Tensor] = None  # int32[tiles, R], the prologue's rank_count_buffer
    copied_topk_idx: Optional[torch.Tensor] = None   # int64[T, K], the kernel's own copy of topk_idx
    slot_map: Optional[torch.Tensor] = None        # int32[T, K]
    recv_src_map: Optional[torch.Tensor] = None    # int32[capacity]
    recv_topk_idx: Optional[torch.Tensor] = None   # int64[capacity]
    recv_topk_weights: Optional[torch.Tensor] = None  # float32[capacity]

    def num_recv_rows(self) -> int:
        """Padded row total; synchronises the stream."""
        return int(self.expert_offsets[-1].item())

    def rank_prefix_matrix(self) -> torch.Tensor:
        """int32[src, dst]: tokens of source chunks 0..src flagged for rank dst, the tokens taken as
        num_ranks equal contiguous chunks (ceil(T / R) tokens each): the notify example's
        rank_prefix_matrix (example047 .cu:128-143,352-360) with chunks of this GPU's tokens standing
        for source ranks.  Written by the layout launch itself, whatever its num_channels."""
        return self.rank_prefix_matrix_


class Buffer:
    """Workspace owner, the one-GPU analogue of the reference's ElasticBuffer
    (example080 bar.py:683-693).  Calls on one Buffer must not overlap in time."""

    def __init__(self, num_max_tokens: int, num_topk: int, num_experts: int, num_ranks: int,
                 device: Union[str, torch.device] = "cuda"):
        _require(0 < num_ranks <= MAX_RANKS, f"num_ranks must be in [1, {MAX_RANKS}]")
        _require(0 < num_topk <= MAX_TOPK, f"num_topk must be in [1, {MAX_TOPK}]")
        _require(num_experts > 0 and num_experts % num_ranks == 0,
                 "num_experts must be divisible by num_ranks")
        _require(num_experts <= MAX_EXPERTS, f"num_experts must be at most {MAX_EXPERTS}")
        self.num_max_tokens = num_max_tokens
        self.num_topk = num_topk
        self.num_experts = num_experts
        self.num_ranks = num_ranks
        self.device = torch.device(device)
        lib = _lib.load()
        nbytes = lib.mi_ep_workspace_bytes(max(num_max_tokens, 1), num_topk, num_experts, num_ranks)
        _require(nbytes > 0, "unsupported shape")
        self.workspace = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        with torch.cuda.device(self.device):
            _lib.check(lib.mi_ep_workspace_init(_ptr(self.workspace), nbytes, _stream()),
                       "mi_ep_workspace_init")

    def set_wait_limit(self, max_polls: int) -> None:
        """Bounds the device-side waits of later layout launches on this buffer (0 = default)."""
        with torch.cuda.device(self.device):
            _lib.check(_lib.load().mi_ep_workspace_set_wait_limit(_ptr(self.workspace), max_polls, _stream()),
                       "mi_ep_workspace_set_wait_limit")

    def status(self) -> None:
        """Raises if a device-side bounded wait ever expired on this workspace."""
        lib = _lib.load()
        with torch.cuda.device(self.device):
            _lib.check(lib.mi_ep_workspace_status(_ptr(self.workspace), _stream()),
                       "mi_ep_workspace_status")

    def dispatch_layout(self, topk_idx: torch.Tensor, expert_alignment: int = 1,
                        num_channels: int = 0, rank_slot_base: Optional[int] = None,
                        route_order: bool = True, tile_rank_counts: bool = False,
                        copy_topk_idx: bool = False,
                        cumulative_expert_stats: Optional[torch.Tensor] = None) -> DispatchHandle:
        """Fused single-pass layout: counts, flags, offsets, per-route segment positions, and
        (unless `route_order` is False) the per-tile destination order that lets dispatch write
        adjacent rows together.

        With `rank_slot_base` (the reference's scaleup_rank_idx * num_max_tokens_per_rank) the
        handle also carries `rank_slot_idx`, the deterministic prologue's per-rank slot table
        (example078 .cu:36-40); `tile_rank_counts` adds its per-tile rank counts (:34-35),
        `copy_topk_idx` the kernel's own copy of the routing table (example080 .cu:33), and
        `cumulative_expert_stats` (int32[E]) has this call's per-expert counts added to it
        (example080 .cu:35,211-212)."""
        T, K = _check_routing(topk_idx, self.num_experts, self.num_ranks)
        _require(K == self.num_topk, "num_topk differs from the buffer's")
        _require(T <= self.num_max_tokens, "more tokens than the buffer was sized for")
        _require(expert_alignment >= 1, "expert_alignment must be positive")
        E, R, dev = self.num_experts, self.num_ranks, topk_idx.device
        h = DispatchHandle(
            num_tokens=T, num_topk=K, num_experts=E, num_ranks=R, expert_alignment=expert_alignment,
            num_tokens_per_rank=torch.empty(R, dtype=torch.int32, device=dev),
            num_tokens_per_expert=torch.empty(E, dtype=torch.int32, device=dev),
            is_token_in_rank=torch.empty((T, R), dtype=torch.bool, device=dev),
            expert_offsets=torch.empty(E + 1, dtype=torch.int32, device=dev),
            psum_rank_rows=torch.empty(R, dtype=torch.int32, device=dev),
            channel_prefix_matrix=(torch.empty((R, num_channels), dtype=torch.int32, device=dev)
                                   if num_channels > 0 else None),
            rank_prefix_matrix_=torch.empty((R, R), dtype=torch.int32, device=dev),
            slot_rel=torch.empty((T, K), dtype=torch.int32, device=dev),
            rank_slot_idx=(torch.empty((T, K), dtype=torch.int32, device=dev)
                           if rank_slot_base is not None else None),
        )
        lib = _lib.load()
        if route_order and T > 0:
            h.route_order = torch.empty((lib.mi_ep_route_order_bytes(T, K) // 16, 4), dtype=torch.int32,
                                        device=dev)
        if tile_rank_counts:
            h.tile_rank_counts = torch.empty(((T + 255) // 256, R), dtype=torch.int32, device=dev)
        if copy_topk_idx:
            h.copied_topk_idx = torch.empty((T, K), dtype=torch.int64, device=dev)
        if cumulative_expert_stats is not None:
            _require(cumulative_expert_stats.is_cuda and cumulative_expert_stats.dtype == torch.int32
                     and cumulative_expert_stats.is_contiguous() and cumulative_expert_stats.numel() == E,
                     "cumulative_expert_stats must be a contiguous int32 [num_experts] GPU tensor")
        _lib.check(lib.mi_ep_dispatch_layout(
            _ptr(topk_idx), T, K, R, E, expert_alignment, num_channels,
            _ptr(h.num_tokens_per_rank), _ptr(h.num_tokens_per_expert), _ptr(h.is_token_in_rank),
            _ptr(h.expert_offsets), _ptr(h.psum_rank_rows), _ptr(h.channel_prefix_matrix),
            _ptr(h.rank_prefix_matrix_), _ptr(h.slot_rel), _ptr(h.rank_slot_idx), rank_slot_base or 0,
            _ptr(h.route_order), _ptr(h.tile_rank_counts), _ptr(h.copied_topk_idx),
            _ptr(cumulative_expert_stats), _ptr(self.workspace), self.workspace.numel(), _stream()),
            "mi_ep_dispatch_layout")
        return h

    def dispatch(self, x: torch.Tensor, scales: Optional[torch.Tensor], topk_idx: torch.Tensor,
                 topk_weights: Optional[torch.Tensor], expert_alignment: int = 1,
                 num_channels: int = 0, handle: Optional[DispatchHandle] = None,
                 capacity_rows: Optional[int] = None, rank_slot_base: Optional[int] = None,
                 zero_pads: bool = False, column_major_recv_scales: bool = False, schedule: str = "auto"):
        """Layout (unless `handle` is given) + permute into the expert-contiguous buffer.

        Returns (recv_x, recv_scales, recv_src_map, handle).  Buffers hold `capacity_rows` rows
        (default: the worst case T*K + E*(alignment-1), so no host sync is needed); rows at and
        beyond handle.num_recv_rows() are unspecified.  With expert_alignment > 1 the pad rows'
        map entries are written (source -1); their payload is left alone, as in the reference's
        receive buffer, unless `zero_pads` asks for zero rows.
        `scales` may be any 2-D float32 view (row- or column-major, padded); with
        `column_major_recv_scales` the returned recv_scales is a [capacity, S] view of a [S, capacity]
        allocation, the layout the reference's TMA-aligned scale tensors have.
        `schedule` picks the copy kernel: "auto" (by shape and device), "token" or "destination";
        the results are identical.
        """
        _require(schedule in _SCHEDULE_FLAGS, 'schedule must be "auto", "token" or "destination"')
        if handle is None:
            handle = self.dispatch_layout(topk_idx, expert_alignment, num_channels, rank_slot_base)
        T, K, E = handle.num_tokens, handle.num_topk, handle.num_experts
        _require(x.is_cuda and x.dim() == 2 and x.is_contiguous() and x.shape[0] == T,
                 "x must be a contiguous [num_tokens, hidden] GPU tensor")
        row_bytes = x.shape[1] * x.element_size()
        _require(row_bytes % 16 == 0, "row size must be a multiple of 16 bytes")
        num_scales = 0
        if scales is not None:
            _require(scales.dtype == torch.float32 and scales.dim() == 2 and scales.shape[0] == T
                     and min(scales.stride()) >= 0, "scales must be a float32 [num_tokens, S] tensor or view")
            num_scales = scales.shape[1]
        if topk_weights is not None:
            _require(topk_weights.dtype == torch.float32 and topk_weights.is_contiguous()
                     and tuple(topk_weights.shape) == (T, K),
                     "topk_weights must be contiguous float32 [num_tokens, num_topk]")
        if capacity_rows is None:
            capacity_rows = T * K + E * (handle.expert_alignment - 1)
        dev = x.device
        recv_x = torch.empty((capacity_rows, x.shape[1]), dtype=x.dtype, device=dev)
        recv_scales = None
        if scales is not None and column_major_recv_scales:
            recv_scales = torch.empty((num_scales, capacity_rows), dtype=torch.float32, device=dev).t()
        elif scales is not None:
            recv_scales = torch.empty((capacity_rows, num_scales), dtype=torch.float32, device=dev)
        xs_strides = scales.stride() if scales is not None else (0, 0)
        rs_strides = recv_scales.stride() if recv_scales is not None else (0, 0)
        handle.recv_src_map = torch.empty(capacity_rows, dtype=torch.int32, device=dev)
        handle.recv_topk_idx = torch.empty(capacity_rows, dtype=torch.int64, device=dev)
        handle.recv_topk_weights = torch.empty(capacity_rows, dtype=torch.float32, device=dev)
        handle.slot_map = torch.empty((T, K), dtype=torch.int32, device=dev)
        lib = _lib.load()
        _lib.check(lib.mi_ep_dispatch_strided_scales(
            _ptr(x), _ptr(scales), xs_strides[0], xs_strides[1], _ptr(topk_idx), _ptr(topk_weights),
            _ptr(handle.expert_offsets), _ptr(handle.slot_rel), _ptr(handle.route_order),
            _ptr(handle.num_tokens_per_expert), T, K, E, handle.expert_alignment, row_bytes, num_scales,
            _ptr(recv_x), _ptr(recv_scales), rs_strides[0], rs_strides[1], _ptr(handle.recv_src_map),
            _ptr(handle.recv_topk_idx), _ptr(handle.recv_topk_weights), _ptr(handle.slot_map), capacity_rows,
            (ZERO_PAD_PAYLOAD if zero_pads else 0) | _SCHEDULE_FLAGS[schedule], _stream()),
            "mi_ep_dispatch_strided_scales")
        return recv_x, recv_scales, handle.recv_src_map, handle


@dataclass
class RankDispatchHandle:
    """What the per-rank dispatch hands to combine (the reference's handle, example082 bar.py:744-755)."""
    layout: DispatchHandle
    psum_rank_tokens: torch.Tensor        # int32[R], inclusive rows per rank
    recv_src_metadata: torch.Tensor       # int32[capacity, 2 + K]
    rank_row_map: torch.Tensor            # int32[T, K], row carrying each route
    combine_map: torch.Tensor             # int32[T, K], each received row once
    recv_scales: Optional[torch.Tensor] = None

    def num_recv_rows(self) -> int:
        """Rows received over all ranks; synchronises the stream."""
        return int(self.psum_rank_tokens[-1].item())


def dispatch_ranks(buffer: "Buffer", x: torch.Tensor, scales: Optional[torch.Tensor], topk_idx: torch.Tensor,
                   topk_weights: Optional[torch.Tensor], num_max_tokens_per_rank: Optional[int] = None,
                   rank_idx: int = 0, local_expert_ids: bool = False, expand: bool = False,
                   column_major_recv_scales: bool = False):
    """The reference's dispatch in its own receive format: one row per (token, destination rank),
    ranks' rows in token order (deterministic mode).  Returns (recv_x, recv_topk_idx,
    recv_topk_weights, handle) as DeepEP's `buffer.dispatch` does (example080 bar.py:725);
    `rank_idx * num_max_tokens_per_rank` offsets the source token ids in the metadata.
    With `expand`, the expert-contiguous dispatch runs too and the metadata names its rows.
    `scales` may be any 2-D float32 view; `column_major_recv_scales` returns them in a [S, rows]
    allocation viewed as [rows, S] (the reference passes token and hidden strides, example081 .cu:31)."""
    T, K = _check_routing(topk_idx, buffer.num_experts, buffer.num_ranks)
    E, R, dev = buffer.num_experts, buffer.num_ranks, topk_idx.device
    max_tokens = T if num_max_tokens_per_rank is None else num_max_tokens_per_rank
    base = rank_idx * max_tokens
    if expand:
        _, _, _, h = buffer.dispatch(x, scales, topk_idx, topk_weights, rank_slot_base=base)
    else:
        h = buffer.dispatch_layout(topk_idx, rank_slot_base=base, route_order=False)
    _require(x.is_cuda and x.dim() == 2 and x.is_contiguous() and x.shape[0] == T,
             "x must be a contiguous [num_tokens, hidden] GPU tensor")
    row_bytes = x.shape[1] * x.element_size()
    _require(row_bytes % 16 == 0, "row size must be a multiple of 16 bytes")
    S = 0
    if scales is not None:
        _require(scales.dtype == torch.float32 and scales.dim() == 2 and scales.shape[0] == T
                 and min(scales.stride()) >= 0, "scales must be a float32 [num_tokens, S] tensor or view")
        S = scales.shape[1]
    cap = T * min(K, R)
    recv_x = torch.empty((cap, x.shape[1]), dtype=x.dtype, device=dev)
    recv_scales = None
    if scales is not None and column_major_recv_scales:
        recv_scales = torch.empty((S, cap), dtype=torch.float32, device=dev).t()
    elif scales is not None:
        recv_scales = torch.empty((cap, S), dtype=torch.float32, device=dev)
    xs_strides = scales.stride() if scales is not None else (0, 0)
    rs_strides = recv_scales.stride() if recv_scales is not None else (0, 0)
    recv_idx = torch.empty((cap, K), dtype=torch.int64, device=dev)
    recv_w = torch.empty((cap, K), dtype=torch.float32, device=dev)
    rh = RankDispatchHandle(
        layout=h, psum_rank_tokens=torch.empty(R, dtype=torch.int32, device=dev),
        recv_src_metadata=torch.empty((cap, 2 + K), dtype=torch.int32, device=dev),
        rank_row_map=torch.empty((T, K), dtype=torch.int32, device=dev),
        combine_map=torch.empty((T, K), dtype=torch.int32, device=dev), recv_scales=recv_scales)
    _lib.check(_lib.load().mi_ep_dispatch_ranks_strided_scales(
        _ptr(x), _ptr(scales), xs_strides[0], xs_strides[1], _ptr(topk_idx), _ptr(topk_weights),
        _ptr(h.rank_slot_idx), base, _ptr(h.num_tokens_per_rank), _ptr(h.slot_map) if expand else None, T, K, R,
        E, row_bytes, S, base, 1 if local_expert_ids else 0, _ptr(recv_x), _ptr(recv_scales), rs_strides[0],
        rs_strides[1], _ptr(recv_idx), _ptr(recv_w), _ptr(rh.recv_src_metadata), _ptr(rh.rank_row_map),
        _ptr(rh.combine_map), _ptr(rh.psum_rank_tokens), cap, _stream()), "mi_ep_dispatch_ranks_strided_scales")
    return recv_x, recv_idx, recv_w, rh


def combine_ranks(y: torch.Tensor, handle: RankDispatchHandle, recv_topk_weights: Optional[torch.Tensor] = None,
                  bias=None, recv_topk_idx: Optional[torch.Tensor] = None):
    """The reference's combine of the per-rank format: the ordered sum of the rows a token sent
    out, one per rank (+ biases); with `recv_topk_weights` also the weights that travelled
    (combined_topk_weights, example082 bar.py:757-765), with `recv_topk_idx` also the expert ids
    (combined_topk_idx, example083 .cu:26).  Returns combined_x, then the weights, then the ids,
    as far as they were asked for."""
    out = combine(y, handle.combine_map, None, bias)
    if recv_topk_weights is None and recv_topk_idx is None:
        return out
    T, K = handle.rank_row_map.shape
    rows = None
    out_w = out_i = None
    if recv_topk_weights is not None:
        _require(recv_topk_weights.dtype == torch.float32 and recv_topk_weights.is_contiguous()
                 and recv_topk_weights.dim() == 2 and recv_topk_weights.shape[1] == K,
                 "recv_topk_weights must be contiguous float32 [rows, num_topk]")
        rows = recv_topk_weights.shape[0]
        out_w = torch.empty((T, K), dtype=torch.float32, device=y.device)
    if recv_topk_idx is not None:
        _require(recv_topk_idx.dtype == torch.int64 and recv_topk_idx.is_contiguous()
                 and recv_topk_idx.dim() == 2 and recv_topk_idx.shape[1] == K
                 and (rows is None or recv_topk_idx.shape[0] == rows),
                 "recv_topk_idx must be contiguous int64 [rows, num_topk]")
        rows = recv_topk_idx.shape[0]
        out_i = torch.empty((T, K), dtype=torch.int64, device=y.device)
    _lib.check(_lib.load().mi_ep_combine_rank_weights(
        _ptr(recv_topk_weights), _ptr(recv_topk_idx), _ptr(handle.rank_row_map), T, K, rows, _ptr(out_w),
        _ptr(out_i), _stream()), "mi_ep_combine_rank_weights")
    return tuple(t for t in (out, out_w, out_i) if t is not None)


def combine(y: torch.Tensor, slot_map: Union[torch.Tensor, DispatchHandle],
            topk_weights: Optional[torch.Tensor] = None,
            bias: Union[None, torch.Tensor, Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]] = None,
            recv_topk_weights: Optional[torch.Tensor] = None,
            recv_topk_idx: Optional[torch.Tensor] = None, stream_output: bool = False):
    """combined_x[t] = bf16(sum_k w[t,k] * y[slot_map[t,k]] (+ biases)), fp32 accumulation.

    topk_weights=None gives the reference's plain ordered sum.  When `recv_topk_weights` (the
    per-row weights that travelled with dispatch) is given, also returns them gathered back to
    [num_tokens, num_topk], as the reference's combined_topk_weights; `recv_topk_idx` (the per-row
    expert ids) likewise comes back as combined_topk_idx, after the weights.
    `stream_output` sends the result straight to HBM instead of through the memory-side cache
    (MI_EP_COMBINE_STREAM_OUTPUT): for outputs that nothing reads soon.
    """
    if isinstance(slot_map, DispatchHandle):
        _require(slot_map.slot_map is not None, "handle has not been through dispatch")
        slot_map = slot_map.slot_map
    _require(y.is_cuda and y.dtype == torch.bfloat16 and y.dim() == 2 and y.is_contiguous(),
             "y must be a contiguous bf16 [rows, hidden] GPU tensor")
    _require(slot_map.dtype == torch.int32 and slot_map.dim() == 2 and slot_map.is_contiguous(),
             "slot_map must be contiguous int32 [num_tokens, num_topk]")
    T, K = slot_map.shape
    _require(0 < K <= MAX_TOPK, f"num_topk must be in [1, {MAX_TOPK}]")
    H = y.shape[1]
    _require(H % 8 == 0, "hidden must be a multiple of 8")
    if topk_weights is not None:
        _require(topk_weights.dtype == torch.float32 and topk_weights.is_contiguous()
                 and tuple(topk_weights.shape) == (T, K),
                 "topk_weights must be contiguous float32 [num_tokens, num_topk]")
    bias_0 = bias_1 = None
    if isinstance(bias, torch.Tensor):
        bias_0 = bias
    elif bias is not None:
        bias_0, bias_1 = bias
    for b in (bias_0, bias_1):
        if b is not None:
            _require(b.dtype == torch.bfloat16 and b.is_contiguous() and tuple(b.shape) == (T, H),
                     "bias must be contiguous bf16 [num_tokens, hidden]")
    dev = y.device
    out = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    out_w = (torch.empty((T, K), dtype=torch.float32, device=dev)
             if recv_topk_weights is not None else None)
    out_i = (torch.empty((T, K), dtype=torch.int64, device=dev)
             if recv_topk_idx is not None else None)
    if recv_topk_idx is not None:
        _require(recv_topk_idx.dtype == torch.int64 and recv_topk_idx.is_contiguous(),
                 "recv_topk_idx must be contiguous int64 [rows]")
    lib = _lib.load()
    _lib.check(lib.mi_ep_combine(_ptr(y), y.shape[0], _ptr(slot_map), _ptr(topk_weights), _ptr(bias_0),
                                 _ptr(bias_1), _ptr(recv_topk_weights), _ptr(recv_topk_idx), T, K, H,
                                 _ptr(out), _ptr(out_w), _ptr(out_i), STREAM_OUTPUT if stream_output else 0,
                                 _stream()), "mi_ep_combine")
    if out_w is None and out_i is None:
        return out
    return tuple(t for t in (out, out_w, out_i) if t is not None)


def dispatch(x: torch.Tensor, scales: Optional[torch.Tensor], topk_idx: torch.Tensor,
             topk_weights: Optional[torch.Tensor], num_experts: int, num_ranks: int,
             expert_alignment: int = 1, num_channels: int = 0):
    """One-shot form: allocates a Buffer for this call's shape.  Prefer Buffer.dispatch in loops."""
    T, K = _check_routing(topk_idx, num_experts, num_ranks)
    buf = Buffer(T, K, num_experts, num_ranks, device=topk_idx.device)
    return buf.dispatch(x, scales, topk_idx, topk_weights, expert_alignment, num_channels)


def dispatch_cached(x: torch.Tensor, scales: Optional[torch.Tensor], recv_src_map: torch.Tensor,
                    num_rows: Optional[int] = None, ready_counters: Optional[torch.Tensor] = None,
                    rows_per_counter: int = 128):
    """Pull-mode dispatch of a new payload with the source map of an earlier dispatch (the
    reference's cached mode).  Returns (recv_x, recv_scales); pad rows are zero.  With
    `ready_counters` (zeroed int32[ceil(rows / rows_per_counter)]) every row bumps its block's
    counter once it is in place, as the ThunderKittens example's pull dispatch does."""
    _require(x.is_cuda and x.dim() == 2 and x.is_contiguous(), "x must be a contiguous 2-D GPU tensor")
    _require(recv_src_map.dtype == torch.int32 and recv_src_map.dim() == 1 and recv_src_map.is_contiguous(),
             "recv_src_map must be contiguous int32 [rows]")
    rows = recv_src_map.shape[0] if num_rows is None else num_rows
    _require(0 <= rows <= recv_src_map.shape[0], "num_rows exceeds the map")
    row_bytes = x.shape[1] * x.element_size()
    _require(row_bytes % 16 == 0, "row size must be a multiple of 16 bytes")
    num_scales = 0
    if scales is not None:
        _require(scales.dtype == torch.float32 and scales.dim() == 2 and scales.is_contiguous()
                 and scales.shape[0] == x.shape[0], "scales must be contiguous float32 [num_tokens, S]")
        num_scales = scales.shape[1]
    recv_x = torch.empty((rows, x.shape[1]), dtype=x.dtype, device=x.device)
    recv_scales = (torch.empty((rows, num_scales), dtype=torch.float32, device=x.device)
                   if scales is not None else None)
    if ready_counters is not None:
        _require(ready_counters.is_cuda and ready_counters.dtype == torch.int32
                 and ready_counters.is_contiguous() and rows_per_counter > 0
                 and ready_counters.numel() * rows_per_counter >= rows,
                 "ready_counters must be contiguous int32 [ceil(rows / rows_per_counter)]")
    lib = _lib.load()
    _lib.check(lib.mi_ep_dispatch_cached(_ptr(x), _ptr(scales), _ptr(recv_src_map), rows, x.shape[0],
                                         row_bytes, num_scales, _ptr(recv_x), _ptr(recv_scales),
                                         _ptr(ready_counters), rows_per_counter, _stream()),
               "mi_ep_dispatch_cached")
    return recv_x, recv_scales


def pull_indices(recv_src_map: torch.Tensor, tokens_per_source_rank: int,
                 num_rows: Optional[int] = None) -> torch.Tensor:
    """The source map as {source rank, token inside the rank} pairs, {-1, -1} for pads: the
    pull_dispatch_indices layout of the reference's ThunderKittens MoE example."""
    _require(recv_src_map.is_cuda and recv_src_map.dtype == torch.int32 and recv_src_map.is_contiguous(),
             "recv_src_map must be a contiguous int32 GPU tensor")
    _require(tokens_per_source_rank > 0, "tokens_per_source_rank must be positive")
    rows = recv_src_map.shape[0] if num_rows is None else num_rows
    out = torch.empty((rows, 2), dtype=torch.int32, device=recv_src_map.device)
    lib = _lib.load()
    _lib.check(lib.mi_ep_pull_indices(_ptr(recv_src_map), rows, tokens_per_source_rank, _ptr(out),
                                      _stream()), "mi_ep_pull_indices")
    return out


def device_traits() -> dict:
    """What the runtime reports for the current device: compute units, accelerator dies, L2 bytes
    per die (the destination-order copy is tuned for 8 dies with 4 MiB each)."""
    import ctypes
    cus, dies, l2 = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
    _lib.check(_lib.load().mi_ep_device_traits(ctypes.byref(cus), ctypes.byref(dies), ctypes.byref(l2), _stream()),
               "mi_ep_device_traits")
    return {"compute_units": cus.value, "dies": dies.value, "l2_bytes": l2.value}


def dispatch_schedule_for(num_tokens: int, num_topk: int, num_experts: int, row_bytes: int) -> str:
    """The copy kernel `schedule="auto"` picks for a shape on the current device."""
    traits = device_traits()
    code = _lib.load().mi_ep_dispatch_schedule_for(num_tokens, num_topk, num_experts, row_bytes,
                                                   traits["dies"], traits["l2_bytes"])
    if code not in (BY_TOKEN, BY_DESTINATION):
        _lib.check(code if code != 0 else -22, "mi_ep_dispatch_schedule_for")
    return "destination" if code == BY_DESTINATION else "token"


def copy_yardstick(dst: torch.Tensor, src: torch.Tensor) -> None:
    """16-byte streaming copy of src into dst (same byte size), the measured-bandwidth yardstick."""
    nbytes = src.numel() * src.element_size()
    _require(dst.numel() * dst.element_size() == nbytes and nbytes % 16 == 0, "size mismatch")
    lib = _lib.load()
    _lib.check(lib.mi_ep_copy_yardstick(_ptr(dst), _ptr(src), nbytes, _stream()),
               "mi_ep_copy_yardstick")


# ---- host-pointer twins: numpy in, numpy out (transfers included; never a measured path) -------

def _np(a, dtype):
    import numpy as np
    if a is None:
        return None
    a = np.ascontiguousarray(a)
    _require(a.dtype == np.dtype(dtype), f"expected a {np.dtype(dtype).name} array")
    return a


def _np_ptr(a):
    return None if a is None else a.ctypes.data


def host_get_dispatch_layout(topk_idx, num_experts: int, num_ranks: int):
    """get_dispatch_layout on host arrays: (num_tokens_per_rank, num_tokens_per_expert, is_token_in_rank)."""
    import numpy as np
    topk_idx = _np(topk_idx, np.int64)
    _require(topk_idx.ndim == 2, "topk_idx must be [num_tokens, num_topk]")
    T, K = topk_idx.shape
    per_rank = np.empty(num_ranks, dtype=np.int32)
    per_expert = np.empty(num_experts, dtype=np.int32)
    flags = np.empty((T, num_ranks), dtype=np.bool_)
    _lib.check(_lib.load().mi_ep_host_get_dispatch_layout(
        _np_ptr(topk_idx), _np_ptr(per_rank), None, _np_ptr(per_expert), _np_ptr(flags), T, K, num_ranks,
        num_experts), "mi_ep_host_get_dispatch_layout")
    return per_rank, per_expert, flags


def host_dispatch_layout(topk_idx, num_experts: int, num_ranks: int, expert_alignment: int = 1,
                         num_channels: int = 0, rank_slot_base: int = 0, cumulative_expert_stats=None):
    """The fused layout on host arrays: a dict with every output of mi_ep_dispatch_layout
    (`cumulative_expert_stats`, int32[E], is updated in place when given)."""
    import numpy as np
    topk_idx = _np(topk_idx, np.int64)
    _require(topk_idx.ndim == 2, "topk_idx must be [num_tokens, num_topk]")
    T, K = topk_idx.shape
    E, R = num_experts, num_ranks
    if cumulative_expert_stats is not None:
        _require(cumulative_expert_stats.dtype == np.int32 and cumulative_expert_stats.flags.c_contiguous
                 and cumulative_expert_stats.shape == (E,), "cumulative_expert_stats must be int32 [num_experts]")
    order_rows = _lib.load().mi_ep_route_order_bytes(T, K) // 16
    out = dict(
        num_tokens_per_rank=np.empty(R, dtype=np.int32), num_tokens_per_expert=np.empty(E, dtype=np.int32),
        is_token_in_rank=np.empty((T, R), dtype=np.bool_), expert_offsets=np.empty(E + 1, dtype=np.int32),
        psum_rank_rows=np.empty(R, dtype=np.int32),
        channel_prefix_matrix=np.empty((R, num_channels), dtype=np.int32) if num_channels > 0 else None,
        rank_prefix_matrix=np.empty((R, R), dtype=np.int32),
        slot_rel=np.empty((T, K), dtype=np.int32), rank_slot_idx=np.empty((T, K), dtype=np.int32),
        route_order=np.empty((order_rows, 4), dtype=np.int32),
        tile_rank_counts=np.empty(((T + 255) // 256, R), dtype=np.int32),
        copied_topk_idx=np.empty((T, K), dtype=np.int64))
    _lib.check(_lib.load().mi_ep_host_dispatch_layout(
        _np_ptr(topk_idx), T, K, R, E, expert_alignment, num_channels, _np_ptr(out["num_tokens_per_rank"]),
        _np_ptr(out["num_tokens_per_expert"]), _np_ptr(out["is_token_in_rank"]), _np_ptr(out["expert_offsets"]),
        _np_ptr(out["psum_rank_rows"]), _np_ptr(out["channel_prefix_matrix"]),
        _np_ptr(out["rank_prefix_matrix"]), _np_ptr(out["slot_rel"]),
        _np_ptr(out["rank_slot_idx"]), rank_slot_base, _np_ptr(out["route_order"]),
        _np_ptr(out["tile_rank_counts"]), _np_ptr(out["copied_topk_idx"]), _np_ptr(cumulative_expert_stats)),
        "mi_ep_host_dispatch_layout")
    return out


def host_dispatch(x, scales, topk_idx, topk_weights, num_experts: int, num_ranks: int,
                  expert_alignment: int = 1):
    """Layout + dispatch on host arrays.  `x` is a [num_tokens, row] array of any 1-, 2- or 4-byte
    dtype; returns a dict with the layout outputs, expert_offsets, slot_map and the recv_* arrays
    trimmed to expert_offsets[-1] rows."""
    import numpy as np
    topk_idx = _np(topk_idx, np.int64)
    T, K = topk_idx.shape
    x = np.ascontiguousarray(x)
    _require(x.ndim == 2 and x.shape[0] == T, "x must be [num_tokens, row]")
    row_bytes = x.shape[1] * x.itemsize
    scales = _np(scales, np.float32)
    topk_weights = _np(topk_weights, np.float32)
    S = 0 if scales is None else scales.shape[1]
    cap = T * K + num_experts * (expert_alignment - 1)
    out = dict(
        num_tokens_per_rank=np.empty(num_ranks, dtype=np.int32),
        num_tokens_per_expert=np.empty(num_experts, dtype=np.int32),
        is_token_in_rank=np.empty((T, num_ranks), dtype=np.bool_),
        expert_offsets=np.empty(num_experts + 1, dtype=np.int32),
        recv_x=np.empty((cap, x.shape[1]), dtype=x.dtype),
        recv_scales=None if scales is None else np.empty((cap, S), dtype=np.float32),
        recv_src_map=np.empty(cap, dtype=np.int32),
        recv_topk_idx=np.empty(cap, dtype=np.int64),
        recv_topk_weights=np.empty(cap, dtype=np.float32),
        slot_map=np.empty((T, K), dtype=np.int32))
    _lib.check(_lib.load().mi_ep_host_dispatch(
        _np_ptr(x), _np_ptr(scales), _np_ptr(topk_idx), _np_ptr(topk_weights), T, K, num_ranks, num_experts,
        expert_alignment, row_bytes, S, _np_ptr(out["num_tokens_per_rank"]),
        _np_ptr(out["num_tokens_per_expert"]), _np_ptr(out["is_token_in_rank"]),
        _np_ptr(out["expert_offsets"]), _np_ptr(out["recv_x"]), _np_ptr(out["recv_scales"]),
        _np_ptr(out["recv_src_map"]), _np_ptr(out["recv_topk_idx"]), _np_ptr(out["recv_topk_weights"]),
        _np_ptr(out["slot_map"]), cap), "mi_ep_host_dispatch")
    rows = int(out["expert_offsets"][-1])
    for key in ("recv_x", "recv_scales", "recv_src_map", "recv_topk_idx", "recv_topk_weights"):
        if out[key] is not None:
            out[key] = out[key][:rows]
    return out


def host_dispatch_ranks(x, scales, topk_idx, topk_weights, num_experts: int, num_ranks: int,
                        source_token_base: int = 0, local_expert_ids: bool = False):
    """Layout + dispatch in the reference's per-rank receive format on host arrays: a dict with
    num_tokens_per_rank, psum_rank_tokens, rank_row_map, combine_map and the recv_* arrays trimmed to
    psum_rank_tokens[-1] rows."""
    import numpy as np
    topk_idx = _np(topk_idx, np.int64)
    T, K = topk_idx.shape
    x = np.ascontiguousarray(x)
    _require(x.ndim == 2 and x.shape[0] == T, "x must be [num_tokens, row]")
    row_bytes = x.shape[1] * x.itemsize
    scales = _np(scales, np.float32)
    topk_weights = _np(topk_weights, np.float32)
    S = 0 if scales is None else scales.shape[1]
    cap = T * min(K, num_ranks)
    out = dict(
        num_tokens_per_rank=np.empty(num_ranks, dtype=np.int32),
        recv_x=np.empty((cap, x.shape[1]), dtype=x.dtype),
        recv_scales=None if scales is None else np.empty((cap, S), dtype=np.float32),
        recv_topk_idx=np.empty((cap, K), dtype=np.int64),
        recv_topk_weights=np.empty((cap, K), dtype=np.float32),
        recv_src_metadata=np.empty((cap, 2 + K), dtype=np.int32),
        rank_row_map=np.empty((T, K), dtype=np.int32),
        combine_map=np.empty((T, K), dtype=np.int32),
        psum_rank_tokens=np.empty(num_ranks, dtype=np.int32))
    _lib.check(_lib.load().mi_ep_host_dispatch_ranks(
        _np_ptr(x), _np_ptr(scales), _np_ptr(topk_idx), _np_ptr(topk_weights), T, K, num_ranks, num_experts,
        row_bytes, S, source_token_base, 1 if local_expert_ids else 0, _np_ptr(out["num_tokens_per_rank"]),
        _np_ptr(out["recv_x"]), _np_ptr(out["recv_scales"]), _np_ptr(out["recv_topk_idx"]),
        _np_ptr(out["recv_topk_weights"]), _np_ptr(out["recv_src_metadata"]), _np_ptr(out["rank_row_map"]),
        _np_ptr(out["combine_map"]), _np_ptr(out["psum_rank_tokens"]), cap), "mi_ep_host_dispatch_ranks")
    rows = int(out["psum_rank_tokens"][-1])
    for key in ("recv_x", "recv_scales", "recv_topk_idx", "recv_topk_weights", "recv_src_metadata"):
        if out[key] is not None:
            out[key] = out[key][:rows]
    return out


def host_dispatch_cached(x, scales, recv_src_map):
    """Pull-form dispatch on host arrays: row i of the result is x[recv_src_map[i]] (zeros where the
    map holds -1), scales likewise."""
    import numpy as np
    recv_src_map = _np(recv_src_map, np.int32)
    x = np.ascontiguousarray(x)
    _require(x.ndim == 2 and recv_src_map.ndim == 1, "x must be [num_tokens, row], recv_src_map [num_rows]")
    T, rows = x.shape[0], recv_src_map.shape[0]
    scales = _np(scales, np.float32)
    S = 0 if scales is None else scales.shape[1]
    recv_x = np.empty((rows, x.shape[1]), dtype=x.dtype)
    recv_scales = None if scales is None else np.empty((rows, S), dtype=np.float32)
    _lib.check(_lib.load().mi_ep_host_dispatch_cached(
        _np_ptr(x), _np_ptr(scales), _np_ptr(recv_src_map), rows, T, x.shape[1] * x.itemsize, S,
        _np_ptr(recv_x), _np_ptr(recv_scales)), "mi_ep_host_dispatch_cached")
    return recv_x, recv_scales


def host_combine(y_bits, slot_map, topk_weights=None, bias_0=None, bias_1=None):
    """combine on host arrays of bf16 bit patterns (uint16): returns uint16 [num_tokens, hidden]."""
    import numpy as np
    y_bits = _np(y_bits, np.uint16)
    slot_map = _np(slot_map, np.int32)
    T, K = slot_map.shape
    H = y_bits.shape[1]
    topk_weights = _np(topk_weights, np.float32)
    bias_0, bias_1 = _np(bias_0, np.uint16), _np(bias_1, np.uint16)
    out = np.empty((T, H), dtype=np.uint16)
    _lib.check(_lib.load().mi_ep_host_combine(
        _np_ptr(y_bits), y_bits.shape[0], _np_ptr(slot_map), _np_ptr(topk_weights), _np_ptr(bias_0),
        _np_ptr(bias_1), T, K, H, _np_ptr(out)), "mi_ep_host_combine")
    return out
