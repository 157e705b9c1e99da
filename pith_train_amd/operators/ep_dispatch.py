"""Expert-parallel dispatch index construction with token dedup, on gfx950.

Drop-in for the single-GPU part of ``pithtrain/operators/ep_dispatch.py``:
``fused_dedup_prepare_dispatch`` (:271-420), ``build_expert_idxs`` (:476-508),
``adjust_expand_idx`` (:553-576) and ``prepare_dispatch`` (:579-676).  The two all-to-alls inside
``prepare_dispatch`` need more than one GPU; with ``ep_size == 1`` it takes the reference's
replicate path, with ``ep_size > 1`` it goes through ``torch.distributed`` exactly as the
reference does.

Order inside an expert bucket is the ascending flat index, inside an EP-rank chunk the ascending
token id (the reference's atomics leave both unspecified).
"""

from __future__ import annotations

from typing import List, NamedTuple, Optional

import torch

from .. import _lib
from .token_scatter import _workspace, get_pinned_buffer, padded_index_gather


class AllToAllSplits(NamedTuple):
    """Row counts of one all-to-all: what this rank sends to / receives from every EP rank."""

    input_splits: List[int]
    output_splits: List[int]


class RoutingInfo(NamedTuple):
    """What stage 1 hands to the later MoE stages (same fields as the reference's
    ``models/interface.py:11-17``)."""

    topk_weight: torch.Tensor
    expert_idxs: torch.Tensor
    moe_local_idxs: Optional[torch.Tensor] = None
    expand_idx: Optional[torch.Tensor] = None
    dispatch_splits: Optional[AllToAllSplits] = None
    combine_splits: Optional[AllToAllSplits] = None


def fused_dedup_prepare_dispatch(topk_ids: torch.Tensor, num_experts: int, ep_size: int, experts_per_rank: int):
    """topk_ids (m, k) int64 -> (tokens_per_ep_rank[ep], dedup_tokens_per_gpu[ep],
    dispatch_token_idxs[m*ep] (first sum(dedup) valid), idxs[m*k], expand_idx[m*k],
    send_meta[ep*(epr+1)]), all int64."""
    _lib.require_cuda(topk_ids)
    m, k = topk_ids.shape
    device = topk_ids.device
    assert ep_size <= 32, f"ep_size={ep_size} exceeds int32 bitmask limit of 32"
    i64 = dict(dtype=torch.int64, device=device)
    if m == 0:
        return (
            torch.zeros(ep_size, **i64), torch.zeros(ep_size, **i64), torch.empty(0, **i64),
            torch.empty(0, **i64), torch.empty(0, **i64),
            torch.zeros(ep_size * (experts_per_rank + 1), **i64),
        )  # fmt: skip
    assert topk_ids.dtype == torch.int64
    if topk_ids.stride(1) != 1:
        topk_ids = topk_ids.contiguous()
    tokens_per_ep_rank = torch.empty(ep_size, **i64)
    dedup_tokens_per_gpu = torch.empty(ep_size, **i64)
    dispatch_token_idxs = torch.empty(m * ep_size, **i64)
    idxs = torch.empty(m * k, **i64)
    expand_idx = torch.empty(m * k, **i64)
    send_meta = torch.empty(ep_size * (experts_per_rank + 1), **i64)
    ws = _workspace(_lib.query("pt_dedup_workspace_bytes", m, k, num_experts, ep_size), device)
    _lib.call(
        "pt_dedup_prepare_dispatch", topk_ids.data_ptr(), topk_ids.stride(0), m, k, num_experts,
        ep_size, experts_per_rank, tokens_per_ep_rank.data_ptr(), dedup_tokens_per_gpu.data_ptr(),
        dispatch_token_idxs.data_ptr(), idxs.data_ptr(), expand_idx.data_ptr(), send_meta.data_ptr(),
        ws.data_ptr(), ws.numel(), _lib.stream_ptr(device),
    )  # fmt: skip
    return tokens_per_ep_rank, dedup_tokens_per_gpu, dispatch_token_idxs, idxs, expand_idx, send_meta


def build_expert_idxs(tokens_per_expert_group: torch.Tensor, ep_size: int, experts_per_rank: int, max_total: int):
    """(expert_idxs[max_total] over-allocated, output_splits[ep]); the caller trims expert_idxs to
    ``sum(output_splits)``."""
    _lib.require_cuda(tokens_per_expert_group)
    num_experts = tokens_per_expert_group.shape[0]
    device = tokens_per_expert_group.device
    expert_idxs = torch.empty(max_total, dtype=torch.int64, device=device)
    output_splits = torch.empty(ep_size, dtype=torch.int64, device=device)
    counts = tokens_per_expert_group.to(torch.int64).contiguous()
    _lib.call(
        "pt_build_expert_idxs", counts.data_ptr(), num_experts, ep_size, experts_per_rank,
        max_total, _lib.ptr(expert_idxs) if max_total else None, output_splits.data_ptr(),
        _lib.stream_ptr(device),
    )  # fmt: skip
    return expert_idxs, output_splits


def adjust_expand_idx(received_expand_idx, dedup_tokens_from_each_gpu, output_splits_tensor):
    """received + exclusive_cumsum(dedup counts)[sender of each slot]."""
    _lib.require_cuda(received_expand_idx)
    N = received_expand_idx.shape[0]
    ep_size = dedup_tokens_from_each_gpu.shape[0]
    out = torch.empty_like(received_expand_idx)
    if N == 0:
        return out
    _lib.call(
        "pt_adjust_expand_idx", received_expand_idx.contiguous().data_ptr(), out.data_ptr(),
        dedup_tokens_from_each_gpu.data_ptr(), dedup_tokens_from_each_gpu.stride(0),
        output_splits_tensor.contiguous().data_ptr(), ep_size, N, _lib.stream_ptr(out.device),
    )  # fmt: skip
    return out


@torch.compiler.disable
def prepare_dispatch(hidden_states, topk_ids, topk_weight, num_experts, ep_size, experts_per_rank, ep_group):
    """Stage-1 dispatch preparation.  ``ep_size == 1``: replicate every token once per selected
    expert.  ``ep_size > 1``: dedup per destination rank, exchange metadata and ``expand_idx`` over
    ``ep_group``, and gather the unique rows to send."""
    import torch.distributed as dist

    hidden_states = hidden_states.view(-1, hidden_states.shape[-1])
    k = topk_ids.shape[1]
    expert_idxs = topk_ids.view(-1)
    if ep_size == 1:
        dispatch_tokens = hidden_states.unsqueeze(1).expand(-1, k, -1).reshape(-1, hidden_states.shape[-1])
        return dispatch_tokens, RoutingInfo(topk_weight, expert_idxs)

    (tokens_per_ep_rank, dedup_tokens_per_gpu, dispatch_token_idxs, idxs, expand_idx, send_meta) = (
        fused_dedup_prepare_dispatch(topk_ids, num_experts, ep_size, experts_per_rank)
    )
    recv_meta = send_meta.new_empty(send_meta.shape[0])
    dist.all_to_all_single(recv_meta, send_meta, group=ep_group)
    recv_meta_2d = recv_meta.view(ep_size, experts_per_rank + 1)
    tokens_per_expert_group = recv_meta_2d[:, :experts_per_rank].reshape(-1)
    dedup_tokens_from_each_gpu = recv_meta_2d[:, experts_per_rank]

    m = topk_ids.shape[0]
    expert_idxs, output_splits_tensor = build_expert_idxs(
        tokens_per_expert_group, ep_size, experts_per_rank, max_total=m * k * ep_size
    )
    names = ("dedup_input_splits", "dedup_output_splits", "input_splits", "output_splits")
    srcs = (dedup_tokens_per_gpu, dedup_tokens_from_each_gpu, tokens_per_ep_rank, output_splits_tensor)
    bufs = [get_pinned_buffer(n, ep_size, s.dtype) for n, s in zip(names, srcs)]
    for b, s in zip(bufs, srcs):
        b.copy_(s, non_blocking=True)
    torch.cuda.current_stream(hidden_states.device).synchronize()
    dedup_input_splits, dedup_output_splits, input_splits, output_splits = (b.tolist() for b in bufs)

    total_output = sum(output_splits)
    expert_idxs = expert_idxs[:total_output]
    received_expand_idx = expand_idx.new_empty(total_output)
    dist.all_to_all_single(received_expand_idx, expand_idx, output_splits, input_splits, ep_group)
    expand_idx = adjust_expand_idx(received_expand_idx, dedup_tokens_from_each_gpu, output_splits_tensor)

    total_dedup = sum(dedup_input_splits)
    dispatch_tokens = padded_index_gather(hidden_states, dispatch_token_idxs[:total_dedup])
    return dispatch_tokens, RoutingInfo(
        topk_weight, expert_idxs, idxs, expand_idx,
        AllToAllSplits(dedup_input_splits, dedup_output_splits),
        AllToAllSplits(input_splits, output_splits),
    )  # fmt: skip
