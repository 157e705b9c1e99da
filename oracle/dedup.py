"""Oracle: expert-parallel dispatch index construction with token dedup.

Test infrastructure only (see ``oracle/__init__.py``).

Follows ``pithtrain/operators/ep_dispatch.py``:
  * ``fused_dedup_prepare_dispatch`` <- :37-268 (three kernels), host :271-420
  * ``build_expert_idxs``            <- :426-508
  * ``adjust_expand_idx``            <- :511-576

The reference places rows with atomics (:231, :256) so the order inside an
expert bucket / inside an EP-rank chunk is not fixed there.  Canonical order
here: ascending flat index inside each expert bucket, ascending token id
inside each EP-rank chunk - the order of ``argsort(stable=True)`` and of
``nonzero()`` which the reference's own CPU simulation uses
(tests/test_ep_dedup_dispatch.py:7-74).
"""

from __future__ import annotations

import torch


def fused_dedup_prepare_dispatch(
    topk_ids: torch.Tensor, num_experts: int, ep_size: int, experts_per_rank: int
):
    """Returns (tokens_per_ep_rank[ep], dedup_tokens_per_gpu[ep], dispatch_token_idxs[m*ep]
    (first sum(dedup) entries valid, rest -1 here), idxs[m*k], expand_idx[m*k],
    send_meta[ep*(epr+1)]), all int64."""
    m, k = topk_ids.shape
    assert ep_size <= 32  # :310
    if m == 0:  # :312-321
        z = torch.zeros(ep_size, dtype=torch.int64)
        e = torch.empty(0, dtype=torch.int64)
        return z, z.clone(), e, e.clone(), e.clone(), torch.zeros(
            ep_size * (experts_per_rank + 1), dtype=torch.int64
        )
    ids = topk_ids.to(torch.int64)
    flat = ids.reshape(-1)
    tokens_per_expert = torch.bincount(flat, minlength=num_experts)[:num_experts]
    tokens_per_ep_rank = tokens_per_expert.view(ep_size, experts_per_rank).sum(1)

    # first-visit dedup: token t is sent to rank g once if any of its experts lives on g (:72-84)
    rank_of = ids // experts_per_rank
    visits = torch.zeros((m, ep_size), dtype=torch.bool)
    visits[torch.arange(m).unsqueeze(1).expand(m, k), rank_of] = True
    dedup_tokens_per_gpu = visits.sum(0).to(torch.int64)
    # local position of token t inside rank g's chunk = number of earlier visiting tokens
    local_pos = visits.to(torch.int64).cumsum(0) - visits.to(torch.int64)
    gpu_starts = dedup_tokens_per_gpu.cumsum(0) - dedup_tokens_per_gpu

    dispatch = torch.full((m * ep_size,), -1, dtype=torch.int64)
    for g in range(ep_size):
        toks = torch.nonzero(visits[:, g]).view(-1)
        dispatch[gpu_starts[g] : gpu_starts[g] + toks.numel()] = toks

    idxs = torch.argsort(flat, stable=True)  # counting sort by expert (:243-256)
    tok = idxs // k
    rank_sorted = flat[idxs] // experts_per_rank
    expand_idx = local_pos[tok, rank_sorted]  # :258-264

    send_meta = torch.empty((ep_size, experts_per_rank + 1), dtype=torch.int64)  # :141-162
    send_meta[:, :experts_per_rank] = tokens_per_expert.view(ep_size, experts_per_rank)
    send_meta[:, experts_per_rank] = dedup_tokens_per_gpu
    return (
        tokens_per_ep_rank,
        dedup_tokens_per_gpu,
        dispatch,
        idxs,
        expand_idx,
        send_meta.view(-1),
    )


def build_expert_idxs(tokens_per_expert_group: torch.Tensor, ep_size: int, experts_per_rank: int):
    """(expert_idxs[sum(counts)], output_splits[ep]): slot s belongs to the bucket e with
    start_e <= s < start_e + count_e and gets e % experts_per_rank. (:426-473)"""
    counts = tokens_per_expert_group.to(torch.int64)
    n = counts.numel()
    local = torch.arange(n, dtype=torch.int64) % experts_per_rank
    expert_idxs = local.repeat_interleave(counts)
    splits = counts.view(ep_size, experts_per_rank).sum(1)
    return expert_idxs, splits


def adjust_expand_idx(
    received_expand_idx: torch.Tensor,
    dedup_tokens_from_each_gpu: torch.Tensor,
    output_splits: torch.Tensor,
) -> torch.Tensor:
    """Add to every slot the exclusive cumsum of dedup counts of the sender it came from;
    slots are laid out sender by sender with ``output_splits`` slots each. (:511-550)"""
    d = dedup_tokens_from_each_gpu.to(torch.int64)
    starts = d.cumsum(0) - d
    return received_expand_idx + starts.repeat_interleave(output_splits.to(torch.int64))


def simulate_receiver_expand_idx(topk_ids_per_sender, receiver: int, ep_size: int, epr: int):
    """Single-process stand-in for the two all-to-alls around the index kernels
    (ep_dispatch.py:616-663): concatenates what every sender would send to ``receiver``.
    Returns (expert_idxs, expand_idx_adjusted, dedup_rows_per_sender list, token-id lists)."""
    num_experts = ep_size * epr
    tpe_group, dedup_from, chunks, dedup_tok = [], [], [], []
    for ids in topk_ids_per_sender:
        tper, dpg, disp, idxs, exp, meta = fused_dedup_prepare_dispatch(
            ids, num_experts, ep_size, epr
        )
        meta = meta.view(ep_size, epr + 1)
        tpe_group.append(meta[receiver, :epr])
        dedup_from.append(meta[receiver, epr])
        in_starts = tper.cumsum(0) - tper
        chunks.append(exp[in_starts[receiver] : in_starts[receiver] + tper[receiver]])
        gs = dpg.cumsum(0) - dpg
        dedup_tok.append(disp[gs[receiver] : gs[receiver] + dpg[receiver]])
    tpe_group = torch.cat(tpe_group)
    expert_idxs, splits = build_expert_idxs(tpe_group, ep_size, epr)
    adjusted = adjust_expand_idx(torch.cat(chunks), torch.stack(dedup_from), splits)
    return expert_idxs, adjusted, [int(x) for x in dedup_from], dedup_tok
