"""Oracle: router gate after the logits GEMM (softmax, top-k, weights of the chosen experts).

Test infrastructure only (see ``oracle/__init__.py``).

  * ``softmax_topk``  <- ``pithtrain/models/qwen3_moe.py:82-88`` (``Qwen3MoeGate.forward``),
    ``models/qwen35_moe.py:217-222``, ``models/deepseek_v2.py:150-164`` (with the
    ``group_limited_greedy`` limit of lines 152-159 and the ``routed_scaling_factor``).
  * ``topk_softmax``  <- ``pithtrain/models/gpt_oss.py:177-182`` (``GptOssTopKRouter.forward``).

The reference calls ``torch.topk(..., sorted=False)``, which fixes neither the order of the result
nor the winner among equal values; the restatement fixes both (descending value, lower expert
index first, i.e. a stable descending sort) and the kernels follow it.  Everything else is the
reference's expression on CPU tensors, so the backward is autograd of that expression.  Pinned in
tests/test_oracle_router.py: selected sets against ``torch.topk`` where no values tie, closed
forms (uniform logits, one dominant expert, weights summing to one or to the scale), a scalar
brute-force loop on small inputs, and the group limit against a hand-worked case.
"""

from __future__ import annotations

import torch


def _stable_topk(values: torch.Tensor, k: int) -> torch.Tensor:
    """Indices of the k largest per row: descending value, ties to the lower index."""
    return torch.sort(values, dim=-1, descending=True, stable=True).indices[:, :k]


def softmax_topk(logits: torch.Tensor, k: int, norm_topk_prob: bool = False, scale: float = 1.0, num_group: int = 1,
                 topk_group: int = 1, forced_idx: torch.Tensor | None = None):
    """Returns (topk_idx int64 [T, k], topk_weight fp32 [T, k], scores fp32 [T, E]); differentiable
    in ``logits`` through ``topk_weight`` and ``scores``."""
    scores = logits.softmax(dim=-1, dtype=torch.float32)
    if num_group > 1:
        n_tokens, E = scores.shape
        group_scores = scores.view(n_tokens, num_group, -1).max(dim=-1).values
        group_idx = _stable_topk(group_scores.detach(), topk_group)
        group_mask = torch.zeros_like(group_scores)
        group_mask.scatter_(1, group_idx, 1)
        score_mask = group_mask.unsqueeze(-1).expand(n_tokens, num_group, E // num_group).reshape(n_tokens, -1)
        scores = scores.masked_fill(~score_mask.bool(), 0.0)
    topk_idx = _stable_topk(scores.detach(), k) if forced_idx is None else forced_idx
    topk_weight = scores.gather(-1, topk_idx)
    if norm_topk_prob:
        topk_weight = topk_weight / topk_weight.sum(dim=-1, keepdim=True)
    topk_weight = topk_weight * scale
    return topk_idx, topk_weight, scores


def topk_softmax(logits: torch.Tensor, k: int, forced_idx: torch.Tensor | None = None):
    """Returns (topk_idx, topk_weight fp32 [T, k], scores = softmax over all experts)."""
    topk_idx = _stable_topk(logits.detach().float(), k) if forced_idx is None else forced_idx
    topk_logits = logits.gather(-1, topk_idx)
    topk_weight = torch.nn.functional.softmax(topk_logits, dim=-1, dtype=torch.float32)
    scores = logits.softmax(dim=-1, dtype=torch.float32)
    return topk_idx, topk_weight, scores
