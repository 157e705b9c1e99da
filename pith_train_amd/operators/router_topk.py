"""Router gate after the logits GEMM: softmax, top-k and the chosen experts' weights in one launch.

Replaces the tensor expressions between ``F.linear`` and the return of the gates' ``forward``:

  * ``softmax_topk`` - ``Qwen3MoeGate`` (models/qwen3_moe.py:81-88), ``Qwen35MoeTopKRouter``
    (models/qwen35_moe.py:216-222), ``DeepSeekV2MoEGate`` (models/deepseek_v2.py:149-164, with
    its ``group_limited_greedy`` limit and ``routed_scaling_factor``);
  * ``topk_softmax`` - ``GptOssTopKRouter`` (models/gpt_oss.py:176-182).

Both return ``(topk_idx int64 [T, k], topk_weight fp32 [T, k])`` and, with ``return_scores``, the
fp32 ``[T, E]`` scores the load-balance loss reads.  The selection comes out sorted by descending
value with ties going to the lower expert index; ``forced_idx`` is the router-replay hook (the
selection is given, the weights are gathered there).  Gradients flow from ``topk_weight`` and
``scores`` back to ``logits``.
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import _lib


class _RouterTopK(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, mode, k, norm, scale, num_group, topk_group, forced_idx, want_scores):
        _lib.require_cuda(logits)
        assert logits.ndim == 2, "logits must be [T, E]"
        if logits.stride(1) != 1:
            logits = logits.contiguous()
        T, E = logits.shape
        dev = logits.device
        if forced_idx is not None:
            assert forced_idx.shape == (T, k) and forced_idx.dtype == torch.int64, "forced_idx must be int64 [T, k]"
            forced_idx = forced_idx.contiguous()
        topk_idx = torch.empty((T, k), device=dev, dtype=torch.int64)
        topk_weight = torch.empty((T, k), device=dev, dtype=torch.float32)
        scores = torch.empty((T, E), device=dev, dtype=torch.float32) if want_scores else None
        _lib.call(
            "pt_router_topk_fwd", logits.data_ptr(), logits.stride(0), _lib.dtype_code(logits.dtype), T, E, k, mode,
            int(norm), float(scale), num_group, topk_group, forced_idx.data_ptr() if forced_idx is not None else None,
            topk_idx.data_ptr(), topk_weight.data_ptr(), scores.data_ptr() if want_scores else None,
            _lib.stream_ptr(dev),
        )  # fmt: skip
        ctx.save_for_backward(logits, topk_idx)
        ctx.cfg = (mode, k, int(norm), float(scale), num_group, topk_group)
        ctx.mark_non_differentiable(topk_idx)
        if want_scores:
            return topk_idx, topk_weight, scores
        return topk_idx, topk_weight

    @staticmethod
    def backward(ctx, _d_idx, d_weight, d_scores=None):
        logits, topk_idx = ctx.saved_tensors
        mode, k, norm, scale, num_group, topk_group = ctx.cfg
        T, E = logits.shape
        if d_weight is None:
            d_weight = torch.zeros((T, k), device=logits.device, dtype=torch.float32)
        d_weight = d_weight.float().contiguous()
        if d_scores is not None:
            d_scores = d_scores.float().contiguous()
        d_logits = torch.empty((T, E), device=logits.device, dtype=logits.dtype)
        _lib.call(
            "pt_router_topk_bwd", logits.data_ptr(), logits.stride(0), _lib.dtype_code(logits.dtype), T, E, k, mode,
            norm, scale, num_group, topk_group, topk_idx.data_ptr(), d_weight.data_ptr(),
            d_scores.data_ptr() if d_scores is not None else None, d_logits.data_ptr(), E, _lib.stream_ptr(logits.device),
        )  # fmt: skip
        return d_logits, None, None, None, None, None, None, None, None


def softmax_topk(logits: torch.Tensor, k: int, *, norm_topk_prob: bool = False, scale: float = 1.0,
                 num_group: int = 1, topk_group: int = 1, forced_idx: Optional[torch.Tensor] = None,
                 return_scores: bool = False):
    """``scores = softmax(logits, fp32)`` [group limit] -> top-k -> ``scores[topk_idx]``
    [``/ sum``] ``* scale``.  With ``num_group > 1`` only the ``topk_group`` groups of
    ``E / num_group`` contiguous experts with the largest maximum score keep their scores; the
    returned ``scores`` are the limited ones, as in the reference."""
    return _RouterTopK.apply(logits, 0, k, norm_topk_prob, scale, num_group, topk_group if num_group > 1 else 1,
                             forced_idx, return_scores)


def topk_softmax(logits: torch.Tensor, k: int, *, forced_idx: Optional[torch.Tensor] = None,
                 return_scores: bool = False):
    """Top-k of the logits, then the fp32 softmax over the k chosen logits; ``scores`` (when asked
    for) is the softmax over all experts."""
    return _RouterTopK.apply(logits, 1, k, False, 1.0, 1, 1, forced_idx, return_scores)
