"""Oracle: top-k weighted combine of the expert outputs with the residual.

Test infrastructure only (see ``oracle/__init__.py``).

  * ``combine_fwd/bwd``  <- ``pithtrain/models/qwen3_moe.py:229-237`` (``forward_stage5``, the
    ``ep_size == 1`` branch): ``residual + (moe.view(T, k, H) * w.unsqueeze(-1)).sum(1).to(dtype)``.

Type promotion makes the products fp32 (bf16 tensor times fp32 tensor); the reference leaves the
order of the k-term fp32 sum to the tensor library, so the restatement fixes it (j = 0..k-1) and
is tolerance-pinned against the tensor expression for k > 2: for k <= 2 the sum has one order
and the two agree bit for bit (checked in tests/test_oracle_combine.py, together with autograd of
the tensor expression for the backward).
"""

from __future__ import annotations

import torch


def combine_fwd(moe: torch.Tensor, topk_weight: torch.Tensor, residual: torch.Tensor) -> torch.Tensor:
    """moe [T*k, H], topk_weight fp32 [T, k], residual [T, H] -> [T, H] in moe's dtype."""
    T, k = topk_weight.shape
    H = moe.shape[1]
    m = moe.view(T, k, H).float()
    w = topk_weight.float()
    acc = torch.zeros((T, H), dtype=torch.float32)
    for j in range(k):
        acc = acc + m[:, j, :] * w[:, j : j + 1]  # fp32 product, fp32 add, in this order
    s = acc.to(moe.dtype)  # the sum is rounded once ...
    return (residual.float() + s.float()).to(moe.dtype)  # ... and the addition once more


def combine_bwd(grad_out: torch.Tensor, moe: torch.Tensor, topk_weight: torch.Tensor):
    """Returns (d_moe [T*k, H] in moe's dtype, d_weight fp32 [T, k], d_residual = grad_out)."""
    T, k = topk_weight.shape
    H = moe.shape[1]
    g = grad_out.float()  # gradient of the rounded sum, passed through the cast
    d_moe = (g[:, None, :] * topk_weight.float()[:, :, None]).to(moe.dtype).reshape(T * k, H)
    d_w = (g[:, None, :].double() * moe.view(T, k, H).double()).sum(-1).float()
    return d_moe, d_w, grad_out
