"""Oracle: in-place fused cross-entropy of the loss head.

Test infrastructure only (see ``oracle/__init__.py``).

  * ``cross_entropy_fwd``  <- ``pithtrain/operators/cross_entropy.py:16-78`` (the Triton kernel
    ``cross_entropy_fwd``) and ``:86-118`` (``CrossEntropy.forward``): blockwise online softmax
    (block = min(32768, next power of two of V)), per-row loss, gradient of the mean loss stored
    in the logits' dtype with the target entry corrected after it was stored.
  * ``cross_entropy_bwd``  <- ``:120-124``: the stored gradient times the incoming scalar rounded
    to the logits' dtype.

Pinned in tests/test_oracle_cross_entropy.py against ``torch.nn.functional.cross_entropy`` in
float64 (loss and autograd gradient), the closed form for uniform logits, and the ignore rules.
"""

from __future__ import annotations

import torch


def cross_entropy_fwd(inp: torch.Tensor, target: torch.Tensor, ignore_index: int = -100):
    """Returns (loss fp32 scalar, grad [N, V] in inp's dtype, loss_rows fp32 [N], n)."""
    N, V = inp.shape
    n = max(1, int((target != ignore_index).sum()))
    block = min(32768, 1 << (V - 1).bit_length())
    x = inp.float()
    m = torch.full((N,), float("-inf"))
    d = torch.zeros(N)
    for i in range(0, V, block):
        xb = x[:, i : i + block]
        m_new = torch.maximum(m, xb.max(dim=1).values)
        d = d * torch.exp(m - m_new) + torch.exp(xb - m_new[:, None]).sum(dim=1)
        m = m_new
    live = target != ignore_index
    rows = torch.arange(N)
    y = target.clamp(min=0)
    grad = ((torch.exp(x - m[:, None]) / d[:, None]) / n).to(inp.dtype)
    grad[rows, y] = (grad[rows, y].float() + (-1.0 / n)).to(inp.dtype)  # corrected after the store
    grad[~live] = 0
    loss_rows = -(x[rows, y] - m - torch.log(d))
    loss_rows[~live] = 0
    loss = loss_rows.sum() / float(n)
    return loss, grad, loss_rows, n


def cross_entropy_bwd(grad: torch.Tensor, grad_output: torch.Tensor) -> torch.Tensor:
    return grad * grad_output.to(grad.dtype)
