"""Oracle: top-k weighted combine of the expert outputs with the residual.

Test infrastructure only (see ``oracle/__init__.py``).

  * ``combine_fwd/bwd``  <- ``pithtrain/models/qwen3_moe.py:229-237`` (``forward_stage5``, the
    ``ep_size == 1`` branch): ``residual + (moe.view(T, k, H) * w.unsqueeze(-1)).sum(1).to(dtype)``.

Type promotion makes the products fp32 (bf16 tensor times fp32 tensor); the reference leaves the
order of the k-term fp32 sum to the tensor library, so the restatement fixes it (j = 0..k-1) and
is tolerance-pinned against the tensor expression for k > 2: for k <= 2 the sum has one order
and the two agree bit for bit (checked in tests/test_oracle_combine.py, together with autograd of
the tensor expression for the backward).

  * ``combine_ep_fwd/bwd``  <- ``pithtrain/models/qwen3_moe.py:238-245`` (the ``ep_size > 1``
    branch): every row weighted in fp32 and rounded, ``scatter_add_`` into a zeroed accumulator of
    the storage type, residual added last.  The reference's adds are device atomics in arbitrary
    order; the restatement adds a token's rows in ascending row order, every partial sum rounded
    (a sequential scatter_add_).  Pinned by tests/test_oracle_combine.py: bit for bit against the
    tensor expression whenever no token has more than two rows (one add, one order), against a
    scalar brute-force loop on small inputs, within rounding of the tensor expression otherwise,
    and the backward against autograd of the tensor expression.
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


def combine_ep_fwd(moe: torch.Tensor, local_idxs: torch.Tensor, topk_weight: torch.Tensor,
                   residual: torch.Tensor) -> torch.Tensor:
    """moe [R, H], local_idxs int64 [R] (distinct flat slots t*k + j), topk_weight fp32 [T, k],
    residual [T, H] -> [T, H] in moe's dtype."""
    T, k = topk_weight.shape
    dt = moe.dtype
    probs = topk_weight.reshape(-1)[local_idxs]
    token = local_idxs // k
    weighted = (moe.float() * probs[:, None]).to(dt)  # rounded row by row
    agg = torch.zeros((T, moe.shape[1]), dtype=dt)
    # ascending r: the j-th pass adds, for every token, its j-th row in row order
    order = torch.argsort(token, stable=True)  # rows grouped by token, ascending r inside
    tok_sorted = token[order]
    first = torch.searchsorted(tok_sorted, tok_sorted)  # start of every row's token run
    nth = torch.arange(order.numel()) - first
    for j in range(int(nth.max().item()) + 1 if order.numel() else 0):
        sel = order[nth == j]
        t = token[sel]
        agg[t] = (agg[t].float() + weighted[sel].float()).to(dt)
    return (residual.float() + agg.float()).to(dt)


def combine_ep_bwd(grad_out: torch.Tensor, moe: torch.Tensor, local_idxs: torch.Tensor, topk_weight: torch.Tensor):
    """Returns (d_moe [R, H], d_weight fp32 [T, k], d_residual = grad_out)."""
    T, k = topk_weight.shape
    token = local_idxs // k
    g = grad_out.float()[token]  # gradient of the accumulator row, through scatter_add_ and the cast
    d_moe = (g * topk_weight.reshape(-1)[local_idxs][:, None]).to(moe.dtype)
    d_w = torch.zeros(T * k, dtype=torch.float32)
    d_w[local_idxs] = (g.double() * moe.double()).sum(-1).float()
    return d_moe, d_w.view(T, k), grad_out
