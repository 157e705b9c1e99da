"""In-place fused cross-entropy of the loss head (operators/cross_entropy.py of the reference).

``cross_entropy(inp, target, ignore_index=-100)`` returns the mean loss over the rows whose target
is not ``ignore_index`` and overwrites ``inp`` with the gradient of that mean during the forward,
so the ``[N, V]`` logits are the only large tensor of the loss head; the backward scales them in
place by the incoming gradient and hands them on (operators/cross_entropy.py:81-124).
"""

from __future__ import annotations

import torch

from .. import _lib


class CrossEntropy(torch.autograd.Function):
    @staticmethod
    def forward(ctx, inp, target, ignore_index):
        _lib.require_cuda(inp, target)
        assert inp.ndim == 2 and target.shape == (inp.shape[0],), "inp must be [N, V], target [N]"
        assert target.dtype == torch.int64, "target must be int64"
        n_rows, n_cols = inp.shape
        if inp.stride(-1) != 1 or inp.stride(-2) != n_cols:
            inp = inp.contiguous()
        if target.stride(-1) != 1:
            target = target.contiguous()
        loss_rows = torch.empty(n_rows, dtype=torch.float32, device=inp.device)
        loss = torch.empty((), dtype=torch.float32, device=inp.device)
        n_non_ignore = torch.empty(1, dtype=torch.int64, device=inp.device)
        _lib.call(
            "pt_cross_entropy_fwd", inp.data_ptr(), n_cols, _lib.dtype_code(inp.dtype), target.data_ptr(), n_rows, n_cols,
            int(ignore_index), loss_rows.data_ptr(), loss.data_ptr(), n_non_ignore.data_ptr(), _lib.stream_ptr(inp.device),
        )  # fmt: skip
        ctx.save_for_backward(inp.detach())
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        (inp,) = ctx.saved_tensors
        n_rows, n_cols = inp.shape
        go = grad_output.detach().reshape(1).float().contiguous()
        _lib.call(
            "pt_cross_entropy_bwd", inp.data_ptr(), n_cols, _lib.dtype_code(inp.dtype), n_rows, n_cols, go.data_ptr(),
            _lib.stream_ptr(inp.device),
        )  # fmt: skip
        return inp, None, None


def cross_entropy(inp: torch.Tensor, target: torch.Tensor, ignore_index: int = -100) -> torch.Tensor:
    """Mean cross-entropy (fp32 scalar) of logits ``inp`` ``[N, V]`` against ``target`` ``[N]``;
    ``inp`` is modified in place (it holds the gradient afterwards)."""
    return CrossEntropy.apply(inp, target, ignore_index)
