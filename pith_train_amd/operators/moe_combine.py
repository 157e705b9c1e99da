"""Top-k weighted combine of the expert outputs with the residual stream.

The memory-bound step right after the expert path: the single-rank branch of ``forward_stage5``
(models/qwen3_moe.py:229-237, and the same expression in the other model files)

    weighted = moe_outs.view(*topk_weight.shape, -1) * topk_weight.unsqueeze(-1)
    return residual + weighted.sum(dim=1).to(moe_outs.dtype).view(*residual.shape)

as one kernel each way instead of a product tensor, a reduction, a cast and an addition, and the
expert-parallel branch (models/qwen3_moe.py:238-245)

    permuted_probs = topk_weight.view(-1)[moe_local_idxs]
    token_indices = moe_local_idxs // topk_weight.shape[1]
    weighted = (moe_outs.float() * permuted_probs.unsqueeze(-1)).to(moe_outs.dtype)
    aggregated = moe_outs.new_zeros(topk_weight.shape[0], moe_outs.shape[-1])
    aggregated.scatter_add_(0, token_indices[:, None].expand_as(weighted), weighted)
    return residual + aggregated.view(*residual.shape)

likewise (:func:`moe_combine_ep`), with the order of the adds fixed: ascending row per token.
"""

from __future__ import annotations

import torch

from .. import _lib


class _MoeCombine(torch.autograd.Function):
    @staticmethod
    def forward(ctx, moe_outs: torch.Tensor, topk_weight: torch.Tensor, residual: torch.Tensor | None) -> torch.Tensor:
        _lib.require_cuda(moe_outs, topk_weight)
        assert moe_outs.ndim == 2 and topk_weight.ndim == 2, "moe_outs must be [T*k, H], topk_weight [T, k]"
        T, k = topk_weight.shape
        H = moe_outs.shape[1]
        assert moe_outs.shape[0] == T * k, f"moe_outs has {moe_outs.shape[0]} rows, expected {T * k}"
        assert topk_weight.dtype == torch.float32, "topk_weight must be float32 (softmax scores)"
        moe_outs = moe_outs.contiguous()
        w = topk_weight.contiguous()
        res_ptr = 0
        if residual is not None:
            _lib.require_cuda(residual)
            assert residual.numel() == T * H and residual.dtype == moe_outs.dtype, "residual must be [T, H] in moe_outs' dtype"
            res2d = residual.reshape(T, H).contiguous()
            res_ptr = res2d.data_ptr()
        out = torch.empty((T, H), dtype=moe_outs.dtype, device=moe_outs.device)
        _lib.call(
            "pt_moe_combine_fwd", moe_outs.data_ptr(), H, w.data_ptr(), res_ptr, H, out.data_ptr(), H,
            T, k, H, _lib.dtype_code(moe_outs.dtype), _lib.stream_ptr(moe_outs.device),
        )  # fmt: skip
        ctx.save_for_backward(moe_outs, w)
        ctx.has_residual = residual is not None
        return out if residual is None else out.view(residual.shape)

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor):
        moe_outs, w = ctx.saved_tensors
        T, k = w.shape
        H = moe_outs.shape[1]
        g = grad_out.reshape(T, H).contiguous()
        d_moe = torch.empty_like(moe_outs)
        d_w = torch.empty_like(w)
        _lib.call(
            "pt_moe_combine_bwd", g.data_ptr(), H, moe_outs.data_ptr(), H, w.data_ptr(), d_moe.data_ptr(), H,
            d_w.data_ptr(), T, k, H, _lib.dtype_code(moe_outs.dtype), _lib.stream_ptr(moe_outs.device),
        )  # fmt: skip
        return d_moe, d_w, (grad_out if ctx.has_residual else None)


def moe_combine(moe_outs: torch.Tensor, topk_weight: torch.Tensor, residual: torch.Tensor | None = None) -> torch.Tensor:
    """``residual + (moe_outs.view(T, k, H) * topk_weight[..., None]).sum(1).to(moe_outs.dtype)``.

    ``moe_outs`` is ``[T*k, H]`` (row ``t*k + j`` = expert output of token t's j-th choice),
    ``topk_weight`` float32 ``[T, k]``, ``residual`` any shape with ``T*H`` elements; the result
    has the residual's shape and ``moe_outs``' dtype.  Without a residual the result is the
    rounded weighted sum ``[T, H]`` itself (the last line of the models' ``reference_forward``,
    models/qwen3_moe.py:119)."""
    return _MoeCombine.apply(moe_outs, topk_weight, residual)


class _MoeCombineEP(torch.autograd.Function):
    @staticmethod
    def forward(ctx, moe_outs, moe_local_idxs, topk_weight, residual):
        _lib.require_cuda(moe_outs, moe_local_idxs, topk_weight, residual)
        assert moe_outs.ndim == 2 and topk_weight.ndim == 2, "moe_outs must be [R, H], topk_weight [T, k]"
        T, k = topk_weight.shape
        R, H = moe_outs.shape
        assert moe_local_idxs.shape == (R,) and moe_local_idxs.dtype == torch.int64, "moe_local_idxs must be int64 [R]"
        assert R <= T * k, f"{R} rows for {T * k} top-k slots"
        assert residual.numel() == T * H and residual.dtype == moe_outs.dtype, "residual must be [T, H] in moe_outs' dtype"
        assert topk_weight.dtype == torch.float32, "topk_weight must be float32 (softmax scores)"
        moe_outs = moe_outs.contiguous()
        res2d = residual.reshape(T, H).contiguous()
        w = topk_weight.contiguous()
        stream = _lib.stream_ptr(moe_outs.device)
        slot_row = torch.empty((T * k,), device=moe_outs.device, dtype=torch.int32)
        _lib.call("pt_moe_combine_ep_index", moe_local_idxs.contiguous().data_ptr(), R, T * k, slot_row.data_ptr(), stream)
        out = torch.empty_like(res2d)
        _lib.call(
            "pt_moe_combine_ep_fwd", moe_outs.data_ptr(), H, R, slot_row.data_ptr(), w.data_ptr(), res2d.data_ptr(), H,
            out.data_ptr(), H, T, k, H, _lib.dtype_code(moe_outs.dtype), stream,
        )  # fmt: skip
        ctx.save_for_backward(moe_outs, w, slot_row)
        return out.view(residual.shape)

    @staticmethod
    def backward(ctx, grad_out):
        moe_outs, w, slot_row = ctx.saved_tensors
        T, k = w.shape
        R, H = moe_outs.shape
        g = grad_out.reshape(T, H).contiguous()
        # rows no slot points to (none when moe_local_idxs is a permutation) get a zero gradient
        d_moe = torch.empty_like(moe_outs) if R == T * k else torch.zeros_like(moe_outs)
        d_w = torch.empty_like(w)
        _lib.call(
            "pt_moe_combine_ep_bwd", g.data_ptr(), H, moe_outs.data_ptr(), H, R, slot_row.data_ptr(), w.data_ptr(),
            d_moe.data_ptr(), H, d_w.data_ptr(), T, k, H, _lib.dtype_code(moe_outs.dtype), _lib.stream_ptr(moe_outs.device),
        )  # fmt: skip
        return d_moe, None, d_w, grad_out


def moe_combine_ep(moe_outs: torch.Tensor, moe_local_idxs: torch.Tensor, topk_weight: torch.Tensor,
                   residual: torch.Tensor) -> torch.Tensor:
    """Expert-parallel combine: row r of ``moe_outs`` ``[R, H]`` is the expert output of the flat
    top-k slot ``moe_local_idxs[r]`` (token ``moe_local_idxs[r] // k``); entries are distinct (the
    dispatch sort's permutation, ep_dispatch.py:669-676).  Every row is weighted in fp32 and
    rounded, a token's rows are added in ascending r with every partial sum rounded to the
    storage type (a sequential ``scatter_add_``), and the residual is added last."""
    return _MoeCombineEP.apply(moe_outs, moe_local_idxs, topk_weight, residual)
