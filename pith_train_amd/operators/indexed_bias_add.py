"""``x + bias[group_ids]`` with a segmented-sum backward for rows already sorted by group.

Drop-in for ``pithtrain/operators/indexed_bias_add.py`` (``indexed_bias_add`` :115-127,
``_IndexedBiasAdd`` :99-112, ``_segment_sum_along_rows`` :54-96).  The forward is one fused
kernel (no materialised ``bias[group_ids]``); its result equals the storage-dtype add bit for bit.
"""

from __future__ import annotations

import torch

from .. import _lib


def _segment_sum_along_rows(x: torch.Tensor, grouped_mm_offs: torch.Tensor, out_dtype: torch.dtype,
                            row_index: torch.Tensor | None = None):
    """(E, H) per-group row sums, fp32 accumulation in a fixed order, stored as ``out_dtype``.
    With ``row_index`` (int32 ``[M]``) grouped row r is ``x[row_index[r]]`` (negative: padding),
    ``x`` being the un-permuted ``[m, H]`` tensor: the same sums, in the same order, as over
    ``x`` gathered into the grouped layout."""
    assert x.is_contiguous(), "x must be contiguous"
    M, H = (row_index.shape[0], x.shape[1]) if row_index is not None else x.shape
    E = grouped_mm_offs.shape[0]
    offs = grouped_mm_offs.to(torch.int32).contiguous()
    direct = (x.dtype, out_dtype) in {
        (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32),
        (torch.float16, torch.float16), (torch.float16, torch.float32),
        (torch.float32, torch.float32), (torch.float32, torch.bfloat16),
    }  # fmt: skip
    kdtype = out_dtype if direct else torch.float32
    out = torch.empty((E, H), dtype=kdtype, device=x.device)
    if E and H and row_index is not None:
        _lib.call(
            "pt_segment_sum_rows", x.data_ptr(), x.shape[0], row_index.contiguous().data_ptr(), offs.data_ptr(), E,
            out.data_ptr(), M, H, _lib.dtype_code(x.dtype), _lib.dtype_code(kdtype), _lib.stream_ptr(x.device),
        )  # fmt: skip
    elif E and H:
        _lib.call(
            "pt_segment_sum", x.data_ptr(), offs.data_ptr(), E, out.data_ptr(), M, H,
            _lib.dtype_code(x.dtype), _lib.dtype_code(kdtype), _lib.stream_ptr(x.device),
        )  # fmt: skip
    return out if kdtype == out_dtype else out.to(out_dtype)


class _IndexedBiasAdd(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, bias, group_ids, grouped_mm_offs):
        _lib.require_cuda(x, bias, group_ids)
        ctx.bias_dtype = bias.dtype
        ctx.save_for_backward(grouped_mm_offs)
        if x.dtype != bias.dtype or x.dim() != 2 or not x.is_contiguous():
            return x + bias[group_ids]  # mixed-dtype promotion is left to torch
        M, H = x.shape
        out = torch.empty_like(x)
        if M * H:
            gid = group_ids.to(torch.int64).contiguous()
            _lib.call(
                "pt_indexed_bias_add_fwd", x.data_ptr(), bias.contiguous().data_ptr(),
                gid.data_ptr(), out.data_ptr(), M, H, _lib.dtype_code(x.dtype),
                _lib.stream_ptr(x.device),
            )  # fmt: skip
        return out

    @staticmethod
    def backward(ctx, grad_out):
        (offs,) = ctx.saved_tensors
        bias_grad = _segment_sum_along_rows(grad_out.contiguous(), offs, ctx.bias_dtype)
        return grad_out, bias_grad, None, None


def indexed_bias_add(x, bias, group_ids, grouped_mm_offs):
    """``x + bias[group_ids]``; ``group_ids`` non-decreasing, ``grouped_mm_offs`` the matching
    cumulative end offsets."""
    return _IndexedBiasAdd.apply(x, bias, group_ids, grouped_mm_offs)
