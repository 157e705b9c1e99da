"""Fused ``silu(gate) * up`` with a one-kernel backward that recomputes the sigmoid.

Drop-in for ``pithtrain/operators/silu_mul.py`` (``silu_mul`` :128-143, ``_SiLUMul`` :93-125):
only ``gate`` and ``up`` are saved for backward.
"""

from __future__ import annotations

import torch

from .. import _lib


class _SiLUMul(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        assert gate.shape == up.shape, f"shape mismatch: {gate.shape} vs {up.shape}"
        assert gate.dtype == up.dtype, f"dtype mismatch: {gate.dtype} vs {up.dtype}"
        assert gate.is_contiguous(), "gate must be contiguous"
        assert up.is_contiguous(), "up must be contiguous"
        _lib.require_cuda(gate, up)
        ctx.save_for_backward(gate, up)
        out = torch.empty_like(gate)
        _lib.call(
            "pt_silu_mul_fwd", gate.data_ptr(), up.data_ptr(), out.data_ptr(), gate.numel(),
            _lib.dtype_code(gate.dtype), _lib.stream_ptr(gate.device),
        )  # fmt: skip
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        gate, up = ctx.saved_tensors
        assert grad_output.shape == gate.shape, (
            f"grad_output shape {grad_output.shape} != gate shape {gate.shape}"
        )
        assert grad_output.dtype == gate.dtype, (
            f"grad_output dtype {grad_output.dtype} != gate dtype {gate.dtype}"
        )
        assert grad_output.is_contiguous(), "grad_output must be contiguous"
        grad_gate = torch.empty_like(gate)
        grad_up = torch.empty_like(up)
        _lib.call(
            "pt_silu_mul_bwd", grad_output.data_ptr(), gate.data_ptr(), up.data_ptr(),
            grad_gate.data_ptr(), grad_up.data_ptr(), gate.numel(), _lib.dtype_code(gate.dtype),
            _lib.stream_ptr(gate.device),
        )  # fmt: skip
        return grad_gate, grad_up


def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """Element-wise ``silu(gate) * up`` in the dtype of the inputs."""
    return _SiLUMul.apply(gate, up)
