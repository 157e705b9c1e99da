"""Fused clamped SwiGLU of gpt-oss: ``(uc + 1) * gc * sigmoid(alpha * gc)`` with
``gc = min(gate, L)``, ``uc = clamp(up, -L, L)``; gate / up are the even / odd columns of
``gate_up[M, 2N]``.

Drop-in for ``pithtrain/operators/clamped_swiglu.py`` (``clamped_swiglu`` :148-155,
``_ClampedSwiGLU`` :95-145): only ``gate_up`` is saved; saturated branches get zero gradient.
"""

from __future__ import annotations

import torch

from .. import _lib


class _ClampedSwiGLU(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gate_up: torch.Tensor, alpha: float, limit: float) -> torch.Tensor:
        assert gate_up.dim() == 2, f"gate_up must be 2-D, got shape {gate_up.shape}"
        M, two_n = gate_up.shape
        assert two_n % 2 == 0, f"gate_up last dim must be even, got {two_n}"
        assert gate_up.is_contiguous(), "gate_up must be contiguous"
        _lib.require_cuda(gate_up)
        N = two_n // 2
        out = torch.empty((M, N), device=gate_up.device, dtype=gate_up.dtype)
        ctx.save_for_backward(gate_up)
        ctx.alpha = float(alpha)
        ctx.limit = float(limit)
        if M * N:
            _lib.call(
                "pt_clamped_swiglu_fwd", gate_up.data_ptr(), out.data_ptr(), M * N, ctx.alpha,
                ctx.limit, _lib.dtype_code(gate_up.dtype), _lib.stream_ptr(gate_up.device),
            )  # fmt: skip
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        (gate_up,) = ctx.saved_tensors
        assert grad_output.shape[0] == gate_up.shape[0]
        assert grad_output.shape[1] * 2 == gate_up.shape[1]
        assert grad_output.dtype == gate_up.dtype
        assert grad_output.is_contiguous(), "grad_output must be contiguous"
        grad_gate_up = torch.empty_like(gate_up)
        n = grad_output.numel()
        if n:
            _lib.call(
                "pt_clamped_swiglu_bwd", grad_output.data_ptr(), gate_up.data_ptr(),
                grad_gate_up.data_ptr(), n, ctx.alpha, ctx.limit, _lib.dtype_code(gate_up.dtype),
                _lib.stream_ptr(gate_up.device),
            )  # fmt: skip
        return grad_gate_up, None, None


def clamped_swiglu(gate_up: torch.Tensor, alpha: float, limit: float) -> torch.Tensor:
    """``gate_up`` (M, 2N) interleaved -> (M, N)."""
    return _ClampedSwiGLU.apply(gate_up, alpha, limit)
