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


class _SiLUMulHalves(torch.autograd.Function):
    """``silu(gate_up[:, :I]) * gate_up[:, I:]`` without materialising the halves.

    Same arithmetic as ``_SiLUMul``; the two halves are read in place through their row stride
    and the backward writes both gradients into one ``[M, 2I]`` buffer, which removes the two
    ``.contiguous()`` copies of ``Qwen35MoeExperts.forward`` (models/qwen35_moe.py:196-199) and
    the zero-fill + slice-copy + add that autograd runs for them in backward.
    """

    @staticmethod
    def forward(ctx, gate_up: torch.Tensor) -> torch.Tensor:
        assert gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, f"bad gate_up shape {tuple(gate_up.shape)}"
        assert gate_up.is_contiguous(), "gate_up must be contiguous"
        _lib.require_cuda(gate_up)
        rows, two_i = gate_up.shape
        inter = two_i // 2
        eb = gate_up.element_size()
        ctx.save_for_backward(gate_up)
        out = torch.empty((rows, inter), dtype=gate_up.dtype, device=gate_up.device)
        _lib.call(
            "pt_silu_mul_fwd_2d", gate_up.data_ptr(), two_i, gate_up.data_ptr() + inter * eb, two_i,
            out.data_ptr(), inter, rows, inter, _lib.dtype_code(gate_up.dtype), _lib.stream_ptr(gate_up.device),
        )  # fmt: skip
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        (gate_up,) = ctx.saved_tensors
        rows, two_i = gate_up.shape
        inter = two_i // 2
        eb = gate_up.element_size()
        assert grad_output.shape == (rows, inter), f"grad_output shape {tuple(grad_output.shape)}"
        assert grad_output.dtype == gate_up.dtype, f"grad_output dtype {grad_output.dtype} != {gate_up.dtype}"
        assert grad_output.is_contiguous(), "grad_output must be contiguous"
        grad = torch.empty_like(gate_up)
        _lib.call(
            "pt_silu_mul_bwd_2d", grad_output.data_ptr(), inter, gate_up.data_ptr(), two_i,
            gate_up.data_ptr() + inter * eb, two_i, grad.data_ptr(), two_i, grad.data_ptr() + inter * eb, two_i,
            rows, inter, _lib.dtype_code(gate_up.dtype), _lib.stream_ptr(gate_up.device),
        )  # fmt: skip
        return grad


def silu_mul_halves(gate_up: torch.Tensor) -> torch.Tensor:
    """``silu_mul(gate_up[:, :I], gate_up[:, I:])`` for a fused ``[M, 2I]`` projection output
    (concatenated halves), bit-identical to the two-tensor form."""
    return _SiLUMulHalves.apply(gate_up)
