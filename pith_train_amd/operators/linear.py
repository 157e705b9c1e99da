"""Dense FP8 linear on gfx950 and the shared forward / backward GEMM recipe.

Drop-in for ``pithtrain/operators/linear.py``: ``fp8_act_weight_gemm`` (:44-60),
``fp8_dgrad_wgrad`` (:63-83), the custom ops ``fp8_linear_fwd`` / ``fp8_linear_bwd`` with fake
kernels so compiled regions can trace through them (:86-167) and ``FP8Linear`` (:170-208).  All
three GEMMs are "1x128-scaled rows times 128x128-scaled rows, NT".
"""

from __future__ import annotations


import torch
import torch.nn as nn

from .. import _lib
from ..dualpipe_utils import FP8WeightCacheControl
from .deepgemm_quantize import (
    fp8cast_blockwise_transpose,
    fp8cast_rowwise_blockwise_transpose,
    fp8cast_rowwise_transpose,
    transposed_pitch,
)

# Kept for importers of the reference module (``from ...linear import ARCH_MAJOR``); nothing in
# this package branches on it.
ARCH_MAJOR = 9


_WORKGROUPS = 256  # one persistent workgroup per compute unit of the MI355X


def _split_k(m: int, n: int, k: int):
    """(splits, split_len) for out[m, n] = a[m, k] @ b[n, k].T.  An output with fewer 256 x 256
    tiles than the GPU has compute units (the weight gradient of a dense linear: small output,
    reduction over all tokens) leaves most of them idle, so its reduction is cut into ranges that
    are computed side by side into fp32 slabs and summed afterwards.  Ranges are multiples of 128
    (whole scale blocks) and at least 1024 long, so the extra slab traffic stays small."""
    tiles = -(-m // 256) * -(-n // 256)
    if tiles * 2 > _WORKGROUPS or k < 2048 or (m * n) % 8:
        return 1, k
    want = min(_WORKGROUPS // tiles, k // 1024)
    split_len = (-(-k // want) + 127) // 128 * 128
    splits = -(-k // split_len)
    return (splits, split_len) if splits > 1 else (1, k)


def _row_pitch(t: torch.Tensor) -> int:
    """Row pitch in bytes of a 2-D FP8 operand whose rows are contiguous."""
    assert t.stride(1) == 1 or t.shape[1] <= 1, "FP8 GEMM operands need contiguous rows"
    return t.stride(0) if t.shape[0] > 1 else max(t.shape[1], 1)


def _fp8_gemm_nt(a_fp8, a_scale, b_fp8, b_scale, m: int, n: int, device, dtype) -> torch.Tensor:
    """out[m, n] = a @ b.T; a: 1x128 scales, b: 128x128 scales.  The operands may be row-padded
    views (the transposed operands of the quantisers are, for some token counts)."""
    k = a_fp8.shape[1]
    if k % 16:
        # The kernels fetch 16-byte chunks along the reduction dimension.  A ragged length (a
        # wgrad over a token count that is not a multiple of 16) is zero-padded; the padding stays
        # inside the last 128-block, so the scale grids are unchanged.
        pad = 16 - k % 16
        a_fp8 = torch.nn.functional.pad(a_fp8.view(torch.uint8), (0, pad)).view(torch.float8_e4m3fn)
        b_fp8 = torch.nn.functional.pad(b_fp8.view(torch.uint8), (0, pad)).view(torch.float8_e4m3fn)
        k += pad
    lda, ldb = _row_pitch(a_fp8), _row_pitch(b_fp8)
    if lda % 16 or ldb % 16:
        a_fp8, b_fp8 = a_fp8.contiguous(), b_fp8.contiguous()
        lda = ldb = k
    out_dtype = dtype if dtype in (torch.bfloat16, torch.float32) else torch.float32
    out = torch.empty((m, n), device=device, dtype=out_dtype)
    splits, split_len = _split_k(m, n, k)
    if splits > 1:
        partial = torch.empty((splits, m, n), device=device, dtype=torch.float32)
        _lib.call(
            "pt_gemm_nt_dense_splitk_ld", a_fp8.data_ptr(), lda, a_scale.data_ptr(), b_fp8.data_ptr(), ldb,
            b_scale.data_ptr(), partial.data_ptr(), splits, split_len, m, n, k, _lib.stream_ptr(device),
        )  # fmt: skip
        _lib.call("pt_sum_partials", partial.data_ptr(), splits, m * n, out.data_ptr(), _lib.dtype_code(out_dtype),
                  _lib.stream_ptr(device))  # fmt: skip
        return out if out_dtype == dtype else out.to(dtype)
    _lib.call(
        "pt_gemm_nt_dense_ld", a_fp8.data_ptr(), lda, a_scale.data_ptr(), b_fp8.data_ptr(), ldb,
        b_scale.data_ptr(), out.data_ptr(), _lib.dtype_code(out_dtype), m, n, k,
        _lib.stream_ptr(device),
    )  # fmt: skip
    return out if out_dtype == dtype else out.to(dtype)


def fp8_act_weight_gemm(input_2d, weight_fp8, scale_weight):
    """y = x @ W.T; returns (output, input_t_fp8[K,M], scale_input_t) - the transposed activation
    is handed back for the later wgrad."""
    m, n = input_2d.shape[0], weight_fp8.shape[0]
    input_fp8, scale_input, input_t_fp8, scale_input_t = fp8cast_rowwise_blockwise_transpose(input_2d, _padded=True)
    output = _fp8_gemm_nt(
        input_fp8, scale_input, weight_fp8, scale_weight, m, n, input_2d.device, input_2d.dtype
    )
    return output, input_t_fp8, scale_input_t


def fp8_dgrad_wgrad(grad_2d, weight_t_fp8, scale_weight_t, input_t_fp8, scale_input_t, k: int):
    """grad_input = grad @ W (through W^T) and weight_grad = grad^T @ x (through x^T), both in
    ``grad_2d``'s dtype."""
    m, n = grad_2d.shape
    grad_fp8, scale_grad, grad_t_fp8, scale_grad_t = fp8cast_rowwise_transpose(grad_2d, _padded=True)
    grad_input = _fp8_gemm_nt(
        grad_fp8, scale_grad, weight_t_fp8, scale_weight_t, m, k, grad_2d.device, grad_2d.dtype
    )
    weight_grad = _fp8_gemm_nt(
        grad_t_fp8, scale_grad_t, input_t_fp8, scale_input_t, n, k, grad_2d.device, grad_2d.dtype
    )
    return grad_input, weight_grad


def _define_ops(namespace: str):
    """Registers ``<namespace>::fp8_linear_fwd`` and ``<namespace>::fp8_linear_bwd`` with the schema
    of the reference's ops (operators/linear.py:86-167): eager kernels, shape-only fake kernels for
    traced regions, and the autograd link from the forward op to the backward op.  Returns the
    two op objects."""
    fwd_schema = ("(Tensor input_2d, Tensor weight, Tensor weight_fp8, Tensor scale_weight, Tensor weight_t_fp8, "
                  "Tensor scale_weight_t) -> (Tensor, Tensor, Tensor)")
    bwd_schema = ("(Tensor grad_output_2d, Tensor weight_t_fp8, Tensor scale_weight_t, Tensor input_t_fp8, "
                  "Tensor scale_input_t, int K) -> (Tensor, Tensor)")

    @torch.library.custom_op(f"{namespace}::fp8_linear_fwd", mutates_args=(), schema=fwd_schema)
    def fwd(input_2d, weight, weight_fp8, scale_weight, weight_t_fp8, scale_weight_t):
        return fp8_act_weight_gemm(input_2d.contiguous(), weight_fp8, scale_weight)

    @fwd.register_fake
    def _(input_2d, weight, weight_fp8, scale_weight, weight_t_fp8, scale_weight_t):
        rows, red = input_2d.shape
        dev = input_2d.device
        return (
            torch.empty((rows, weight.shape[0]), dtype=input_2d.dtype, device=dev),
            torch.empty_strided((red, rows), (transposed_pitch(rows), 1), dtype=torch.float8_e4m3fn, device=dev),
            torch.empty((-(-red // 128), -(-rows // 128)), dtype=torch.float32, device=dev),
        )

    @torch.library.custom_op(f"{namespace}::fp8_linear_bwd", mutates_args=(), schema=bwd_schema)
    def bwd(grad_output_2d, weight_t_fp8, scale_weight_t, input_t_fp8, scale_input_t, K):
        return fp8_dgrad_wgrad(grad_output_2d.contiguous(), weight_t_fp8, scale_weight_t, input_t_fp8, scale_input_t, K)

    @bwd.register_fake
    def _(grad_output_2d, weight_t_fp8, scale_weight_t, input_t_fp8, scale_input_t, K):
        rows, cols = grad_output_2d.shape
        like = dict(dtype=grad_output_2d.dtype, device=grad_output_2d.device)
        return torch.empty((rows, K), **like), torch.empty((cols, K), **like)

    def remember(ctx, inputs, output):
        # what the backward op reads: the transposed quantised weight and the transposed quantised
        # activation the forward op handed back
        ctx.save_for_backward(inputs[4], inputs[5], output[1], output[2])
        ctx.K = inputs[0].shape[1]
        # The quantised activation and its scales are outputs only so that the backward op can read
        # them: nothing flows back through them, and autograd must not fill a zero "gradient" of
        # their size (64 MB of FP8 per 32k-token linear) before every backward call.
        ctx.set_materialize_grads(False)

    def backward(ctx, grad_output, _grad_input_t, _grad_scale_t):
        if grad_output is None:
            return None, None, None, None, None, None
        grad_input, weight_grad = bwd(grad_output, *ctx.saved_tensors, ctx.K)
        return grad_input, weight_grad, None, None, None, None

    fwd.register_autograd(backward, setup_context=remember)
    return fwd, bwd


_fp8_linear_fwd, _fp8_linear_bwd = _define_ops("pith_train_amd")
# The reference registers the same two ops as pithtrain::fp8_linear_fwd / fp8_linear_bwd; code that
# finds them by qualified name (torch.ops.pithtrain.*) gets these kernels when this module is
# imported first.  When the reference's own module was imported first the names are taken and stay
# the reference's; importing the reference's module after this one fails in its own registration.
# PITHTRAIN_OPS_OWNER says which of the two happened ("pith_train_amd" or "other").
try:
    _define_ops("pithtrain")
    PITHTRAIN_OPS_OWNER = "pith_train_amd"
except RuntimeError as exc:
    import warnings

    PITHTRAIN_OPS_OWNER = "other"
    warnings.warn(
        "pithtrain::fp8_linear_fwd / fp8_linear_bwd were registered before pith_train_amd was imported "
        f"and keep their first implementation ({exc}); FP8Linear of this package is unaffected "
        "(it calls pith_train_amd::fp8_linear_*)", RuntimeWarning, stacklevel=2)


class FP8Linear(nn.Linear):
    """``nn.Linear`` whose three GEMMs run in FP8; the bf16 weight is quantised once per
    ``FP8WeightCacheControl.version`` and reused across micro-batches."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self._wq_cache = None
        self._wq_version: int = -1

    def _get_quantized_weight(self):
        if torch.compiler.is_compiling():
            return fp8cast_blockwise_transpose(self.weight)
        ver = FP8WeightCacheControl.version
        if self._wq_version == ver and self._wq_cache is not None:
            return self._wq_cache
        result = fp8cast_blockwise_transpose(self.weight)
        self._wq_cache = result
        self._wq_version = ver
        return result

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        if input.numel() == 0:
            return torch.nn.functional.linear(input, self.weight, self.bias)
        weight_fp8, scale_weight, weight_t_fp8, scale_weight_t = self._get_quantized_weight()
        input_2d = input.flatten(0, -2)
        output_2d, _, _ = _fp8_linear_fwd(
            input_2d, self.weight, weight_fp8, scale_weight, weight_t_fp8, scale_weight_t
        )
        output = output_2d.view(*input.shape[:-1], self.weight.shape[0])
        if self.bias is not None:
            output = output + self.bias
        return output
