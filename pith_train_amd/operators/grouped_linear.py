"""Grouped (per-expert) linear layers: FP8 on the gfx950 matrix cores, and the BF16 baseline.

Drop-in for ``pithtrain/operators/grouped_linear.py``: ``GroupedLinearFunc`` / ``GroupedLinear``
(:18-85) and ``FP8GroupedLinearFunc`` / ``FP8GroupedLinear`` (:104-284) keep their signatures,
including the deferred weight-gradient closure handed to ``WeightGradStore`` and the direct write
to ``weight.grad``.

Differences that stay behind the interface:
  * the colwise copies kept for the wgrad GEMM are stored transposed ([N, M]); that is the operand
    layout of ``pt_gemm_k_grouped_wgrad``;
  * the wgrad GEMM rounds to bf16 and (when ``weight.grad`` exists) accumulates in its epilogue,
    instead of fp32 zeros -> GEMM -> cast -> add as four passes over a [G, N, K] tensor;
  * ``group_indices`` is accepted and ignored (the kernels search ``grouped_mm_offs`` themselves).
"""

from __future__ import annotations

from functools import partial
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import _lib
from ..dualpipe_utils import FP8WeightCacheControl, WeightGradStore
from .deepgemm_quantize import (
    fp8cast_blockwise_transpose_batched,
    fp8cast_blockwise_transpose_batched_cat,
    fp8cast_grouped_weight,
    weight_twin_enabled,
    fp8cast_rowwise_colwise_t,
    fp8cast_rowwise_colwise_t_rows,
)


_GROUPED_MM_USABLE: dict = {}  # (device type, dtype) -> whether torch's grouped_mm runs there


def _torch_grouped_mm_usable(a: torch.Tensor) -> bool:
    """Decided once per device type and dtype with a one-group 16 x 16 product, so that an error
    on real operands (out of memory, a shape mismatch) is raised instead of being turned into the
    slow per-group loop."""
    key = (a.device.type, a.dtype)
    if key not in _GROUPED_MM_USABLE:
        ok = hasattr(F, "grouped_mm")
        if ok:
            try:
                t = torch.zeros((16, 16), dtype=a.dtype, device=a.device)
                F.grouped_mm(t, t.unsqueeze(0), offs=torch.tensor([16], dtype=torch.int32, device=a.device))
            except (RuntimeError, NotImplementedError):
                ok = False
        _GROUPED_MM_USABLE[key] = ok
    return _GROUPED_MM_USABLE[key]


def _grouped_mm(a: torch.Tensor, b: torch.Tensor, offs: torch.Tensor) -> torch.Tensor:
    """``F.grouped_mm`` where torch provides it for the device, otherwise the per-group loop it
    stands for (which reads the offsets on the host)."""
    if a.device.type != "cuda":
        # host tensors (tests, the CPU reference path): torch's CPU grouped_mm rejects some layouts
        # it could compute; the loop below is as good there
        if hasattr(F, "grouped_mm"):
            try:
                return F.grouped_mm(a, b, offs=offs)
            except (RuntimeError, NotImplementedError):
                pass
    elif _torch_grouped_mm_usable(a):
        return F.grouped_mm(a, b, offs=offs)
    bounds = [0] + offs.tolist()
    if a.dim() == 2 and b.dim() == 3:  # jagged on rows of a
        out = a.new_zeros((a.shape[0], b.shape[2]))
        for g in range(b.shape[0]):
            s, e = bounds[g], bounds[g + 1]
            if e > s:
                out[s:e] = a[s:e] @ b[g]
        return out
    out = a.new_zeros((len(bounds) - 1, a.shape[0], b.shape[1]))  # jagged on the reduction dim
    for g in range(len(bounds) - 1):
        s, e = bounds[g], bounds[g + 1]
        if e > s:
            out[g] = a[:, s:e] @ b[s:e]
    return out


class GroupedLinearFunc(torch.autograd.Function):
    """BF16 grouped linear; wgrad split off so it can be deferred (grouped_linear.py:18-55)."""

    @staticmethod
    def forward(ctx, input: torch.Tensor, weight: torch.Tensor, grouped_mm_offs: torch.Tensor):
        output = _grouped_mm(input, weight.transpose(1, 2), grouped_mm_offs)
        ctx.save_for_backward(input, weight, grouped_mm_offs)
        return output

    @staticmethod
    def backward(ctx, dy):
        input, weight, offs = ctx.saved_tensors
        dgrad = _grouped_mm(dy, weight, offs)

        def wgrad_fn(dy, x, offs):
            wgrad = _grouped_mm(dy.transpose(0, 1), x, offs)
            weight.grad = wgrad if weight.grad is None else weight.grad.add_(wgrad)

        if WeightGradStore.enabled:
            WeightGradStore.put(partial(wgrad_fn, dy.detach(), input.detach(), offs.detach()))
        else:
            wgrad_fn(dy, input, offs)
        return dgrad, None, None


class GroupedLinear(nn.Module):
    """One linear map per group of rows (MoE experts), BF16."""

    def __init__(self, num_groups: int, in_features: int, out_features: int):
        super().__init__()
        self.num_groups = num_groups
        self.in_features = in_features
        self.out_features = out_features
        self.weight = nn.Parameter(torch.empty((num_groups, out_features, in_features)))

    def forward(
        self,
        input: torch.Tensor,
        grouped_mm_offs: torch.Tensor,
        ks: Optional[list] = None,
        ks_tensor: Optional[torch.Tensor] = None,
        group_indices: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        if input.shape[0] == 0:
            return input @ self.weight[0].T  # keeps a grad_fn with zero rows
        return GroupedLinearFunc.apply(input, self.weight, grouped_mm_offs)


# ------------------------------------------------------------------------------------------------
# FP8
# ------------------------------------------------------------------------------------------------
def m_grouped_fp8_gemm_nt(a, b, out: torch.Tensor, grouped_mm_offs: torch.Tensor,
                          out_rows: torch.Tensor | None = None, bias: torch.Tensor | None = None) -> torch.Tensor:
    """out[rows_g] = a[rows_g] @ b[g].T with a=(fp8[M,K], scale[M,K/128]), b=(fp8[G,N,K],
    scale[G,N/128,K/128]).  Rows at or past ``grouped_mm_offs[-1]`` are left untouched.  With
    ``out_rows`` (int32 [M]) result row r is written to ``out[out_rows[r]]`` instead (negative:
    dropped).  With ``bias`` ([G, N] in ``out``'s dtype) the bias row of a row's group is added
    to the rounded result (``out + bias[group_ids]`` in the output dtype, as one kernel).  Both
    may be given."""
    (a_fp8, a_s), (b_fp8, b_s) = a, b
    M, K = a_fp8.shape
    G, N, _ = b_fp8.shape
    if bias is not None:
        assert bias.shape == (G, N) and bias.dtype == out.dtype and bias.is_contiguous()
    if bias is not None and out_rows is not None:
        assert out_rows.dtype == torch.int32 and out_rows.shape == (M,)
        _lib.call(
            "pt_gemm_m_grouped_nt_scatter_bias", a_fp8.data_ptr(), a_s.data_ptr(), b_fp8.data_ptr(), b_s.data_ptr(),
            out.data_ptr(), _lib.dtype_code(out.dtype), grouped_mm_offs.data_ptr(), G, M, N, K,
            out_rows.contiguous().data_ptr(), out.shape[0], bias.data_ptr(), _lib.stream_ptr(out.device),
        )  # fmt: skip
        return out
    if bias is not None:
        _lib.call(
            "pt_gemm_m_grouped_nt_bias", a_fp8.data_ptr(), a_s.data_ptr(), b_fp8.data_ptr(), b_s.data_ptr(),
            out.data_ptr(), _lib.dtype_code(out.dtype), grouped_mm_offs.data_ptr(), G, M, N, K, bias.data_ptr(),
            _lib.stream_ptr(out.device),
        )  # fmt: skip
        return out
    if out_rows is not None:
        _lib.call(
            "pt_gemm_m_grouped_nt_scatter", a_fp8.data_ptr(), a_s.data_ptr(), b_fp8.data_ptr(),
            b_s.data_ptr(), out.data_ptr(), _lib.dtype_code(out.dtype), grouped_mm_offs.data_ptr(), G,
            M, N, K, out_rows.data_ptr(), out.shape[0], _lib.stream_ptr(out.device),
        )  # fmt: skip
        return out
    _lib.call(
        "pt_gemm_m_grouped_nt", a_fp8.data_ptr(), a_s.data_ptr(), b_fp8.data_ptr(), b_s.data_ptr(),
        out.data_ptr(), _lib.dtype_code(out.dtype), grouped_mm_offs.data_ptr(), G, M, N, K,
        _lib.stream_ptr(out.device),
    )  # fmt: skip
    return out


def k_grouped_fp8_wgrad(dy_t, x_t, out: torch.Tensor, grouped_mm_offs, accumulate: bool):
    """out[g] (+)= dY_g^T X_g with dy_t=(fp8[N,M], scale[M/128,N]), x_t=(fp8[K,M], scale[M/128,K]).
    The fp8 operands are contiguous; the scale arrays may be column slices of wider arrays (their
    row stride is passed on)."""
    (dy_fp8, dy_s), (x_fp8, x_s) = dy_t, x_t
    N, M = dy_fp8.shape
    K = x_fp8.shape[0]
    G = out.shape[0]
    assert dy_fp8.is_contiguous() and x_fp8.is_contiguous() and dy_s.stride(-1) == 1 and x_s.stride(-1) == 1
    ld_dy = dy_s.stride(0) if dy_s.shape[0] > 1 else N
    ld_x = x_s.stride(0) if x_s.shape[0] > 1 else K
    if ld_dy == N and ld_x == K:
        _lib.call(
            "pt_gemm_k_grouped_wgrad", dy_fp8.data_ptr(), dy_s.data_ptr(), x_fp8.data_ptr(),
            x_s.data_ptr(), out.data_ptr(), _lib.dtype_code(out.dtype), int(accumulate),
            grouped_mm_offs.data_ptr(), G, M, N, K, _lib.stream_ptr(out.device),
        )  # fmt: skip
    else:
        _lib.call(
            "pt_gemm_k_grouped_wgrad_ld", dy_fp8.data_ptr(), dy_s.data_ptr(), ld_dy, x_fp8.data_ptr(),
            x_s.data_ptr(), ld_x, out.data_ptr(), _lib.dtype_code(out.dtype), int(accumulate),
            grouped_mm_offs.data_ptr(), G, M, N, K, _lib.stream_ptr(out.device),
        )  # fmt: skip
    return out


def schedule_wgrad(weight: torch.Tensor, a_wgrad: tuple, b_wgrad: tuple, offs: torch.Tensor) -> None:
    """Run - or, when ``WeightGradStore`` is enabled, queue - the weight-gradient GEMM of one
    grouped linear (``grad_weight_fn``, grouped_linear.py:202-234): ``a_wgrad`` / ``b_wgrad`` are the
    colwise-quantised transposed copies (fp8 ``[N, M]`` / ``[K, M]`` and their scales).  The result is
    written to ``weight.grad`` (assigned if None, accumulated otherwise)."""
    num_groups, N, K = weight.shape

    def grad_weight_fn(a, b, offs):
        # bf16(sum) is formed in the GEMM epilogue; an existing grad is accumulated there too
        if weight.grad is None:
            wg = torch.empty((num_groups, N, K), device=a[0].device, dtype=torch.bfloat16)
            k_grouped_fp8_wgrad(a, b, wg, offs, accumulate=False)
            weight.grad = wg if weight.dtype == torch.bfloat16 else wg.to(weight.dtype)
        elif weight.grad.dtype == torch.bfloat16 and weight.grad.is_contiguous():
            k_grouped_fp8_wgrad(a, b, weight.grad, offs, accumulate=True)
        else:
            wg = torch.empty((num_groups, N, K), device=a[0].device, dtype=torch.bfloat16)
            k_grouped_fp8_wgrad(a, b, wg, offs, accumulate=False)
            weight.grad += wg

    if WeightGradStore.enabled:
        WeightGradStore.put(
            partial(
                grad_weight_fn,
                (a_wgrad[0].detach(), a_wgrad[1].detach()),
                (b_wgrad[0].detach(), b_wgrad[1].detach()),
                offs.detach(),
            )
        )
    else:
        grad_weight_fn(a_wgrad, b_wgrad, offs)


def m_grouped_fp8_gemm_nn(a, b, out: torch.Tensor, grouped_mm_offs: torch.Tensor,
                          out_rows: torch.Tensor | None = None) -> torch.Tensor:
    """out[rows_g] = a[rows_g] @ b[g] with a=(fp8[M,K], scale[M,K/128]) and b=(fp8[G,K,N],
    scale[G,K/128,N/128]) reduction-major: a weight ``[G, out, in]`` in its forward layout, read by
    the input-gradient GEMM (K = out features, N = in features).  Same bits as
    :func:`m_grouped_fp8_gemm_nt` on the transposed operand.  ``out_rows`` as there."""
    (a_fp8, a_s), (b_fp8, b_s) = a, b
    M, K = a_fp8.shape
    G, Kb, N = b_fp8.shape
    assert Kb == K, (b_fp8.shape, a_fp8.shape)
    if out_rows is not None:
        _lib.call(
            "pt_gemm_m_grouped_nn_scatter", a_fp8.data_ptr(), a_s.data_ptr(), b_fp8.data_ptr(),
            b_s.data_ptr(), out.data_ptr(), _lib.dtype_code(out.dtype), grouped_mm_offs.data_ptr(), G,
            M, N, K, out_rows.data_ptr(), out.shape[0], _lib.stream_ptr(out.device),
        )  # fmt: skip
        return out
    _lib.call(
        "pt_gemm_m_grouped_nn", a_fp8.data_ptr(), a_s.data_ptr(), b_fp8.data_ptr(), b_s.data_ptr(),
        out.data_ptr(), _lib.dtype_code(out.dtype), grouped_mm_offs.data_ptr(), G, M, N, K,
        _lib.stream_ptr(out.device),
    )  # fmt: skip
    return out


# limits of the kernel that reads a weight in its forward layout (32-bit byte offsets, group table)
_NN_MAX_GRAD_BYTES = 2**31
_NN_MAX_OUT_BYTES = 2**32
_NN_MAX_GROUPS = 2048


def dgrad_operand(quantized_weight: tuple, weight=None, rows: int = 0):
    """(fp8, scale, forward_layout) of the weight operand the input-gradient GEMM reads: the
    transposed twin when the tuple has one, else the forward-layout tensors themselves.

    The kernel that reads the forward layout addresses its operands through 32-bit byte offsets:
    the quantised gradient ``[rows, out_features]`` must stay below 2 GiB and the result
    ``[rows, in_features]`` (2 bytes per element) below 4 GiB.  Past that (``rows`` and the bf16
    ``weight``, or the tuple of weights whose rows the quantised operand concatenates, are given by
    the forward for this check) the twin is built here, once, instead of failing in the backward."""
    w_fp8, w_scale, w_t_fp8, w_t_scale = quantized_weight
    if w_t_fp8 is None and weight is not None:
        n_out, n_in = w_fp8.shape[1], w_fp8.shape[2]
        if rows * n_out >= _NN_MAX_GRAD_BYTES or rows * n_in * 2 >= _NN_MAX_OUT_BYTES or w_fp8.shape[0] > _NN_MAX_GROUPS:
            if isinstance(weight, (tuple, list)):
                _, _, w_t_fp8, w_t_scale = fp8cast_blockwise_transpose_batched_cat([p_.detach() for p_ in weight])
            else:
                _, _, w_t_fp8, w_t_scale = fp8cast_blockwise_transpose_batched(weight)
    if w_t_fp8 is None:
        return w_fp8, w_scale, True
    return w_t_fp8, w_t_scale, False


def m_grouped_fp8_dgrad(grad, w_fp8: torch.Tensor, w_scale: torch.Tensor, forward_layout: bool, out: torch.Tensor,
                        grouped_mm_offs: torch.Tensor, out_rows: torch.Tensor | None = None) -> torch.Tensor:
    """dX = dY W per group, from whichever weight operand :func:`dgrad_operand` returned."""
    if forward_layout:
        # (the NN form exists in the kernel with 32-bit offsets only: a gradient of 2 GiB or an
        # output of 4 GiB and more needs PITHTRAIN_FP8_WEIGHT_TWIN=1, and the library says so)
        return m_grouped_fp8_gemm_nn(grad, (w_fp8, w_scale), out, grouped_mm_offs, out_rows)
    return m_grouped_fp8_gemm_nt(grad, (w_fp8, w_scale), out, grouped_mm_offs, out_rows)


class FP8GroupedLinearFunc(torch.autograd.Function):
    """FP8 grouped linear (grouped_linear.py:104-236): forward and dgrad are m-grouped NT GEMMs on
    1x128-scaled activations against 128x128-scaled weights, wgrad a k-grouped GEMM on the colwise
    copies."""

    @staticmethod
    def forward(
        ctx,
        input: torch.Tensor,
        weight: torch.Tensor,
        grouped_mm_offs: torch.Tensor,
        ks: list,
        ks_tensor: torch.Tensor,
        quantized_weight: tuple,
        group_indices: torch.Tensor | None = None,
        in_rows: torch.Tensor | None = None,
        out_rows: torch.Tensor | None = None,
        out_m: int | None = None,
        bias: torch.Tensor | None = None,
    ):
        """``bias`` (extension; ``[G, N]`` in the input's dtype): ``indexed_bias_add`` of the result
        folded into the GEMM's store (same bits as the two operators in a row; its gradient is the
        per-group row sum of the incoming gradient).

        ``in_rows`` / ``out_rows`` (extension; int32 ``[M]`` source-row maps as produced by the
        scatter, every non-negative value occurring once) fold the token permutation into this
        layer: with ``in_rows`` the input is the un-permuted ``[m, K]`` tensor and grouped row r is
        read from ``input[in_rows[r]]``; with ``out_rows`` the result is returned un-permuted
        (``[out_m, N]``, row ``out_rows[r]`` holding grouped row r).  Backward mirrors both."""
        weight_fp8, scale_weight, weight_t_fp8, scale_weight_t = quantized_weight
        num_groups, N, K = weight.shape
        if in_rows is not None:
            M = in_rows.shape[0]
            input_fp8, scale_input, input_ch_t, scale_input_ch = fp8cast_rowwise_colwise_t_rows(input, in_rows)
        else:
            M = input.shape[0]
            input_fp8, scale_input, input_ch_t, scale_input_ch = fp8cast_rowwise_colwise_t(input)
        if out_rows is not None:
            assert out_m is not None, "out_rows needs out_m, the row count of the un-permuted result"
            output = torch.empty((out_m, N), device=input.device, dtype=input.dtype)
        else:
            output = torch.empty((M, N), device=input.device, dtype=input.dtype)
        m_grouped_fp8_gemm_nt(
            (input_fp8, scale_input), (weight_fp8, scale_weight), output, grouped_mm_offs, out_rows,
            bias.detach().contiguous() if bias is not None else None,
        )
        ctx.bias_dtype = bias.dtype if bias is not None else None
        dg_fp8, dg_scale, ctx.dgrad_forward_layout = dgrad_operand(quantized_weight, weight, M)
        ctx.save_for_backward(
            dg_fp8, dg_scale, grouped_mm_offs, input_ch_t, scale_input_ch, ks_tensor,
            in_rows, out_rows,
        )
        ctx.weight_ref = weight
        ctx.ks = ks
        ctx.dims = (M, K, N, num_groups)
        ctx.in_m = input.shape[0]
        return output

    @staticmethod
    def backward(ctx, grad_output):
        (dg_fp8, dg_scale, offs, input_ch_t, scale_input_ch, ks_tensor, in_rows,
         out_rows) = ctx.saved_tensors  # fmt: skip
        weight = ctx.weight_ref
        M, K, N, num_groups = ctx.dims
        grad_output = grad_output.contiguous()
        if out_rows is not None:  # the gradient arrives un-permuted: gather while quantising
            grad_fp8, scale_grad, grad_ch_t, scale_grad_ch = fp8cast_rowwise_colwise_t_rows(grad_output, out_rows)
        else:
            grad_fp8, scale_grad, grad_ch_t, scale_grad_ch = fp8cast_rowwise_colwise_t(grad_output)

        rows_in = ctx.in_m if in_rows is not None else M
        grad_input = torch.empty((rows_in, K), device=grad_output.device, dtype=grad_output.dtype)
        m_grouped_fp8_dgrad((grad_fp8, scale_grad), dg_fp8, dg_scale, ctx.dgrad_forward_layout, grad_input, offs, in_rows)

        schedule_wgrad(weight, (grad_ch_t, scale_grad_ch), (input_ch_t, scale_input_ch), offs)
        grad_bias = None
        if ctx.bias_dtype is not None:
            from .indexed_bias_add import _segment_sum_along_rows

            # un-permuted gradient: summed in the grouped order of its rows through the row map
            grad_bias = _segment_sum_along_rows(grad_output, offs, ctx.bias_dtype, out_rows)
        return grad_input, None, None, None, None, None, None, None, None, None, grad_bias


class FP8GroupedLinear(nn.Module):
    """FP8 grouped linear for MoE experts; weight ``(num_groups, out_features, in_features)``.
    The quantised weight is cached per ``FP8WeightCacheControl.version``."""

    def __init__(self, num_groups: int, in_features: int, out_features: int):
        super().__init__()
        self.num_groups = num_groups
        self.in_features = in_features
        self.out_features = out_features
        self.weight = nn.Parameter(torch.empty((num_groups, out_features, in_features)))
        self._wq_cache = None
        self._wq_version: int = -1

    def _get_quantized_weight(self):
        if torch.compiler.is_compiling():
            return fp8cast_grouped_weight(self.weight)
        ver = FP8WeightCacheControl.version
        cache = self._wq_cache
        # a cached tuple is reused only in the shape the twin switch asks for now
        if self._wq_version == ver and cache is not None and (cache[2] is not None) == weight_twin_enabled():
            return cache
        result = fp8cast_grouped_weight(self.weight)
        self._wq_cache = result
        self._wq_version = ver
        return result

    def forward(
        self,
        input: torch.Tensor,
        grouped_mm_offs: torch.Tensor,
        ks: list | None = None,
        ks_tensor: torch.Tensor | None = None,
        group_indices: torch.Tensor | None = None,
        in_rows: torch.Tensor | None = None,
        out_rows: torch.Tensor | None = None,
        out_m: int | None = None,
    ) -> torch.Tensor:
        if input.shape[0] == 0:
            return input @ self.weight[0].T  # keeps a grad_fn with zero rows
        return FP8GroupedLinearFunc.apply(
            input, self.weight, grouped_mm_offs, ks, ks_tensor, self._get_quantized_weight(),
            group_indices, in_rows, out_rows, out_m,
        )  # fmt: skip
