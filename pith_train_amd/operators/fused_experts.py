"""A whole SwiGLU expert block (fused gate_up projection -> SwiGLU -> down projection) as one
autograd node, for the FP8 path.

Composition and arithmetic are those of ``Qwen35MoeExperts.forward``
(models/qwen35_moe.py:190-200) built from ``FP8GroupedLinearFunc`` (grouped_linear.py:104-236) and
``silu_mul`` (silu_mul.py:93-143); the results are bit-identical to that composition.  Being one
node lets two intermediate bf16 tensors stay out of memory: the SwiGLU output ``h`` (forward) and
its gradient ``[dgate | dup]`` (backward) are produced inside the kernels that quantise them.
The token permutation can be folded in as well (``row_map``, see ``FP8GroupedLinearFunc``).
"""

from __future__ import annotations

import torch

from .. import _lib
from .deepgemm_quantize import FP8, fp8cast_rowwise_colwise_t, fp8cast_rowwise_colwise_t_rows
from .grouped_linear import dgrad_operand, m_grouped_fp8_dgrad, m_grouped_fp8_gemm_nt, schedule_wgrad
from .token_scatter import _GEMM_ALLOC_ALIGNMENT, _PaddedIndexGather


def _cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def _last(offs):
    """Device pointer to the last entry of the inclusive group offsets (= the number of grouped rows)."""
    return None if offs is None or offs.numel() == 0 else offs.data_ptr() + 4 * (offs.numel() - 1)


def silu_mul_quant(gate_up: torch.Tensor, grouped_mm_offs: torch.Tensor | None = None):
    """``fp8cast_rowwise_colwise_t(silu_mul(gate_up[:, :I], gate_up[:, I:]))`` in one pass.  With
    ``grouped_mm_offs`` only the rows below its last entry are processed (the tensors may be sized
    for more rows than the routing produced)."""
    M, two_i = gate_up.shape
    half = two_i // 2
    dev = gate_up.device
    tok = torch.empty((M, half), dtype=FP8, device=dev)
    tok_s = torch.empty((M, _cdiv(half, 128)), dtype=torch.float32, device=dev)
    ch_t = torch.empty((half, M), dtype=FP8, device=dev)
    ch_s = torch.empty((M // 128, half), dtype=torch.float32, device=dev)
    _lib.call(
        "pt_silu_mul_quant_rowwise_colwise", gate_up.data_ptr(), M, half, gate_up.stride(0),
        tok.data_ptr(), tok_s.data_ptr(), ch_t.data_ptr(), ch_s.data_ptr(), _last(grouped_mm_offs),
        _lib.stream_ptr(dev),
    )  # fmt: skip
    return tok, tok_s, ch_t, ch_s


def silu_mul_bwd_quant(grad_h: torch.Tensor, gate_up: torch.Tensor, grouped_mm_offs: torch.Tensor | None = None):
    """``fp8cast_rowwise_colwise_t`` of the SwiGLU gradient ``[dgate | dup]`` in one pass (rows
    limited as in :func:`silu_mul_quant`)."""
    M, two_i = gate_up.shape
    half = two_i // 2
    dev = gate_up.device
    tok = torch.empty((M, two_i), dtype=FP8, device=dev)
    tok_s = torch.empty((M, _cdiv(two_i, 128)), dtype=torch.float32, device=dev)
    ch_t = torch.empty((two_i, M), dtype=FP8, device=dev)
    ch_s = torch.empty((M // 128, two_i), dtype=torch.float32, device=dev)
    _lib.call(
        "pt_silu_mul_bwd_quant_rowwise_colwise", grad_h.data_ptr(), grad_h.stride(0), gate_up.data_ptr(),
        gate_up.stride(0), M, half, tok.data_ptr(), tok_s.data_ptr(), ch_t.data_ptr(), ch_s.data_ptr(),
        _last(grouped_mm_offs), _lib.stream_ptr(dev),
    )  # fmt: skip
    return tok, tok_s, ch_t, ch_s


def clamped_swiglu_quant(gate_up: torch.Tensor, alpha: float, limit: float, grouped_mm_offs: torch.Tensor | None = None):
    """``fp8cast_rowwise_colwise_t(clamped_swiglu(gate_up, alpha, limit))`` in one pass (interleaved
    (gate, up) pairs, clamped_swiglu.py:95-155); rows limited as in :func:`silu_mul_quant`."""
    M, two_i = gate_up.shape
    half = two_i // 2
    dev = gate_up.device
    tok = torch.empty((M, half), dtype=FP8, device=dev)
    tok_s = torch.empty((M, _cdiv(half, 128)), dtype=torch.float32, device=dev)
    ch_t = torch.empty((half, M), dtype=FP8, device=dev)
    ch_s = torch.empty((M // 128, half), dtype=torch.float32, device=dev)
    _lib.call(
        "pt_clamped_swiglu_quant_rowwise_colwise", gate_up.data_ptr(), M, half, gate_up.stride(0), alpha, limit,
        tok.data_ptr(), tok_s.data_ptr(), ch_t.data_ptr(), ch_s.data_ptr(), _last(grouped_mm_offs),
        _lib.stream_ptr(dev),
    )  # fmt: skip
    return tok, tok_s, ch_t, ch_s


def clamped_swiglu_bwd_quant(grad_h: torch.Tensor, gate_up: torch.Tensor, alpha: float, limit: float,
                             grouped_mm_offs: torch.Tensor | None = None):
    """``fp8cast_rowwise_colwise_t`` of the clamped SwiGLU's input gradient in one pass, plus
    ``col_sum`` ``[M / 128, 2I]`` fp32: the column sums of every 128-row tile of that (bf16-rounded)
    gradient, from which the bias gradient of the projection before it is summed per group."""
    M, two_i = gate_up.shape
    half = two_i // 2
    dev = gate_up.device
    tok = torch.empty((M, two_i), dtype=FP8, device=dev)
    tok_s = torch.empty((M, _cdiv(two_i, 128)), dtype=torch.float32, device=dev)
    ch_t = torch.empty((two_i, M), dtype=FP8, device=dev)
    ch_s = torch.empty((M // 128, two_i), dtype=torch.float32, device=dev)
    col_sum = torch.empty((M // 128, two_i), dtype=torch.float32, device=dev)
    _lib.call(
        "pt_clamped_swiglu_bwd_quant_rowwise_colwise", grad_h.data_ptr(), grad_h.stride(0), gate_up.data_ptr(),
        gate_up.stride(0), M, half, alpha, limit, tok.data_ptr(), tok_s.data_ptr(), ch_t.data_ptr(), ch_s.data_ptr(),
        col_sum.data_ptr(), _last(grouped_mm_offs), _lib.stream_ptr(dev),
    )  # fmt: skip
    return tok, tok_s, ch_t, ch_s, col_sum


def supported(x: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor) -> bool:
    """bf16 activations, half width and hidden size multiples of 8 (16-byte accesses)."""
    half = w_gate_up.shape[1] // 2
    return (x.dtype == torch.bfloat16 and w_gate_up.shape[1] % 2 == 0 and half % 8 == 0
            and w_down.shape[1] % 8 == 0 and w_down.shape[2] == half)


def compose_row_maps(row_map: torch.Tensor, expand_idx: torch.Tensor, n_src: int) -> torch.Tensor:
    """``expand_idx[row_map]`` with the negative (padding) entries of ``row_map`` kept negative:
    the source row (among ``n_src``) of every grouped row when the routed rows are themselves an
    expansion (``expand_idx``) of deduplicated rows."""
    assert row_map.dtype == torch.int32 and expand_idx.dtype == torch.int64
    out = torch.empty_like(row_map)
    _lib.call(
        "pt_compose_row_map", row_map.contiguous().data_ptr(), row_map.numel(), expand_idx.contiguous().data_ptr(),
        expand_idx.numel(), n_src, out.data_ptr(), _lib.stream_ptr(row_map.device),
    )  # fmt: skip
    return out


def _forward(ctx, x, gate_up_weights, w_down, grouped_mm_offs, q_gate_up, q_down, row_map, expand_idx=None):
    """Shared forward of the two autograd nodes below.  ``gate_up_weights``: the parameters whose
    gradients the gate_up weight gradient is written to, one fused ``[G, 2I, K]`` tensor or the
    pair ``(gate [G, I, K], up [G, I, K])``.  ``expand_idx`` (with ``row_map``): ``x`` holds
    deduplicated rows and routed row i is ``x[expand_idx[i]]``; the result has one row per routed
    row, and the backward sums the gradients of the rows that share a source row."""
    _lib.require_cuda(x)
    gu_fp8, gu_scale, gu_t_fp8, gu_t_scale = q_gate_up
    dn_fp8, dn_scale, dn_t_fp8, dn_t_scale = q_down
    two_i = gu_fp8.shape[1]
    H = w_down.shape[1]
    out_m = x.shape[0]
    if row_map is not None:
        M = row_map.shape[0]
        in_map = row_map
        if expand_idx is not None:
            in_map = compose_row_maps(row_map, expand_idx, x.shape[0])
            out_m = expand_idx.shape[0]
        x_fp8, x_s, x_ch_t, x_ch_s = fp8cast_rowwise_colwise_t_rows(x, in_map, grouped_mm_offs)
    else:
        assert expand_idx is None, "expand_idx needs the row map of the scatter"
        M = x.shape[0]
        x_fp8, x_s, x_ch_t, x_ch_s = fp8cast_rowwise_colwise_t(x)
    gate_up = torch.empty((M, two_i), device=x.device, dtype=x.dtype)
    m_grouped_fp8_gemm_nt((x_fp8, x_s), (gu_fp8, gu_scale), gate_up, grouped_mm_offs)
    del x_fp8, x_s
    h_fp8, h_s, h_ch_t, h_ch_s = silu_mul_quant(gate_up, grouped_mm_offs if row_map is not None else None)
    out = torch.empty((out_m, H), device=x.device, dtype=x.dtype)
    m_grouped_fp8_gemm_nt((h_fp8, h_s), (dn_fp8, dn_scale), out, grouped_mm_offs, row_map)
    gu_dg, gu_dg_s, ctx.gu_forward_layout = dgrad_operand(q_gate_up, gate_up_weights, M)
    dn_dg, dn_dg_s, ctx.dn_forward_layout = dgrad_operand(q_down, w_down, M)
    ctx.save_for_backward(gu_dg, gu_dg_s, dn_dg, dn_dg_s, grouped_mm_offs, x_ch_t, x_ch_s,
                          gate_up, h_ch_t, h_ch_s, row_map, expand_idx)
    ctx.gate_up_weights, ctx.w_down = gate_up_weights, w_down
    ctx.rows = (M, out_m, x.shape[0])
    return out


def _backward(ctx, grad_out):
    """Shared backward: returns the gradient of ``x``; the weight gradients go to ``.grad`` (or to
    the ``WeightGradStore`` queue) through :func:`schedule_wgrad`."""
    (gu_dg, gu_dg_s, dn_dg, dn_dg_s, offs, x_ch_t, x_ch_s, gate_up, h_ch_t, h_ch_s,
     row_map, expand_idx) = ctx.saved_tensors  # fmt: skip
    M, rows_x, rows_src = ctx.rows
    half = gate_up.shape[1] // 2
    K = gu_dg.shape[2] if ctx.gu_forward_layout else gu_dg.shape[1]
    grad_out = grad_out.contiguous()
    if row_map is not None:
        dy_fp8, dy_s, dy_ch_t, dy_ch_s = fp8cast_rowwise_colwise_t_rows(grad_out, row_map, offs)
    else:
        dy_fp8, dy_s, dy_ch_t, dy_ch_s = fp8cast_rowwise_colwise_t(grad_out)
    grad_h = torch.empty((M, half), device=grad_out.device, dtype=grad_out.dtype)
    m_grouped_fp8_dgrad((dy_fp8, dy_s), dn_dg, dn_dg_s, ctx.dn_forward_layout, grad_h, offs)
    schedule_wgrad(ctx.w_down, (dy_ch_t, dy_ch_s), (h_ch_t, h_ch_s), offs)
    del dy_fp8, dy_s
    dgu_fp8, dgu_s, dgu_ch_t, dgu_ch_s = silu_mul_bwd_quant(grad_h, gate_up, offs if row_map is not None else None)
    grad_x = torch.empty((rows_x, K), device=grad_out.device, dtype=grad_out.dtype)
    m_grouped_fp8_dgrad((dgu_fp8, dgu_s), gu_dg, gu_dg_s, ctx.gu_forward_layout, grad_x, offs, row_map)
    if expand_idx is not None:
        # one gradient row per routed row so far: rows that expand the same source row are summed
        # (the backward of the expanding gather, token_scatter.py:311-325)
        grad_x = _PaddedIndexGather.scatter_sum(grad_x, expand_idx, rows_src, _GEMM_ALLOC_ALIGNMENT)
    if isinstance(ctx.gate_up_weights, tuple):
        # separate gate and up parameters: each gets the weight-gradient GEMM of its half of the
        # colwise twin (rows of the transposed bytes, columns of the scale array)
        w_gate, w_up = ctx.gate_up_weights
        schedule_wgrad(w_gate, (dgu_ch_t[:half], dgu_ch_s[:, :half]), (x_ch_t, x_ch_s), offs)
        schedule_wgrad(w_up, (dgu_ch_t[half:], dgu_ch_s[:, half:]), (x_ch_t, x_ch_s), offs)
    else:
        schedule_wgrad(ctx.gate_up_weights, (dgu_ch_t, dgu_ch_s), (x_ch_t, x_ch_s), offs)
    return grad_x


class FP8SwiGLUExpertsFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w_gate_up, w_down, grouped_mm_offs, ks, ks_tensor, q_gate_up, q_down, row_map=None, expand_idx=None):
        """``x`` is ``[M, K]`` grouped rows, or with ``row_map`` (int32 ``[M]``) the un-permuted
        ``[m, K]`` tokens; the result has the same row layout as ``x``.  ``row_map`` may be longer
        than the grouped rows (its tail negative): every kernel takes the real row count from
        ``grouped_mm_offs`` on the device, so no host-side size is needed (``ks`` may be None)."""
        return _forward(ctx, x, w_gate_up, w_down, grouped_mm_offs, q_gate_up, q_down, row_map, expand_idx)

    @staticmethod
    def backward(ctx, grad_out):
        return _backward(ctx, grad_out), None, None, None, None, None, None, None, None, None


class FP8SwiGLUSplitExpertsFunc(torch.autograd.Function):
    """The same node for experts that keep gate and up as separate parameters
    (``Qwen3MoeExperts`` / ``DeepSeekV2Experts``, models/qwen3_moe.py:45-65): ``q_gate_up`` is the
    two weights quantised into one fused operand (:func:`fp8cast_blockwise_transpose_batched_cat`),
    so the tokens are quantised once and one GEMM each way serves both projections; the weight
    gradients are written to the two parameters separately."""

    @staticmethod
    def forward(ctx, x, w_gate, w_up, w_down, grouped_mm_offs, q_gate_up, q_down, row_map=None, expand_idx=None):
        return _forward(ctx, x, (w_gate, w_up), w_down, grouped_mm_offs, q_gate_up, q_down, row_map, expand_idx)

    @staticmethod
    def backward(ctx, grad_out):
        return _backward(ctx, grad_out), None, None, None, None, None, None, None, None


def supported_split(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> bool:
    """As :func:`supported`, and the halves must be whole 128-row blocks of the fused operand."""
    half = w_gate.shape[1]
    return (x.dtype == torch.bfloat16 and w_gate.shape == w_up.shape and half % 128 == 0
            and w_down.shape[1] % 8 == 0 and w_down.shape[2] == half)


class FP8ClampedSwiGLUExpertsFunc(torch.autograd.Function):
    """The GPT-OSS expert block (models/gpt_oss.py:139-157: gate_up projection + bias, clamped
    SwiGLU on interleaved pairs, down projection + bias) as one node.  Outputs, input gradient,
    weight gradients and the down bias gradient have the bits of the composition of
    ``FP8GroupedLinearFunc`` (biases in the GEMM stores) and ``clamped_swiglu``; the activation
    and its gradient are never written as bf16 tensors, and the gate_up bias gradient is summed
    from per-tile column sums that the backward's quantisation produces (fp32, another order of
    additions than the segmented sum over the materialised gradient: same value up to fp32
    rounding before the cast to the bias dtype).

    ``row_map`` (int32 ``[M]``, from the scatter): ``x`` is the un-permuted ``[m, K]`` token tensor;
    with ``scatter_output`` the result comes back un-permuted as well."""

    @staticmethod
    def forward(ctx, x, w_gate_up, b_gate_up, w_down, b_down, grouped_mm_offs, q_gate_up, q_down, alpha, limit,
                row_map=None, scatter_output=False):
        _lib.require_cuda(x)
        gu_fp8, gu_scale, gu_t_fp8, gu_t_scale = q_gate_up
        dn_fp8, dn_scale, dn_t_fp8, dn_t_scale = q_down
        two_i = gu_fp8.shape[1]
        H = w_down.shape[1]
        assert not scatter_output or row_map is not None, "scatter_output needs the row map"
        if row_map is not None:
            M = row_map.shape[0]
            # row_map may be sized for more rows than the routing produced (its tail negative):
            # every kernel below takes the real row count from grouped_mm_offs on the device
            x_fp8, x_s, x_ch_t, x_ch_s = fp8cast_rowwise_colwise_t_rows(x, row_map, grouped_mm_offs)
        else:
            M = x.shape[0]
            x_fp8, x_s, x_ch_t, x_ch_s = fp8cast_rowwise_colwise_t(x)
        limit_rows = grouped_mm_offs if row_map is not None else None
        gate_up = torch.empty((M, two_i), device=x.device, dtype=x.dtype)
        m_grouped_fp8_gemm_nt((x_fp8, x_s), (gu_fp8, gu_scale), gate_up, grouped_mm_offs, None,
                              b_gate_up.detach().contiguous())
        del x_fp8, x_s
        h_fp8, h_s, h_ch_t, h_ch_s = clamped_swiglu_quant(gate_up, alpha, limit, limit_rows)
        out_rows = row_map if scatter_output else None
        out = torch.empty((x.shape[0] if scatter_output else M, H), device=x.device, dtype=x.dtype)
        m_grouped_fp8_gemm_nt((h_fp8, h_s), (dn_fp8, dn_scale), out, grouped_mm_offs, out_rows,
                              b_down.detach().contiguous())
        gu_dg, gu_dg_s, ctx.gu_forward_layout = dgrad_operand(q_gate_up, w_gate_up, M)
        dn_dg, dn_dg_s, ctx.dn_forward_layout = dgrad_operand(q_down, w_down, M)
        ctx.save_for_backward(gu_dg, gu_dg_s, dn_dg, dn_dg_s, grouped_mm_offs, x_ch_t, x_ch_s,
                              gate_up, h_ch_t, h_ch_s, row_map)
        ctx.weights = (w_gate_up, w_down)
        ctx.consts = (float(alpha), float(limit), bool(scatter_output), M, x.shape[0], b_gate_up.dtype, b_down.dtype)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        from .indexed_bias_add import _segment_sum_along_rows

        (gu_dg, gu_dg_s, dn_dg, dn_dg_s, offs, x_ch_t, x_ch_s, gate_up, h_ch_t, h_ch_s,
         row_map) = ctx.saved_tensors  # fmt: skip
        w_gate_up, w_down = ctx.weights
        alpha, limit, scatter_output, M, rows_x, gu_bias_dtype, dn_bias_dtype = ctx.consts
        half = gate_up.shape[1] // 2
        K = gu_dg.shape[2] if ctx.gu_forward_layout else gu_dg.shape[1]
        grad_out = grad_out.contiguous()
        out_rows = row_map if scatter_output else None
        if out_rows is not None:
            dy_fp8, dy_s, dy_ch_t, dy_ch_s = fp8cast_rowwise_colwise_t_rows(grad_out, out_rows, offs)
        else:
            dy_fp8, dy_s, dy_ch_t, dy_ch_s = fp8cast_rowwise_colwise_t(grad_out)
        grad_b_down = _segment_sum_along_rows(grad_out, offs, dn_bias_dtype, out_rows)
        grad_h = torch.empty((M, half), device=grad_out.device, dtype=grad_out.dtype)
        m_grouped_fp8_dgrad((dy_fp8, dy_s), dn_dg, dn_dg_s, ctx.dn_forward_layout, grad_h, offs)
        schedule_wgrad(w_down, (dy_ch_t, dy_ch_s), (h_ch_t, h_ch_s), offs)
        del dy_fp8, dy_s
        dgu_fp8, dgu_s, dgu_ch_t, dgu_ch_s, col_sum = clamped_swiglu_bwd_quant(
            grad_h, gate_up, alpha, limit, offs if row_map is not None else None)
        # groups are whole 128-row tiles: their ends in tiles index the per-tile column sums
        grad_b_gate_up = _segment_sum_along_rows(col_sum, offs // 128, gu_bias_dtype)
        grad_x = torch.empty((rows_x if row_map is not None else M, K), device=grad_out.device, dtype=grad_out.dtype)
        m_grouped_fp8_dgrad((dgu_fp8, dgu_s), gu_dg, gu_dg_s, ctx.gu_forward_layout, grad_x, offs, row_map)
        schedule_wgrad(w_gate_up, (dgu_ch_t, dgu_ch_s), (x_ch_t, x_ch_s), offs)
        return grad_x, None, grad_b_gate_up, None, grad_b_down, None, None, None, None, None, None, None
