"""Oracle: FP8 GEMMs on dequantised operands.

Test infrastructure only (see ``oracle/__init__.py``).

The reference's GEMM arithmetic is in the third-party DeepGEMM package
(``pyproject.toml:6,28`` - git ``main``, no pinned commit); what the reference
itself fixes is the operand convention at its call sites:

  * dense NT           ``linear.py:26-41``   out[m,n] = a[m,:] . b[n,:]
                        a: 1x128 scales [m, ceil(k/128)], b: 128x128 scales
  * m-grouped NT       ``grouped_linear.py:88-101,146-154,192-200``
                        rows [offs[g-1], offs[g]) use b[g]
  * k-grouped wgrad    ``grouped_linear.py:202-221``
                        d[g] = c[g] + dY_g^T X_g, both operands colwise-scaled

The oracle is the mathematical definition with products of dequantised values
accumulated in float64 (``accum=torch.float64``) or float32, rounded once to
the output dtype.  It is **pinned to tolerance only** against the reference
(no bit-level vectors exist for DeepGEMM's accumulation order).
"""

from __future__ import annotations

import torch

from . import fp8 as _q


def gemm_nt_dense(a_fp8, a_scale, b_fp8, b_scale, out_dtype=torch.bfloat16, accum=torch.float64):
    """out[m,n] = sum_k a[m,k] b[n,k]; a rowwise-scaled, b blockwise-scaled. (linear.py:26-41)"""
    a = _q.dequant_rowwise(a_fp8, a_scale, accum)
    b = _q.dequant_blockwise(b_fp8, b_scale, accum)
    return (a @ b.T).to(out_dtype)


def _group_bounds(offs: torch.Tensor):
    start = 0
    for g, end in enumerate(offs.tolist()):
        yield g, start, int(end)
        start = int(end)


def gemm_m_grouped_nt(
    a_fp8, a_scale, b_fp8, b_scale, offs, out_dtype=torch.bfloat16, accum=torch.float64
):
    """d[rows_g] = a[rows_g] @ b[g].T; rows past offs[-1] are left zero.
    (grouped_linear.py:88-101)"""
    M = a_fp8.shape[0]
    N = b_fp8.shape[1]
    a = _q.dequant_rowwise(a_fp8, a_scale, accum)
    out = torch.zeros((M, N), dtype=accum)
    for g, s, e in _group_bounds(offs):
        if e > s:
            bg = _q.dequant_blockwise(b_fp8[g], b_scale[g], accum)
            out[s:e] = a[s:e] @ bg.T
    return out.to(out_dtype)


def gemm_k_grouped_wgrad(
    dy_ch_fp8, dy_ch_scale, x_ch_fp8, x_ch_scale, offs, num_groups, accum=torch.float64
):
    """dW[g][n,k] = sum_{m in g} dY[m,n] X[m,k]; colwise-quantised operands with one scale
    per (128-row chunk, column).  Returns float32 [G, N, K]. (grouped_linear.py:202-216)"""
    dy = _q.dequant_colwise(dy_ch_fp8, dy_ch_scale, accum)
    x = _q.dequant_colwise(x_ch_fp8, x_ch_scale, accum)
    N, K = dy.shape[1], x.shape[1]
    out = torch.zeros((num_groups, N, K), dtype=accum)
    for g, s, e in _group_bounds(offs):
        if e > s:
            out[g] = dy[s:e].T @ x[s:e]
    return out.to(torch.float32)


def wgrad_to_param_grad(wgrad_f32: torch.Tensor, existing_grad: torch.Tensor | None):
    """fp32 wgrad -> bf16, assign or accumulate in bf16. (grouped_linear.py:217-221)"""
    w = wgrad_f32.to(torch.bfloat16)
    if existing_grad is None:
        return w
    return existing_grad + w


# ---------------------------------------------------------------------------
# whole linear layers (quantise + GEMM), forward and backward
# ---------------------------------------------------------------------------
def fp8_linear_forward(x2d: torch.Tensor, weight: torch.Tensor, accum=torch.float64):
    """y = x W^T for the dense FP8 linear; returns (y, saved-for-backward). (linear.py:44-60)"""
    w_fp8, w_s, w_t_fp8, w_t_s = _q.fp8cast_blockwise_transpose(weight)
    x_fp8, x_s, x_t_fp8, x_t_s = _q.fp8cast_rowwise_blockwise_transpose(x2d)
    y = gemm_nt_dense(x_fp8, x_s, w_fp8, w_s, x2d.dtype, accum)
    return y, (w_t_fp8, w_t_s, x_t_fp8, x_t_s)


def fp8_linear_backward(grad2d: torch.Tensor, saved, accum=torch.float64):
    """(grad_input, weight_grad) for the dense FP8 linear. (linear.py:63-83)"""
    w_t_fp8, w_t_s, x_t_fp8, x_t_s = saved
    g_fp8, g_s, g_t_fp8, g_t_s = _q.fp8cast_rowwise_transpose(grad2d)
    grad_input = gemm_nt_dense(g_fp8, g_s, w_t_fp8, w_t_s, grad2d.dtype, accum)
    weight_grad = gemm_nt_dense(g_t_fp8, g_t_s, x_t_fp8, x_t_s, grad2d.dtype, accum)
    return grad_input, weight_grad


def fp8_grouped_linear_forward(x, weight, offs, accum=torch.float64):
    """FP8GroupedLinearFunc.forward. (grouped_linear.py:114-167)"""
    w_fp8, w_s, w_t_fp8, w_t_s = _q.fp8cast_blockwise_transpose_batched(weight)
    x_fp8, x_s, x_ch, x_ch_s = _q.fp8cast_rowwise_colwise(x)
    y = gemm_m_grouped_nt(x_fp8, x_s, w_fp8, w_s, offs, x.dtype, accum)
    return y, (w_t_fp8, w_t_s, x_ch, x_ch_s)


def fp8_grouped_linear_backward(grad, saved, offs, num_groups, accum=torch.float64):
    """FP8GroupedLinearFunc.backward -> (grad_input, weight_grad bf16). (grouped_linear.py:169-236)"""
    w_t_fp8, w_t_s, x_ch, x_ch_s = saved
    g_fp8, g_s, g_ch, g_ch_s = _q.fp8cast_rowwise_colwise(grad)
    grad_input = gemm_m_grouped_nt(g_fp8, g_s, w_t_fp8, w_t_s, offs, grad.dtype, accum)
    wgrad = gemm_k_grouped_wgrad(g_ch, g_ch_s, x_ch, x_ch_s, offs, num_groups, accum)
    return grad_input, wgrad.to(torch.bfloat16)


# ---------------------------------------------------------------------------
# BF16 grouped linear (the reference's pure-PyTorch path; grouped_linear.py:18-55)
# ---------------------------------------------------------------------------
def bf16_grouped_mm(x, weight, offs):
    """F.grouped_mm(x, weight.transpose(1, 2), offs) as a per-group loop."""
    out = torch.zeros((x.shape[0], weight.shape[1]), dtype=x.dtype)
    for g, s, e in _group_bounds(offs):
        if e > s:
            out[s:e] = x[s:e] @ weight[g].T
    return out


def calc_diff(x: torch.Tensor, y: torch.Tensor) -> float:
    """1 - 2<x,y>/(|x|^2+|y|^2), the similarity metric of the reference's FP8 tests
    (tests/test_deepgemm_fp8_linear_correctness.py:22-28)."""
    x, y = x.double(), y.double()
    den = (x * x + y * y).sum()
    if den == 0:
        return 0.0
    return float(1 - 2 * (x * y).sum() / den)
