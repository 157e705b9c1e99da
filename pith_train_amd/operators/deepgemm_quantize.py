"""Blockwise FP8 quantisation (e4m3fn, power-of-two fp32 scales) on gfx950.

Drop-in for ``pithtrain/operators/deepgemm_quantize.py``: same six entry points, same return
tuples, layouts and dtypes (``:16-23``).  ``fp8cast_rowwise_colwise_t`` is this package's own
variant that stores the colwise twin transposed, which is the operand layout of the wgrad GEMM
here.
"""

from __future__ import annotations

import torch

from .. import _lib

__all__ = [
    "fp8cast_rowwise_colwise",
    "fp8cast_rowwise_kmajor",
    "fp8cast_rowwise_transpose",
    "fp8cast_rowwise_blockwise_transpose",
    "fp8cast_blockwise_transpose",
    "fp8cast_blockwise_transpose_batched",
    "fp8cast_blockwise_batched",
    "fp8cast_grouped_weight",
    "fp8cast_grouped_weight_cat",
    "fp8cast_rowwise_colwise_t",
    "fp8cast_rowwise_colwise_t_rows",
]

FP8 = torch.float8_e4m3fn


def _prep2d(x: torch.Tensor) -> torch.Tensor:
    _lib.require_cuda(x)
    if x.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise TypeError(f"fp8cast: expected bfloat16, float16 or float32 input, got {x.dtype}")
    if x.shape[-1] > 0 and x.stride(-1) != 1:
        x = x.contiguous()
    return x


def _cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def transposed_pitch(m: int) -> int:
    """Row pitch (bytes) of a transposed FP8 operand ``[N, m]`` of a dense linear.  The weight
    gradient reads these operands along rows, 128 bytes of every row per step; with a pitch that
    is a multiple of 256 the rows of a step fall onto few memory channels (measured: 25 % slower
    at 5 * 2**14 than at 579 * 128), so such pitches get one more 128-byte column."""
    return m + 128 if (m >= 2048 and m % 256 == 0) else m


def _empty_transposed(rows: int, m: int, dev, padded: bool) -> torch.Tensor:
    """``[rows, m]`` FP8, packed, or (``padded``) with the row pitch of :func:`transposed_pitch`
    (then a view of a wider buffer when that pitch differs from ``m``)."""
    ld = transposed_pitch(m) if padded else m
    buf = torch.empty((rows, ld), dtype=FP8, device=dev)
    return buf if ld == m else buf[:, :m]


def _rowwise_colwise(x: torch.Tensor, layout: int, offs: torch.Tensor | None):
    assert x.ndim == 2 and x.shape[0] % 128 == 0, (
        f"Expected 2D tensor with M%128==0, got shape {tuple(x.shape)}"
    )
    x = _prep2d(x)
    M, N = x.shape
    dev = x.device
    out_tok = torch.empty((M, N), dtype=FP8, device=dev)
    scale_tok = torch.empty((M, _cdiv(N, 128)), dtype=torch.float32, device=dev)
    if layout == _lib.PT_CH_ROWMAJOR:
        out_ch = torch.empty((M, N), dtype=FP8, device=dev)
        scale_ch = torch.empty((M // 128, N), dtype=torch.float32, device=dev)
    elif layout == _lib.PT_CH_TRANSPOSED:
        out_ch = torch.empty((N, M), dtype=FP8, device=dev)
        scale_ch = torch.empty((M // 128, N), dtype=torch.float32, device=dev)
    else:
        out_ch = torch.empty(M * N, dtype=FP8, device=dev)
        scale_ch = torch.empty((N, M // 128), dtype=torch.float32, device=dev)
    if M == 0 or N == 0:
        return out_tok, scale_tok, out_ch, scale_ch
    ld = x.stride(0) if M > 1 else N
    _lib.call(
        "pt_quant_rowwise_colwise", x.data_ptr(), _lib.dtype_code(x.dtype), M, N, ld,
        out_tok.data_ptr(), scale_tok.data_ptr(), out_ch.data_ptr(), scale_ch.data_ptr(), layout,
        _lib.ptr(offs), 0 if offs is None else offs.shape[0], _lib.stream_ptr(dev),
    )  # fmt: skip
    return out_tok, scale_tok, out_ch, scale_ch


def fp8cast_rowwise_colwise(x: torch.Tensor):
    """(tok_fp8[M,N], tok_scale[M,ceil(N/128)], ch_fp8[M,N], ch_scale[M//128,N]); M % 128 == 0."""
    return _rowwise_colwise(x, _lib.PT_CH_ROWMAJOR, None)


def fp8cast_rowwise_colwise_t_rows(x: torch.Tensor, row_index: torch.Tensor, grouped_mm_offs: torch.Tensor | None = None):
    """:func:`fp8cast_rowwise_colwise_t` of ``x[row_index]`` (rows with a negative index are zero)
    without materialising the gathered tensor.  ``row_index`` is int32 ``[M]``, ``M % 128 == 0``.
    With ``grouped_mm_offs`` (int32, inclusive) only the rows below its last entry are written:
    ``M`` may then be an upper bound of the row count that is only known on the device."""
    assert x.ndim == 2 and row_index.ndim == 1 and row_index.dtype == torch.int32
    assert row_index.shape[0] % 128 == 0, f"row count {row_index.shape[0]} must be a multiple of 128"
    x = _prep2d(x)
    _lib.require_cuda(row_index)
    row_index = row_index.contiguous()
    M, N = row_index.shape[0], x.shape[1]
    dev = x.device
    out_tok = torch.empty((M, N), dtype=FP8, device=dev)
    scale_tok = torch.empty((M, _cdiv(N, 128)), dtype=torch.float32, device=dev)
    out_ch = torch.empty((N, M), dtype=FP8, device=dev)
    scale_ch = torch.empty((M // 128, N), dtype=torch.float32, device=dev)
    if M and N:
        ld = x.stride(0) if x.shape[0] > 1 else N
        _lib.call(
            "pt_quant_rowwise_colwise_rows", x.data_ptr(), _lib.dtype_code(x.dtype), M, N, ld,
            row_index.data_ptr(), out_tok.data_ptr(), scale_tok.data_ptr(), out_ch.data_ptr(),
            scale_ch.data_ptr(), _lib.PT_CH_TRANSPOSED, _lib.ptr(grouped_mm_offs),
            0 if grouped_mm_offs is None else grouped_mm_offs.numel(), _lib.stream_ptr(dev),
        )  # fmt: skip
    return out_tok, scale_tok, out_ch, scale_ch


def fp8cast_rowwise_colwise_t(x: torch.Tensor):
    """As :func:`fp8cast_rowwise_colwise` with the colwise bytes stored transposed: ch_t_fp8[N,M]
    (``ch_t_fp8 == ch_fp8.T`` byte for byte), ch_scale[M//128,N] unchanged."""
    return _rowwise_colwise(x, _lib.PT_CH_TRANSPOSED, None)


def fp8cast_rowwise_kmajor(x: torch.Tensor, grouped_mm_offs: torch.Tensor):
    """Rowwise outputs as above; colwise bytes per group as (N, K_g) blocks in a flat 1-D buffer,
    colwise scales transposed to (N, M//128)."""
    assert grouped_mm_offs.dtype == torch.int32 and grouped_mm_offs.ndim == 1
    return _rowwise_colwise(x, _lib.PT_CH_KMAJOR, grouped_mm_offs.contiguous())


def fp8cast_rowwise_transpose(x: torch.Tensor, *, _padded: bool = False):
    """(tok_fp8[M,N], tok_scale[M,ceil(N/128)], t_fp8[N,M], t_scale[N,ceil(M/128)]), all freshly
    allocated and contiguous.  ``_padded`` is for this package's dense linear only: ``t_fp8`` may
    then be a row-padded view (see :func:`transposed_pitch`)."""
    assert x.ndim == 2, f"Expected 2D tensor, got {x.ndim}D"
    x = _prep2d(x)
    M, N = x.shape
    dev = x.device
    out_tok = torch.empty((M, N), dtype=FP8, device=dev)
    scale_tok = torch.empty((M, _cdiv(N, 128)), dtype=torch.float32, device=dev)
    out_t = _empty_transposed(N, M, dev, _padded)
    scale_t = torch.empty((N, _cdiv(M, 128)), dtype=torch.float32, device=dev)
    if M and N:
        _lib.call(
            "pt_quant_rowwise_transpose_ld", x.data_ptr(), _lib.dtype_code(x.dtype), M, N,
            x.stride(0) if M > 1 else N, out_tok.data_ptr(), scale_tok.data_ptr(), out_t.data_ptr(),
            out_t.stride(0) if N > 1 else M, scale_t.data_ptr(), _lib.stream_ptr(dev),
        )  # fmt: skip
    return out_tok, scale_tok, out_t, scale_t


def fp8cast_rowwise_blockwise_transpose(x: torch.Tensor, *, _padded: bool = False):
    """(tok_fp8[M,K], tok_scale[M,ceil(K/128)], blk_t_fp8[K,M], blk_t_scale[ceil(K/128),ceil(M/128)]),
    all freshly allocated and contiguous; ``_padded`` as in :func:`fp8cast_rowwise_transpose`."""
    assert x.ndim == 2, f"Expected 2D tensor, got {x.ndim}D"
    x = _prep2d(x)
    M, K = x.shape
    dev = x.device
    out_tok = torch.empty((M, K), dtype=FP8, device=dev)
    scale_tok = torch.empty((M, _cdiv(K, 128)), dtype=torch.float32, device=dev)
    out_blk_t = _empty_transposed(K, M, dev, _padded)
    scale_blk_t = torch.empty((_cdiv(K, 128), _cdiv(M, 128)), dtype=torch.float32, device=dev)
    if M and K:
        _lib.call(
            "pt_quant_rowwise_blockwise_transpose_ld", x.data_ptr(), _lib.dtype_code(x.dtype), M, K,
            x.stride(0) if M > 1 else K, out_tok.data_ptr(), scale_tok.data_ptr(),
            out_blk_t.data_ptr(), out_blk_t.stride(0) if K > 1 else M, scale_blk_t.data_ptr(),
            _lib.stream_ptr(dev),
        )  # fmt: skip
    return out_tok, scale_tok, out_blk_t, scale_blk_t


def _blockwise_batched(x3: torch.Tensor, twin: bool = True):
    G, N, K = x3.shape
    dev = x3.device
    out = torch.empty((G, N, K), dtype=FP8, device=dev)
    scale = torch.empty((G, _cdiv(N, 128), _cdiv(K, 128)), dtype=torch.float32, device=dev)
    out_t = torch.empty((G, K, N), dtype=FP8, device=dev) if twin else None
    scale_t = torch.empty((G, _cdiv(K, 128), _cdiv(N, 128)), dtype=torch.float32, device=dev) if twin else None
    if G and N and K:
        _lib.call(
            "pt_quant_blockwise_transpose_batched", x3.data_ptr(), _lib.dtype_code(x3.dtype), G, N, K,
            x3.stride(0) if G > 1 else N * K, x3.stride(1) if N > 1 else K, out.data_ptr(),
            scale.data_ptr(), out_t.data_ptr() if twin else 0, scale_t.data_ptr() if twin else 0, _lib.stream_ptr(dev),
        )  # fmt: skip
    return out, scale, out_t, scale_t


def fp8cast_blockwise_transpose_batched_cat(parts, twin: bool = True):
    """:func:`fp8cast_blockwise_transpose_batched` of ``torch.cat(parts, dim=1)`` without the
    concatenation: each ``[G, N_i, K]`` part is quantised straight into its rows of the fused
    outputs (and its columns of the transposed twin).  ``N_i % 128 == 0`` so that the 128x128
    blocks of the fused tensor are blocks of the parts; separate gate and up weights become one
    fused projection operand this way.  ``twin=False``: see :func:`fp8cast_blockwise_batched`."""
    G, _, K = parts[0].shape
    dev = parts[0].device
    assert all(p_.ndim == 3 and p_.shape[0] == G and p_.shape[2] == K and p_.shape[1] % 128 == 0 for p_ in parts)
    N = sum(p_.shape[1] for p_ in parts)
    nb, kb = N // 128, _cdiv(K, 128)
    out = torch.empty((G, N, K), dtype=FP8, device=dev)
    scale = torch.empty((G, nb, kb), dtype=torch.float32, device=dev)
    out_t = torch.empty((G, K, N), dtype=FP8, device=dev) if twin else None
    scale_t = torch.empty((G, kb, nb), dtype=torch.float32, device=dev) if twin else None
    row = 0
    for part in parts:
        x3 = _prep2d(part.detach())
        n = x3.shape[1]
        if G and n and K:
            _lib.call(
                "pt_quant_blockwise_transpose_batched_into", x3.data_ptr(), _lib.dtype_code(x3.dtype), G, n, K,
                x3.stride(0) if G > 1 else n * K, x3.stride(1) if n > 1 else K,
                out.data_ptr() + row * K, N * K, scale.data_ptr() + 4 * (row // 128) * kb, nb * kb,
                out_t.data_ptr() + row if twin else 0, N, K * N, scale_t.data_ptr() + 4 * (row // 128) if twin else 0, nb, kb * nb,
                _lib.stream_ptr(dev),
            )  # fmt: skip
        row += n
    return out, scale, out_t, scale_t


def fp8cast_blockwise_transpose(x: torch.Tensor):
    """(fp8[M,K], scale[ceil(M/128),ceil(K/128)], fp8_t[K,M], scale_t[ceil(K/128),ceil(M/128)])."""
    assert x.ndim == 2, f"Expected 2D tensor, got {x.ndim}D"
    x = _prep2d(x.detach())
    out, scale, out_t, scale_t = _blockwise_batched(x.unsqueeze(0))
    return out[0], scale[0], out_t[0], scale_t[0]


def fp8cast_blockwise_transpose_batched(x: torch.Tensor):
    """(fp8[G,N,K], scale[G,ceil(N/128),ceil(K/128)], fp8_t[G,K,N], scale_t[G,ceil(K/128),ceil(N/128)])."""
    assert x.ndim == 3, f"Expected 3D tensor, got {x.ndim}D"
    return _blockwise_batched(_prep2d(x.detach()))


def fp8cast_blockwise_batched(x: torch.Tensor):
    """(fp8[G,N,K], scale[G,ceil(N/128),ceil(K/128)], None, None): the first half of
    :func:`fp8cast_blockwise_transpose_batched`, in the same four-slot tuple.  The transposed twin
    of a 128x128-blockwise quantisation holds the same bytes and the transposed scale grid; the
    grouped input-gradient GEMM reads the forward layout directly (``m_grouped_fp8_gemm_nn``), so
    the grouped-expert weights are quantised without it: a quarter less traffic in this kernel and
    half the FP8 weight cache."""
    assert x.ndim == 3, f"Expected 3D tensor, got {x.ndim}D"
    return _blockwise_batched(_prep2d(x.detach()), twin=False)


def weight_twin_enabled() -> bool:
    """``PITHTRAIN_FP8_WEIGHT_TWIN=1`` keeps the transposed FP8 copy of the grouped-expert weights
    (the reference's data flow: the input-gradient GEMM then runs in the NT form on it)."""
    import os

    return os.environ.get("PITHTRAIN_FP8_WEIGHT_TWIN", "0") == "1"


def fp8cast_grouped_weight(x: torch.Tensor):
    """The quantised operand tuple of a grouped-expert weight ``[G, N, K]`` as the grouped linears
    and fused expert nodes take it: with or without the transposed twin (``weight_twin_enabled``)."""
    return fp8cast_blockwise_transpose_batched(x) if weight_twin_enabled() else fp8cast_blockwise_batched(x)


def fp8cast_grouped_weight_cat(parts):
    """:func:`fp8cast_grouped_weight` of ``torch.cat(parts, dim=1)`` without the concatenation."""
    return fp8cast_blockwise_transpose_batched_cat(parts, twin=weight_twin_enabled())
