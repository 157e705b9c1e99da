"""Oracle: routing-driven token permute / unpermute.

Test infrastructure only (see ``oracle/__init__.py``).

Follows ``pithtrain/operators/token_scatter.py``:
  * ``group_offsets``            <- ``_compute_group_offsets_kernel`` (:38-71)
  * ``scatter_for_grouped_gemm`` <- ``_scatter_for_grouped_gemm_kernel`` (:74-153),
                                    ``ScatterForGroupedGemm`` (:156-284)
  * ``padded_index_gather``      <- ``_PaddedIndexGather`` (:287-336)
  * ``precompute_group_indices`` <- :370-384 (and models/gpt_oss.py:146-150)

The reference assigns slots inside a group with ``tl.atomic_add`` (:95), so its
row order inside a group varies from run to run.  The oracle fixes the
canonical order: ascending source row inside each group (stable counting
sort), which is one of the reference's legal outcomes.
"""

from __future__ import annotations

import torch

GEMM_ALLOC_ALIGNMENT = 1024  # token_scatter.py:23


def group_offsets(expert_idxs: torch.Tensor, num_groups: int, padding_alignment: int = 128):
    """(counts i64[G], ks i32[G], offs i32[G]) - bincount, pad to alignment, inclusive cumsum."""
    counts = torch.bincount(expert_idxs.to(torch.int64), minlength=num_groups)[:num_groups]
    padded = (counts + padding_alignment - 1) // padding_alignment * padding_alignment
    offs = padded.cumsum(0)
    return counts, padded.to(torch.int32), offs.to(torch.int32)


def scatter_for_grouped_gemm(
    input_tokens: torch.Tensor,
    expert_idxs: torch.Tensor,
    num_groups: int,
    padding_alignment: int = 128,
):
    """Returns (out[sum(ks),H], reverse i64[m], offs i32[G], ks list, ks_tensor i32[G],
    buffer[M_rounded,H]) - the last item is the 1024-row-aligned zero-tailed buffer that
    ``out`` is a view of (:243-251 zero pad rows, :133-153 zero tail)."""
    m, H = input_tokens.shape
    if m == 0:  # :181-187
        return (
            torch.empty((0, H), dtype=input_tokens.dtype),
            torch.empty((0,), dtype=torch.int64),
            torch.empty((0,), dtype=torch.int32),
            [],
            torch.empty((0,), dtype=torch.int32),
            torch.empty((0, H), dtype=input_tokens.dtype),
        )
    counts, ks_tensor, offs = group_offsets(expert_idxs, num_groups, padding_alignment)
    starts = offs.to(torch.int64) - ks_tensor.to(torch.int64)
    order = torch.argsort(expert_idxs.to(torch.int64), stable=True)  # sorted pos -> source row
    sorted_e = expert_idxs.to(torch.int64)[order]
    excl = counts.cumsum(0) - counts
    pos_in_group = torch.arange(m, dtype=torch.int64) - excl[sorted_e]
    dest = starts[sorted_e] + pos_in_group
    reverse = torch.empty(m, dtype=torch.int64)
    reverse[order] = dest
    actual_M = int(offs[-1])
    M_rounded = (actual_M + GEMM_ALLOC_ALIGNMENT - 1) // GEMM_ALLOC_ALIGNMENT * GEMM_ALLOC_ALIGNMENT
    buf = torch.zeros((M_rounded, H), dtype=input_tokens.dtype)
    buf[reverse] = input_tokens
    return buf[:actual_M], reverse, offs, ks_tensor.tolist(), ks_tensor, buf


def scatter_backward(grad_out: torch.Tensor, reverse: torch.Tensor) -> torch.Tensor:
    """grad_in[i] = grad_out[reverse[i]]. (:271-284)"""
    return grad_out[reverse]


def padded_index_gather(input: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
    """input[index]. (:297-309)"""
    return input.index_select(0, index)


def padded_index_gather_backward(
    grad_out: torch.Tensor, index: torch.Tensor, rows: int, accum=torch.float32
) -> torch.Tensor:
    """grad_in[r] = sum_{j: index[j]==r} grad_out[j].  The reference sums duplicates with
    ``scatter_add_`` in the gradient dtype (:311-325), whose order is not deterministic on a
    GPU; the oracle accumulates in ``accum`` and rounds once."""
    buf = torch.zeros((rows,) + tuple(grad_out.shape[1:]), dtype=accum)
    buf.index_add_(0, index, grad_out.to(accum))
    return buf.to(grad_out.dtype)


def precompute_group_indices(grouped_mm_offs: torch.Tensor, M: int) -> torch.Tensor:
    """searchsorted(offs, arange(M), right=True).clamp(max=G-1) as int32. (:379-383)"""
    rows = torch.arange(M, dtype=torch.int64)
    gi = torch.searchsorted(grouped_mm_offs.to(torch.int64), rows, right=True)
    return gi.clamp_(max=grouped_mm_offs.shape[0] - 1).to(torch.int32)
