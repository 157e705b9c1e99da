"""Routing-driven token permute / unpermute on gfx950.

Drop-in for ``pithtrain/operators/token_scatter.py``: ``scatter_for_grouped_gemm`` (:339-367),
``padded_index_gather`` (:328-336), ``precompute_group_indices`` (:370-384),
``get_pinned_buffer`` (:26-35).

Row order inside a group is the ascending source row (the reference's atomics leave it
unspecified), so every output is reproducible bit for bit.
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import _lib

_pinned_buffers: dict[tuple[str, torch.dtype, int], torch.Tensor] = {}
_GEMM_ALLOC_ALIGNMENT = 1024


def get_pinned_buffer(name: str, numel: int, dtype: torch.dtype) -> torch.Tensor:
    """Process-wide cache of pinned host buffers for small device-to-host read-backs."""
    key = (name, dtype, numel)
    buf = _pinned_buffers.get(key)
    if buf is None:
        buf = torch.empty(numel, dtype=dtype, device="cpu", pin_memory=True)
        _pinned_buffers[key] = buf
    return buf


def _workspace(nbytes: int, device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def group_rows(expert_idxs: torch.Tensor, num_groups: int, padding_alignment: int, cap: int):
    """Index half of the scatter: (reverse i64[m], offs i32[G], ks i32[G], src_of i32[cap])."""
    m = expert_idxs.shape[0]
    dev = expert_idxs.device
    reverse = torch.empty((m,), device=dev, dtype=torch.int64)
    offs = torch.empty((num_groups,), device=dev, dtype=torch.int32)
    ks_tensor = torch.empty((num_groups,), device=dev, dtype=torch.int32)
    src_of = torch.empty((cap,), device=dev, dtype=torch.int32)
    ws_bytes = _lib.query("pt_group_rows_workspace_bytes", m, num_groups)
    ws = _workspace(ws_bytes, dev)
    _lib.call(
        "pt_group_rows", expert_idxs.data_ptr(), m, num_groups, padding_alignment, offs.data_ptr(),
        ks_tensor.data_ptr(), reverse.data_ptr(), src_of.data_ptr(), cap, ws.data_ptr(), ws.numel(),
        _lib.stream_ptr(dev),
    )  # fmt: skip
    return reverse, offs, ks_tensor, src_of


def group_rows_with_sizes(expert_idxs: torch.Tensor, num_groups: int, padding_alignment: int = 128, device=None,
                          host_sizes: bool = True):
    """The index half of :func:`scatter_for_grouped_gemm` on its own: returns ``(reverse i64[m],
    grouped_mm_offs i32[G], ks list[int], ks_tensor i32[G], src_of i32[sum(ks)])`` where
    ``src_of[r]`` is the source row of grouped row r (-1 for a padding row).  No rows are moved.

    ``host_sizes=False`` skips the device-to-host copy of the group sizes and the stream
    synchronisation it needs: ``ks`` is None and ``src_of`` keeps its full capacity (the largest
    padded row count ``m`` rows in ``num_groups`` groups can give, -1 past the real rows).  Callers
    that size their buffers by ``src_of`` and take the real row count from ``grouped_mm_offs`` on
    the device (the fused expert path) then never wait for the GPU."""
    _lib.require_cuda(expert_idxs)
    expert_idxs = expert_idxs.contiguous()
    assert expert_idxs.dtype == torch.int64, "expert_idxs must be int64"
    m = expert_idxs.shape[0]
    dev = expert_idxs.device
    max_m_padded = m + num_groups * (padding_alignment - 1)
    if not host_sizes:
        # Capacity = the largest padded row count, as an odd multiple of 128.  The colwise twins
        # are [N, capacity] matrices read along rows at this pitch: with a large power of two in
        # it, consecutive rows fall onto a few memory channels (measured: 81920 = 5 * 2**14 makes
        # the weight-gradient GEMM 25 % slower than 74112 = 579 * 128).
        cap = -(-max_m_padded // 128) * 128
        if (cap // 128) % 2 == 0:
            cap += 128
        alloc = -(-cap // _GEMM_ALLOC_ALIGNMENT) * _GEMM_ALLOC_ALIGNMENT
        reverse, offs, ks_tensor, src_of = group_rows(expert_idxs, num_groups, padding_alignment, alloc)
        return reverse, offs, None, ks_tensor, src_of[:cap]
    max_m_padded = -(-max_m_padded // _GEMM_ALLOC_ALIGNMENT) * _GEMM_ALLOC_ALIGNMENT
    reverse, offs, ks_tensor, src_of = group_rows(expert_idxs, num_groups, padding_alignment, max_m_padded)
    ks_cpu = get_pinned_buffer("ks", num_groups, torch.int32)
    ks_cpu.copy_(ks_tensor, non_blocking=True)
    torch.cuda.current_stream(dev).synchronize()
    ks = ks_cpu.tolist()
    return reverse, offs, ks, ks_tensor, src_of[: sum(ks)]


def permute_rows(input_tokens, src_of, out, offs_last, pre_index=None):
    """out[r] = input[src_of[r]] (optionally through ``pre_index``), zero where src_of[r] < 0."""
    H = input_tokens.shape[1]
    _lib.call(
        "pt_permute_rows", input_tokens.data_ptr(), input_tokens.stride(0), out.data_ptr(),
        out.stride(0), src_of.data_ptr(), _lib.ptr(pre_index), _lib.ptr(offs_last),
        _GEMM_ALLOC_ALIGNMENT, out.shape[0], H, input_tokens.element_size(),
        _lib.stream_ptr(out.device),
    )  # fmt: skip
    return out


def gather_rows(input: torch.Tensor, index: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    n = index.shape[0]
    if n == 0 or input.shape[1] == 0:
        return out
    _lib.call(
        "pt_gather_rows", input.data_ptr(), input.stride(0), out.data_ptr(), out.stride(0),
        index.data_ptr(), n, input.shape[1], input.element_size(), _lib.stream_ptr(out.device),
    )  # fmt: skip
    return out


class ScatterForGroupedGemm(torch.autograd.Function):
    """Forward: rows grouped by expert, groups zero-padded to the alignment.  Backward: gather."""

    @staticmethod
    def forward(ctx, input_tokens, expert_idxs, num_groups, padding_alignment=128, pre_index=None):
        _lib.require_cuda(input_tokens, expert_idxs)
        m = expert_idxs.shape[0]
        hidden_size = input_tokens.shape[1]
        device = input_tokens.device
        ctx.pre_index = pre_index
        ctx.in_rows = input_tokens.shape[0]
        if m == 0:
            output_tokens = torch.empty((0, hidden_size), device=device, dtype=input_tokens.dtype)
            reverse = torch.empty((0,), device=device, dtype=torch.int64)
            offs = torch.empty((0,), device=device, dtype=torch.int32)
            ks_tensor = torch.empty((0,), device=device, dtype=torch.int32)
            ctx.save_for_backward(reverse)
            ctx.src_of = None
            return output_tokens, reverse, offs, ks_tensor, []
        if input_tokens.stride(1) != 1:
            input_tokens = input_tokens.contiguous()
        expert_idxs = expert_idxs.contiguous()
        assert expert_idxs.dtype == torch.int64, "expert_idxs must be int64"

        max_m_padded = m + num_groups * (padding_alignment - 1)
        max_m_padded = -(-max_m_padded // _GEMM_ALLOC_ALIGNMENT) * _GEMM_ALLOC_ALIGNMENT
        reverse, offs, ks_tensor, src_of = group_rows(
            expert_idxs, num_groups, padding_alignment, max_m_padded
        )
        # ks goes to the host on a side stream while the row copy runs
        ks_cpu = get_pinned_buffer("ks", num_groups, torch.int32)
        copy_stream, copy_event = _copy_stream_and_event(device)
        copy_event.record()
        output_tokens = torch.empty((max_m_padded, hidden_size), device=device, dtype=input_tokens.dtype)
        permute_rows(input_tokens, src_of, output_tokens, offs[num_groups - 1 :], pre_index)
        with torch.cuda.stream(copy_stream):
            copy_stream.wait_event(copy_event)
            ks_cpu.copy_(ks_tensor, non_blocking=True)
        copy_stream.synchronize()
        ks = ks_cpu.tolist()
        actual_M = sum(ks)
        output_tokens = output_tokens[:actual_M]
        ctx.save_for_backward(reverse)
        ctx.mark_non_differentiable(reverse, offs, ks_tensor)
        return output_tokens, reverse, offs, ks_tensor, ks

    @staticmethod
    def backward(ctx, grad_output_tokens, *unused):
        (reverse,) = ctx.saved_tensors
        m = reverse.shape[0]
        grad_output_tokens = grad_output_tokens.contiguous()
        H = grad_output_tokens.shape[1]
        grad = torch.empty((m, H), device=grad_output_tokens.device, dtype=grad_output_tokens.dtype)
        gather_rows(grad_output_tokens, reverse, grad)
        if ctx.pre_index is not None:
            grad = _PaddedIndexGather.scatter_sum(grad, ctx.pre_index, ctx.in_rows, _GEMM_ALLOC_ALIGNMENT)
        return grad, None, None, None, None


_copy_stream: Optional[torch.cuda.Stream] = None
_copy_event: Optional[torch.cuda.Event] = None


def _copy_stream_and_event(device):
    global _copy_stream, _copy_event
    if _copy_stream is None:
        _copy_stream = torch.cuda.Stream(device=device)
        _copy_event = torch.cuda.Event()
    return _copy_stream, _copy_event


class _PaddedIndexGather(torch.autograd.Function):
    """``input[index]`` into a buffer whose row count is padded; the input is not saved, backward
    sums the rows that share an index."""

    @staticmethod
    def forward(ctx, input: torch.Tensor, index: torch.Tensor, pad_to_multiple: int):
        _lib.require_cuda(input, index)
        ctx.save_for_backward(index)
        ctx.input_shape = input.shape
        ctx.pad_to_multiple = pad_to_multiple
        actual = index.shape[0]
        padded = -(-actual // pad_to_multiple) * pad_to_multiple
        buf = input.new_empty(padded, *input.shape[1:])
        if actual:
            src = input.reshape(input.shape[0], -1)
            if src.stride(-1) != 1:
                src = src.contiguous()
            gather_rows(src, index.contiguous(), buf[:actual].view(actual, -1))
        return buf[:actual]

    @staticmethod
    def scatter_sum(grad_output, index, rows: int, pad_to_multiple: int):
        padded_rows = -(-rows // pad_to_multiple) * pad_to_multiple
        tail = tuple(grad_output.shape[1:])
        grad_buf = torch.empty((padded_rows,) + tail, dtype=grad_output.dtype, device=grad_output.device)
        n = index.shape[0]
        H = 1
        for d in tail:
            H *= d
        if rows and H:
            go = grad_output.contiguous().view(n, H)
            ws_bytes = _lib.query("pt_gather_rows_backward_workspace_bytes", n, rows)
            ws = _workspace(ws_bytes, grad_output.device)
            _lib.call(
                "pt_gather_rows_backward", go.data_ptr(), H, grad_buf.data_ptr(), H,
                index.contiguous().data_ptr(), n, rows, H, _lib.dtype_code(grad_output.dtype),
                ws.data_ptr(), ws.numel(), _lib.stream_ptr(grad_output.device),
            )  # fmt: skip
        return grad_buf[:rows]

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        (index,) = ctx.saved_tensors
        grad = _PaddedIndexGather.scatter_sum(
            grad_output, index, ctx.input_shape[0], ctx.pad_to_multiple
        )
        return grad, None, None


def padded_index_gather(input: torch.Tensor, index: torch.Tensor, pad_to_multiple: int = 1024):
    """Memory-lean ``input[index]`` with a padded allocation."""
    return _PaddedIndexGather.apply(input, index, pad_to_multiple)


def scatter_for_grouped_gemm(
    input_tokens: torch.Tensor,
    expert_idxs: torch.Tensor,
    num_groups: int,
    padding_alignment: int = 128,
    pre_index: torch.Tensor | None = None,
):
    """Group rows by expert with per-group zero padding.

    Returns ``(output_tokens[sum(ks), H], reverse_shuffle_idxs[m] i64, grouped_mm_offs[G] i32,
    ks list[int], ks_tensor[G] i32)``.  ``output_tokens`` is a view of a buffer whose row count is
    a multiple of 1024 with a zeroed tail.

    ``pre_index`` (extension): when given, row ``i`` is read from ``input_tokens[pre_index[i]]`` -
    the dedup expand and the scatter in one pass over the data.
    """
    out, reverse, offs, ks_tensor, ks = ScatterForGroupedGemm.apply(
        input_tokens, expert_idxs, num_groups, padding_alignment, pre_index
    )
    return out, reverse, offs, ks, ks_tensor


def precompute_group_indices(grouped_mm_offs: torch.Tensor, M: int) -> Optional[torch.Tensor]:
    """Per-row group ids were an input of the reference's Hopper GEMM; the kernels here locate
    groups from ``grouped_mm_offs`` themselves, so nothing is precomputed."""
    return None


def group_indices(grouped_mm_offs: torch.Tensor, M: int, dtype=torch.int64) -> torch.Tensor:
    """``searchsorted(offs, arange(M), right=True).clamp(max=G-1)`` as one kernel."""
    assert dtype in (torch.int32, torch.int64)
    out = torch.empty((M,), device=grouped_mm_offs.device, dtype=dtype)
    if M:
        _lib.call(
            "pt_group_indices", grouped_mm_offs.data_ptr(), grouped_mm_offs.shape[0], M,
            out.data_ptr(), out.element_size(), _lib.stream_ptr(out.device),
        )  # fmt: skip
    return out
