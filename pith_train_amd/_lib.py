"""ctypes binding of ``libpithtrain_hip.so`` (the C-ABI declared in ``include/pithtrain_hip.h``).

The library is built in-tree by ``pith_train_amd/csrc/Makefile``.  There is no CPU fallback:
if the library is missing, every operator of this package raises.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# PITHTRAIN_HIP_LIB: another build of the library (measurement builds, see csrc/Makefile)
LIB_PATH = os.environ.get("PITHTRAIN_HIP_LIB") or os.path.join(_HERE, "libpithtrain_hip.so")

PT_BF16, PT_F32, PT_F16 = 0, 1, 2
PT_CH_ROWMAJOR, PT_CH_TRANSPOSED, PT_CH_KMAJOR = 0, 1, 2

_DTYPE_CODE = {torch.bfloat16: PT_BF16, torch.float32: PT_F32, torch.float16: PT_F16}

P, I32, I64, F = c_void_p, c_int32, c_int64, c_float

# name -> (restype, argtypes); mirrors include/pithtrain_hip.h one to one
SIGNATURES = {
    "pt_last_error": (c_char_p, []),
    "pt_abi_version": (c_int, []),
    "pt_quant_rowwise_colwise": (c_int, [P, c_int, I64, I64, I64, P, P, P, P, c_int, P, I32, P]),
    "pt_quant_rowwise_colwise_rows": (c_int, [P, c_int, I64, I64, I64, P, P, P, P, P, c_int, P, I32, P]),
    "pt_silu_mul_quant_rowwise_colwise": (c_int, [P, I64, I64, I64, P, P, P, P, P, P]),
    "pt_silu_mul_bwd_quant_rowwise_colwise": (c_int, [P, I64, P, I64, I64, I64, P, P, P, P, P, P]),
    "pt_clamped_swiglu_quant_rowwise_colwise": (c_int, [P, I64, I64, I64, F, F, P, P, P, P, P, P]),
    "pt_clamped_swiglu_bwd_quant_rowwise_colwise": (c_int, [P, I64, P, I64, I64, I64, F, F, P, P, P, P, P, P, P]),
    "pt_quant_rowwise_transpose": (c_int, [P, c_int, I64, I64, I64, P, P, P, P, P]),
    "pt_quant_rowwise_blockwise_transpose": (c_int, [P, c_int, I64, I64, I64, P, P, P, P, P]),
    "pt_quant_rowwise_transpose_ld": (c_int, [P, c_int, I64, I64, I64, P, P, P, I64, P, P]),
    "pt_quant_rowwise_blockwise_transpose_ld": (c_int, [P, c_int, I64, I64, I64, P, P, P, I64, P, P]),
    "pt_quant_blockwise_transpose_batched": (c_int, [P, c_int, I64, I64, I64, I64, I64, P, P, P, P, P]),
    "pt_quant_blockwise_transpose_batched_into": (c_int, [P, c_int, I64, I64, I64, I64, I64, P, I64, P, I64, P, I64, I64, P, I64,
                                                          I64, P]),
    "pt_gemm_nt_dense": (c_int, [P, P, P, P, P, c_int, I64, I64, I64, P]),
    "pt_gemm_nt_dense_splitk": (c_int, [P, P, P, P, P, I32, I64, I64, I64, I64, P]),
    "pt_gemm_nt_dense_ld": (c_int, [P, I64, P, P, I64, P, P, c_int, I64, I64, I64, P]),
    "pt_gemm_nt_dense_splitk_ld": (c_int, [P, I64, P, P, I64, P, P, I32, I64, I64, I64, I64, P]),
    "pt_sum_partials": (c_int, [P, I32, I64, P, c_int, P]),
    "pt_gemm_m_grouped_nt": (c_int, [P, P, P, P, P, c_int, P, I32, I64, I64, I64, P]),
    "pt_gemm_m_grouped_nn": (c_int, [P, P, P, P, P, c_int, P, I32, I64, I64, I64, P]),
    "pt_gemm_m_grouped_nn_scatter": (c_int, [P, P, P, P, P, c_int, P, I32, I64, I64, I64, P, I64, P]),
    "pt_gemm_m_grouped_nt_bias": (c_int, [P, P, P, P, P, c_int, P, I32, I64, I64, I64, P, P]),
    "pt_gemm_m_grouped_nt_scatter_bias": (c_int, [P, P, P, P, P, c_int, P, I32, I64, I64, I64, P, I64, P, P]),
    "pt_gemm_m_grouped_nt_scatter": (c_int, [P, P, P, P, P, c_int, P, I32, I64, I64, I64, P, I64, P]),
    "pt_gemm_k_grouped_wgrad": (c_int, [P, P, P, P, P, c_int, c_int, P, I32, I64, I64, I64, P]),
    "pt_gemm_k_grouped_wgrad_ld": (c_int, [P, P, I64, P, P, I64, P, c_int, c_int, P, I32, I64, I64, I64, P]),
    "pt_gemm_select_kernel": (c_int, [ctypes.c_char_p]),
    "pt_moe_combine_fwd": (c_int, [P, I64, P, P, I64, P, I64, I64, I32, I64, c_int, P]),
    "pt_moe_combine_bwd": (c_int, [P, I64, P, I64, P, P, I64, P, I64, I32, I64, c_int, P]),
    "pt_router_topk_fwd": (c_int, [P, I64, c_int, I64, I32, I32, c_int, c_int, F, I32, I32, P, P, P, P, P]),
    "pt_router_topk_bwd": (c_int, [P, I64, c_int, I64, I32, I32, c_int, c_int, F, I32, I32, P, P, P, P, I64, P]),
    "pt_compose_row_map": (c_int, [P, I64, P, I64, I64, P, P]),
    "pt_cross_entropy_fwd": (c_int, [P, I64, c_int, P, I64, I64, I64, P, P, P, P]),
    "pt_cross_entropy_bwd": (c_int, [P, I64, c_int, I64, I64, P, P]),
    "pt_moe_combine_ep_index": (c_int, [P, I64, I64, P, P]),
    "pt_moe_combine_ep_fwd": (c_int, [P, I64, I64, P, P, P, I64, P, I64, I64, I32, I64, c_int, P]),
    "pt_moe_combine_ep_bwd": (c_int, [P, I64, P, I64, I64, P, P, P, I64, P, I64, I32, I64, c_int, P]),
    "pt_group_rows_workspace_bytes": (I64, [I64, I32]),
    "pt_group_rows": (c_int, [P, I64, I32, I32, P, P, P, P, I64, P, I64, P]),
    "pt_group_rows_static": (c_int, [P, I64, I32, I32, P, P, P, P, I64, P]),
    "pt_permute_rows": (c_int, [P, I64, P, I64, P, P, P, I32, I64, I64, I32, P]),
    "pt_gather_rows": (c_int, [P, I64, P, I64, P, I64, I64, I32, P]),
    "pt_gather_rows_backward_workspace_bytes": (I64, [I64, I64]),
    "pt_gather_rows_backward": (c_int, [P, I64, P, I64, P, I64, I64, I64, c_int, P, I64, P]),
    "pt_group_indices": (c_int, [P, I32, I64, P, I32, P]),
    "pt_dedup_workspace_bytes": (I64, [I64, I32, I32, I32]),
    "pt_dedup_prepare_dispatch": (c_int, [P, I64, I64, I32, I32, I32, I32, P, P, P, P, P, P, P, I64, P]),
    "pt_build_expert_idxs": (c_int, [P, I32, I32, I32, I64, P, P, P]),
    "pt_adjust_expand_idx": (c_int, [P, P, P, I64, P, I32, I64, P]),
    "pt_silu_mul_fwd": (c_int, [P, P, P, I64, c_int, P]),
    "pt_silu_mul_bwd": (c_int, [P, P, P, P, P, I64, c_int, P]),
    "pt_silu_mul_fwd_2d": (c_int, [P, I64, P, I64, P, I64, I64, I64, c_int, P]),
    "pt_silu_mul_bwd_2d": (c_int, [P, I64, P, I64, P, I64, P, I64, P, I64, I64, I64, c_int, P]),
    "pt_clamped_swiglu_fwd": (c_int, [P, P, I64, F, F, c_int, P]),
    "pt_clamped_swiglu_bwd": (c_int, [P, P, P, I64, F, F, c_int, P]),
    "pt_indexed_bias_add_fwd": (c_int, [P, P, P, P, I64, I64, c_int, P]),
    "pt_segment_sum": (c_int, [P, P, I32, P, I64, I64, c_int, c_int, P]),
    "pt_segment_sum_rows": (c_int, [P, I64, P, P, I32, P, I64, I64, c_int, c_int, P]),
}

_lib = None


class PithTrainHipError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise PithTrainHipError(
            f"{LIB_PATH} not found: build it with `make -C pith_train_amd/csrc` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`). "
            "This package has no CPU fallback."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {dtype}") from None


def ptr(t: torch.Tensor | None):
    return None if t is None else t.data_ptr()


def stream_ptr(device=None):
    return torch.cuda.current_stream(device).cuda_stream


def require_cuda(*tensors: torch.Tensor):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise PithTrainHipError(
                "pith_train_amd operators run on the GPU only (got a tensor on "
                f"{t.device}); there is no CPU path"
            )


def call(name: str, *args):
    """Invoke an int-returning entry point and raise on a non-zero status."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib.pt_last_error().decode("utf-8", "replace")
        raise PithTrainHipError(f"{name} failed ({rc}): {msg}")


def query(name: str, *args) -> int:
    """Invoke a size-returning entry point (workspace queries)."""
    return int(getattr(load(), name)(*args))
