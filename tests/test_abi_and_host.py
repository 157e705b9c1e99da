"""CPU-only checks: the C-ABI library loads and exports every symbol the header declares, the
ctypes table mirrors the header, and the host-side logic that needs no GPU behaves."""

import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "pithtrain_hip.h")


def _declared():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(pt_[a-z0-9_]+)\s*\(", src)))


def test_header_declares_what_ctypes_binds():
    from pith_train_amd import _lib

    assert sorted(_lib.SIGNATURES) == _declared()


def test_library_exports_every_declared_symbol():
    from pith_train_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built yet (run __graft_entry__.build())")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), name
    assert _lib.load().pt_abi_version() == 1
    assert _lib.load().pt_last_error() is not None


def test_workspace_queries_need_no_gpu():
    from pith_train_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built yet")
    assert _lib.query("pt_group_rows_workspace_bytes", 65536, 128) >= 65536 // 256 * 128 * 4
    assert _lib.query("pt_gather_rows_backward_workspace_bytes", 1000, 300) >= 1000 * 4 + 3 * 300 * 4
    assert _lib.query("pt_dedup_workspace_bytes", 2048, 8, 128, 8) > 0


def test_gemm_kernel_selection_validates_names_without_a_gpu():
    from pith_train_amd import _lib

    lib = _lib.load()
    for name in (b"auto", b"p0", b"q0", b"q1", b"r0", b"t", None):
        assert lib.pt_gemm_select_kernel(name) == 0
    assert lib.pt_gemm_select_kernel(b"fastest") != 0
    assert b"fastest" in lib.pt_last_error()
    assert lib.pt_gemm_select_kernel(None) == 0


def test_fused_gemm_stores_refuse_outputs_beyond_the_32_bit_store_offsets():
    """The persistent GEMM kernels address the output through an unsigned 32-bit byte offset.  A
    biased or scattered store has no 64-bit fallback, so an output of 4 GiB or more is refused on
    the host, before any launch (the pointers below are never dereferenced)."""
    from pith_train_amd import _lib

    lib = _lib.load()
    p = ctypes.c_void_p(0x10000)
    I64, I32 = ctypes.c_int64, ctypes.c_int32
    M, N, K, G = 128 * 20000, 1024, 128, 4  # operands 328 MB and 0.5 MB, bf16 output 5.2 GB
    assert M * N * 2 >= 1 << 32 and M * K < (1 << 31)
    lib.pt_gemm_m_grouped_nt_bias.argtypes = [ctypes.c_void_p] * 5 + [ctypes.c_int, ctypes.c_void_p, I32, I64, I64, I64,
                                              ctypes.c_void_p, ctypes.c_void_p]
    rc = lib.pt_gemm_m_grouped_nt_bias(p, p, p, p, p, 0, p, G, M, N, K, p, None)
    assert rc != 0 and b"4 GiB" in lib.pt_last_error()
    lib.pt_gemm_m_grouped_nt_scatter.argtypes = [ctypes.c_void_p] * 5 + [ctypes.c_int, ctypes.c_void_p, I32, I64, I64, I64,
                                                 ctypes.c_void_p, I64, ctypes.c_void_p]
    rc = lib.pt_gemm_m_grouped_nt_scatter(p, p, p, p, p, 0, p, G, 1024, N, K, p, M, None)
    assert rc != 0 and b"4 GiB" in lib.pt_last_error()


def test_reduction_major_gemm_validates_its_operand_on_the_host():
    """pt_gemm_m_grouped_nn reads b[g] as [K, N] through 16-byte chunks of its rows and exists only
    in the kernel with 32-bit offsets: a row length that is not a multiple of 16 and an output of
    4 GiB or more are refused before any launch (the pointers below are never dereferenced)."""
    from pith_train_amd import _lib

    lib = _lib.load()
    p = ctypes.c_void_p(0x10000)
    I64, I32 = ctypes.c_int64, ctypes.c_int32
    lib.pt_gemm_m_grouped_nn.argtypes = [ctypes.c_void_p] * 5 + [ctypes.c_int, ctypes.c_void_p, I32, I64, I64, I64, ctypes.c_void_p]
    assert lib.pt_gemm_m_grouped_nn(p, p, p, p, p, 0, p, 2, 256, 24, 128, None) != 0
    assert b"multiple of 16" in lib.pt_last_error()
    M, N, K = 128 * 20000, 1024, 128  # bf16 output 5.2 GB
    assert lib.pt_gemm_m_grouped_nn(p, p, p, p, p, 0, p, 4, M, N, K, None) != 0
    assert b"row-split kernel" in lib.pt_last_error() and b"NT entry point" in lib.pt_last_error()
    assert lib.pt_gemm_m_grouped_nn(p, p, p, p, p, 0, p, 4, 0, N, K, None) == 0  # nothing to do


def test_operators_refuse_cpu_tensors_loudly():
    from pith_train_amd import _lib
    from pith_train_amd.operators.deepgemm_quantize import fp8cast_rowwise_colwise
    from pith_train_amd.operators.silu_mul import silu_mul
    from pith_train_amd.operators.token_scatter import scatter_for_grouped_gemm

    x = torch.zeros((128, 128), dtype=torch.bfloat16)
    with pytest.raises(_lib.PithTrainHipError):
        fp8cast_rowwise_colwise(x)
    with pytest.raises(_lib.PithTrainHipError):
        silu_mul(x, x)
    with pytest.raises(_lib.PithTrainHipError):
        scatter_for_grouped_gemm(x, torch.zeros(128, dtype=torch.int64), 4)


def test_weight_grad_store_and_cache_control():
    from pith_train_amd.dualpipe_utils import FP8WeightCacheControl, WeightGradStore

    WeightGradStore.clear()
    order = []
    WeightGradStore.put(lambda: order.append(1))
    WeightGradStore.put(lambda: order.append(2))
    WeightGradStore.flush()
    WeightGradStore.put(lambda: order.append(3))
    WeightGradStore.flush()
    WeightGradStore.pop()
    assert order == [1, 2]
    WeightGradStore.pop()
    assert order == [1, 2, 3]
    with pytest.raises(AssertionError):
        WeightGradStore.pop()
    v = FP8WeightCacheControl.version
    FP8WeightCacheControl.step()
    assert FP8WeightCacheControl.version == v + 1

    class M(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self._wq_cache = (1, 2, 3, 4)

    m = torch.nn.Sequential(M(), M())
    FP8WeightCacheControl.clear(m)
    assert all(x._wq_cache is None for x in m)


def test_bf16_grouped_linear_on_cpu_matches_loop():
    from pith_train_amd.operators.grouped_linear import GroupedLinear

    torch.manual_seed(0)
    gl = GroupedLinear(3, 16, 8)
    torch.nn.init.normal_(gl.weight, std=0.1)
    offs = torch.tensor([4, 4, 10], dtype=torch.int32)
    x = torch.randn(10, 16, requires_grad=True)
    y = gl(x, offs)
    ref = torch.cat([x[:4] @ gl.weight[0].T, x[4:10] @ gl.weight[2].T])
    assert torch.allclose(y, ref, atol=1e-5)
    y.sum().backward()
    assert gl.weight.grad is not None and torch.all(gl.weight.grad[1] == 0)
    empty = gl(torch.empty(0, 16, requires_grad=True), torch.empty(0, dtype=torch.int32))
    assert empty.shape == (0, 8) and empty.grad_fn is not None


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_bench_times_every_gemm_entry_point_of_the_library():
    """The roofline figure is only valid if no GEMM launch escapes the timer."""
    import re

    import bench

    header = open(os.path.join(os.path.dirname(__file__), "..", "include", "pithtrain_hip.h")).read()
    declared = set(re.findall(r"\bint (pt_gemm_(?!select_kernel)\w+)\(", header))
    assert declared == set(bench.GemmTimer.NAMES), declared ^ set(bench.GemmTimer.NAMES)
