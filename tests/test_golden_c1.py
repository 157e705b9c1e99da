"""The committed C1 fixture (toy FP8 grouped linear, forward only; tests/golden/) against the
oracle (CPU) and against the HIP path (GPU)."""

import importlib.util
import os

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
FIX = os.path.join(HERE, "golden", "c1_toy_fp8_grouped_linear.npz")

_spec = importlib.util.spec_from_file_location("make_c1_fixture", os.path.join(HERE, "golden", "make_c1_fixture.py"))
gen = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(gen)


@pytest.fixture(scope="module")
def fixture():
    return np.load(FIX, allow_pickle=False)


def test_oracle_reproduces_the_fixture(fixture):
    got = gen.compute()
    assert str(got["input_sha256"]) == str(fixture["input_sha256"]), "the seeded inputs changed (generator drift)"
    for key in fixture.files:
        if key.endswith("sha256"):
            assert str(got[key]) == str(fixture[key]), key
        else:
            assert np.array_equal(got[key], fixture[key]), key


def test_fixture_invariants(fixture):
    """Independent of the oracle's code: scales are powers of two, every group is padded to 128
    rows, pad rows are zero bytes, the permutation is injective."""
    offs, rev = fixture["offs"], fixture["reverse"]
    assert (offs % 128 == 0).all() and (np.diff(np.concatenate([[0], offs])) >= 0).all()
    assert len(np.unique(rev)) == len(rev) == gen.T * gen.TOPK and rev.max() < offs[-1]
    for name in ("x_scale", "w_scale"):
        m, _ = np.frexp(fixture[name])
        assert (m == 0.5).all(), f"{name} holds a value that is not a power of two"
    pad = np.ones(offs[-1], dtype=bool)
    pad[rev] = False
    assert (fixture["x_fp8"][pad] == 0).all()
    assert (fixture["x_fp8"] & 0x7F).max() <= 0x7E, "e4m3fn has no byte above 448"


@pytest.mark.gpu
def test_hip_path_matches_the_fixture(fixture):
    from pith_train_amd.operators.deepgemm_quantize import fp8cast_blockwise_transpose_batched, fp8cast_rowwise_colwise
    from pith_train_amd.operators.grouped_linear import m_grouped_fp8_gemm_nt
    from pith_train_amd.operators.token_scatter import scatter_for_grouped_gemm

    tokens, eidx, w = gen.make_inputs()
    xp, reverse, offs, ks, ks_tensor = scatter_for_grouped_gemm(tokens.cuda(), eidx.cuda(), gen.E)
    assert np.array_equal(offs.cpu().numpy(), fixture["offs"])
    assert np.array_equal(reverse.cpu().numpy(), fixture["reverse"])
    x_fp8, x_scale, _, _ = fp8cast_rowwise_colwise(xp)
    w_fp8, w_scale, _, _ = fp8cast_blockwise_transpose_batched(w.cuda())
    assert np.array_equal(x_fp8.view(torch.uint8).cpu().numpy(), fixture["x_fp8"])
    assert np.array_equal(x_scale.cpu().numpy(), fixture["x_scale"])
    assert np.array_equal(w_fp8.view(torch.uint8).cpu().numpy(), fixture["w_fp8"])
    assert np.array_equal(w_scale.cpu().numpy(), fixture["w_scale"])
    out = torch.empty((xp.shape[0], gen.N), dtype=torch.bfloat16, device="cuda")
    m_grouped_fp8_gemm_nt((x_fp8, x_scale), (w_fp8, w_scale), out, offs)
    ref = torch.from_numpy(fixture["out_bf16_bits_head"].view(np.int16).copy()).view(torch.bfloat16).float()
    got = out[:256].float().cpu()
    # fp32 accumulation on the GPU against float64 in the fixture: max rel-err <= 1e-2 of the scale
    assert (got - ref).abs().max() <= 1e-2 * ref.abs().max()
    assert (got != ref).float().mean() < 0.05, "more than 5% of bf16 outputs differ in the last bit"
