"""The committed fixture of the steps beside the expert path (router gate, expert-parallel combine,
cross-entropy; tests/golden/) against the oracle (CPU) and against the HIP path (GPU)."""

import importlib.util
import os

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
FIX = os.path.join(HERE, "golden", "next_rows_router_combine_ce.npz")

_spec = importlib.util.spec_from_file_location("make_next_rows_fixture", os.path.join(HERE, "golden", "make_next_rows_fixture.py"))
gen = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(gen)


@pytest.fixture(scope="module")
def fixture():
    return np.load(FIX, allow_pickle=False)


def _bf16(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def test_oracle_reproduces_the_fixture(fixture):
    got = gen.compute()
    assert str(got["input_sha256"]) == str(fixture["input_sha256"]), "the seeded inputs changed (generator drift)"
    for key in fixture.files:
        if key.endswith("sha256"):
            continue
        a, b = got[key], fixture[key]
        if a.dtype.kind == "f":  # the host's exp / softmax may differ in the last bits between builds
            np.testing.assert_allclose(a, b, rtol=2e-6, atol=1e-9, err_msg=key)
        else:
            assert np.array_equal(a, b), key


def test_fixture_invariants(fixture):
    """Independent of the oracle's code: distinct experts per token in descending weight order,
    normalised weights summing to one (to the scaling factor where there is one), grouped
    choices inside three groups of eight, gradient rows summing to zero."""
    for name, k, total in (("router", gen.K_TOP, 1.0), ("router_topk_softmax", 4, 1.0)):
        idx, w = fixture[name + "_idx"], fixture[name + "_weight"]
        assert idx.shape == w.shape == (gen.T, k)
        assert all(len(set(r)) == k for r in idx.tolist())
        assert (np.diff(w, axis=1) <= 0).all()
        np.testing.assert_allclose(w.sum(1), total, rtol=1e-5)
    gidx = fixture["router_grouped_idx"]
    assert all(len({e // 8 for e in r}) <= 3 for r in gidx.tolist())
    assert (fixture["router_grouped_weight"] > 0).all() and (fixture["router_grouped_weight"] <= 16.0).all()
    grad = _bf16(fixture["ce_grad"]).float()
    n = int(fixture["ce_rows"])
    assert n == gen.T - len(range(0, gen.T, 9))
    assert (grad[::9] == 0).all()
    live = np.ones(gen.T, dtype=bool)
    live[::9] = False
    assert (grad[torch.from_numpy(live)].sum(-1).abs() * n < 2e-2).all()


@pytest.mark.gpu
def test_hip_path_matches_the_fixture(fixture):
    from pith_train_amd.operators.cross_entropy import cross_entropy
    from pith_train_amd.operators.moe_combine import moe_combine_ep
    from pith_train_amd.operators.router_topk import softmax_topk, topk_softmax

    logits, logits_g, perm, moe, res, ce_logits, target = gen.make_inputs()
    idx, w = softmax_topk(logits.cuda(), gen.K_TOP, norm_topk_prob=True)
    assert np.array_equal(idx.cpu().numpy(), fixture["router_idx"])
    np.testing.assert_allclose(w.cpu().numpy(), fixture["router_weight"], rtol=1e-5)
    gidx, gw = softmax_topk(logits_g.cuda(), 6, scale=16.0, num_group=8, topk_group=3)
    assert np.array_equal(gidx.cpu().numpy(), fixture["router_grouped_idx"])
    np.testing.assert_allclose(gw.cpu().numpy(), fixture["router_grouped_weight"], rtol=1e-5)
    tidx, tw = topk_softmax(logits[:, :32].bfloat16().cuda(), 4)
    assert np.array_equal(tidx.cpu().numpy(), fixture["router_topk_softmax_idx"])
    np.testing.assert_allclose(tw.cpu().numpy(), fixture["router_topk_softmax_weight"], rtol=1e-5)
    # the combine takes the fixture's weights, so that the check is of the combine alone: bit-exact
    out = moe_combine_ep(moe.cuda(), perm.cuda(), torch.from_numpy(fixture["router_weight"]).cuda(), res.cuda())
    assert torch.equal(out.cpu(), _bf16(fixture["combined"]))
    buf = ce_logits.cuda()
    loss = cross_entropy(buf, target.cuda())
    np.testing.assert_allclose(float(loss), float(fixture["ce_loss"]), rtol=1e-5)
    got, ref = buf.float().cpu(), _bf16(fixture["ce_grad"]).float()
    assert ((got - ref).abs() <= ref.abs() * 2.0**-7 + 1e-30).all()
    assert (got == ref).float().mean() > 0.98
