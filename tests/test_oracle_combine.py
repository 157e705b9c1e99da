"""Pins of the top-k combine oracle (CPU): the restatement against the reference's tensor
expression (models/qwen3_moe.py:235-237), where the mathematics leaves no freedom."""

import pytest
import torch

from oracle import combine as C


def _inputs(T, k, H, seed):
    g = torch.Generator().manual_seed(seed)
    moe = torch.randn((T * k, H), generator=g).bfloat16()
    w = torch.softmax(torch.randn((T, 4 * k), generator=g), -1).topk(k, -1).values.float()
    res = torch.randn((T, H), generator=g).bfloat16()
    return moe, w, res


def _expression(moe, w, res):
    """The reference's forward, verbatim in structure."""
    weighted = moe.view(*w.shape, -1) * w.unsqueeze(-1)
    return res + weighted.sum(dim=1).to(moe.dtype).view(*res.shape)


@pytest.mark.parametrize("k", [1, 2])
def test_forward_equals_the_tensor_expression_where_the_sum_has_one_order(k):
    moe, w, res = _inputs(64, k, 96, k)
    assert torch.equal(C.combine_fwd(moe, w, res), _expression(moe, w, res))


def test_forward_matches_the_tensor_expression_to_one_rounding_for_k8():
    moe, w, res = _inputs(128, 8, 256, 3)
    got, ref = C.combine_fwd(moe, w, res).float(), _expression(moe, w, res).float()
    # a different order of eight fp32 additions can move the bf16 rounding of the sum by one step
    s_mag = (ref - res.float()).abs()
    assert ((got - ref).abs() <= (s_mag + ref.abs()) * 2.0**-7 + 1e-6).all()
    assert (got == ref).float().mean() > 0.99


def test_known_answers():
    # two experts with weights 0.25 / 0.75 on constant rows: 0.25*4 + 0.75*8 = 7, plus residual 1
    moe = torch.tensor([[4.0] * 8, [8.0] * 8]).bfloat16()
    w = torch.tensor([[0.25, 0.75]])
    res = torch.ones((1, 8)).bfloat16()
    assert torch.equal(C.combine_fwd(moe, w, res), torch.full((1, 8), 8.0).bfloat16())
    # The sum is rounded to bf16 before the residual is added: 1 + 2**-8 rounds to 1 (tie to even),
    # and 2**-8 + 1 rounds to 1 again; a single rounding of 1 + 2**-8 + 2**-8 would give 1.0078125.
    moe = torch.tensor([[1.0] * 8, [2.0**-8] * 8]).bfloat16()
    w = torch.tensor([[1.0, 1.0]])
    res = torch.full((1, 8), 2.0**-8).bfloat16()
    assert torch.equal(C.combine_fwd(moe, w, res), torch.ones((1, 8)).bfloat16())


def test_backward_matches_autograd_of_the_tensor_expression():
    moe, w, res = _inputs(32, 4, 64, 7)
    g = torch.randn((32, 64), generator=torch.Generator().manual_seed(8)).bfloat16()
    m, ww, r = moe.clone().requires_grad_(True), w.clone().requires_grad_(True), res.clone().requires_grad_(True)
    _expression(m, ww, r).backward(g)
    d_moe, d_w, d_res = C.combine_bwd(g, moe, w)
    assert torch.equal(d_moe, m.grad)  # one product, one rounding: no freedom
    assert torch.equal(d_res, r.grad)
    torch.testing.assert_close(d_w, ww.grad, rtol=1e-5, atol=1e-5)  # fp32 sum over H: order-dependent last bits
