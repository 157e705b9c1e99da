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


# ---- expert-parallel branch (models/qwen3_moe.py:238-245) ----


def _ep_inputs(T, k, H, seed, rows=None):
    g = torch.Generator().manual_seed(seed)
    R = T * k if rows is None else rows
    idx = torch.randperm(T * k, generator=g)[:R].contiguous()
    moe = torch.randn((R, H), generator=g).bfloat16()
    w = torch.softmax(torch.randn((T, 4 * k), generator=g), -1).topk(k, -1).values.float()
    res = torch.randn((T, H), generator=g).bfloat16()
    return moe, idx, w, res


def _ep_expression(moe, idx, w, res):
    """The reference's expert-parallel forward, verbatim in structure."""
    permuted_probs = w.view(-1)[idx]
    token_indices = idx // w.shape[1]
    weighted = (moe.float() * permuted_probs.unsqueeze(-1)).to(moe.dtype)
    aggregated = moe.new_zeros(w.shape[0], moe.shape[-1])
    aggregated.scatter_add_(0, token_indices[:, None].expand_as(weighted), weighted)
    return res + aggregated.view(*res.shape)


@pytest.mark.parametrize("k", [1, 2])
def test_ep_forward_equals_the_tensor_expression_where_the_sum_has_one_order(k):
    moe, idx, w, res = _ep_inputs(64, k, 96, 10 + k)
    assert torch.equal(C.combine_ep_fwd(moe, idx, w, res), _ep_expression(moe, idx, w, res))


def test_ep_forward_equals_a_scalar_loop_in_row_order():
    """Brute force: one bf16 accumulator per (token, column), rows visited in ascending r."""
    T, k, H = 5, 4, 3
    moe, idx, w, res = _ep_inputs(T, k, H, 21, rows=17)  # three slots without a row
    acc = [[torch.zeros((), dtype=torch.bfloat16) for _ in range(H)] for _ in range(T)]
    for r in range(moe.shape[0]):
        t = int(idx[r]) // k
        p = w.reshape(-1)[idx[r]]
        for h in range(H):
            weighted = (moe[r, h].float() * p).bfloat16()
            acc[t][h] = (acc[t][h].float() + weighted.float()).bfloat16()
    want = torch.stack([torch.stack([(res[t, h].float() + acc[t][h].float()).bfloat16() for h in range(H)]) for t in range(T)])
    assert torch.equal(C.combine_ep_fwd(moe, idx, w, res), want)


def test_ep_forward_is_within_the_rounding_of_the_tensor_expression_for_k8():
    moe, idx, w, res = _ep_inputs(128, 8, 256, 23)
    got, ref = C.combine_ep_fwd(moe, idx, w, res).float(), _ep_expression(moe, idx, w, res).float()
    # Seven bf16-rounded partial sums against whatever order and width the library uses: each
    # rounding is at most 2**-9 of a partial sum, none larger than the token's sum of magnitudes.
    mag = torch.zeros((128, 256)).index_add_(0, idx // 8, (moe.float() * w.view(-1)[idx][:, None]).abs())
    assert ((got - ref).abs() <= mag * 2.0**-5 + ref.abs() * 2.0**-7 + 1e-6).all()
    assert (got == ref).float().mean() > 0.8


def test_ep_rounds_every_partial_sum():
    # token 0, three rows 1, 2**-8, 2**-8 with weight 1: the accumulator stays 1 after each add
    # (tie to even), where a single rounding of the sum would give 1.0078125
    moe = torch.tensor([[1.0] * 4, [2.0**-8] * 4, [2.0**-8] * 4]).bfloat16()
    idx = torch.tensor([0, 1, 2])
    w = torch.ones((1, 3))
    res = torch.zeros((1, 4)).bfloat16()
    assert torch.equal(C.combine_ep_fwd(moe, idx, w, res), torch.ones((1, 4)).bfloat16())
    # The order is by row, not by slot: rows 2**-8, 2**-8, 1 (held by slots 2, 1, 0) give 2**-7
    # first, then 1 + 2**-7; walking the slots in order would start from 1 and stay there.
    assert torch.equal(C.combine_ep_fwd(moe.flip(0), torch.tensor([2, 1, 0]), w, res),
                       torch.full((1, 4), 1.0078125).bfloat16())


def test_ep_backward_matches_autograd_of_the_tensor_expression():
    moe, idx, w, res = _ep_inputs(32, 4, 64, 27)
    g = torch.randn((32, 64), generator=torch.Generator().manual_seed(28)).bfloat16()
    m, ww, r = moe.clone().requires_grad_(True), w.clone().requires_grad_(True), res.clone().requires_grad_(True)
    _ep_expression(m, idx, ww, r).backward(g)
    d_moe, d_w, d_res = C.combine_ep_bwd(g, moe, idx, w)
    assert torch.equal(d_moe, m.grad)
    assert torch.equal(d_res, r.grad)
    torch.testing.assert_close(d_w, ww.grad, rtol=1e-5, atol=1e-5)
