"""GPU parity: top-k combine through the C-ABI vs the oracle (bit-exact where the arithmetic has a
fixed order: forward, d_moe; fp32 reduction over H for d_weight within 1e-5)."""

import pytest
import torch

from oracle import combine as C

pytestmark = pytest.mark.gpu


def _inputs(T, k, H, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    moe = torch.randn((T * k, H), generator=g).to(dtype)
    w = torch.softmax(torch.randn((T, max(2 * k, 4)), generator=g), -1).topk(k, -1).values.float()
    w = w / w.sum(-1, keepdim=True)
    res = torch.randn((T, H), generator=g).to(dtype)
    go = torch.randn((T, H), generator=g).to(dtype)
    return moe, w, res, go


@pytest.mark.parametrize("T,k,H", [(64, 8, 2048), (33, 2, 256), (7, 1, 128), (16, 6, 2880), (5, 4, 100), (1, 16, 8), (0, 8, 64)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_combine_forward_backward(T, k, H, dtype):
    from pith_train_amd.operators.moe_combine import moe_combine

    moe, w, res, go = _inputs(T, k, H, T + k + H, dtype)
    m, ww, r = (t.cuda().requires_grad_(True) for t in (moe, w, res))
    out = moe_combine(m, ww, r)
    assert out.shape == res.shape and out.dtype == dtype
    assert torch.equal(out.detach().cpu(), C.combine_fwd(moe, w, res))
    if T == 0:
        return
    out.backward(go.cuda())
    d_moe, d_w, d_res = C.combine_bwd(go, moe, w)
    assert torch.equal(m.grad.cpu(), d_moe)
    assert torch.equal(r.grad.cpu(), d_res)
    torch.testing.assert_close(ww.grad.cpu(), d_w, rtol=1e-5, atol=1e-5 * H**0.5)


def test_combine_full_size_follows_stage3_and_is_deterministic():
    """At the benchmark's size (8192 tokens x top-8 x 2048): two runs give the same bits, and the
    result agrees with the tensor expression of the reference evaluated by torch on the GPU."""
    from pith_train_amd.operators.moe_combine import moe_combine

    T, k, H = 8192, 8, 2048
    moe, w, res, go = _inputs(T, k, H, 1)
    m, ww, r = moe.cuda(), w.cuda(), res.cuda()
    a = moe_combine(m, ww, r)
    b = moe_combine(m, ww, r)
    assert torch.equal(a, b)
    ref = r + (m.view(T, k, H) * ww.unsqueeze(-1)).sum(dim=1).to(m.dtype)
    # another order of the eight fp32 additions can move the bf16 rounding of the sum by one step of
    # the sum, and that of the result by one step of the result
    diff = (a.float() - ref.float()).abs()
    s_mag = (ref.float() - r.float()).abs()
    assert (diff <= (s_mag + ref.float().abs()) * 2.0**-7 + 1e-6).all()
    assert (a == ref).float().mean().item() > 0.99


# ---- expert-parallel branch ----


def _ep_inputs(T, k, H, seed, dtype=torch.bfloat16, rows=None):
    g = torch.Generator().manual_seed(seed)
    R = T * k if rows is None else rows
    idx = torch.randperm(T * k, generator=g)[:R].contiguous()
    moe = torch.randn((R, H), generator=g).to(dtype)
    w = torch.softmax(torch.randn((T, max(2 * k, 4)), generator=g), -1).topk(k, -1).values.float()
    res = torch.randn((T, H), generator=g).to(dtype)
    go = torch.randn((T, H), generator=g).to(dtype)
    return moe, idx, w, res, go


@pytest.mark.parametrize("T,k,H,rows", [(64, 8, 2048, None), (33, 2, 256, None), (7, 1, 128, None), (16, 6, 2880, None),
                                        (5, 4, 100, 17), (3, 16, 8, None), (40, 8, 512, 0), (0, 8, 64, None)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_combine_ep_forward_backward(T, k, H, rows, dtype):
    """Bit-exact against the oracle's sequential accumulation (a token's rows in ascending row
    order, every partial sum rounded); slots without a row contribute nothing and get a zero
    weight gradient."""
    from pith_train_amd.operators.moe_combine import moe_combine_ep

    moe, idx, w, res, go = _ep_inputs(T, k, H, T + k + H, dtype, rows)
    m, ww, r = (t.cuda().requires_grad_(True) for t in (moe, w, res))
    out = moe_combine_ep(m, idx.cuda(), ww, r)
    assert out.shape == res.shape and out.dtype == dtype
    assert torch.equal(out.detach().cpu(), C.combine_ep_fwd(moe, idx, w, res))
    if T == 0:
        return
    out.backward(go.cuda())
    d_moe, d_w, d_res = C.combine_ep_bwd(go, moe, idx, w)
    assert torch.equal(m.grad.cpu(), d_moe)
    assert torch.equal(r.grad.cpu(), d_res)
    torch.testing.assert_close(ww.grad.cpu(), d_w, rtol=1e-5, atol=1e-5 * H**0.5)


def test_combine_ep_full_size_against_the_tensor_expression():
    """8192 tokens x top-8 x 2048 with the dispatch sort's permutation (rows ordered by expert):
    deterministic, and within the rounding of the partial sums of the reference's expression
    evaluated by torch on the GPU (whose scatter_add_ order is not fixed)."""
    from pith_train_amd.operators.moe_combine import moe_combine_ep

    T, k, H, E = 8192, 8, 2048, 128
    g = torch.Generator().manual_seed(5)
    topk_ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    idx = torch.argsort(topk_ids.view(-1), stable=True)
    moe = torch.randn((T * k, H), generator=g).bfloat16().cuda()
    w = torch.softmax(torch.randn((T, k), generator=g), -1).cuda()
    res = torch.randn((T, H), generator=g).bfloat16().cuda()
    idx = idx.cuda()
    a = moe_combine_ep(moe, idx, w, res)
    assert torch.equal(a, moe_combine_ep(moe, idx, w, res))
    weighted = (moe.float() * w.view(-1)[idx].unsqueeze(-1)).to(moe.dtype)
    agg = moe.new_zeros(T, H)
    agg.scatter_add_(0, (idx // k)[:, None].expand_as(weighted), weighted)
    ref = (res + agg).float()
    mag = torch.zeros((T, H), device="cuda").index_add_(0, idx // k, weighted.float().abs())
    assert ((a.float() - ref).abs() <= mag * 2.0**-5 + ref.abs() * 2.0**-7 + 1e-6).all()
    assert (a.float() == ref).float().mean().item() > 0.8
