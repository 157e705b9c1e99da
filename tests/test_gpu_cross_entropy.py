"""GPU parity: in-place fused cross-entropy through the C-ABI vs the oracle.

The loss agrees to 1e-5 (fp32 statistics in another summation order, hardware exp2); a gradient
entry is the oracle's to one rounding step of the logits' dtype, and bit-equal wherever the
arithmetic is exact (uniform logits, ignored rows, the scaling of the backward)."""

import math

import pytest
import torch

from oracle import cross_entropy as CE

pytestmark = pytest.mark.gpu


def _case(N, V, seed, dtype, ignore_frac=0.2):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn((N, V), generator=g) * 3).to(dtype)
    y = torch.randint(0, V, (N,), generator=g)
    y[torch.rand(N, generator=g) < ignore_frac] = -100
    return x, y


def _check_grad(got, ref, dtype):
    got, ref = got.float().cpu(), ref.float()
    assert got.shape == ref.shape
    if got.numel() == 0:
        return
    if dtype == torch.float32:
        torch.testing.assert_close(got, ref, rtol=2e-5, atol=1e-10)
        return
    step = 2.0**-7 if dtype == torch.bfloat16 else 2.0**-10
    assert ((got - ref).abs() <= ref.abs() * step + 1e-30).all(), "more than one rounding step apart"
    assert (got == ref).float().mean() > 0.98


@pytest.mark.parametrize("N,V,dtype", [
    (64, 4096, torch.bfloat16), (33, 151936, torch.bfloat16), (16, 50000, torch.float32), (9, 1000, torch.float16),
    (7, 1003, torch.bfloat16),   # V not a multiple of 8: element-wise path
    (3, 5, torch.float32), (1, 201088, torch.bfloat16), (0, 128, torch.bfloat16),
])
def test_forward_backward(N, V, dtype):
    from pith_train_amd.operators.cross_entropy import cross_entropy

    x, y = _case(N, V, N + V, dtype)
    o_loss, o_grad, _, _ = CE.cross_entropy_fwd(x, y)
    leaf = x.cuda().requires_grad_(True)
    buf = leaf.clone()  # the operator overwrites its input: hand it a non-leaf
    loss = cross_entropy(buf, y.cuda())
    assert loss.dtype == torch.float32 and loss.shape == ()
    torch.testing.assert_close(loss.cpu(), o_loss, rtol=1e-5, atol=1e-6)
    _check_grad(buf.detach(), o_grad, dtype)  # the forward already left the gradient in place
    stored = buf.detach().clone()
    (loss * 0.3).backward()
    assert torch.equal(leaf.grad, stored * torch.tensor(0.3).to(dtype))  # one multiplication: no freedom
    if N:
        # a unit incoming gradient leaves the stored gradient as it is
        leaf2 = x.cuda().requires_grad_(True)
        buf2 = leaf2.clone()
        cross_entropy(buf2, y.cuda()).backward()
        assert torch.equal(leaf2.grad, stored)


def test_exact_cases():
    from pith_train_amd.operators.cross_entropy import cross_entropy

    N, V = 4, 512
    x = torch.full((N, V), 1.25, dtype=torch.bfloat16).cuda()
    y = torch.tensor([0, 5, 511, 7])
    loss = cross_entropy(x, y.cuda())
    assert abs(float(loss) - math.log(V)) < 1e-6
    want = torch.full((N, V), 2.0**-11).bfloat16()
    want[torch.arange(N), y] = torch.tensor(2.0**-11 - 0.25).bfloat16()
    assert torch.equal(x.cpu(), want)
    # two roundings at the target: the stored softmax term is corrected afterwards
    x = torch.tensor([[0.0, math.log(3.0)] + [-1e4] * 6]).bfloat16().cuda()
    cross_entropy(x, torch.tensor([1]).cuda())
    assert float(x[0, 1]) == float((torch.tensor(0.75).bfloat16().float() - 1.0).bfloat16())


def test_ignore_rules_and_masked_vocabulary():
    from pith_train_amd.operators.cross_entropy import cross_entropy

    x, y = _case(9, 304, 1, torch.bfloat16, ignore_frac=0.0)
    y[[2, 5]] = -100
    buf = x.cuda()
    loss = cross_entropy(buf, y.cuda())
    o_loss, o_grad, _, _ = CE.cross_entropy_fwd(x, y)
    torch.testing.assert_close(loss.cpu(), o_loss, rtol=1e-5, atol=1e-6)
    assert buf[[2, 5]].abs().max() == 0
    buf = x.cuda()
    loss = cross_entropy(buf, torch.full((9,), -100).cuda())  # nothing counts: n clamps to 1
    assert float(loss) == 0 and buf.abs().max() == 0
    buf = x.cuda()
    loss = cross_entropy(buf, torch.full((9,), 7).cuda(), ignore_index=7)
    assert float(loss) == 0 and buf.abs().max() == 0
    # a vocabulary whose tail is masked with -inf: zero probability there, finite loss
    xm = x.clone()
    xm[:, 200:] = float("-inf")
    ym = y.clamp(min=0) % 200
    o_loss, o_grad, _, _ = CE.cross_entropy_fwd(xm, ym)
    buf = xm.cuda()
    loss = cross_entropy(buf, ym.cuda())
    torch.testing.assert_close(loss.cpu(), o_loss, rtol=1e-5, atol=1e-6)
    assert buf[:, 200:].abs().max() == 0 and torch.isfinite(buf).all()


def test_full_size_rows_sum_to_zero_and_loss_matches_torch():
    """2048 rows of a 151 936-entry vocabulary: the loss equals torch's cross_entropy on the same
    device, every gradient row of a counted token sums to zero (softmax minus one-hot) within the
    bf16 rounding of its entries, and two runs give the same bits."""
    import torch.nn.functional as F

    from pith_train_amd.operators.cross_entropy import cross_entropy

    N, V = 2048, 151936
    g = torch.Generator(device="cuda").manual_seed(5)
    x = (torch.randn((N, V), device="cuda", generator=g) * 2).bfloat16()
    y = torch.randint(0, V, (N,), device="cuda", generator=g)
    y[::7] = -100
    ref = F.cross_entropy(x.float(), y, ignore_index=-100)
    a, b = x.clone(), x.clone()
    la, lb = cross_entropy(a, y), cross_entropy(b, y)
    assert torch.equal(la, lb) and torch.equal(a, b)
    torch.testing.assert_close(la, ref, rtol=1e-5, atol=1e-6)
    n = int((y != -100).sum())
    sums = a.float().sum(-1) * n
    assert sums[y == -100].abs().max() == 0
    assert sums[y != -100].abs().max() < 2e-2
