"""Pins of the cross-entropy oracle (CPU): against torch's own cross_entropy in float64, the
closed form for uniform logits, and the ignore rules."""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import cross_entropy as CE


def _case(N, V, seed, dtype=torch.float32, ignore_frac=0.2):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn((N, V), generator=g) * 3).to(dtype)
    y = torch.randint(0, V, (N,), generator=g)
    y[torch.rand(N, generator=g) < ignore_frac] = -100
    return x, y


@pytest.mark.parametrize("N,V", [(17, 1000), (8, 40000), (5, 70001)])  # one block, two blocks, ragged third block
def test_against_torch_cross_entropy_in_float64(N, V):
    x, y = _case(N, V, N + V)
    loss, grad, loss_rows, n = CE.cross_entropy_fwd(x, y)
    xd = x.double().requires_grad_(True)
    ref = F.cross_entropy(xd, y, ignore_index=-100, reduction="mean")
    ref.backward()
    assert n == int((y != -100).sum())
    torch.testing.assert_close(loss.double(), ref.detach(), rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(grad.double(), xd.grad, rtol=1e-4, atol=1e-9)
    torch.testing.assert_close(loss_rows.double(), F.cross_entropy(x.double(), y, ignore_index=-100, reduction="none"),
                               rtol=1e-6, atol=1e-6)


def test_uniform_logits_closed_form():
    N, V = 4, 512
    x = torch.full((N, V), 1.25, dtype=torch.bfloat16)
    y = torch.tensor([0, 5, 511, 7])
    loss, grad, _, n = CE.cross_entropy_fwd(x, y)
    assert n == 4 and abs(float(loss) - math.log(V)) < 1e-6
    # softmax 1/512, over n = 4: 2**-11 exactly; the target entry 2**-11 - 0.25 rounded to bf16
    want = torch.full((N, V), 2.0**-11).bfloat16()
    want[torch.arange(N), y] = torch.tensor(2.0**-11 - 0.25).bfloat16()
    assert torch.equal(grad, want)


def test_target_entry_is_corrected_after_the_store():
    # one row, two logits 0 and log(3): softmax 0.25 / 0.75; bf16 holds both; n = 1
    x = torch.tensor([[0.0, math.log(3.0)]]).bfloat16()
    loss, grad, _, _ = CE.cross_entropy_fwd(x, torch.tensor([1]))
    p = torch.softmax(x.float(), -1)
    assert torch.equal(grad[0, 0], p[0, 0].bfloat16())
    assert torch.equal(grad[0, 1], (p[0, 1].bfloat16().float() - 1.0).bfloat16())  # two roundings, not one


def test_ignore_rules():
    x, y = _case(9, 300, 1, torch.bfloat16, ignore_frac=0.0)
    y[[2, 5]] = -100
    loss, grad, loss_rows, n = CE.cross_entropy_fwd(x, y)
    assert n == 7 and grad[[2, 5]].abs().max() == 0 and loss_rows[[2, 5]].abs().max() == 0
    y[:] = -100  # nothing counts: n clamps to 1, loss 0, all gradients 0
    loss, grad, _, n = CE.cross_entropy_fwd(x, y)
    assert n == 1 and float(loss) == 0 and grad.abs().max() == 0
    y[3] = 7  # a custom ignore value
    loss2, grad2, _, n2 = CE.cross_entropy_fwd(x, torch.full((9,), 7), ignore_index=7)
    assert n2 == 1 and float(loss2) == 0 and grad2.abs().max() == 0


def test_backward_scales_by_the_rounded_scalar():
    x, y = _case(6, 128, 3, torch.bfloat16)
    _, grad, _, _ = CE.cross_entropy_fwd(x, y)
    s = torch.tensor(0.3)
    assert torch.equal(CE.cross_entropy_bwd(grad, s), grad * s.bfloat16())
