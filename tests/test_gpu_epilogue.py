"""GPU parity: silu_mul, clamped SwiGLU, indexed bias add / segmented sum vs the CPU oracle.

Tolerances are the reference's own (tests/test_silu_mul.py: atol=rtol=1e-2;
tests/test_clamped_swiglu.py: atol 3e-1 / rtol 5e-2 in bf16; tests/test_indexed_bias_add.py:
forward exact, bias grad 5e-1 / 5e-2) - and much tighter where fp32 math allows: outputs must be
within one storage-dtype ulp of the oracle (sigmoid's last bit differs between back ends).
"""

import pytest
import torch

from oracle import epilogue as E

pytestmark = pytest.mark.gpu


def _close_ulp(got, ref, dtype, what):
    got, ref = got.float().cpu(), ref.float()
    eps = {torch.bfloat16: 2.0**-7, torch.float16: 2.0**-10, torch.float32: 2.0**-20}[dtype]
    err = (got - ref).abs()
    bound = ref.abs() * eps + 1e-30 + (1e-6 if dtype == torch.float32 else 0) * ref.abs().max()
    sub = {torch.bfloat16: 1e-38, torch.float16: 6.2e-5, torch.float32: 1e-37}[dtype]
    bad = err > bound + sub
    assert not bad.any(), f"{what}: {int(bad.sum())} elements off, max err {err.max().item():.3e}"


@pytest.mark.parametrize("shape", [(8192, 4096), (1023, 777), (1, 1), (128, 768), (5, 8)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_silu_mul(shape, dtype):
    from pith_train_amd.operators.silu_mul import silu_mul

    if shape[0] * shape[1] > 1e7 and dtype != torch.bfloat16:
        pytest.skip("large shape covered in bf16")
    g = torch.Generator().manual_seed(shape[0])
    gate = (torch.randn(shape, generator=g) * 3).to(dtype)
    up = torch.randn(shape, generator=g).to(dtype)
    do = torch.randn(shape, generator=g).to(dtype)
    a = gate.cuda().requires_grad_(True)
    b = up.cuda().requires_grad_(True)
    out = silu_mul(a, b)
    _close_ulp(out, E.silu_mul_fwd(gate, up), dtype, "fwd")
    out.backward(do.cuda())
    rg, ru = E.silu_mul_bwd(do, gate, up)
    _close_ulp(a.grad, rg, dtype, "grad_gate")
    _close_ulp(b.grad, ru, dtype, "grad_up")
    # textbook autograd of F.silu(g) * u at the reference's tolerance
    g32 = gate.float().requires_grad_(True)
    u32 = up.float().requires_grad_(True)
    (torch.nn.functional.silu(g32) * u32).backward(do.float())
    assert torch.allclose(a.grad.float().cpu(), g32.grad, atol=1e-2, rtol=1e-2)
    assert torch.allclose(b.grad.float().cpu(), u32.grad, atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("rows,inter", [(8192, 768), (1000, 100), (3, 4), (129, 1408), (7, 5)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_silu_mul_halves_matches_two_tensor_form(rows, inter, dtype):
    """The in-place-halves form is bit-identical (outputs and both gradients) to silu_mul on
    contiguous copies of the halves, and within an ulp of the oracle."""
    from pith_train_amd.operators.silu_mul import silu_mul, silu_mul_halves

    g = torch.Generator().manual_seed(rows + inter)
    gu = (torch.randn((rows, 2 * inter), generator=g) * 2).to(dtype)
    do = torch.randn((rows, inter), generator=g).to(dtype)
    a = gu.cuda().requires_grad_(True)
    out = silu_mul_halves(a)
    out.backward(do.cuda())
    b = gu.cuda().requires_grad_(True)
    ref = silu_mul(b[:, :inter].contiguous(), b[:, inter:].contiguous())
    ref.backward(do.cuda())
    assert torch.equal(out, ref)
    assert torch.equal(a.grad, b.grad)
    _close_ulp(out, E.silu_mul_fwd(gu[:, :inter].contiguous(), gu[:, inter:].contiguous()), dtype, "fwd")


def test_silu_mul_asserts():
    from pith_train_amd.operators.silu_mul import silu_mul

    a = torch.randn(4, 8, device="cuda")
    with pytest.raises(AssertionError):
        silu_mul(a, a[:, :4])
    with pytest.raises(AssertionError):
        silu_mul(a.t(), a.t())


@pytest.mark.parametrize("M,N", [(4096, 2880), (7, 5), (1, 1), (128, 768), (1000, 33)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_clamped_swiglu(M, N, dtype):
    from pith_train_amd.operators.clamped_swiglu import clamped_swiglu

    alpha, limit = 1.702, 7.0
    g = torch.Generator().manual_seed(M + N)
    gu = (torch.randn((M, 2 * N), generator=g) * 4).to(dtype)
    do = torch.randn((M, N), generator=g).to(dtype)
    x = gu.cuda().requires_grad_(True)
    out = clamped_swiglu(x, alpha, limit)
    _close_ulp(out, E.clamped_swiglu_fwd(gu, alpha, limit), dtype, "fwd")
    out.backward(do.cuda())
    ref = E.clamped_swiglu_bwd(do, gu, alpha, limit)
    _close_ulp(x.grad, ref, dtype, "bwd")
    # saturated branches: exactly zero gradient (tests/test_clamped_swiglu.py:61-95)
    gsat = gu[:, 0::2].float() > limit
    usat = gu[:, 1::2].float().abs() > limit
    assert (x.grad[:, 0::2].cpu()[gsat] == 0).all() and (x.grad[:, 1::2].cpu()[usat] == 0).all()
    # textbook expression through autograd
    y = gu.float().requires_grad_(True)
    gg, uu = y[:, 0::2].clamp(max=limit), y[:, 1::2].clamp(-limit, limit)
    ((uu + 1) * gg * torch.sigmoid(alpha * gg)).backward(do.float())
    assert torch.allclose(x.grad.float().cpu(), y.grad, atol=3e-1, rtol=5e-2)


@pytest.mark.parametrize("sizes,H", [([128, 0, 256, 128], 5760), ([128] * 32, 2880), ([256, 128], 100), ([0, 0, 128], 8)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_indexed_bias_add(sizes, H, dtype):
    from pith_train_amd.operators.indexed_bias_add import indexed_bias_add
    from pith_train_amd.operators.token_scatter import group_indices

    offs = torch.tensor(sizes).cumsum(0).to(torch.int32)
    M, G = int(offs[-1]), len(sizes)
    g = torch.Generator().manual_seed(M + H)
    x = torch.randn((M, H), generator=g).to(dtype)
    bias = (torch.randn((G, H), generator=g) * 0.02).to(dtype)
    gid = group_indices(offs.cuda(), M, torch.int64)
    xc = x.cuda().requires_grad_(True)
    bc = bias.cuda().requires_grad_(True)
    out = indexed_bias_add(xc, bc, gid, offs.cuda())
    ref = E.indexed_bias_add_fwd(x, bias, gid.cpu())
    assert torch.equal(out.cpu().view(torch.uint8), ref.view(torch.uint8))  # forward exact
    do = torch.randn((M, H), generator=g).to(dtype)
    out.backward(do.cuda())
    assert torch.equal(xc.grad.cpu(), do)  # identity
    truth = E.segment_sum(do, offs, torch.float32, accum=torch.float64)
    got = bc.grad.float().cpu()
    assert bc.grad.dtype == dtype
    tol = 2.0**-7 if dtype == torch.bfloat16 else 1e-5
    assert ((got - truth).abs() <= tol * truth.abs() + 1e-4 * truth.abs().max()).all()
    for gi, s in enumerate(sizes):  # empty groups: exactly zero rows (test_indexed_bias_add.py:141-163)
        if s == 0:
            assert (bc.grad[gi] == 0).all()
