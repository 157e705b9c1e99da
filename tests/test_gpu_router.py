"""GPU parity: router gate (softmax / top-k / weights) through the C-ABI vs the oracle.

Indices are compared exactly on every row whose answer does not hang on the last bits of an fp32
softmax (adjacent scores among the best k+1 either tie exactly, which the tie rule decides, or
differ by more than a few ulp); the kernel's selection is also checked bit-exactly against its own
scores on every row.  Weights and scores: rtol 1e-5.  Gradients: autograd of the oracle on the
same selection, to the rounding of the logits' dtype."""

import pytest
import torch

from oracle import router as R

pytestmark = pytest.mark.gpu


def _logits(T, E, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn((T, E), generator=g) * 2).to(dtype)


def _decidable_rows(values, k):
    """Rows of the oracle's fp32 values whose descending order over the best k+1 is safe against
    last-bit differences: neighbours equal, or apart by more than 1e-5 relative."""
    top = torch.sort(values.double(), dim=-1, descending=True, stable=True).values[:, : k + 1]
    gap = top[:, :-1] - top[:, 1:]
    ok = (gap == 0) | (gap > 1e-5 * top[:, :-1].abs().clamp(min=1e-30))
    return ok.all(-1)


def _grad_tol(dtype):
    return dict(rtol=2.0**-6, atol=2e-4) if dtype != torch.float32 else dict(rtol=2e-4, atol=1e-6)


SOFTMAX_CASES = [
    # E, k, T, dtype, norm, scale, num_group, topk_group
    (128, 8, 1000, torch.bfloat16, True, 1.0, 1, 1),     # Qwen3-30B-A3B gate (bf16 logits: exact ties happen)
    (128, 8, 257, torch.bfloat16, False, 1.0, 1, 1),
    (64, 6, 513, torch.float32, False, 16.0, 1, 1),      # DeepSeek-V2-Lite: greedy, scaling factor
    (160, 6, 300, torch.float32, False, 16.0, 8, 3),     # DeepSeek-V2: group_limited_greedy
    (512, 10, 130, torch.bfloat16, True, 1.0, 1, 1),     # Qwen3.5-size expert count
    (48, 3, 77, torch.float16, True, 2.0, 4, 2),         # ragged: E not a multiple of 64, T not of 4
    (8, 8, 5, torch.float32, True, 1.0, 1, 1),           # k = E
    (128, 8, 0, torch.bfloat16, True, 1.0, 1, 1),        # empty
]


@pytest.mark.parametrize("with_scores_grad", [False, True])
@pytest.mark.parametrize("E,k,T,dtype,norm,scale,ng,tg", SOFTMAX_CASES)
def test_softmax_topk(E, k, T, dtype, norm, scale, ng, tg, with_scores_grad):
    from pith_train_amd.operators.router_topk import softmax_topk

    lg = _logits(T, E, E + k + T, dtype)
    x = lg.cuda().requires_grad_(True)
    idx, w, scores = softmax_topk(x, k, norm_topk_prob=norm, scale=scale, num_group=ng, topk_group=tg, return_scores=True)
    assert idx.shape == (T, k) and idx.dtype == torch.int64 and w.dtype == torch.float32 and scores.shape == (T, E)
    if T == 0:
        return
    o_idx, o_w, o_scores = R.softmax_topk(lg, k, norm, scale, ng, tg)
    # the kernel's selection is the stable descending order of the kernel's own scores, bit for bit
    assert torch.equal(idx.cpu(), R._stable_topk(scores.detach().cpu(), k))
    raw = scores.detach().gather(-1, idx)
    own_w = (raw / raw.sum(-1, keepdim=True) if norm else raw) * scale
    torch.testing.assert_close(w.detach(), own_w, rtol=2e-6, atol=0)
    # decidability is judged on the float64 softmax, where two scores tie only if their logits do
    # (an fp32 softmax can round two different logits to one score: no exact tie for the kernel)
    exact = torch.softmax(lg.double(), -1)
    rows = _decidable_rows(torch.where(o_scores > 0, exact, torch.zeros_like(exact)) if ng > 1 else exact, k)
    if ng > 1:  # the group choice must be decidable too
        rows &= _decidable_rows(exact.view(T, ng, -1).amax(-1), tg)
    assert rows.float().mean() > 0.9
    assert torch.equal(idx.cpu()[rows], o_idx[rows])
    torch.testing.assert_close(scores.detach().cpu()[rows], o_scores[rows], rtol=1e-5, atol=1e-9)
    torch.testing.assert_close(w.detach().cpu()[rows], o_w[rows], rtol=1e-5, atol=1e-9)
    # backward on the kernel's own selection
    g = torch.Generator().manual_seed(3)
    dw = torch.randn((T, k), generator=g)
    ds = torch.randn((T, E), generator=g) * 0.1 if with_scores_grad else None
    loss = (w * dw.cuda()).sum() + ((scores * ds.cuda()).sum() if ds is not None else 0)
    loss.backward()
    ref = lg.clone().requires_grad_(True)
    _, r_w, r_scores = R.softmax_topk(ref, k, norm, scale, ng, tg, forced_idx=idx.cpu())
    ((r_w * dw).sum() + ((r_scores * ds).sum() if ds is not None else 0)).backward()
    assert x.grad.dtype == dtype
    if ng > 1:
        torch.testing.assert_close(x.grad.cpu()[rows].float(), ref.grad[rows].float(), **_grad_tol(dtype))
    else:
        torch.testing.assert_close(x.grad.cpu().float(), ref.grad.float(), **_grad_tol(dtype))


@pytest.mark.parametrize("with_scores_grad", [False, True])
@pytest.mark.parametrize("E,k,T,dtype", [(32, 4, 1000, torch.bfloat16), (128, 4, 301, torch.bfloat16), (32, 4, 64, torch.float32),
                                         (20, 5, 33, torch.float16), (32, 4, 0, torch.bfloat16)])
def test_topk_softmax(E, k, T, dtype, with_scores_grad):
    from pith_train_amd.operators.router_topk import topk_softmax

    lg = _logits(T, E, E + k + T, dtype)
    x = lg.cuda().requires_grad_(True)
    idx, w, scores = topk_softmax(x, k, return_scores=True)
    if T == 0:
        assert idx.shape == (0, k)
        return
    o_idx, o_w, o_scores = R.topk_softmax(lg, k)
    assert torch.equal(idx.cpu(), o_idx)  # logits are compared as they are: nothing to round
    torch.testing.assert_close(w.detach().cpu(), o_w, rtol=1e-5, atol=1e-9)
    torch.testing.assert_close(scores.detach().cpu(), o_scores, rtol=1e-5, atol=1e-9)
    g = torch.Generator().manual_seed(3)
    dw = torch.randn((T, k), generator=g)
    ds = torch.randn((T, E), generator=g) * 0.1 if with_scores_grad else None
    ((w * dw.cuda()).sum() + ((scores * ds.cuda()).sum() if ds is not None else 0)).backward()
    ref = lg.clone().requires_grad_(True)
    _, r_w, r_scores = R.topk_softmax(ref, k)
    ((r_w * dw).sum() + ((r_scores * ds).sum() if ds is not None else 0)).backward()
    torch.testing.assert_close(x.grad.cpu().float(), ref.grad.float(), **_grad_tol(dtype))


def test_ties_go_to_the_lower_index_and_results_are_sorted():
    from pith_train_amd.operators.router_topk import softmax_topk, topk_softmax

    lg = torch.zeros((5, 128), dtype=torch.bfloat16)
    lg[1, [100, 7, 64]] = 1.0     # three equal winners, then the tie among the zeros
    lg[2, 127] = 3.0
    lg[3] = -1.0
    lg[4, [5, 3]] = torch.tensor([2.0, 4.0]).bfloat16()
    want = torch.tensor([[0, 1, 2, 3], [7, 64, 100, 0], [127, 0, 1, 2], [0, 1, 2, 3], [3, 5, 0, 1]])
    for fn in (softmax_topk, topk_softmax):
        idx, w = fn(lg.cuda(), 4)
        assert torch.equal(idx.cpu(), want)
        assert (w[:, :-1] >= w[:, 1:]).all()


def test_router_replay_gathers_at_the_given_experts():
    from pith_train_amd.operators.router_topk import softmax_topk, topk_softmax

    T, E, k = 200, 128, 8
    lg = _logits(T, E, 11, torch.bfloat16)
    forced = torch.stack([torch.randperm(E, generator=torch.Generator().manual_seed(i))[:k] for i in range(T)])
    idx, w, scores = softmax_topk(lg.cuda(), k, forced_idx=forced.cuda(), return_scores=True)
    assert torch.equal(idx.cpu(), forced)
    assert torch.equal(w, scores.gather(-1, idx))
    _, o_w, _ = R.softmax_topk(lg, k, forced_idx=forced)
    torch.testing.assert_close(w.cpu(), o_w, rtol=1e-5, atol=1e-9)
    idx, w = topk_softmax(lg.cuda(), k, forced_idx=forced.cuda())
    _, o_w, _ = R.topk_softmax(lg, k, forced_idx=forced)
    assert torch.equal(idx.cpu(), forced)
    torch.testing.assert_close(w.cpu(), o_w, rtol=1e-5, atol=1e-9)


def _reference_gate(kind, x, weight, bias, k, lb_fn, **kw):
    """The reference gates' tensor expressions, evaluated by torch on the GPU."""
    import torch.nn.functional as F

    if kind == "gpt_oss":
        logits = F.linear(x, weight, bias)
        top_l, idx = torch.topk(logits, k=k, dim=-1, sorted=True)
        w = F.softmax(top_l, dim=-1, dtype=torch.float32)
        scores = logits.softmax(dim=-1, dtype=torch.float32)
    else:
        logits = F.linear(x.float(), weight.float()) if kind == "deepseek" else F.linear(x, weight)
        scores = logits.softmax(dim=-1, dtype=torch.float32)
        w, idx = torch.topk(scores, k=k, dim=-1, sorted=True)
        if kw.get("norm"):
            w = w / w.sum(dim=-1, keepdim=True)
        w = w * kw.get("scale", 1.0)
    lb = lb_fn(scores, idx, weight.shape[0], k) if lb_fn is not None else None
    return idx, w, lb


@pytest.mark.parametrize("kind", ["qwen3", "deepseek", "gpt_oss"])
@pytest.mark.parametrize("with_lb", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gate_modules_against_the_tensor_expressions(kind, with_lb, dtype):
    """The gate modules (library logits GEMM + the kernel) against the reference's expressions on
    the same device.  fp32 parameters (no two logits tie): the same experts on every row, the same
    weights and the same gradients of the gate weight and the hidden states, load-balance hook
    included.  bf16 parameters (logits tie now and then and torch.topk picks its own winner): the
    same multiset of weights on every row, the same experts on most."""
    from pith_train_amd.modules import gates as G

    T, H, E, k = 512, 256, {"qwen3": 128, "deepseek": 64, "gpt_oss": 32}[kind], {"qwen3": 8, "deepseek": 6, "gpt_oss": 4}[kind]
    g = torch.Generator().manual_seed(17)
    x = torch.randn((T, H), generator=g).to(dtype).cuda()
    wt = (torch.randn((E, H), generator=g) * 0.1).to(dtype).cuda()
    if kind == "qwen3":
        mod, kw = G.Qwen3MoeGate(E, H, k, norm_topk_prob=True), dict(norm=True)
    elif kind == "deepseek":
        mod, kw = G.DeepSeekV2MoEGate(E, H, k, routed_scaling_factor=16.0), dict(scale=16.0)
    else:
        mod, kw = G.GptOssTopKRouter(E, H, k), {}
    mod = mod.cuda().to(dtype)
    with torch.no_grad():
        mod.weight.copy_(wt)
        if kind == "gpt_oss":
            mod.bias.copy_((torch.randn(E, generator=g) * 0.1).to(dtype))

    def lb_fn(scores, idx, n_exp, top_k):  # Switch-style: fraction routed x mean probability
        f = torch.zeros(n_exp, device=scores.device).index_add_(0, idx.reshape(-1), torch.ones(idx.numel(), device=scores.device))
        return 0.01 * n_exp * (f / idx.numel() * scores.mean(0)).sum()

    mod.load_balance_loss_fn = lb_fn if with_lb else None
    dw = torch.randn((T, k), generator=g).cuda()
    xa = x.clone().requires_grad_(True)
    idx, w, lb = mod(xa)
    assert (lb is None) == (not with_lb)
    (w * dw).sum().backward()
    xb = x.clone().requires_grad_(True)
    wb = mod.weight.detach().clone().requires_grad_(True)
    bb = mod.bias.detach().clone().requires_grad_(True) if kind == "gpt_oss" else None
    r_idx, r_w, r_lb = _reference_gate(kind, xb, wb, bb, k, lb_fn if with_lb else None, **kw)
    ((r_w * dw).sum() + (r_lb * T if with_lb else 0)).backward()
    same = (idx.sort(-1).values == r_idx.sort(-1).values).all(-1)
    torch.testing.assert_close(w.sort(-1).values, r_w.sort(-1).values, rtol=1e-5, atol=1e-8)
    if with_lb:
        torch.testing.assert_close(lb, r_lb, rtol=1e-4, atol=1e-8)
    if dtype == torch.bfloat16:
        assert same.float().mean() > 0.9
        return
    assert same.all()
    assert torch.equal(idx, r_idx)  # no ties: descending order is unique
    torch.testing.assert_close(mod.weight.grad, wb.grad, rtol=1e-3, atol=1e-4 * float(wb.grad.abs().max()))
    torch.testing.assert_close(xa.grad, xb.grad, rtol=1e-3, atol=1e-4 * float(xb.grad.abs().max()))
    if kind == "gpt_oss":
        torch.testing.assert_close(mod.bias.grad, bb.grad, rtol=1e-3, atol=1e-4 * float(bb.grad.abs().max()))
