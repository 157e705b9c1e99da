"""Pins the non-quantisation oracles on the CPU against independent formulations."""

import pytest
import torch

from oracle import dedup as OD
from oracle import epilogue as E
from oracle import fp8 as Q
from oracle import gemm as G
from oracle import moe as OM
from oracle import permute as OP


def test_gemm_oracle_vs_elementwise_definition():
    torch.manual_seed(0)
    M, N, K = 5, 130, 200
    x = torch.randn(M, K).bfloat16()
    w = (torch.randn(N, K) * 0.1).bfloat16()
    a, sa, _, _ = Q.fp8cast_rowwise_transpose(x)
    b, sb, _, _ = Q.fp8cast_blockwise_transpose(w)
    out = G.gemm_nt_dense(a, sa, b, sb, torch.float64)
    for m, n in [(0, 0), (4, 129), (2, 128), (3, 7)]:
        acc = 0.0
        for k in range(K):
            acc += float(a[m, k].float()) * float(sa[m, k // 128]) * float(b[n, k].float()) * float(sb[n // 128, k // 128])
        assert abs(acc - float(out[m, n])) <= 1e-9 * max(1.0, abs(acc))
    # quantise -> dequantise -> matmul stays close to the unquantised product
    assert G.calc_diff(out, x.double() @ w.double().T) < 1e-3


def test_grouped_gemm_oracles_vs_per_group_matmul():
    torch.manual_seed(1)
    offs = torch.tensor([128, 128, 384], dtype=torch.int32)
    M, K, N, Gn = 384, 256, 128, 3
    x, dy = torch.randn(M, K).bfloat16(), torch.randn(M, N).bfloat16()
    w = (torch.randn(Gn, N, K) * 0.05).bfloat16()
    y, saved = G.fp8_grouped_linear_forward(x, w, offs)
    ref = torch.cat([x[:128].double() @ w[0].double().T, x[128:].double() @ w[2].double().T])
    assert G.calc_diff(y, ref) < 1e-3
    gi, gw = G.fp8_grouped_linear_backward(dy, saved, offs, Gn)
    assert torch.all(gw[1] == 0)
    assert G.calc_diff(gw[2], dy[128:].double().T @ x[128:].double()) < 1e-3
    assert G.calc_diff(gi[:128], dy[:128].double() @ w[0].double()) < 1e-3
    assert G.calc_diff(G.bf16_grouped_mm(x, w, offs), ref) < 1e-4


@pytest.mark.parametrize("m,G", [(1000, 8), (5, 3), (4096, 128)])
def test_scatter_oracle_invariants(m, G):
    g = torch.Generator().manual_seed(m)
    x = torch.randn((m, 16), generator=g)
    e = torch.randint(0, G, (m,), generator=g)
    out, rev, offs, ks, kst, buf = OP.scatter_for_grouped_gemm(x, e, G)
    assert torch.equal(out[rev], x)  # out[reverse] == in
    counts = torch.bincount(e, minlength=G)
    assert ks == ((counts + 127) // 128 * 128).tolist() and offs.tolist() == torch.tensor(ks).cumsum(0).tolist()
    start = 0
    for gi in range(G):  # rows of a group are its tokens in ascending source order, then zeros
        rows = (e == gi).nonzero().view(-1)
        assert torch.equal(out[start : start + rows.numel()], x[rows])
        assert torch.all(out[start + rows.numel() : start + ks[gi]] == 0)
        start += ks[gi]
    assert buf.shape[0] % 1024 == 0 and torch.all(buf[out.shape[0] :] == 0)
    assert torch.equal(OP.precompute_group_indices(offs, out.shape[0]).long(),
                       torch.repeat_interleave(torch.arange(G), torch.tensor(ks)))
    go = torch.randn(out.shape, generator=g)
    assert torch.equal(OP.scatter_backward(go, rev), go[rev])
    idx = torch.randint(0, 50, (300,), generator=g)
    gg = torch.randn((300, 4), generator=g)
    ref = torch.zeros(50, 4).index_add_(0, idx, gg)
    assert torch.allclose(OP.padded_index_gather_backward(gg, idx, 50), ref)


@pytest.mark.parametrize("m,k,E,ep", [(32, 8, 32, 8), (100, 8, 32, 4), (10, 4, 8, 2), (1, 2, 8, 4), (64, 1, 8, 4)])
def test_dedup_oracle_vs_bruteforce(m, k, E, ep):
    g = torch.Generator().manual_seed(m * 7 + k)
    epr = E // ep
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(m)])
    tper, dpg, disp, idxs, exp, meta = OD.fused_dedup_prepare_dispatch(ids, E, ep, epr)
    flat = ids.view(-1).tolist()
    # python brute force
    per_e = [[f for f, e in enumerate(flat) if e == ee] for ee in range(E)]
    assert idxs.tolist() == [f for lst in per_e for f in lst]
    sent = [[t for t in range(m) if any(e // epr == gg for e in ids[t].tolist())] for gg in range(ep)]
    assert dpg.tolist() == [len(s) for s in sent]
    assert disp[: sum(len(s) for s in sent)].tolist() == [t for s in sent for t in s]
    assert tper.tolist() == [sum(len(per_e[gg * epr + j]) for j in range(epr)) for gg in range(ep)]
    want = [sent[flat[f] // epr].index(f // k) for f in idxs.tolist()]
    assert exp.tolist() == want
    mm = meta.view(ep, epr + 1)
    assert mm[:, epr].tolist() == dpg.tolist() and mm[:, :epr].reshape(-1).tolist() == [len(l) for l in per_e]


def test_build_and_adjust_oracles():
    counts = torch.tensor([2, 0, 1, 3])
    idx, splits = OD.build_expert_idxs(counts, 2, 2)
    assert idx.tolist() == [0, 0, 0, 1, 1, 1] and splits.tolist() == [2, 4]
    adj = OD.adjust_expand_idx(torch.tensor([0, 1, 0, 1, 2, 0]), torch.tensor([5, 7]), splits)
    assert adj.tolist() == [0, 1, 5, 6, 7, 5]


def test_epilogue_oracles_vs_autograd():
    torch.manual_seed(0)
    g = (torch.randn(64, 32) * 3).requires_grad_(True)
    u = torch.randn(64, 32).requires_grad_(True)
    do = torch.randn(64, 32)
    (torch.nn.functional.silu(g) * u).backward(do)
    dg, du = E.silu_mul_bwd(do, g.detach(), u.detach())
    assert torch.allclose(dg, g.grad, atol=1e-5) and torch.allclose(du, u.grad, atol=1e-5)
    assert torch.allclose(E.silu_mul_fwd(g.detach(), u.detach()), torch.nn.functional.silu(g) * u, atol=1e-6)
    gu = (torch.randn(16, 40) * 5).requires_grad_(True)
    gg, uu = gu[:, 0::2].clamp(max=7.0), gu[:, 1::2].clamp(-7.0, 7.0)
    out = (uu + 1) * gg * torch.sigmoid(1.702 * gg)
    do2 = torch.randn(16, 20)
    out.backward(do2)
    assert torch.allclose(E.clamped_swiglu_fwd(gu.detach(), 1.702, 7.0), out, atol=1e-5)
    assert torch.allclose(E.clamped_swiglu_bwd(do2, gu.detach(), 1.702, 7.0), gu.grad, atol=1e-5)
    x = torch.randn(6, 4)
    offs = torch.tensor([2, 2, 6], dtype=torch.int32)
    s = E.segment_sum(x, offs, torch.float32)
    assert torch.allclose(s[0], x[:2].sum(0)) and torch.all(s[1] == 0) and torch.allclose(s[2], x[2:].sum(0))
    assert torch.allclose(E.segment_sum(x, torch.tensor([2, 2, 9], dtype=torch.int32), torch.float32)[2], x[2:].sum(0))


@pytest.mark.parametrize("kind", ["split", "fused", "gpt_oss"])
def test_moe_oracle_fp8_close_to_bf16_and_autograd(kind):
    """The FP8 layer oracle agrees with the BF16 one (calc_diff), and the BF16 one with autograd."""
    E_, H, I, T, k = 4, 128, 128, 96, 2
    ids = OM.make_routing(T, E_, k, seed=0)
    g = torch.Generator().manual_seed(0)
    x = torch.randn((T, H), generator=g).bfloat16()
    tokens = x.unsqueeze(1).expand(-1, k, -1).reshape(-1, H).contiguous()
    eidx = ids.reshape(-1)
    dy = torch.randn((T * k, H), generator=g).bfloat16()
    r = lambda *s: (torch.randn(s, generator=g) * 0.05).bfloat16()  # noqa: E731
    if kind == "split":
        w = {"gate_proj": r(E_, I, H), "up_proj": r(E_, I, H), "down_proj": r(E_, H, I)}
    elif kind == "fused":
        w = {"gate_up_proj": r(E_, 2 * I, H), "down_proj": r(E_, H, I)}
    else:
        w = {"gate_up_proj": r(E_, 2 * I, H), "gate_up_proj_bias": r(E_, 2 * I), "down_proj": r(E_, H, I), "down_proj_bias": r(E_, H)}
    a = OM.moe_layer_fwd_bwd(tokens, eidx, w, dy, E_, kind=kind, fp8=True)
    b = OM.moe_layer_fwd_bwd(tokens, eidx, w, dy, E_, kind=kind, fp8=False)
    for key in ["out", "grad_tokens"] + list(w):
        lim = 5e-3 if "bias" not in key else 1e-2
        assert G.calc_diff(a[key].float(), b[key].float()) < lim, key
    # fp32 autograd of the textbook expression
    wf = {n: v.float().requires_grad_(True) for n, v in w.items()}
    tf = tokens.float().requires_grad_(True)
    outs = torch.zeros(T * k, H)
    for e in range(E_):
        rows = (eidx == e).nonzero().view(-1)
        xe = tf[rows]
        if kind == "split":
            h = torch.nn.functional.silu(xe @ wf["gate_proj"][e].T) * (xe @ wf["up_proj"][e].T)
            ye = h @ wf["down_proj"][e].T
        elif kind == "fused":
            gu = xe @ wf["gate_up_proj"][e].T
            ye = (torch.nn.functional.silu(gu[:, :I]) * gu[:, I:]) @ wf["down_proj"][e].T
        else:
            gu = xe @ wf["gate_up_proj"][e].T + wf["gate_up_proj_bias"][e]
            gg, uu = gu[:, 0::2].clamp(max=7.0), gu[:, 1::2].clamp(-7.0, 7.0)
            ye = ((uu + 1) * gg * torch.sigmoid(1.702 * gg)) @ wf["down_proj"][e].T + wf["down_proj_bias"][e]
        outs = outs.index_add(0, rows, ye)
    outs.backward(dy.float())
    assert G.calc_diff(b["out"].float(), outs.detach()) < 1e-3
    assert G.calc_diff(b["grad_tokens"].float(), tf.grad) < 1e-3
    for n in w:
        assert G.calc_diff(b[n].float(), wf[n].grad) < (1e-3 if "bias" not in n else 1e-2), n
