"""GPU parity: permute / unpermute and dedup index construction vs the CPU oracle, bit for bit.

Also re-expresses the invariants the reference's own tests assert
(tests/test_grouped_linear_correctness.py:330-429, tests/test_ep_dedup_dispatch.py:134-171).
"""

import pytest
import torch

from oracle import dedup as OD
from oracle import permute as OP

pytestmark = pytest.mark.gpu


def _ts():
    from pith_train_amd.operators import token_scatter as T

    return T


SCATTER = [(1024, 8, 256, torch.bfloat16), (100, 4, 100, torch.float32), (5000, 128, 64, torch.bfloat16),
           (1, 8, 1, torch.float32), (777, 1, 128, torch.bfloat16), (4096, 64, 2048, torch.bfloat16),
           (300, 300, 16, torch.float16), (65536, 128, 128, torch.bfloat16),
           (40000, 2048, 8, torch.bfloat16), (20000, 1001, 8, torch.float32)]


@pytest.mark.parametrize("m,G,H,dtype", SCATTER)
def test_scatter_for_grouped_gemm(m, G, H, dtype):
    T = _ts()
    g = torch.Generator().manual_seed(m + G)
    x = torch.randn((m, H), generator=g).to(dtype)
    e = torch.randint(0, G, (m,), generator=g)
    if G > 2:
        e[e == 1] = 0  # force an empty group
    ref_out, ref_rev, ref_offs, ref_ks, ref_kst, ref_buf = OP.scatter_for_grouped_gemm(x, e, G)
    out, rev, offs, ks, kst = T.scatter_for_grouped_gemm(x.cuda(), e.cuda(), G)
    assert ks == ref_ks and isinstance(ks, list)
    assert torch.equal(offs.cpu(), ref_offs) and offs.dtype == torch.int32 and offs.shape == (G,)
    assert torch.equal(kst.cpu(), ref_kst) and kst.dtype == torch.int32
    assert torch.equal(rev.cpu(), ref_rev) and rev.dtype == torch.int64
    assert out.shape == ref_out.shape and out.dtype == dtype
    assert torch.equal(out.cpu().view(torch.uint8), ref_out.contiguous().view(torch.uint8))
    # the view sits on a buffer padded to 1024 rows whose tail is zero
    rows = out.untyped_storage().nbytes() // (H * out.element_size())
    assert rows % 1024 == 0 and rows >= ref_buf.shape[0]
    full = torch.as_strided(out, (ref_buf.shape[0], H), (H, 1))
    assert torch.equal(full.cpu().view(torch.uint8), ref_buf.view(torch.uint8))
    # invariants of the reference's _verify_scatter_result
    assert torch.equal(out[rev].cpu(), x)
    assert int(offs[-1]) == out.shape[0] and all(k % 128 == 0 for k in ks)


def test_scatter_empty_and_backward():
    T = _ts()
    out, rev, offs, ks, kst = T.scatter_for_grouped_gemm(
        torch.empty((0, 64), device="cuda"), torch.empty((0,), dtype=torch.int64, device="cuda"), 8)
    assert out.shape == (0, 64) and rev.shape == (0,) and offs.shape == (0,) and ks == [] and kst.shape == (0,)
    g = torch.Generator().manual_seed(1)
    x = torch.randn((500, 96), generator=g).bfloat16().cuda().requires_grad_(True)
    e = torch.randint(0, 6, (500,), generator=g).cuda()
    out, rev, offs, ks, kst = T.scatter_for_grouped_gemm(x, e, 6)
    go = torch.randn(out.shape, generator=g).bfloat16().cuda()
    out.backward(go)
    assert torch.equal(x.grad, go[rev])


@pytest.mark.parametrize("rows,n,H,dtype", [(1000, 4000, 128, torch.bfloat16), (64, 10, 100, torch.float32),
                                             (300, 300, 2048, torch.bfloat16), (50, 5000, 8, torch.float32)])
def test_padded_index_gather_fwd_bwd(rows, n, H, dtype):
    T = _ts()
    g = torch.Generator().manual_seed(rows + n)
    x = torch.randn((rows, H), generator=g).to(dtype)
    idx = torch.randint(0, rows, (n,), generator=g)
    xc = x.cuda().requires_grad_(True)
    out = T.padded_index_gather(xc, idx.cuda())
    assert torch.equal(out.cpu(), OP.padded_index_gather(x, idx))
    assert out.untyped_storage().nbytes() // (H * out.element_size()) % 1024 == 0
    go = torch.randn((n, H), generator=g).to(dtype)
    out.backward(go.cuda())
    ref = OP.padded_index_gather_backward(go, idx, rows)
    # sums run in ascending source order in fp32 on both sides: bit-exact
    assert torch.equal(xc.grad.cpu().view(torch.uint8), ref.view(torch.uint8))


def test_fused_expand_scatter_matches_two_step():
    T = _ts()
    g = torch.Generator().manual_seed(9)
    uniq = torch.randn((700, 256), generator=g).bfloat16().cuda()
    expand = torch.randint(0, 700, (2000,), generator=g).cuda()
    e = torch.randint(0, 16, (2000,), generator=g).cuda()
    a = uniq.clone().requires_grad_(True)
    b = uniq.clone().requires_grad_(True)
    o1, r1, f1, k1, t1 = T.scatter_for_grouped_gemm(T.padded_index_gather(a, expand), e, 16)
    o2, r2, f2, k2, t2 = T.scatter_for_grouped_gemm(b, e, 16, pre_index=expand)
    assert torch.equal(o1, o2) and torch.equal(r1, r2) and torch.equal(f1, f2) and k1 == k2
    go = torch.randn(o1.shape, generator=torch.Generator().manual_seed(3)).bfloat16().cuda()
    o1.backward(go)
    o2.backward(go)
    assert torch.equal(a.grad, b.grad)


def test_group_indices():
    T = _ts()
    offs = torch.tensor([128, 128, 512, 640], dtype=torch.int32)
    for M in (640, 700, 1):
        ref = OP.precompute_group_indices(offs, M)
        got = T.group_indices(offs.cuda(), M, torch.int32)
        assert torch.equal(got.cpu(), ref)
        assert torch.equal(T.group_indices(offs.cuda(), M, torch.int64).cpu(), ref.long())


DEDUP = [(32, 8, 32, 8), (64, 4, 16, 4), (128, 8, 64, 8), (16, 2, 8, 4), (100, 8, 32, 4), (256, 8, 128, 16), (10, 4, 8, 2),
         (32, 1, 8, 4), (32, 4, 8, 2), (2, 2, 4, 2), (1, 2, 8, 4), (2048, 8, 128, 2), (32768, 8, 128, 8), (1000, 6, 64, 32)]


@pytest.mark.parametrize("m,k,E,ep", DEDUP)
@pytest.mark.parametrize("seed", [0, 42])
def test_fused_dedup_prepare_dispatch(m, k, E, ep, seed):
    from pith_train_amd.operators.ep_dispatch import fused_dedup_prepare_dispatch

    g = torch.Generator().manual_seed(seed)
    epr = E // ep
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(min(m, 4096))])
    if m > 4096:
        ids = ids.repeat(m // 4096, 1)[torch.randperm(m, generator=g)]
    ref = OD.fused_dedup_prepare_dispatch(ids, E, ep, epr)
    got = fused_dedup_prepare_dispatch(ids.cuda(), E, ep, epr)
    names = ("tokens_per_ep_rank", "dedup_tokens_per_gpu", "dispatch_token_idxs", "idxs", "expand_idx", "send_meta")
    total_dedup = int(ref[1].sum())
    for name, a, r in zip(names, got, ref):
        a = a.cpu()
        assert a.dtype == torch.int64 and a.shape == r.shape, name
        if name == "dispatch_token_idxs":
            a, r = a[:total_dedup], r[:total_dedup]
        assert torch.equal(a, r), name
    # invariant: dispatch_token_idxs[gpu_start + expand_idx] == token id of the sorted slot
    tper, dpg, disp, idxs, exp, meta = (t.cpu() for t in got)
    gs = dpg.cumsum(0) - dpg
    rank = ids.view(-1)[idxs] // epr
    assert torch.equal(disp[gs[rank] + exp], idxs // k)


def test_dedup_duplicate_experts_in_a_row_and_empty():
    from pith_train_amd.operators.ep_dispatch import fused_dedup_prepare_dispatch

    ids = torch.tensor([[3, 3, 1], [0, 7, 7], [5, 5, 5]])
    ref = OD.fused_dedup_prepare_dispatch(ids, 8, 4, 2)
    got = fused_dedup_prepare_dispatch(ids.cuda(), 8, 4, 2)
    n = int(ref[1].sum())
    for i, (a, r) in enumerate(zip(got, ref)):
        a = a.cpu()
        assert torch.equal(a[:n], r[:n]) if i == 2 else torch.equal(a, r), i
    z = fused_dedup_prepare_dispatch(torch.empty((0, 4), dtype=torch.int64, device="cuda"), 8, 2, 4)
    assert z[0].tolist() == [0, 0] and z[2].numel() == 0 and z[5].numel() == 2 * 5 and not z[5].any()


@pytest.mark.parametrize("ep,epr", [(2, 4), (8, 16), (4, 1), (32, 2)])
def test_build_expert_idxs_and_adjust(ep, epr):
    from pith_train_amd.operators.ep_dispatch import adjust_expand_idx, build_expert_idxs

    g = torch.Generator().manual_seed(ep * 10 + epr)
    counts = torch.randint(0, 50, (ep * epr,), generator=g)
    counts[0] = 0
    ref_idx, ref_splits = OD.build_expert_idxs(counts, ep, epr)
    idx, splits = build_expert_idxs(counts.cuda(), ep, epr, max_total=int(counts.sum()) + 100)
    assert torch.equal(splits.cpu(), ref_splits)
    assert torch.equal(idx[: ref_idx.numel()].cpu(), ref_idx)
    n = int(ref_splits.sum())
    recv = torch.randint(0, 20, (n,), generator=g)
    dedup = torch.randint(0, 30, (ep, 3), generator=g)[:, 1]  # strided view like recv_meta_2d[:, epr]
    ref = OD.adjust_expand_idx(recv, dedup, ref_splits)
    got = adjust_expand_idx(recv.cuda(), dedup.cuda(), splits)
    assert torch.equal(got.cpu(), ref)
    zi, zs = build_expert_idxs(torch.zeros(ep * epr, dtype=torch.int64, device="cuda"), ep, epr, 0)
    assert zs.tolist() == [0] * ep


def test_receiver_simulation_roundtrip():
    """Sender -> receiver in one process (the technique of tests/test_ep_dedup_dispatch.py:174-231):
    rows expanded with the adjusted expand_idx equal the rows a non-dedup dispatch would deliver."""
    from pith_train_amd.operators.ep_dispatch import adjust_expand_idx, build_expert_idxs, fused_dedup_prepare_dispatch

    ep, epr, k, m, H = 4, 8, 6, 200, 32
    E = ep * epr
    g = torch.Generator().manual_seed(4)
    hs = [torch.randn((m, H), generator=g) for _ in range(ep)]
    ids = [torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(m)]) for _ in range(ep)]
    outs = [fused_dedup_prepare_dispatch(i.cuda(), E, ep, epr) for i in ids]
    for recv in range(ep):
        metas = [o[5].view(ep, epr + 1)[recv] for o in outs]
        tpe = torch.cat([mm[:epr] for mm in metas])
        dedup_from = torch.stack([mm[epr] for mm in metas])
        eidx, splits = build_expert_idxs(tpe, ep, epr, max_total=m * k * ep)
        chunks, rows, refs = [], [], []
        for s, o in enumerate(outs):
            tper, dpg, disp, idxs, exp, _ = o
            st = int((tper.cumsum(0) - tper)[recv]); n = int(tper[recv])
            chunks.append(exp[st : st + n])
            gs = int((dpg.cumsum(0) - dpg)[recv]); nd = int(dpg[recv])
            rows.append(hs[s].cuda()[disp[gs : gs + nd]])
            refs.append(hs[s].cuda()[idxs[st : st + n] // k])
        adj = adjust_expand_idx(torch.cat(chunks), dedup_from, splits)
        assert torch.equal(torch.cat(rows)[adj], torch.cat(refs))
        ref_e, ref_adj, _, _ = OD.simulate_receiver_expand_idx(ids, recv, ep, epr)
        assert torch.equal(adj.cpu(), ref_adj) and torch.equal(eidx[: ref_e.numel()].cpu(), ref_e)
