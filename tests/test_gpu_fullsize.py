"""Parity at the benchmark's full sizes (Qwen3-30B-A3B MoE layer: 8192 tokens x top-8, 128 experts,
hidden 2048, intermediate 768).

The whole layer is too large for the CPU oracle in a test, so parity is shown two ways:
  * the oracle recomputes the layer for a few experts only (their rows, their weights): an
    expert's rows never interact with another expert's in forward, dgrad or wgrad, and its 128-row
    column-scale blocks depend only on the stable order of its own rows;
  * size-independent properties: the fused and unfused compositions agree bit for bit, every
    routed row is written exactly once, quantisation round-trips within half an FP8 step.
"""

import pytest
import torch

from oracle import gemm as G
from oracle import moe as OM

pytestmark = pytest.mark.gpu

E, H, I, T, K_TOP = 128, 2048, 768, 8192, 8


def _inputs():
    ids = OM.make_routing(T, E, K_TOP, seed=0)
    g = torch.Generator().manual_seed(0)
    x = torch.randn((T, H), generator=g).bfloat16()
    dy = torch.randn((T * K_TOP, H), generator=g).bfloat16()
    w = {"gate_up_proj": (torch.randn((E, 2 * I, H), generator=g) * 0.02).bfloat16(),
         "down_proj": (torch.randn((E, H, I), generator=g) * 0.02).bfloat16()}
    tokens = x.unsqueeze(1).expand(-1, K_TOP, -1).reshape(-1, H).contiguous()
    return tokens, ids.reshape(-1), dy, w


def _run(tokens, eidx, dy, w, **kw):
    from pith_train_amd.dualpipe_utils import FP8WeightCacheControl
    from pith_train_amd.modules import experts as X

    mod = X.Qwen35MoeExperts(H, I, E).cuda().to(torch.bfloat16)
    with torch.no_grad():
        mod.gate_up_proj.weight.copy_(w["gate_up_proj"].cuda())
        mod.down_proj.weight.copy_(w["down_proj"].cuda())
    FP8WeightCacheControl.step()
    tok = tokens.cuda().requires_grad_(True)
    out = X.forward_stage3(mod, tok, eidx.cuda(), E, **kw)
    out.backward(dy.cuda())
    return out.detach(), tok.grad, mod.gate_up_proj.weight.grad, mod.down_proj.weight.grad


def _close(got, ref, what, rel=5e-2, diff=1e-3):
    got, ref = got.float().cpu().double(), ref.double()
    assert torch.isfinite(got).all(), what
    d = G.calc_diff(got, ref)
    assert d < diff, f"{what}: calc_diff {d:.3e}"
    assert (got - ref).abs().max() <= rel * ref.abs().max() + 1e-30, f"{what}: max err"


def test_full_size_layer_against_the_oracle_on_sampled_experts():
    tokens, eidx, dy, w = _inputs()
    out, gtok, g_gu, g_dn = _run(tokens, eidx, dy, w)
    assert out.shape == (T * K_TOP, H) and torch.isfinite(out.float()).all()
    for e in (0, 37, 127):
        rows = (eidx == e).nonzero().flatten()  # ascending = the stable order inside the group
        assert rows.numel() > 0
        sub_w = {k: v[e : e + 1] for k, v in w.items()}
        ref = OM.moe_layer_fwd_bwd(tokens[rows], torch.zeros_like(rows), sub_w, dy[rows], 1, kind="fused", fp8=True,
                                   accum=torch.float64)
        _close(out[rows.cuda()], ref["out"], f"expert {e} out")
        _close(gtok[rows.cuda()], ref["grad_tokens"], f"expert {e} grad_tokens")
        _close(g_gu[e], ref["gate_up_proj"][0], f"expert {e} gate_up grad")
        _close(g_dn[e], ref["down_proj"][0], f"expert {e} down grad")


def test_full_size_fused_and_unfused_compositions_agree_bit_for_bit():
    tokens, eidx, dy, w = _inputs()
    a = _run(tokens, eidx, dy, w, fuse_permute=True)
    b = _run(tokens, eidx, dy, w, fuse_permute=False)
    for x, y, what in zip(a, b, ("out", "grad_tokens", "gate_up grad", "down grad")):
        assert torch.equal(x, y), what


def test_full_size_scatter_covers_every_row_once_and_quant_round_trips():
    from pith_train_amd.operators.deepgemm_quantize import fp8cast_rowwise_colwise
    from pith_train_amd.operators.token_scatter import group_rows_with_sizes, scatter_for_grouped_gemm

    tokens, eidx, _, _ = _inputs()
    tok = tokens.cuda()
    xp, reverse, offs, ks, ks_tensor = scatter_for_grouped_gemm(tok, eidx.cuda(), E)
    _, offs2, ks2, _, src_of = group_rows_with_sizes(eidx.cuda(), E)
    assert torch.equal(offs, offs2) and ks == ks2 and sum(ks) == xp.shape[0] and all(k % 128 == 0 for k in ks)
    valid = src_of >= 0
    assert int(valid.sum()) == T * K_TOP
    assert torch.equal(torch.sort(src_of[valid].long()).values, torch.arange(T * K_TOP, device="cuda"))
    assert torch.equal(reverse[src_of[valid].long()], valid.nonzero().flatten())  # the two maps are inverses
    assert torch.equal(xp[reverse], tok)                                          # encode -> decode round trip
    assert not xp[~valid].any()                                                   # padding rows are zero
    q, s, qc, sc = fp8cast_rowwise_colwise(xp)
    assert (torch.frexp(s)[0] == 0.5).all() and (torch.frexp(sc)[0] == 0.5).all()  # powers of two
    deq = q.float().view(xp.shape[0], -1, 128) * s.unsqueeze(-1)
    err = (deq.view_as(xp) - xp.float()).abs().view(xp.shape[0], -1, 128)
    # an e4m3 value is within 2**-4 relative (half a step of the 3-bit mantissa) or half a subnormal step
    bound = xp.float().abs().view(xp.shape[0], -1, 128) * 2.0**-4 + s.unsqueeze(-1) * 2.0**-10
    assert (err <= bound).all()


def test_full_size_dense_weight_gradient_split_over_the_reduction_matches_the_single_pass():
    """The k/v and q projections' weight gradients at 32768 tokens (512 x 2048 and 4096 x 2048
    outputs, reduction 32768): the operator cuts the reduction into ranges; the sum of the ranges
    equals the single-pass kernel's result up to fp32 summation order, and sampled output rows
    equal the oracle's float64 product."""
    from oracle import fp8 as Q
    from pith_train_amd import _lib
    from pith_train_amd.operators import deepgemm_quantize as DQ
    from pith_train_amd.operators.linear import _fp8_gemm_nt, _split_k

    tokens = 32768
    g = torch.Generator().manual_seed(3)
    for n_out, n_in in ((512, 2048), (4096, 2048)):
        grad = torch.randn((tokens, n_out), generator=g).bfloat16().cuda()
        x = torch.randn((tokens, n_in), generator=g).bfloat16().cuda()
        _, _, gt, gt_s = DQ.fp8cast_rowwise_transpose(grad)            # grad^T rows, 1x128 scales
        _, _, xt, xt_s = DQ.fp8cast_rowwise_blockwise_transpose(x)     # x^T, 128x128 scales
        assert _split_k(n_out, n_in, tokens)[0] > 1
        split = _fp8_gemm_nt(gt, gt_s, xt, xt_s, n_out, n_in, "cuda", torch.float32)
        single = torch.empty((n_out, n_in), device="cuda", dtype=torch.float32)
        _lib.call("pt_gemm_nt_dense", gt.data_ptr(), gt_s.data_ptr(), xt.data_ptr(), xt_s.data_ptr(), single.data_ptr(),
                  _lib.dtype_code(torch.float32), n_out, n_in, tokens, _lib.stream_ptr("cuda"))
        scale = single.abs().mean().item()
        assert (split - single).abs().max().item() <= 1e-4 * scale * 50, "more than fp32 reordering noise"
        rows = torch.tensor([0, 127, 128, n_out - 1])
        ref = G.gemm_nt_dense(gt[rows].cpu(), gt_s[rows].cpu(), xt.cpu(), xt_s.cpu(), torch.float64)
        got = split[rows].cpu().double()
        assert ((got - ref).abs() <= 1e-2 * ref.abs() + 1e-2 * ref.pow(2).mean().sqrt()).all()
