"""GPU parity: the FP8 decompression of the MLA latent (kv_b) and its backward against the oracle's
dense FP8 linear (same quantised operands, fp64 accumulation), at DeepSeek-V2-Lite's shapes."""

import pytest
import torch

from oracle import gemm as G

pytestmark = pytest.mark.gpu


def _close(got, ref, what, rel=1e-2, diff=1e-3):
    got, ref = got.detach().float().cpu().double(), ref.double()
    assert got.shape == ref.shape, f"{what}: {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert G.calc_diff(got, ref) < diff, what
    assert (got - ref).abs().max() <= rel * ref.abs().max() + 1e-30, what


@pytest.mark.parametrize("b,n,heads,nope,vdim,rank", [(1, 4096, 16, 128, 128, 512), (2, 384, 4, 64, 32, 256)])
def test_decompress_forward_backward(b, n, heads, nope, vdim, rank):
    from pith_train_amd.operators.deepgemm_quantize import fp8cast_blockwise_transpose
    from pith_train_amd.operators.mla_decompress import mla_decompress, mla_decompress_backward

    out_features = heads * (nope + vdim)
    g = torch.Generator().manual_seed(n)
    nkv = torch.randn((b, n, rank), generator=g).bfloat16()
    w = (torch.randn((out_features, rank), generator=g) * 0.02).bfloat16()
    dk = torch.randn((b, n, heads, nope), generator=g).bfloat16()
    dv = torch.randn((b, n, heads, vdim), generator=g).bfloat16()
    y_ref, saved = G.fp8_linear_forward(nkv.reshape(b * n, rank), w)
    dy = torch.cat([dk, dv], dim=-1).reshape(b * n, out_features)
    gi_ref, gw_ref = G.fp8_linear_backward(dy, saved)

    w_fp8, w_s, w_t_fp8, w_t_s = fp8cast_blockwise_transpose(w.cuda())
    k_nope, value = mla_decompress(nkv.cuda(), w.cuda(), heads, nope, vdim, use_fp8=True, weight_fp8=w_fp8, scale_weight=w_s)
    assert k_nope.shape == (b, n, heads, nope) and value.shape == (b, n, heads, vdim) and value.is_contiguous()
    kv_ref = y_ref.view(b, n, heads, nope + vdim)
    _close(k_nope, kv_ref[..., :nope], "k_nope")
    _close(value, kv_ref[..., nope:], "value")
    # the bf16 branch is the plain linear
    k2, v2 = mla_decompress(nkv.cuda(), w.cuda(), heads, nope, vdim)
    ref2 = torch.nn.functional.linear(nkv.cuda(), w.cuda()).view(b, n, heads, nope + vdim)
    assert torch.equal(k2, ref2[..., :nope]) and torch.equal(v2, ref2[..., nope:])

    d_nkv, dW = mla_decompress_backward(dk.cuda(), dv.cuda(), nkv.cuda(), w_t_fp8, w_t_s)
    assert d_nkv.dtype == torch.float32 and dW.dtype == torch.float32
    assert d_nkv.shape == (b, n, rank) and dW.shape == (out_features, rank)
    _close(d_nkv, gi_ref.view(b, n, rank), "d_nkv")
    _close(dW, gw_ref, "dW")
