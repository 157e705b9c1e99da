"""Pins the quantisation oracle (CPU only).

What is checked against what:
  * scale rule: every positive bf16 amax, against the rule DeepGEMM publishes for
    ``use_ue8m0=True`` - ``2**ceil(log2(max(amax,1e-4)/448))`` - evaluated in float64, and
    against the known answers amax=448 -> 1, 224 -> 0.5, 3.5 -> 2**-7, 0 -> 2**-22.
  * e4m3 cast: torch's library cast against an integer-only encoder written from the format
    definition, over every bf16 bit pattern times every reciprocal scale that can occur.
  * layouts: per-element Python loops on small ragged shapes; transposed twins; the
    ``scale_t == scale.T`` symmetry the reference's tests assert
    (tests/operators/test_deepgemm_quantize.py:290-297,376-383); all-zero input (:95-103).
"""

import math

import numpy as np
import pytest
import torch

from oracle import fp8 as Q


def all_bf16_nonneg_finite():
    bits = torch.arange(0, 0x7F80, dtype=torch.int32).to(torch.int16)
    return bits.view(torch.bfloat16)


def test_scale_known_answers():
    amax = torch.tensor([448.0, 224.0, 3.5, 0.0, 1e-4, 448.0 * 4, 449.0])
    scale, rcp = Q.compute_fp8_scale(amax)
    expect = torch.tensor([1.0, 0.5, 2.0**-7, 2.0**-22, 2.0**-22, 4.0, 2.0])
    assert torch.equal(scale, expect)
    assert torch.equal(scale * rcp, torch.ones_like(scale))


def test_scale_exhaustive_vs_published_rule():
    amax = all_bf16_nonneg_finite().float()
    scale, rcp = Q.compute_fp8_scale(amax)
    a64 = amax.double().clamp(min=float(np.float32(1e-4)))
    # fp32 division as DeepGEMM does it, then ceil(log2()) in float64 (exact for fp32 inputs)
    sf = (a64.float() / 448.0).double()
    expect = torch.pow(2.0, torch.ceil(torch.log2(sf)))
    # log2 of an exact power of two is exact in float64, otherwise ceil is insensitive
    assert torch.equal(scale.double(), expect)
    assert torch.equal((scale.double() * rcp.double()), torch.ones_like(expect))
    # quantised magnitude never exceeds 448
    assert float((amax * rcp).max()) <= 448.0
    # and uses the top binade whenever the clamp is inactive
    active = amax > 1e-4 * 448
    assert float((amax * rcp)[active].min()) > 224.0 - 1e-3


def test_e4m3_cast_exhaustive_vs_integer_encoder():
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16).float()
    x = x[torch.isfinite(x)]
    checked = 0
    for e in range(-40, 24):
        y = x * (2.0**e)
        y = y[y.abs() <= 448.0]
        got = Q.cast_e4m3(y).view(torch.uint8).numpy()
        ref = Q.cast_e4m3_numpy(y.numpy())
        assert np.array_equal(got, ref), f"exponent {e}"
        checked += y.numel()
    assert checked > 1_000_000
    # spot values from the format definition (ties to even, subnormals)
    probe = torch.tensor([17.0, 19.0, 2.0**-10, 1.5 * 2.0**-9, -0.0, 448.0, 2.0**-9, 0.0])
    assert Q.cast_e4m3(probe).view(torch.uint8).tolist() == [88, 90, 0, 2, 128, 126, 1, 0]


def _loop_rowwise(x):
    M, N = x.shape
    nb = (N + 127) // 128
    q = torch.zeros((M, N), dtype=torch.uint8)
    s = torch.zeros((M, nb), dtype=torch.float32)
    for i in range(M):
        for b in range(nb):
            seg = x[i, b * 128 : min(N, (b + 1) * 128)].float()
            amax = max(float(seg.abs().max()), 1e-4)
            sc = 2.0 ** math.ceil(math.log2(np.float32(amax) / np.float32(448.0)))
            s[i, b] = sc
            q[i, b * 128 : b * 128 + seg.numel()] = (seg / sc).to(torch.float8_e4m3fn).view(
                torch.uint8
            )
    return q, s


@pytest.mark.parametrize("shape", [(128, 128), (128, 300), (256, 130), (7, 300), (1, 128), (64, 64)])
def test_layouts_vs_loops(shape):
    torch.manual_seed(shape[0] * 1000 + shape[1])
    M, N = shape
    x = (torch.randn(M, N) * torch.exp(torch.randn(M, 1) * 2)).bfloat16()
    x[0, 0] = -0.0
    q_ref, s_ref = _loop_rowwise(x)
    qt_ref, st_ref = _loop_rowwise(x.T.contiguous())

    tok, tok_s, t, t_s = Q.fp8cast_rowwise_transpose(x)
    assert torch.equal(tok.view(torch.uint8), q_ref) and torch.equal(tok_s, s_ref)
    assert torch.equal(t.view(torch.uint8), qt_ref) and torch.equal(t_s, st_ref)
    assert t.shape == (N, M) and t_s.shape == (N, (M + 127) // 128)

    if M % 128 == 0:
        tok2, tok_s2, ch, ch_s = Q.fp8cast_rowwise_colwise(x)
        assert torch.equal(tok2.view(torch.uint8), q_ref) and torch.equal(tok_s2, s_ref)
        assert torch.equal(ch.view(torch.uint8), qt_ref.T) and torch.equal(ch_s, st_ref.T)

    tok3, tok_s3, blk_t, blk_t_s = Q.fp8cast_rowwise_blockwise_transpose(x)
    assert torch.equal(tok3.view(torch.uint8), q_ref) and torch.equal(tok_s3, s_ref)
    b, b_s, b_t, b_t_s = Q.fp8cast_blockwise_transpose(x)
    assert torch.equal(b_t.view(torch.uint8), b.view(torch.uint8).T)
    assert torch.equal(b_s, b_t_s.T)
    assert torch.equal(blk_t.view(torch.uint8), b_t.view(torch.uint8))
    assert torch.equal(blk_t_s, b_t_s)
    # block scale = max of the rowwise scales inside the block; bytes follow from it
    mb, kb = (M + 127) // 128, (N + 127) // 128
    for i in range(mb):
        for j in range(kb):
            tile = x[i * 128 : (i + 1) * 128, j * 128 : (j + 1) * 128].float()
            assert float(b_s[i, j]) == float(s_ref[i * 128 : (i + 1) * 128, j].max())
            qq = (tile / b_s[i, j]).to(torch.float8_e4m3fn).view(torch.uint8)
            assert torch.equal(b.view(torch.uint8)[i * 128 : (i + 1) * 128, j * 128 : (j + 1) * 128], qq)


def test_batched_matches_2d_and_symmetry():
    torch.manual_seed(3)
    w = (torch.randn(3, 200, 300) * 0.02).bfloat16()
    q, s, qt, st = Q.fp8cast_blockwise_transpose_batched(w)
    assert q.shape == (3, 200, 300) and s.shape == (3, 2, 3)
    assert qt.shape == (3, 300, 200) and st.shape == (3, 3, 2)
    assert torch.equal(st, s.transpose(1, 2))
    for g in range(3):
        a, b, c, d = Q.fp8cast_blockwise_transpose(w[g])
        assert torch.equal(q[g].view(torch.uint8), a.view(torch.uint8))
        assert torch.equal(qt[g].view(torch.uint8), c.view(torch.uint8))


def test_all_zero_input():
    x = torch.zeros((128, 256), dtype=torch.bfloat16)
    tok, tok_s, ch, ch_s = Q.fp8cast_rowwise_colwise(x)
    assert torch.all(tok.view(torch.uint8) == 0) and torch.all(ch.view(torch.uint8) == 0)
    assert torch.all(tok_s == 2.0**-22) and torch.all(ch_s == 2.0**-22)


def test_kmajor_layout_invariant():
    torch.manual_seed(5)
    offs = torch.tensor([128, 128, 512, 640], dtype=torch.int32)  # one empty group
    M, N = 640, 200
    x = torch.randn(M, N).bfloat16()
    tok, tok_s, flat, s_t = Q.fp8cast_rowwise_kmajor(x, offs)
    _, _, ch, ch_s = Q.fp8cast_rowwise_colwise(x)
    assert torch.equal(s_t, ch_s.T)
    fb, cb = flat.view(torch.uint8), ch.view(torch.uint8)
    start = 0
    for end in offs.tolist():
        kg = end - start
        for n in (0, 7, N - 1):
            for r in (0, kg // 2, kg - 1) if kg else ():
                assert fb[start * N + n * kg + r] == cb[start + r, n]
        start = end


def test_dequant_roundtrip_error_bound():
    torch.manual_seed(11)
    x = torch.randn(256, 384).bfloat16()
    q, s, _, _ = Q.fp8cast_rowwise_colwise(x)
    back = Q.dequant_rowwise(q, s)
    # e4m3 has 3 mantissa bits: relative error <= 2**-4 for normals of the top binades
    err = (back - x.float()).abs()
    bound = x.float().abs() * 2.0**-4 + s.repeat_interleave(128, 1) * 2.0**-10
    assert torch.all(err <= bound)
