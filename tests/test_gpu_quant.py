"""GPU parity: the six quantisers through the C-ABI vs the CPU oracle, bit for bit.

Shapes follow the reference's own lists (tests/operators/test_deepgemm_quantize.py:50-61,
111-122,169-182,229-240,305-315) plus ragged / strided / fp32 / extreme-magnitude cases.
"""

import pytest
import torch

from oracle import fp8 as Q

pytestmark = pytest.mark.gpu


def _ops():
    from pith_train_amd.operators import deepgemm_quantize as D

    return D


def _mk(shape, seed, dtype=torch.bfloat16, spread=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g)
    if spread:  # per-row magnitudes over many binades so many different scales occur
        x = x * torch.exp2(torch.randint(-12, 12, (shape[0],) + (1,) * (len(shape) - 1), generator=g).float())
    x = x.to(dtype)
    x.view(-1)[0] = -0.0
    return x


def _eq(got, ref, what):
    got = got.cpu()
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert got.dtype == ref.dtype, f"{what}: dtype {got.dtype} vs {ref.dtype}"
    if got.dtype == torch.float8_e4m3fn:
        got, ref = got.view(torch.uint8), ref.view(torch.uint8)
    bad = (got != ref).sum().item()
    assert bad == 0, f"{what}: {bad} of {got.numel()} elements differ"


ROWCOL = [(128, 128), (128, 256), (256, 256), (256, 512), (384, 384), (128, 300), (256, 7168), (128, 7), (1024, 2880)]


@pytest.mark.parametrize("M,N", ROWCOL)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rowwise_colwise(M, N, dtype):
    D = _ops()
    x = _mk((M, N), M * 7 + N, dtype)
    ref = Q.fp8cast_rowwise_colwise(x)
    got = D.fp8cast_rowwise_colwise(x.cuda())
    for g, r, w in zip(got, ref, ("tok_fp8", "tok_scale", "ch_fp8", "ch_scale")):
        _eq(g, r, w)
    got_t = D.fp8cast_rowwise_colwise_t(x.cuda())
    _eq(got_t[0], ref[0], "tok_fp8")
    _eq(got_t[1], ref[1], "tok_scale")
    _eq(got_t[2], ref[2].view(torch.uint8).T.contiguous().view(torch.float8_e4m3fn), "ch_t_fp8")
    _eq(got_t[3], ref[3], "ch_scale")


@pytest.mark.parametrize("M", [63 * 128, 64 * 128, 65 * 128, 72 * 128, 130 * 128 + 40])
def test_row_scaled_kernels_cover_every_tile_under_each_tile_order(M):
    """The row-scaled kernels hand their 128 x 128 tiles to workgroups in three orders, chosen by the
    number of row blocks: octets of row blocks per XCD (from 64 row blocks on), single row blocks
    per XCD (the next multiple of 8), plain order (the rest).  Row counts on either side of every
    switch, one of them ragged, against the oracle bit for bit."""
    D = _ops()
    N = 392  # three full column tiles and a ragged one
    x = _mk((M, N), M + 5)
    ref = Q.fp8cast_rowwise_transpose(x)
    got = D.fp8cast_rowwise_transpose(x.cuda())
    for g, r, w in zip(got, ref, ("tok_fp8", "tok_scale", "t_fp8", "t_scale")):
        _eq(g, r, w)
    if M % 128 == 0:
        ref = Q.fp8cast_rowwise_colwise(x)
        got = D.fp8cast_rowwise_colwise_t(x.cuda())
        _eq(got[0], ref[0], "tok_fp8")
        _eq(got[1], ref[1], "tok_scale")
        _eq(got[2], ref[2].view(torch.uint8).T.contiguous().view(torch.float8_e4m3fn), "ch_t_fp8")
        _eq(got[3], ref[3], "ch_scale")


def test_transposed_outputs_are_contiguous_as_in_the_reference():
    """The public quantisers return freshly allocated contiguous tensors whatever the token count
    (reference: operators/deepgemm_quantize.py:429-482,575-629); only the private form that the
    dense linear uses pads the rows of the transposed operand, and it holds the same bytes."""
    D = _ops()
    for shape, seed in (((4096, 256), 5), ((300, 256), 6), ((2048, 384), 7)):
        x = _mk(shape, seed).cuda()
        for fn in (D.fp8cast_rowwise_transpose, D.fp8cast_rowwise_blockwise_transpose):
            got = fn(x)
            for t in got:
                assert t.is_contiguous() and t.storage_offset() == 0
            assert got[2].shape == (shape[1], shape[0]) and got[2].view(-1).numel() == shape[0] * shape[1]
            padded = fn(x, _padded=True)
            if shape[0] >= 2048 and shape[0] % 256 == 0:
                assert padded[2].stride() == (shape[0] + 128, 1)
            for a, b in zip(got, padded):
                assert torch.equal(a.view(torch.uint8) if a.dtype != torch.float32 else a,
                                   b.view(torch.uint8) if b.dtype != torch.float32 else b)


def test_rowwise_colwise_all_zero_and_strided():
    D = _ops()
    z = torch.zeros((128, 256), dtype=torch.bfloat16)
    tok, tok_s, ch, ch_s = D.fp8cast_rowwise_colwise(z.cuda())
    assert (tok.view(torch.uint8) == 0).all() and (ch.view(torch.uint8) == 0).all()
    assert (tok_s == 2.0**-22).all() and (ch_s == 2.0**-22).all()
    big = _mk((256, 512), 3)
    view = big[:, 128:384]  # row stride 512, 256 columns
    ref = Q.fp8cast_rowwise_colwise(view.contiguous())
    got = D.fp8cast_rowwise_colwise(big.cuda()[:, 128:384])
    for g, r, w in zip(got, ref, ("tok_fp8", "tok_scale", "ch_fp8", "ch_scale")):
        _eq(g, r, w)


def test_rowwise_kmajor():
    D = _ops()
    offs = torch.tensor([128, 128, 512, 640, 1024], dtype=torch.int32)
    x = _mk((1024, 200), 17)
    ref = Q.fp8cast_rowwise_kmajor(x, offs)
    got = D.fp8cast_rowwise_kmajor(x.cuda(), offs.cuda())
    for g, r, w in zip(got, ref, ("tok_fp8", "tok_scale", "kmajor_fp8", "kmajor_scale")):
        _eq(g, r, w)


TRANS = [(128, 128), (128, 256), (256, 256), (64, 256), (7, 300), (1, 128), (256, 7168), (64, 64), (300, 130), (4096, 512),
         (2048, 200), (8192, 384)]  # the last three: token counts whose transposed outputs get a padded row pitch


@pytest.mark.parametrize("M,N", TRANS)
def test_rowwise_transpose(M, N):
    D = _ops()
    x = _mk((M, N), M * 11 + N)
    ref = Q.fp8cast_rowwise_transpose(x)
    got = D.fp8cast_rowwise_transpose(x.cuda())
    for g, r, w in zip(got, ref, ("tok_fp8", "tok_scale", "t_fp8", "t_scale")):
        _eq(g, r, w)


@pytest.mark.parametrize("M,K", TRANS)
def test_rowwise_blockwise_transpose(M, K):
    D = _ops()
    x = _mk((M, K), M * 13 + K)
    ref = Q.fp8cast_rowwise_blockwise_transpose(x)
    got = D.fp8cast_rowwise_blockwise_transpose(x.cuda())
    for g, r, w in zip(got, ref, ("tok_fp8", "tok_scale", "blk_t_fp8", "blk_t_scale")):
        _eq(g, r, w)


@pytest.mark.parametrize("M,K", TRANS + [(2880, 2880)])
def test_blockwise_transpose(M, K):
    D = _ops()
    x = _mk((M, K), M * 17 + K)
    ref = Q.fp8cast_blockwise_transpose(x)
    got = D.fp8cast_blockwise_transpose(x.cuda())
    for g, r, w in zip(got, ref, ("fp8", "scale", "fp8_t", "scale_t")):
        _eq(g, r, w)
    assert torch.equal(got[1], got[3].T)


@pytest.mark.parametrize("G,N,K", [(1, 128, 128), (4, 256, 128), (3, 200, 300), (8, 512, 256), (2, 2880, 320)])
def test_blockwise_transpose_batched(G, N, K):
    D = _ops()
    g = torch.Generator().manual_seed(G * 100 + N + K)
    w = (torch.randn((G, N, K), generator=g) * 0.02).bfloat16()
    ref = Q.fp8cast_blockwise_transpose_batched(w)
    got = D.fp8cast_blockwise_transpose_batched(w.cuda())
    for a, r, name in zip(got, ref, ("fp8", "scale", "fp8_t", "scale_t")):
        _eq(a, r, name)
    assert torch.equal(got[1], got[3].transpose(1, 2))


def test_all_six_quantisers_take_fp16_sources():
    """The reference's kernels take any float input (deepgemm_quantize.py:141-152 loads and
    converts to fp32); fp16 sources must give the oracle's bytes and scales as bf16 and fp32 do,
    on full tiles and on ragged edges, subnormal halves included."""
    D = _ops()
    g = torch.Generator().manual_seed(16)

    def mk(*shape):
        x = torch.randn(shape, generator=g) * torch.exp2(torch.randint(-20, 8, shape[:-1] + (1,), generator=g).float())
        return x.to(torch.float16)

    for M, N in ((256, 384), (128, 200), (384, 7168)):
        x = mk(M, N)
        for a, r, w in zip(D.fp8cast_rowwise_colwise(x.cuda()), Q.fp8cast_rowwise_colwise(x), ("tok", "tok_s", "ch", "ch_s")):
            _eq(a, r, f"rowwise_colwise fp16 {w}")
    offs = torch.tensor([128, 128, 512], dtype=torch.int32)
    x = mk(512, 256)
    for a, r, w in zip(D.fp8cast_rowwise_kmajor(x.cuda(), offs.cuda()), Q.fp8cast_rowwise_kmajor(x, offs), ("tok", "tok_s", "km", "km_s")):
        _eq(a, r, f"rowwise_kmajor fp16 {w}")
    for M, N in ((7, 300), (256, 512)):
        x = mk(M, N)
        for name in ("fp8cast_rowwise_transpose", "fp8cast_rowwise_blockwise_transpose", "fp8cast_blockwise_transpose"):
            for a, r, w in zip(getattr(D, name)(x.cuda()), getattr(Q, name)(x), "abcd"):
                _eq(a, r, f"{name} fp16 {M}x{N} output {w}")
    w3 = mk(3, 200, 300)
    for a, r, w in zip(D.fp8cast_blockwise_transpose_batched(w3.cuda()), Q.fp8cast_blockwise_transpose_batched(w3), "abcd"):
        _eq(a, r, f"blockwise_transpose_batched fp16 output {w}")


def test_every_bf16_value_roundtrips_like_the_oracle():
    """All 65280 finite bf16 bit patterns in one tensor (rows sorted by magnitude so scales vary)."""
    D = _ops()
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16)
    x = x[torch.isfinite(x.float())]
    x = x[torch.argsort(x.float().abs(), stable=True)]
    n = (x.numel() // (128 * 128)) * 128 * 128
    x = x[-n:].reshape(-1, 128).contiguous()
    x = x[: (x.shape[0] // 128) * 128]
    ref = Q.fp8cast_rowwise_colwise(x)
    got = D.fp8cast_rowwise_colwise(x.cuda())
    for g, r, w in zip(got, ref, ("tok_fp8", "tok_scale", "ch_fp8", "ch_scale")):
        _eq(g, r, w)


def test_row_limit_from_device_offsets_leaves_the_tail_untouched():
    """With the group offsets given, only the rows below their last entry are quantised: the
    tensors may be sized for more rows than the routing produced, without the host knowing how
    many (no device-to-host copy).  Rows below the limit carry the same bytes as a plain call."""
    from pith_train_amd import _lib
    from pith_train_amd.operators import deepgemm_quantize as DQ
    from pith_train_amd.operators import fused_experts as FE

    g = torch.Generator().manual_seed(11)
    cap, real, N = 1024, 640, 384
    x = torch.randn((700, N), generator=g).bfloat16().cuda()
    row_index = torch.full((cap,), -1, dtype=torch.int32)
    row_index[:real] = torch.randint(0, 700, (real,), generator=g, dtype=torch.int32)
    row_index[real - 40 : real] = -1  # padding rows inside the last group
    row_index = row_index.cuda()
    offs = torch.tensor([256, 256, real], dtype=torch.int32).cuda()
    full = DQ.fp8cast_rowwise_colwise_t_rows(x, row_index[:real].contiguous())
    lim = DQ.fp8cast_rowwise_colwise_t_rows(x, row_index, offs)
    u8 = lambda t: t.view(torch.uint8)  # noqa: E731
    assert torch.equal(u8(lim[0])[:real], u8(full[0])) and torch.equal(lim[1][:real], full[1])
    assert torch.equal(u8(lim[2])[:, :real], u8(full[2])) and torch.equal(lim[3][: real // 128], full[3])

    # the kernels must not have written past the limit: pre-filled outputs keep their sentinel
    M, half = cap, 256
    gate_up = torch.randn((M, 2 * half), generator=g).bfloat16().cuda()
    gate_up[real:] = float("nan")  # rows the routing never produced hold garbage
    ref = FE.silu_mul_quant(gate_up[:real].contiguous())
    tok = torch.full((M, half), 0x55, dtype=torch.uint8, device="cuda")
    tok_s = torch.full((M, half // 128), -7.0, device="cuda")
    ch_t = torch.full((half, M), 0x55, dtype=torch.uint8, device="cuda")
    ch_s = torch.full((M // 128, half), -7.0, device="cuda")
    _lib.call("pt_silu_mul_quant_rowwise_colwise", gate_up.data_ptr(), M, half, gate_up.stride(0), tok.data_ptr(),
              tok_s.data_ptr(), ch_t.data_ptr(), ch_s.data_ptr(), offs.data_ptr() + 8, _lib.stream_ptr())
    assert torch.equal(tok[:real], u8(ref[0])) and torch.equal(tok_s[:real], ref[1])
    assert torch.equal(ch_t[:, :real], u8(ref[2])) and torch.equal(ch_s[: real // 128], ref[3])
    assert (tok[real:] == 0x55).all() and (tok_s[real:] == -7.0).all()
    assert (ch_t[:, real:] == 0x55).all() and (ch_s[real // 128 :] == -7.0).all()


def test_weights_quantised_into_a_fused_operand_equal_the_quantised_concatenation():
    from pith_train_amd.operators import deepgemm_quantize as DQ

    g = torch.Generator().manual_seed(21)
    parts = [(torch.randn((3, n, 320), generator=g) * 0.02).bfloat16().cuda() for n in (128, 256, 128)]
    got = DQ.fp8cast_blockwise_transpose_batched_cat(parts)
    ref = DQ.fp8cast_blockwise_transpose_batched(torch.cat(parts, dim=1))
    for a, b in zip(got, ref):
        assert a.shape == b.shape
        assert torch.equal(a.view(torch.uint8) if a.dtype != torch.float32 else a, b.view(torch.uint8) if b.dtype != torch.float32 else b)


@pytest.mark.parametrize("M,half", [(384, 256), (256, 200), (128, 2880)])
def test_clamped_swiglu_fused_into_the_quantisation_has_the_bits_of_the_two_steps(M, half):
    """The GPT-OSS activation computed inside the quantisation kernels: forward bytes and scales,
    backward bytes and scales equal those of clamped_swiglu (tested against the oracle on its own)
    followed by the rowwise + colwise quantiser; the per-tile column sums equal the float64 sums
    of the materialised bf16 gradient to fp32 rounding."""
    from pith_train_amd.operators import deepgemm_quantize as DQ
    from pith_train_amd.operators import fused_experts as FE
    from pith_train_amd.operators.clamped_swiglu import clamped_swiglu

    g = torch.Generator().manual_seed(M + half)
    gate_up = (torch.randn((M, 2 * half), generator=g) * 4).bfloat16().cuda().requires_grad_(True)
    grad_h = torch.randn((M, half), generator=g).bfloat16().cuda()
    h = clamped_swiglu(gate_up, 1.702, 7.0)
    h.backward(grad_h)
    u8 = lambda t: t.view(torch.uint8) if t.dtype == torch.float8_e4m3fn else t  # noqa: E731
    for got, ref in zip(FE.clamped_swiglu_quant(gate_up.detach(), 1.702, 7.0), DQ.fp8cast_rowwise_colwise_t(h.detach())):
        assert got.shape == ref.shape and torch.equal(u8(got), u8(ref))
    *quant, col_sum = FE.clamped_swiglu_bwd_quant(grad_h, gate_up.detach(), 1.702, 7.0)
    for got, ref in zip(quant, DQ.fp8cast_rowwise_colwise_t(gate_up.grad)):
        assert got.shape == ref.shape and torch.equal(u8(got), u8(ref))
    tiles = gate_up.grad.double().reshape(M // 128, 128, 2 * half)
    want, mag = tiles.sum(1), tiles.abs().sum(1)
    assert col_sum.shape == want.shape
    assert ((col_sum.double() - want).abs() <= 1e-6 * mag + 1e-30).all()
    assert (gate_up.grad == 0).any() and (gate_up.grad != 0).any()  # both sides of the clamps occur


@pytest.mark.parametrize("G,N,K", [(3, 256, 384), (2, 200, 300), (1, 128, 128), (4, 1536, 2048)])
def test_blockwise_batched_without_the_twin_is_the_first_half_of_the_transposing_quantiser(G, N, K):
    """The grouped-expert weights are quantised without the transposed twin (the input-gradient
    GEMM reads the forward layout): bytes and scales equal those of the quantiser that writes
    both, and the fused gate/up form agrees with the concatenation."""
    from pith_train_amd.operators import deepgemm_quantize as D

    w = (torch.randn((G, N, K), generator=torch.Generator().manual_seed(G + N + K)) * 0.02).bfloat16().cuda()
    full = D.fp8cast_blockwise_transpose_batched(w)
    half = D.fp8cast_blockwise_batched(w)
    assert half[2] is None and half[3] is None
    assert torch.equal(half[0].view(torch.uint8), full[0].view(torch.uint8)) and torch.equal(half[1], full[1])
    # the twin of a 128x128-blockwise quantisation is the byte transpose with the transposed scale grid
    assert torch.equal(full[2].view(torch.uint8), full[0].view(torch.uint8).transpose(1, 2))
    assert torch.equal(full[3], full[1].transpose(1, 2))
    if N % 256 == 0:
        parts = (w[:, : N // 2].contiguous(), w[:, N // 2 :].contiguous())
        cat = D.fp8cast_blockwise_transpose_batched_cat(parts, twin=False)
        assert cat[2] is None and torch.equal(cat[0].view(torch.uint8), full[0].view(torch.uint8)) and torch.equal(cat[1], full[1])
