"""GPU parity: FP8 GEMMs through the C-ABI vs the float64 dequantised oracle.

Tolerance (stated by the task): every element within 1e-2 relative of the fp32/fp64-dequantised
reference (with an absolute floor of 1e-2 x rms(ref) for elements near zero), and the reference
test-suite's similarity metric ``calc_diff < 1e-3``
(tests/test_deepgemm_fp8_linear_correctness.py:14,22-28).  In practice the only differences are
the fp32 accumulation order and the single bf16 rounding (2**-9).
"""

import pytest
import torch

from oracle import fp8 as Q
from oracle import gemm as G

pytestmark = pytest.mark.gpu

REL = 1e-2


@pytest.fixture(autouse=True, params=["auto", "p0", "q0", "q1", "r0", "t"])
def gemm_kernel(request):
    """Every test runs once per GEMM kernel of the library (and once with the library's own choice)."""
    from pith_train_amd import _lib

    _lib.call("pt_gemm_select_kernel", request.param.encode())
    yield request.param
    _lib.call("pt_gemm_select_kernel", None)


def _check(got, ref, what):
    got = got.float().cpu().double()
    ref = ref.double()
    assert got.shape == ref.shape
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    rms = ref.pow(2).mean().sqrt().item()
    err = (got - ref).abs()
    bound = REL * ref.abs() + REL * rms
    worst = (err - bound).max().item()
    assert worst <= 0, f"{what}: max violation {worst:.3e} (rms {rms:.3e}, max err {err.max().item():.3e})"
    assert G.calc_diff(got, ref) < 1e-3, f"{what}: calc_diff {G.calc_diff(got, ref):.3e}"


def _rand(shape, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).bfloat16()


@pytest.mark.parametrize("M,N,K", [(128, 128, 128), (256, 384, 512), (1024, 512, 256), (300, 200, 384), (7, 128, 256),
                                   (512, 2880, 2880), (2048, 4096, 2048), (130, 64, 64)])
def test_dense_nt(M, N, K):
    from pith_train_amd.operators.linear import _fp8_gemm_nt

    x, w = _rand((M, K), M + K), _rand((N, K), N + K + 1, 0.02)
    a, sa, _, _ = Q.fp8cast_rowwise_transpose(x)
    b, sb, _, _ = Q.fp8cast_blockwise_transpose(w)
    ref = G.gemm_nt_dense(a, sa, b, sb, torch.float64)
    out = _fp8_gemm_nt(a.cuda(), sa.cuda(), b.cuda(), sb.cuda(), M, N, "cuda", torch.bfloat16)
    _check(out, ref, f"dense {M}x{N}x{K}")
    out32 = _fp8_gemm_nt(a.cuda(), sa.cuda(), b.cuda(), sb.cuda(), M, N, "cuda", torch.float32)
    _check(out32, ref, f"dense fp32 {M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K", [(512, 256, 4096), (300, 200, 4000), (128, 128, 20000), (256, 1024, 2048)])
def test_dense_nt_with_the_reduction_split_over_workgroups(M, N, K):
    """Small outputs with a long reduction (a dense weight gradient) are computed as several
    ranges of the reduction side by side and summed: same result within the GEMM tolerance, through
    the operator's own rule and through the C-ABI with other range lengths (ragged last range,
    one range)."""
    from pith_train_amd import _lib
    from pith_train_amd.operators.linear import _fp8_gemm_nt, _split_k

    x, w = _rand((M, K), M + K + 2), _rand((N, K), N + K + 3, 0.02)
    a, sa, _, _ = Q.fp8cast_rowwise_transpose(x)
    b, sb, _, _ = Q.fp8cast_blockwise_transpose(w)
    ref = G.gemm_nt_dense(a, sa, b, sb, torch.float64)
    assert _split_k(M, N, K)[0] > 1, "the case is meant to take the split path"
    ad, sad, bd, sbd = a.cuda(), sa.cuda(), b.cuda(), sb.cuda()
    _check(_fp8_gemm_nt(ad, sad, bd, sbd, M, N, "cuda", torch.bfloat16), ref, f"split dense {M}x{N}x{K}")
    for split_len in (128, 640, (K + 127) // 128 * 128):
        splits = (K + split_len - 1) // split_len
        partial = torch.full((splits, M, N), float("nan"), device="cuda")
        _lib.call("pt_gemm_nt_dense_splitk", ad.data_ptr(), sad.data_ptr(), bd.data_ptr(), sbd.data_ptr(), partial.data_ptr(),
                  splits, split_len, M, N, K, _lib.stream_ptr("cuda"))
        for dt in (torch.float32, torch.bfloat16):
            out = torch.empty((M, N), device="cuda", dtype=dt)
            _lib.call("pt_sum_partials", partial.data_ptr(), splits, M * N, out.data_ptr(), _lib.dtype_code(dt),
                      _lib.stream_ptr("cuda"))
            _check(out, ref, f"split dense {M}x{N}x{K} in {splits} ranges of {split_len} as {dt}")
        # the slabs are the partial products of their ranges: they add up in float64 as well
        _check(partial.double().sum(0), ref, "slabs")


def _dense_rows_against_oracle(M, N, K, rows, what):
    from pith_train_amd.operators.linear import _fp8_gemm_nt

    x, w = _rand((M, K), M + K + 4), _rand((N, K), N + K + 5, 0.02)
    a, sa, _, _ = Q.fp8cast_rowwise_transpose(x)
    b, sb, _, _ = Q.fp8cast_blockwise_transpose(w)
    out = _fp8_gemm_nt(a.cuda(), sa.cuda(), b.cuda(), sb.cuda(), M, N, "cuda", torch.bfloat16)
    assert out.shape == (M, N)
    ref = G.gemm_nt_dense(a[rows], sa[rows], b, sb, torch.float64)
    _check(out[rows.cuda()], ref, what)


def test_dense_nt_with_more_tiles_per_workgroup_than_the_tile_table_holds(gemm_kernel):
    """32768 x 25600 is 12800 tiles of 256 x 256, 50 per workgroup of the persistent kernels: the
    last tiles of every workgroup are decoded on the fly instead of read from the table built at
    kernel start.  Two rows of every 256-row tile are compared over all columns, so every tile of
    the launch is checked."""
    M, N, K = 32768, 25600, 128
    rows = torch.arange(0, M, 256).repeat_interleave(2) + torch.tensor([5, 201]).repeat(M // 256)
    _dense_rows_against_oracle(M, N, K, rows, f"dense {M}x{N}x{K}, {gemm_kernel}")


def test_dense_nt_with_an_output_beyond_the_32_bit_store_offsets(gemm_kernel):
    """A 65536 x 32896 bf16 result is 4.3 GB: past the unsigned 32-bit byte offsets the persistent
    kernels store through, so the library must route the call to its kernel with 64-bit addresses
    whatever kernel was asked for.  One row of every 128-row tile, all columns."""
    if gemm_kernel not in ("auto", "q0"):
        pytest.skip("the route does not depend on the requested kernel; run twice")
    M, N, K = 65536, 32896, 128
    assert M * N * 2 >= 1 << 32
    rows = torch.arange(0, M, 128) + (torch.arange(M // 128) * 37) % 128
    _dense_rows_against_oracle(M, N, K, rows, f"dense {M}x{N}x{K} (64-bit route)")


def test_dense_scale_extremes():
    """Rows with very different magnitudes: the E8M0 exponents given to the MFMA must be per row."""
    from pith_train_amd.operators.linear import _fp8_gemm_nt

    M, N, K = 256, 256, 512
    g = torch.Generator().manual_seed(5)
    x = (torch.randn((M, K), generator=g) * torch.exp2(torch.randint(-20, 20, (M, 1), generator=g).float())).bfloat16()
    w = (torch.randn((N, K), generator=g) * torch.exp2(torch.randint(-10, 10, (N // 128, 1), generator=g).float())
         .repeat_interleave(128, 0)).bfloat16()
    a, sa, _, _ = Q.fp8cast_rowwise_transpose(x)
    b, sb, _, _ = Q.fp8cast_blockwise_transpose(w)
    ref = G.gemm_nt_dense(a, sa, b, sb, torch.float64)
    out = _fp8_gemm_nt(a.cuda(), sa.cuda(), b.cuda(), sb.cuda(), M, N, "cuda", torch.float32).cpu().double()
    # compare row by row relative to each row's own scale
    rel = (out - ref).abs().amax(1) / ref.abs().amax(1).clamp_min(1e-300)
    assert rel.max().item() < 1e-4, rel.max().item()


def _groups(sizes):
    ks = torch.tensor([(s + 127) // 128 * 128 for s in sizes], dtype=torch.int32)
    return ks, ks.cumsum(0).to(torch.int32)


GROUPED = [
    ([128, 128], 256, 128),
    ([100, 0, 300, 128, 1], 512, 256),
    ([0, 0, 640], 384, 384),
    ([256] * 8, 512, 256),
    ([512, 640, 128, 0, 384], 1536, 2048),
    ([300, 200], 2880, 2880),
    ([1536, 1700], 256, 2048),  # large groups + long reduction: the pipelined loop by the library's own choice
]


# More than 256 groups: the kernels' group scan gives every lane more than four groups (its long
# path), and the list of tiles is full of empty and single-block groups.
MANY_GROUPS = [([0 if i % 7 == 3 else (256 if i % 5 == 0 else 128) for i in range(320)], 256, 256)]


@pytest.mark.parametrize("sizes,N,K", GROUPED + MANY_GROUPS)
def test_m_grouped_nt(sizes, N, K):
    from pith_train_amd.operators.grouped_linear import m_grouped_fp8_gemm_nt

    ks, offs = _groups(sizes)
    M, Gn = int(offs[-1]), len(sizes)
    x = _rand((M, K), M + K)
    start = 0
    for s, k in zip(sizes, ks.tolist()):  # zero pad rows like the scatter does
        x[start + s : start + k] = 0
        start += k
    w = _rand((Gn, N, K), N + K + 3, 0.02)
    a, sa, _, _ = Q.fp8cast_rowwise_colwise(x)
    b, sb, _, _ = Q.fp8cast_blockwise_transpose_batched(w)
    ref = G.gemm_m_grouped_nt(a, sa, b, sb, offs, torch.float64)
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    m_grouped_fp8_gemm_nt((a.cuda(), sa.cuda()), (b.cuda(), sb.cuda()), out, offs.cuda())
    _check(out, ref, f"m-grouped {sizes} N={N} K={K}")


@pytest.mark.parametrize("sizes,N,K", GROUPED)
def test_m_grouped_nt_scattered_rows(sizes, N, K, gemm_kernel):
    """The un-permute folded into the store: result row r lands in output row out_rows[r]; rows of
    a group's padding (negative index) are dropped and rows nobody maps to stay untouched."""
    from pith_train_amd.operators.grouped_linear import m_grouped_fp8_gemm_nt

    if gemm_kernel == "t":
        pytest.skip("the tile-per-workgroup kernel has no scattered store (the library refuses it)")
    ks, offs = _groups(sizes)
    M, Gn = int(offs[-1]), len(sizes)
    x = _rand((M, K), M + K + 17)
    w = _rand((Gn, N, K), N + K + 5, 0.02)
    a, sa, _, _ = Q.fp8cast_rowwise_colwise(x)
    b, sb, _, _ = Q.fp8cast_blockwise_transpose_batched(w)
    ref = G.gemm_m_grouped_nt(a, sa, b, sb, offs, torch.float64)
    real = torch.zeros(M, dtype=torch.bool)
    start = 0
    for s_, k_ in zip(sizes, ks.tolist()):
        real[start : start + s_] = True
        start += k_
    n_real = int(real.sum())
    out_m = n_real + 3  # three rows that no result row maps to
    g = torch.Generator().manual_seed(M)
    dst = torch.randperm(out_m, generator=g)[:n_real].to(torch.int32)
    out_rows = torch.full((M,), -1, dtype=torch.int32)
    out_rows[real] = dst
    out = torch.full((out_m, N), 7.0, dtype=torch.bfloat16, device="cuda")
    m_grouped_fp8_gemm_nt((a.cuda(), sa.cuda()), (b.cuda(), sb.cuda()), out, offs.cuda(), out_rows.cuda())
    out = out.cpu()
    _check(out[dst.long()], ref[real], f"m-grouped scattered {sizes} N={N} K={K}")
    untouched = torch.ones(out_m, dtype=torch.bool)
    untouched[dst.long()] = False
    assert (out[untouched] == 7.0).all()


@pytest.mark.parametrize("sizes,N,K", GROUPED + MANY_GROUPS + [([256], 272, 400), ([600] * 16, 768, 2048)])
def test_m_grouped_nn_reads_the_forward_layout_weight_with_the_bits_of_nt(sizes, N, K, gemm_kernel):
    """The input-gradient form: b given reduction-major ([G, K, N], scales [G, K/128, N/128]) is the
    same product as the NT form on its transpose, accumulated in the same order: equal to the
    oracle within the GEMM tolerance and to the NT kernel bit for bit, plain and with scattered
    rows, for ragged N and K too."""
    from pith_train_amd.operators.grouped_linear import m_grouped_fp8_gemm_nn, m_grouped_fp8_gemm_nt

    ks, offs = _groups(sizes)
    M, Gn = int(offs[-1]), len(sizes)
    x = _rand((M, K), M + K + 29)
    w = _rand((Gn, N, K), N + K + 31, 0.02)
    a, sa, _, _ = Q.fp8cast_rowwise_colwise(x)
    b, sb, _, _ = Q.fp8cast_blockwise_transpose_batched(w)
    ref = G.gemm_m_grouped_nt(a, sa, b, sb, offs, torch.float64)
    bt, sbt = b.transpose(1, 2).contiguous().cuda(), sb.transpose(1, 2).contiguous().cuda()
    out_nn = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    out_nt = out_nn.clone()
    m_grouped_fp8_gemm_nn((a.cuda(), sa.cuda()), (bt, sbt), out_nn, offs.cuda())
    _check(out_nn, ref, f"m-grouped nn {sizes} N={N} K={K}")
    if gemm_kernel in ("auto", "r0"):  # the NT launch of the same kernel family
        m_grouped_fp8_gemm_nt((a.cuda(), sa.cuda()), (b.cuda(), sb.cuda()), out_nt, offs.cuda())
        assert torch.equal(out_nn[: int(offs[-1])], out_nt[: int(offs[-1])])
    if N % 8 == 0:
        g = torch.Generator().manual_seed(M + 1)
        dst = torch.randperm(M + 5, generator=g)[:M].to(torch.int32)
        dst[::7] = -1  # dropped rows
        out_s = torch.full((M + 5, N), 7.0, dtype=torch.bfloat16, device="cuda")
        m_grouped_fp8_gemm_nn((a.cuda(), sa.cuda()), (bt, sbt), out_s, offs.cuda(), dst.cuda())
        keep = (dst >= 0).nonzero().flatten()
        assert torch.equal(out_s[dst[keep].long().cuda()], out_nn[keep.cuda()])
        untouched = torch.ones(M + 5, dtype=torch.bool)
        untouched[dst[keep].long()] = False
        assert (out_s.cpu()[untouched] == 7.0).all()


@pytest.mark.parametrize("sizes", [[256], [256, 384]])
def test_m_grouped_nn_reads_nothing_past_a_ragged_reduction(sizes):
    """The reduction-major b operand of a ragged reduction (K = 400: 16 rows into the last
    128-block) lies inside a larger buffer whose every other byte is 0xFF, an e4m3 NaN: the rows of
    a reduction block past a group's K rows belong to the next group or to that padding, and the
    loader leaves them to the range check of the group's buffer descriptor.  A byte read from
    there would meet a zero of the a operand and give NaN; the result must be finite and equal to
    the NT form's bit for bit."""
    from pith_train_amd.operators.grouped_linear import m_grouped_fp8_gemm_nn, m_grouped_fp8_gemm_nt

    N, K = 272, 400
    ks, offs = _groups(sizes)
    M, Gn = int(offs[-1]), len(sizes)
    x = _rand((M, K), 71)
    w = _rand((Gn, N, K), 73, 0.02)
    a, sa, _, _ = Q.fp8cast_rowwise_colwise(x)
    b, sb, _, _ = Q.fp8cast_blockwise_transpose_batched(w)
    big = torch.full((Gn * K * N + 256 * N,), 0xFF, dtype=torch.uint8, device="cuda")
    bt = big[: Gn * K * N].view(Gn, K, N)
    bt.copy_(b.transpose(1, 2).contiguous().view(torch.uint8).cuda())
    bt = bt.view(torch.float8_e4m3fn)
    sbt = sb.transpose(1, 2).contiguous().cuda()
    out_nn = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    out_nt = out_nn.clone()
    m_grouped_fp8_gemm_nn((a.cuda(), sa.cuda()), (bt, sbt), out_nn, offs.cuda())
    m_grouped_fp8_gemm_nt((a.cuda(), sa.cuda()), (b.cuda(), sb.cuda()), out_nt, offs.cuda())
    rows = int(offs[-1])
    assert torch.isfinite(out_nn[:rows].float()).all(), "a byte past the group's reduction rows was read"
    assert torch.equal(out_nn[:rows], out_nt[:rows])
    assert (big[Gn * K * N :] == 0xFF).all()


def test_m_grouped_nt_with_more_tiles_per_workgroup_than_the_tile_table_holds(gemm_kernel):
    """Four groups of 25600 rows x 8192 columns: 12800 tiles, 50 per workgroup, so the grouped
    tile decode (group search, row tile inside the group) also runs on the fly for the last tiles.
    Two rows of every 256-row tile against the oracle, all columns."""
    from pith_train_amd.operators.grouped_linear import m_grouped_fp8_gemm_nt

    sizes, N, K = [25600] * 4, 8192, 128
    ks, offs = _groups(sizes)
    M, Gn = int(offs[-1]), len(sizes)
    x, w = _rand((M, K), M + K + 6), _rand((Gn, N, K), N + K + 7, 0.02)
    a, sa, _, _ = Q.fp8cast_rowwise_colwise(x)
    b, sb, _, _ = Q.fp8cast_blockwise_transpose_batched(w)
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    m_grouped_fp8_gemm_nt((a.cuda(), sa.cuda()), (b.cuda(), sb.cuda()), out, offs.cuda())
    rows = torch.arange(0, M, 256).repeat_interleave(2) + torch.tensor([9, 250]).repeat(M // 256)
    grp = rows // 25600
    for g in range(Gn):
        r = rows[grp == g]
        ref = G.gemm_nt_dense(a[r], sa[r], b[g], sb[g], torch.float64)
        _check(out[r.cuda()], ref, f"m-grouped group {g} of {sizes} N={N} K={K}, {gemm_kernel}")


def test_k_grouped_wgrad_with_more_tiles_per_workgroup_than_the_tile_table_holds(gemm_kernel):
    """200 groups of one 128-row block, 2048 x 2048 results: 12800 tiles, 50 per workgroup.  Groups
    spread over the whole list (the on-the-fly decode handles the end of every XCD's share) are
    compared with the oracle; all others must at least be finite and non-trivial."""
    from pith_train_amd.operators.grouped_linear import k_grouped_fp8_wgrad

    if gemm_kernel == "t":
        pytest.skip("the tile-per-workgroup kernel has no tile table")
    Gn, N, K = 200, 2048, 2048
    ks, offs = _groups([128] * Gn)
    M = int(offs[-1])
    dy, x = _rand((M, N), M + N + 1), _rand((M, K), M + K + 2)
    _, _, dy_ch, dy_s = Q.fp8cast_rowwise_colwise(dy)
    _, _, x_ch, x_s = Q.fp8cast_rowwise_colwise(x)
    tr = lambda q: q.view(torch.uint8).T.contiguous().view(torch.float8_e4m3fn).cuda()  # noqa: E731
    out = torch.full((Gn, N, K), float("nan"), dtype=torch.bfloat16, device="cuda")
    k_grouped_fp8_wgrad((tr(dy_ch), dy_s.cuda()), (tr(x_ch), x_s.cuda()), out, offs.cuda(), False)
    assert torch.isfinite(out).all()
    assert (out.float().abs().amax(dim=(1, 2)) > 0).all()
    for g in list(range(23, Gn, 25)) + [0, Gn - 1]:  # 24, 49, ..., 199: the last group of every eighth of the list
        sl = slice(g * 128, (g + 1) * 128)
        ref = G.gemm_k_grouped_wgrad(dy_ch[sl], dy_s[g : g + 1], x_ch[sl], x_s[g : g + 1], torch.tensor([128], dtype=torch.int32), 1,
                                     torch.float64).double()
        _check(out[g : g + 1], ref, f"wgrad group {g} of {Gn}, {gemm_kernel}")


# Skewed group sizes: the weight-gradient tiles are shared out over the XCDs by cost (a tile's
# reduction length), so the cuts fall inside groups, at empty groups and at the ends of the list.
SKEWED = [
    ([0] * 5 + [4096] + [0] * 10 + [130, 1, 1, 1], 512, 512),
    ([3, 900, 0, 17, 2500, 128, 0, 0, 1, 640] * 7, 256, 256),
    ([2000], 768, 256),
    ([1] * 9, 256, 512),
]


@pytest.mark.parametrize("sizes,N,K", GROUPED + SKEWED + MANY_GROUPS)
@pytest.mark.parametrize("accumulate", [False, True])
def test_k_grouped_wgrad(sizes, N, K, accumulate):
    from pith_train_amd.operators.grouped_linear import k_grouped_fp8_wgrad

    if N * K > 4e6 and accumulate:
        pytest.skip("covered by the non-accumulating case")
    ks, offs = _groups(sizes)
    M, Gn = int(offs[-1]), len(sizes)
    dy, x = _rand((M, N), M + N), _rand((M, K), M + K + 9)
    _, _, dy_ch, dy_s = Q.fp8cast_rowwise_colwise(dy)
    _, _, x_ch, x_s = Q.fp8cast_rowwise_colwise(x)
    ref = G.gemm_k_grouped_wgrad(dy_ch, dy_s, x_ch, x_s, offs, Gn, torch.float64).double()
    tr = lambda q: q.view(torch.uint8).T.contiguous().view(torch.float8_e4m3fn).cuda()  # noqa: E731
    a, b = (tr(dy_ch), dy_s.cuda()), (tr(x_ch), x_s.cuda())
    if not accumulate:
        out = torch.full((Gn, N, K), float("nan"), dtype=torch.bfloat16, device="cuda")
        k_grouped_fp8_wgrad(a, b, out, offs.cuda(), False)
        _check(out, ref, "wgrad bf16")
        out32 = torch.full((Gn, N, K), float("nan"), dtype=torch.float32, device="cuda")
        k_grouped_fp8_wgrad(a, b, out32, offs.cuda(), False)
        _check(out32, ref, "wgrad fp32")
        for g, s in enumerate(sizes):
            if s == 0:
                assert (out[g] == 0).all(), "empty group must give exactly zero"
    else:
        old = _rand((Gn, N, K), 77, 30.0)
        out = old.clone().cuda()
        k_grouped_fp8_wgrad(a, b, out, offs.cuda(), True)
        # bf16(old + bf16(sum)): same two roundings as `weight.grad += wgrad.to(bf16)`
        expect = (old.float() + ref.float().bfloat16().float()).bfloat16()
        diff = (out.cpu().float() - expect.float()).abs()
        # one bf16 ulp of slack: the kernel's fp32 sum may round to the neighbouring bf16 value
        # (relative to the operands, not to the possibly cancelling result)
        # plus the fp32 accumulation-order noise of the sum itself (matters where it cancels to ~0)
        ulp = (old.float().abs() + ref.float().abs()) * 2.0**-6 + 1e-3 * ref.float().pow(2).mean().sqrt()
        assert (diff <= ulp).all(), diff.max().item()
        old32 = old.float()
        out32 = old32.clone().cuda()
        k_grouped_fp8_wgrad(a, b, out32, offs.cuda(), True)
        _check(out32.cpu().double() - old32.double(), ref, "wgrad fp32 accumulate")


def test_k_grouped_wgrad_on_column_slices_of_the_scale_array():
    """The weight gradient of one half of a fused projection: rows of the transposed bytes (contiguous)
    and a column slice of the scale array (its row stride is passed to the library)."""
    from pith_train_amd.operators.grouped_linear import k_grouped_fp8_wgrad

    sizes, N, K = [300, 0, 200, 128], 256, 128
    ks, offs = _groups(sizes)
    M, Gn = int(offs[-1]), len(sizes)
    dy, x = _rand((M, N), 31), _rand((M, K), 32)
    _, _, dy_ch, dy_s = Q.fp8cast_rowwise_colwise(dy)
    _, _, x_ch, x_s = Q.fp8cast_rowwise_colwise(x)
    tr = lambda q: q.view(torch.uint8).T.contiguous().view(torch.float8_e4m3fn).cuda()  # noqa: E731
    dy_t, dy_sc, x_t, x_sc = tr(dy_ch), dy_s.cuda(), tr(x_ch), x_s.cuda()
    half = N // 2
    for lo in (0, half):
        ref = G.gemm_k_grouped_wgrad(dy_ch[:, lo : lo + half].contiguous(), dy_s[:, lo : lo + half].contiguous(), x_ch, x_s,
                                     offs, Gn, torch.float64).double()
        out = torch.full((Gn, half, K), float("nan"), dtype=torch.bfloat16, device="cuda")
        k_grouped_fp8_wgrad((dy_t[lo : lo + half], dy_sc[:, lo : lo + half]), (x_t, x_sc), out, offs.cuda(), False)
        _check(out, ref, f"wgrad on scale columns {lo}..{lo + half}")
