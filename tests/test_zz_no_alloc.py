"""GPU parity of the entry point that allocates nothing: ``pt_group_rows_static`` against
``pt_group_rows`` (bit-exact: integer work), two calls in a row, the second with a smaller input,
plus the refusal of a problem beyond the built-in scratch."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _run(entry, keys, G, alignment, cap):
    from pith_train_amd import _lib

    m = keys.numel()
    dev = keys.device
    offs = torch.full((G,), -7, dtype=torch.int32, device=dev)
    ks = torch.full((G,), -7, dtype=torch.int32, device=dev)
    reverse = torch.full((m,), -7, dtype=torch.int64, device=dev)
    src_of = torch.full((cap,), -7, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    if entry == "pt_group_rows":
        nbytes = _lib.query("pt_group_rows_workspace_bytes", m, G)
        ws = torch.empty((nbytes,), dtype=torch.uint8, device=dev)
        _lib.call(entry, keys.data_ptr(), m, G, alignment, offs.data_ptr(), ks.data_ptr(), reverse.data_ptr(),
                  src_of.data_ptr(), cap, ws.data_ptr(), nbytes, stream)
    else:
        _lib.call(entry, keys.data_ptr(), m, G, alignment, offs.data_ptr(), ks.data_ptr(), reverse.data_ptr(),
                  src_of.data_ptr(), cap, stream)
    torch.cuda.synchronize()
    return offs, ks, reverse, src_of


def _keys(m, G, seed):
    g = torch.Generator().manual_seed(seed)
    k = torch.randint(0, G, (m,), generator=g, dtype=torch.int64)
    k[k == 3 % G] = (5 % G)  # one empty group when G > 5
    return k.cuda()


def test_group_rows_static_matches_workspace_entry_twice():
    from oracle import permute as OP

    # first call: the benchmark's routing size; second call: a smaller, ragged one that leaves most of
    # the first call's scratch contents in place
    for m, G, alignment, seed in ((65536, 128, 128, 0), (1000, 7, 16, 1)):
        keys = _keys(m, G, seed)
        cap = m + G * (alignment - 1)
        want = _run("pt_group_rows", keys, G, alignment, cap)
        got = _run("pt_group_rows_static", keys, G, alignment, cap)
        for name, a, b in zip(("offs", "ks", "reverse", "src_of"), got, want):
            assert torch.equal(a, b), f"{name} differs at m={m} G={G}"
        # and against the oracle's stable sort (rows of a group in ascending source order)
        _, ref_rev, ref_offs, _, ref_ks, _ = OP.scatter_for_grouped_gemm(torch.zeros((m, 1)), keys.cpu(), G, alignment)
        ref_src = torch.full((cap,), -1, dtype=torch.int32)
        ref_src[ref_rev] = torch.arange(m, dtype=torch.int32)
        assert torch.equal(got[0].cpu(), ref_offs) and torch.equal(got[1].cpu(), ref_ks)
        assert torch.equal(got[2].cpu(), ref_rev) and torch.equal(got[3].cpu(), ref_src)


def test_group_rows_static_refuses_oversized_problem():
    from pith_train_amd import _lib

    m, G = 1 << 20, 2048  # 4096 chunks x 2048 groups x 4 B = 32 MiB of counters
    assert _lib.query("pt_group_rows_workspace_bytes", m, G) > (1 << 20) + 8192
    keys = torch.zeros((m,), dtype=torch.int64, device="cuda")
    with pytest.raises(_lib.PithTrainHipError, match="scratch"):
        _run("pt_group_rows_static", keys, G, 128, m + G * 127)
