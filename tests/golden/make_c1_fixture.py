#!/usr/bin/env python3
"""Writes tests/golden/c1_toy_fp8_grouped_linear.npz: the toy FP8 grouped linear (forward only)
of the benchmark's first configuration - 8 experts, K=256, N=512, 1024 tokens, top-2 routing,
seed 0 - computed with the CPU oracle after the oracle passed its known-answer tests.

Inputs are regenerated from the seed by the tests; their SHA-256 is stored so that a drift of the
random generator is told apart from a change of the arithmetic.  Stored outputs: grouped offsets
and the row permutation, the FP8 bytes and power-of-two scales of the scattered activations and of
the weights (bit-exact targets), and the bf16 output - its first 256 rows and the SHA-256 of all of
it (tolerance target for the GPU on the stored rows, bit-exact for the oracle itself).

Run from the repository root:  python tests/golden/make_c1_fixture.py
"""

import hashlib
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import fp8 as F  # noqa: E402
from oracle import gemm as G  # noqa: E402
from oracle import moe as OM  # noqa: E402
from oracle import permute as P  # noqa: E402

E, K, N, T, TOPK, SEED = 8, 256, 512, 1024, 2, 0
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c1_toy_fp8_grouped_linear.npz")


def make_inputs():
    ids = OM.make_routing(T, E, TOPK, seed=SEED)
    g = torch.Generator().manual_seed(SEED)
    x = torch.randn((T, K), generator=g).bfloat16()
    w = (torch.randn((E, N, K), generator=g) * 0.02).bfloat16()
    tokens = x.unsqueeze(1).expand(-1, TOPK, -1).reshape(-1, K).contiguous()
    return tokens, ids.reshape(-1), w


def bits(t: torch.Tensor) -> np.ndarray:
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.float8_e4m3fn:
        return t.view(torch.uint8).numpy()
    return t.numpy()


def digest(*arrays) -> str:
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()


def compute():
    tokens, eidx, w = make_inputs()
    xp, reverse, offs, ks, ks_tensor, _ = P.scatter_for_grouped_gemm(tokens, eidx, E)
    x_fp8, x_scale, _, _ = F.fp8cast_rowwise_colwise(xp)
    w_fp8, w_scale, _, _ = F.fp8cast_blockwise_transpose_batched(w)
    out = G.gemm_m_grouped_nt(x_fp8, x_scale, w_fp8, w_scale, offs, torch.bfloat16)
    return {
        "input_sha256": np.array(digest(bits(tokens), eidx.numpy(), bits(w))),
        "offs": offs.numpy().astype(np.int32),
        "reverse": reverse.numpy().astype(np.int64),
        "x_fp8": bits(x_fp8),
        "x_scale": x_scale.numpy().astype(np.float32),
        "w_fp8": bits(w_fp8),
        "w_scale": w_scale.numpy().astype(np.float32),
        "out_bf16_bits_head": bits(out)[:256].copy(),  # first 256 grouped rows in full
        "out_sha256": np.array(digest(bits(out))),     # all rows
    }


if __name__ == "__main__":
    np.savez_compressed(OUT, **compute())
    print(f"wrote {OUT} ({os.path.getsize(OUT) / 1e6:.2f} MB)")
