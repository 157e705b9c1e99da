#!/usr/bin/env python3
"""Writes tests/golden/next_rows_router_combine_ce.npz: seeded small cases of the three steps on
either side of the expert path - router gate, expert-parallel combine, fused cross-entropy -
computed with the CPU oracle after its pins passed (tests/test_oracle_router.py,
test_oracle_combine.py, test_oracle_cross_entropy.py).

Inputs are regenerated from the seed by the tests; their SHA-256 is stored so that a drift of the
random generator is told apart from a change of the arithmetic.  Stored outputs: the router's
expert indices and weights (both flavours), the combined rows, the loss and the in-place gradient.

Run from the repository root:  python tests/golden/make_next_rows_fixture.py
"""

import hashlib
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import combine as C  # noqa: E402
from oracle import cross_entropy as CE  # noqa: E402
from oracle import router as R  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "next_rows_router_combine_ce.npz")
T, E, K_TOP, H, V = 96, 128, 8, 256, 3000


def make_inputs():
    g = torch.Generator().manual_seed(0)
    logits = (torch.randn((T, E), generator=g) * 2).float()      # fp32 logits: no two scores tie
    logits_g = (torch.randn((T, 64), generator=g) * 2).float()   # DeepSeek flavour: 8 groups of 8, best 3
    perm = torch.randperm(T * K_TOP, generator=g)                 # arrival order of the expert outputs
    moe = torch.randn((T * K_TOP, H), generator=g).bfloat16()
    res = torch.randn((T, H), generator=g).bfloat16()
    ce_logits = (torch.randn((T, V), generator=g) * 3).bfloat16()
    target = torch.randint(0, V, (T,), generator=g)
    target[::9] = -100
    return logits, logits_g, perm, moe, res, ce_logits, target


def bits(t: torch.Tensor) -> np.ndarray:
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def digest(*arrays) -> str:
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()


def compute():
    logits, logits_g, perm, moe, res, ce_logits, target = make_inputs()
    idx, w, _ = R.softmax_topk(logits, K_TOP, norm_topk_prob=True)
    gidx, gw, _ = R.softmax_topk(logits_g, 6, scale=16.0, num_group=8, topk_group=3)
    tidx, tw, _ = R.topk_softmax(logits[:, :32].bfloat16(), 4)
    combined = C.combine_ep_fwd(moe, perm, w, res)
    loss, grad, loss_rows, n = CE.cross_entropy_fwd(ce_logits, target)
    return {
        "input_sha256": np.array(digest(*[bits(t) for t in (logits, logits_g, perm, moe, res, ce_logits, target)])),
        "router_idx": idx.numpy(), "router_weight": w.numpy(),
        "router_grouped_idx": gidx.numpy(), "router_grouped_weight": gw.numpy(),
        "router_topk_softmax_idx": tidx.numpy(), "router_topk_softmax_weight": tw.numpy(),
        "combined": bits(combined),
        "ce_loss": loss.numpy(), "ce_rows": np.array(n), "ce_grad": bits(grad),
    }


if __name__ == "__main__":
    np.savez_compressed(OUT, **compute())
    print("wrote", OUT, os.path.getsize(OUT), "bytes")
