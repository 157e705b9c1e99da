"""Oracle: whole MoE expert layer (stage 3), forward and backward, on the CPU.

Test infrastructure only (see ``oracle/__init__.py``).  Composition follows

  * ``forward_stage3``      models/qwen3_moe.py:216-227  (expand -> scatter -> experts -> gather)
  * ``Qwen3MoeExperts``     models/qwen3_moe.py:45-65    kind="split"  (gate, up, down)
  * ``Qwen35MoeExperts``    models/qwen35_moe.py:179-200 kind="fused"  (gate_up halves, down)
  * ``GptOssExperts``       models/gpt_oss.py:95-157     kind="gpt_oss" (interleaved, biases)

with the per-operator oracles of this package.  ``fp8=False`` runs the BF16 grouped-linear
semantics of ``GroupedLinearFunc`` (grouped_linear.py:18-55) instead: that is the reference's
pure-PyTorch path and what ``bench.py`` times as the CPU baseline.
"""

from __future__ import annotations

import torch

from . import epilogue as E
from . import gemm as G
from . import permute as P


def _lin_fwd(x, w, offs, fp8, accum):
    if fp8:
        return G.fp8_grouped_linear_forward(x, w, offs, accum)
    return G.bf16_grouped_mm(x, w, offs), (x, w)


def _lin_bwd(dy, saved, offs, num_groups, fp8, accum):
    if fp8:
        return G.fp8_grouped_linear_backward(dy, saved, offs, num_groups, accum)
    x, w = saved
    dx = torch.zeros_like(x)
    dw = torch.zeros_like(w)
    start = 0
    for g, end in enumerate(offs.tolist()):
        if end > start:
            dx[start:end] = dy[start:end] @ w[g]
            dw[g] = dy[start:end].T @ x[start:end]
        start = end
    return dx, dw


def moe_layer_fwd_bwd(
    tokens: torch.Tensor,
    expert_idxs: torch.Tensor,
    weights: dict,
    grad_out: torch.Tensor | None,
    num_groups: int,
    kind: str = "split",
    fp8: bool = True,
    expand_idx: torch.Tensor | None = None,
    accum=torch.float32,
    alpha: float = 1.702,
    limit: float = 7.0,
):
    """Returns a dict with ``out`` [m,H] and, when ``grad_out`` is given, ``grad_tokens`` and one
    gradient per entry of ``weights`` (same keys)."""
    src = tokens if expand_idx is None else P.padded_index_gather(tokens, expand_idx)
    xp, reverse, offs, ks, ks_tensor, _ = P.scatter_for_grouped_gemm(src, expert_idxs, num_groups)
    Mp = xp.shape[0]
    res = {"offs": offs, "reverse": reverse}
    if kind == "split":
        g, sg = _lin_fwd(xp, weights["gate_proj"], offs, fp8, accum)
        u, su = _lin_fwd(xp, weights["up_proj"], offs, fp8, accum)
        h = E.silu_mul_fwd(g, u)
        y, sd = _lin_fwd(h, weights["down_proj"], offs, fp8, accum)
    elif kind == "fused":
        gu, sgu = _lin_fwd(xp, weights["gate_up_proj"], offs, fp8, accum)
        inter = gu.shape[1] // 2
        g, u = gu[:, :inter].contiguous(), gu[:, inter:].contiguous()
        h = E.silu_mul_fwd(g, u)
        y, sd = _lin_fwd(h, weights["down_proj"], offs, fp8, accum)
    elif kind == "gpt_oss":
        gid = P.precompute_group_indices(offs, Mp).long()
        gu0, sgu = _lin_fwd(xp, weights["gate_up_proj"], offs, fp8, accum)
        gu = E.indexed_bias_add_fwd(gu0, weights["gate_up_proj_bias"], gid)
        h = E.clamped_swiglu_fwd(gu, alpha, limit)
        y0, sd = _lin_fwd(h, weights["down_proj"], offs, fp8, accum)
        y = E.indexed_bias_add_fwd(y0, weights["down_proj_bias"], gid)
    else:
        raise ValueError(kind)
    res["out"] = P.padded_index_gather(y, reverse)
    if grad_out is None:
        return res

    dy = P.padded_index_gather_backward(grad_out, reverse, Mp)
    if kind == "gpt_oss":
        res["down_proj_bias"] = E.segment_sum(dy, offs, weights["down_proj_bias"].dtype)
    dh, res["down_proj"] = _lin_bwd(dy, sd, offs, num_groups, fp8, accum)
    if kind == "split":
        dg, du = E.silu_mul_bwd(dh, g, u)
        dx1, res["gate_proj"] = _lin_bwd(dg, sg, offs, num_groups, fp8, accum)
        dx2, res["up_proj"] = _lin_bwd(du, su, offs, num_groups, fp8, accum)
        dxp = dx1 + dx2  # autograd sums the two uses of x in the storage dtype
    elif kind == "fused":
        dg, du = E.silu_mul_bwd(dh, g, u)
        dgu = torch.cat([dg, du], dim=1)
        dxp, res["gate_up_proj"] = _lin_bwd(dgu, sgu, offs, num_groups, fp8, accum)
    else:
        dgu = E.clamped_swiglu_bwd(dh, gu, alpha, limit)
        res["gate_up_proj_bias"] = E.segment_sum(dgu, offs, weights["gate_up_proj_bias"].dtype)
        dxp, res["gate_up_proj"] = _lin_bwd(dgu, sgu, offs, num_groups, fp8, accum)
    dsrc = P.scatter_backward(dxp, reverse)
    if expand_idx is not None:
        dsrc = P.padded_index_gather_backward(dsrc, expand_idx, tokens.shape[0])
    res["grad_tokens"] = dsrc
    return res


def gemm_flops(m_rows: int, hidden: int, inter: int, fwd_bwd: bool = True) -> float:
    """Algorithmic GEMM FLOPs of one layer: 2*M*H*2I + 2*M*I*H forward, x3 with dgrad and wgrad;
    padding rows are not counted (convention of benchmarks/operators/fp8/test_deepgemm.py:10-14)."""
    fwd = 2.0 * m_rows * hidden * 2 * inter + 2.0 * m_rows * inter * hidden
    return fwd * (3 if fwd_bwd else 1)


def make_routing(num_tokens: int, num_experts: int, top_k: int, seed: int = 0, zipf_s: float | None = None,
                 return_scale: bool = False):
    """Router logits ~N(0,1) (+ optional Zipf(s) popularity bias) -> softmax -> top-k ids [T,k].

    The Zipf bias is ``b_e = log p_e - mean(log p)`` with ``p_e`` proportional to ``rank_e ** -s``
    (ranks from a seeded permutation).  The skewed configuration asks for routing in which some
    expert gets no token and another more than four times the mean; when the bias as stated does
    not produce that, it is multiplied by 1.25, 1.5, ... until it does (``return_scale`` also
    returns that factor)."""
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn((num_tokens, num_experts), generator=g)
    scale = 1.0
    if zipf_s is None:
        idx = torch.topk(logits.softmax(dim=-1), k=top_k, dim=-1).indices
    else:
        ranks = torch.randperm(num_experts, generator=g).float() + 1.0
        logp = -zipf_s * ranks.log()
        bias = logp - logp.mean()
        while True:
            idx = torch.topk((logits + scale * bias).softmax(dim=-1), k=top_k, dim=-1).indices
            counts = torch.bincount(idx.reshape(-1), minlength=num_experts)
            if ((counts == 0).any() and counts.max() > 4 * counts.float().mean()) or scale >= 8.0:
                break
            scale += 0.25
    return (idx, scale) if return_scale else idx
