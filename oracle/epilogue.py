"""Oracle: fused activation / bias epilogues of the expert path.

Test infrastructure only (see ``oracle/__init__.py``).

  * ``silu_mul_fwd/bwd``        <- ``pithtrain/operators/silu_mul.py:28-87``
  * ``clamped_swiglu_fwd/bwd``  <- ``pithtrain/operators/clamped_swiglu.py:18-89``
  * ``indexed_bias_add_fwd``    <- ``pithtrain/operators/indexed_bias_add.py:100-104``
  * ``segment_sum``             <- ``pithtrain/operators/indexed_bias_add.py:20-96``

All math in float32 (or ``accum``), one rounding to the storage dtype, as in the
kernels.  The last ulp of ``sigmoid`` differs between back ends, so these are
tolerance-pinned (the bf16 rounding of the result hides almost all of it).
"""

from __future__ import annotations

import torch


def silu_mul_fwd(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    g, u = gate.float(), up.float()
    return (g * torch.sigmoid(g) * u).to(up.dtype)


def silu_mul_bwd(grad_out, gate, up):
    """grad_up = do*silu(g); grad_gate = do*u*sig*(1 + g - silu(g)). (silu_mul.py:62-87)"""
    do, g, u = grad_out.float(), gate.float(), up.float()
    sig = torch.sigmoid(g)
    silu = g * sig
    grad_up = do * silu
    grad_gate = do * u * sig * (1.0 + g - silu)
    return grad_gate.to(gate.dtype), grad_up.to(up.dtype)


def clamped_swiglu_fwd(gate_up: torch.Tensor, alpha: float, limit: float) -> torch.Tensor:
    """gate = even columns, up = odd columns. (clamped_swiglu.py:27-46)"""
    g = gate_up[:, 0::2].float()
    u = gate_up[:, 1::2].float()
    gc = torch.clamp(g, max=limit)
    uc = torch.clamp(u, min=-limit, max=limit)
    sig = torch.sigmoid(alpha * gc)
    return ((uc + 1.0) * (gc * sig)).to(gate_up.dtype)


def clamped_swiglu_bwd(grad_out, gate_up, alpha: float, limit: float) -> torch.Tensor:
    """(clamped_swiglu.py:58-89)"""
    do = grad_out.float()
    g = gate_up[:, 0::2].float()
    u = gate_up[:, 1::2].float()
    gc = torch.clamp(g, max=limit)
    uc = torch.clamp(u, min=-limit, max=limit)
    sig = torch.sigmoid(alpha * gc)
    glu = gc * sig
    grad_uc = do * glu
    grad_gc = do * (uc + 1.0) * sig * (1.0 + alpha * gc * (1.0 - sig))
    grad_g = torch.where(g <= limit, grad_gc, torch.zeros_like(grad_gc))
    grad_u = torch.where((u >= -limit) & (u <= limit), grad_uc, torch.zeros_like(grad_uc))
    out = torch.empty_like(gate_up)
    out[:, 0::2] = grad_g.to(gate_up.dtype)
    out[:, 1::2] = grad_u.to(gate_up.dtype)
    return out


def indexed_bias_add_fwd(x, bias, group_ids):
    """x + bias[group_ids] in the storage dtype. (indexed_bias_add.py:100-104)"""
    return x + bias[group_ids.to(torch.int64)]


def segment_sum(x, grouped_mm_offs, out_dtype, accum=torch.float32):
    """Row sums per group [offs[g-1], offs[g]) with offs clamped to M; accumulate in ``accum``,
    cast to ``out_dtype``. (indexed_bias_add.py:54-96)"""
    M, H = x.shape
    E = grouped_mm_offs.shape[0]
    out = torch.zeros((E, H), dtype=accum)
    start = 0
    for g, end in enumerate(grouped_mm_offs.tolist()):
        end = min(int(end), M)
        if end > start:
            out[g] = x[start:end].to(accum).sum(0)
        start = end
    return out.to(out_dtype)
