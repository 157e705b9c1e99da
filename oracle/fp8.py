"""Oracle: blockwise FP8 (e4m3fn) quantisation with power-of-two fp32 scales.

Test infrastructure only (see ``oracle/__init__.py``).

Follows ``pithtrain/operators/deepgemm_quantize.py``:
  * ``compute_fp8_scale``                      <- ``_compute_fp8_scale`` (:36-83)
  * ``fp8cast_rowwise_colwise``                <- :91-259
  * ``fp8cast_rowwise_kmajor``                 <- :174-194, :262-333
  * ``fp8cast_rowwise_transpose``              <- :341-482
  * ``fp8cast_rowwise_blockwise_transpose``    <- :490-629
  * ``fp8cast_blockwise_transpose``            <- :637-756
  * ``fp8cast_blockwise_transpose_batched``    <- :764-899

All tensors are CPU tensors.  FP8 outputs are ``torch.float8_e4m3fn``.
"""

from __future__ import annotations

import numpy as np
import torch

BLOCK = 128
FP8_MAX_RCP = np.float32(1.0 / 448.0)  # the fp32 constant the kernels multiply by (:48-51)
AMAX_CLAMP = np.float32(1e-4)  # :50


# --------------------------------------------------------------------------
# scale rule
# --------------------------------------------------------------------------
def compute_fp8_scale(amax: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """(scale, 1/scale) from per-group amax; both exact powers of two.

    deepgemm_quantize.py:50-51  scale_input = max(amax, 1e-4) * fl32(1/448)
    deepgemm_quantize.py:69-73  clear mantissa, +1 exponent if mantissa != 0
    deepgemm_quantize.py:76-77  clamp to 2**-126
    deepgemm_quantize.py:80-81  reciprocal by exponent flip (254<<23) - bits
    """
    a = amax.to(torch.float32)
    s_in = torch.maximum(a, torch.tensor(float(AMAX_CLAMP), dtype=torch.float32)) * torch.tensor(
        float(FP8_MAX_RCP), dtype=torch.float32
    )
    bits = s_in.contiguous().view(torch.int32)
    mant = bits & 0x007FFFFF
    pow2 = (bits & 0x7F800000) + torch.where(mant != 0, 0x00800000, 0).to(torch.int32)
    scale = pow2.view(torch.float32)
    scale = torch.maximum(scale, torch.tensor(2.0**-126, dtype=torch.float32))
    rcp_bits = (254 << 23) - scale.contiguous().view(torch.int32)
    rcp = rcp_bits.view(torch.float32)
    return scale, rcp


# --------------------------------------------------------------------------
# e4m3fn encoder: integer-only numpy (independent of torch's cast)
# --------------------------------------------------------------------------
def cast_e4m3_numpy(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even float32 -> OCP e4m3fn byte, finite |x| <= 448 assumed
    (saturates to 448 above, NaN -> 0x7F).  Written from the format definition:
    1 sign, 4 exponent (bias 7), 3 mantissa, subnormals at exponent 0, no inf.
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    b = x.view(np.uint32)
    sign = ((b >> 24) & 0x80).astype(np.uint8)
    mag = (b & 0x7FFFFFFF).astype(np.uint64)
    out = np.zeros(x.shape, dtype=np.uint8)

    exp = (mag >> 23).astype(np.int64) - 127  # unbiased
    man = (mag & 0x7FFFFF) | 0x800000  # 24-bit significand with hidden one (normals)
    # fp32 subnormals are < 2**-126: far below half the smallest e4m3 subnormal -> 0
    # target: value = q * 2**-9 for e4m3 subnormals (q in 0..7), normal: (8+m) * 2**(e-3)
    # number of fp32 significand bits to drop so the result is in units of the e4m3 ulp
    e_eff = np.maximum(exp, -6)  # below 2**-6 the ulp is fixed at 2**-9
    shift = (23 - 3) + (e_eff - exp)  # >= 20
    shift = np.minimum(shift, 40)
    sig = man.astype(np.uint64)
    q = sig >> shift.astype(np.uint64)
    rem = sig & ((np.uint64(1) << shift.astype(np.uint64)) - np.uint64(1))
    half = np.uint64(1) << (shift.astype(np.uint64) - np.uint64(1))
    round_up = (rem > half) | ((rem == half) & ((q & np.uint64(1)) == 1))
    q = q + round_up.astype(np.uint64)
    # q is in units of ulp(e_eff): normal numbers have q in [8, 16], subnormals q in [0, 8]
    # encode: for e_eff >= -6 and q >= 8: biased exponent (e_eff + 7), mantissa q - 8;
    # q == 16 carries into the next exponent; adding works because the fields are adjacent.
    biased = (e_eff + 7).astype(np.int64)
    code = np.where(q >= 8, (biased << 3) + (q.astype(np.int64) - 8), q.astype(np.int64))
    # when exp < -6 the "hidden one" was shifted as a normal bit, so q<8 is the subnormal
    # mantissa directly and q == 8 means the smallest normal (biased 1, mantissa 0) = code 8,
    # which the first branch yields too because biased == 1 there.
    code = np.where(mag == 0, 0, code)
    code = np.where(exp < -127 + 1, 0, code)  # fp32 zero / subnormal
    code = np.minimum(code, 0x7E)  # saturate to 448
    isnan = mag > 0x7F800000
    out = (code.astype(np.uint8) | sign).astype(np.uint8)
    out = np.where(isnan, np.uint8(0x7F), out)
    return out


def cast_e4m3(x: torch.Tensor) -> torch.Tensor:
    """float32 -> e4m3fn (round-to-nearest-even), the library cast used by the oracle."""
    return x.to(torch.float8_e4m3fn)


# --------------------------------------------------------------------------
# building blocks
# --------------------------------------------------------------------------
def _cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def _pad2d(x: torch.Tensor, rows: int, cols: int) -> torch.Tensor:
    """Zero-pad like the kernels' masked loads with other=0.0 (:140-141)."""
    M, N = x.shape
    if M == rows and N == cols:
        return x
    p = torch.zeros((rows, cols), dtype=x.dtype)
    p[:M, :N] = x
    return p


def _rowwise(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """1x128 scaling along the last dim of a 2-D tensor. (:145-164)"""
    M, N = x.shape
    nb = _cdiv(N, BLOCK)
    xp = _pad2d(x, M, nb * BLOCK).view(M, nb, BLOCK)
    amax = xp.abs().amax(dim=2).float() if M > 0 else torch.zeros((0, nb))
    scale, rcp = compute_fp8_scale(amax)
    q = cast_e4m3(xp.float() * rcp[:, :, None]).view(M, nb * BLOCK)[:, :N].contiguous()
    return q, scale


def _colwise(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """128-row groups, one scale per column per group; ragged M is zero padded. (:166-201)"""
    M, N = x.shape
    mb = _cdiv(M, BLOCK)
    xp = _pad2d(x, mb * BLOCK, N).view(mb, BLOCK, N)
    amax = xp.abs().amax(dim=1).float() if N > 0 else torch.zeros((mb, 0))
    scale, rcp = compute_fp8_scale(amax)
    q = cast_e4m3(xp.float() * rcp[:, None, :]).view(mb * BLOCK, N)[:M].contiguous()
    return q, scale


def _blockwise(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """128x128 tiles, one scale per tile. (:678-706)"""
    M, K = x.shape
    mb, kb = _cdiv(M, BLOCK), _cdiv(K, BLOCK)
    xp = _pad2d(x, mb * BLOCK, kb * BLOCK).view(mb, BLOCK, kb, BLOCK)
    amax = xp.abs().amax(dim=(1, 3)).float()
    scale, rcp = compute_fp8_scale(amax)
    q = cast_e4m3(xp.float() * rcp[:, None, :, None]).view(mb * BLOCK, kb * BLOCK)[:M, :K]
    return q.contiguous(), scale


# --------------------------------------------------------------------------
# the six entry points
# --------------------------------------------------------------------------
def fp8cast_rowwise_colwise(x: torch.Tensor):
    """(tok_fp8[M,N], tok_scale[M,ceil(N/128)], ch_fp8[M,N], ch_scale[M/128,N]). (:204-259)"""
    assert x.ndim == 2 and x.shape[0] % BLOCK == 0
    tok, tok_s = _rowwise(x)
    ch, ch_s = _colwise(x)
    return tok, tok_s, ch, ch_s


def fp8cast_rowwise_kmajor(x: torch.Tensor, grouped_mm_offs: torch.Tensor):
    """Rowwise as above; colwise bytes re-laid per group as (N, K_g) blocks concatenated
    into a flat 1-D buffer, scales transposed to (N, M/128). (:174-194, :262-333)"""
    tok, tok_s, ch, ch_s = fp8cast_rowwise_colwise(x)
    M, N = x.shape
    flat = torch.empty(M * N, dtype=torch.uint8)
    chb = ch.view(torch.uint8)
    start = 0
    covered = 0
    for end in grouped_mm_offs.tolist():
        end = int(end)
        if end > start:
            flat[start * N : end * N] = chb[start:end].T.contiguous().view(-1)
            covered = end
        start = max(start, end)
    # Rows past the last offset belong to the last group per the clamped searchsorted
    # (:300-305); the kernel would index them relative to that group's start with its
    # K_g, which only stays in bounds when offs[-1] == M.  The oracle requires that.
    assert covered == M or M == 0, "grouped_mm_offs[-1] must equal M"
    return tok, tok_s, flat.view(torch.float8_e4m3fn), ch_s.T.contiguous()


def fp8cast_rowwise_transpose(x: torch.Tensor):
    """(tok_fp8[M,N], tok_scale[M,ceil(N/128)], t_fp8[N,M], t_scale[N,ceil(M/128)]). (:429-482)"""
    assert x.ndim == 2
    tok, tok_s = _rowwise(x)
    ch, ch_s = _colwise(x)  # axis-0 reduction of the tile == rowwise of x.T (:406-426)
    return tok, tok_s, ch.view(torch.uint8).T.contiguous().view(torch.float8_e4m3fn), ch_s.T.contiguous()


def fp8cast_rowwise_blockwise_transpose(x: torch.Tensor):
    """(tok_fp8[M,K], tok_scale[M,ceil(K/128)], blk_t_fp8[K,M], blk_t_scale[ceil(K/128),ceil(M/128)]).
    (:575-629)"""
    assert x.ndim == 2
    tok, tok_s = _rowwise(x)
    blk, blk_s = _blockwise(x)
    return (
        tok,
        tok_s,
        blk.view(torch.uint8).T.contiguous().view(torch.float8_e4m3fn),
        blk_s.T.contiguous(),
    )


def fp8cast_blockwise_transpose(x: torch.Tensor):
    """(fp8[M,K], scale[ceil(M/128),ceil(K/128)], fp8_t[K,M], scale_t = scale.T). (:709-756)"""
    assert x.ndim == 2
    blk, blk_s = _blockwise(x)
    return (
        blk,
        blk_s,
        blk.view(torch.uint8).T.contiguous().view(torch.float8_e4m3fn),
        blk_s.T.contiguous(),
    )


def fp8cast_blockwise_transpose_batched(x: torch.Tensor):
    """Per-group blockwise + transpose for (G, N, K). (:846-899)"""
    assert x.ndim == 3
    G, N, K = x.shape
    nb, kb = _cdiv(N, BLOCK), _cdiv(K, BLOCK)
    out = torch.empty((G, N, K), dtype=torch.float8_e4m3fn)
    scale = torch.empty((G, nb, kb), dtype=torch.float32)
    out_t = torch.empty((G, K, N), dtype=torch.float8_e4m3fn)
    scale_t = torch.empty((G, kb, nb), dtype=torch.float32)
    for g in range(G):
        q, s, qt, st = fp8cast_blockwise_transpose(x[g])
        out[g], scale[g], out_t[g], scale_t[g] = q, s, qt, st
    return out, scale, out_t, scale_t


# --------------------------------------------------------------------------
# dequantisation helpers (used by the GEMM oracle)
# --------------------------------------------------------------------------
def dequant_rowwise(q: torch.Tensor, scale: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
    """q[M,N] e4m3 with scale[M,ceil(N/128)] -> real values."""
    M, N = q.shape
    s = scale.repeat_interleave(BLOCK, dim=1)[:, :N]
    return q.to(dtype) * s.to(dtype)


def dequant_colwise(q: torch.Tensor, scale: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
    """q[M,N] e4m3 with scale[ceil(M/128),N] -> real values."""
    M, N = q.shape
    s = scale.repeat_interleave(BLOCK, dim=0)[:M]
    return q.to(dtype) * s.to(dtype)


def dequant_blockwise(q: torch.Tensor, scale: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
    """q[...,M,K] e4m3 with scale[...,ceil(M/128),ceil(K/128)] -> real values."""
    M, K = q.shape[-2:]
    s = scale.repeat_interleave(BLOCK, dim=-2).repeat_interleave(BLOCK, dim=-1)[..., :M, :K]
    return q.to(dtype) * s.to(dtype)
