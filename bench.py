#!/usr/bin/env python3
"""Benchmark of the FP8 grouped-expert path on one MI355X.

One "step" = one full MoE expert layer (stage 3) forward + backward over one batch of synthetic
tokens resident in HBM: weight quantisation (every step - nothing is cached across steps), token
scatter, gate/up grouped GEMM, SwiGLU, down grouped GEMM, unpermute, and the whole backward
(dgrad + wgrad GEMMs, epilogue backward, gathers).

Prints ONE JSON line.  ``value`` is algorithmic GEMM TFLOP/s of the whole step (padding rows not
counted); ``roofline`` describes the dominant kernel (the FP8 MFMA GEMM) from HIP-event timings
taken around every GEMM launch inside the timed region; ``cpu_baseline`` is the CPU oracle of the
same layer (the reference's pure-PyTorch BF16 grouped-linear semantics) on a bounded sample.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

FP8_DENSE_PEAK_TFLOPS = 5000.0  # MI355X dense FP8 MFMA
HBM_PEAK_GBS = 8000.0

# Average HBM bytes moved by one GEMM launch (fetch + write), from the FETCH_SIZE / WRITE_SIZE
# counter runs summarised under profiles/ (scaled by the same counters' readings for a plain copy
# of known size).  FETCH_SIZE counts what the L2 asks of the fabric, whether the memory-side cache
# or HBM answers: where successive waves of tiles re-read operand panels that the 4 MiB L2 of an
# XCD cannot keep (GPT-OSS: 2.5x the algorithmic bytes) most of the excess is served by that cache.
GEMM_TRAFFIC_BYTES_PER_LAUNCH = {"qwen3-30b-a3b-moe": 747e6, "dsv2-lite-moe": 477e6, "gpt-oss-20b-moe": 2831e6,
                                 "qwen3-decoder-linears-32k": 923e6}

WORKLOADS = {
    # name: (kind, hidden, intermediate, experts, top_k, tokens, zipf)
    "qwen3-30b-a3b-moe": ("fused", 2048, 768, 128, 8, 8192, None),
    "toy": ("split", 256, 512, 8, 2, 1024, None),
    "dsv2-lite-moe": ("split", 2048, 1408, 64, 6, 8192, 1.2),
    "gpt-oss-20b-moe": ("gpt_oss", 2880, 2880, 32, 4, 16384, None),
    "qwen3-decoder-linears-32k": ("fused", 2048, 768, 128, 8, 32768, None),
}
# Parts of a workload beyond the routed experts (all on the same tokens):
#   shared_mlp: width of a dense FP8 SwiGLU MLP (DeepSeek-V2-Lite's two shared experts run as one);
#   dense_linears: (in, out) of dense FP8 linears (q, k, v, o projections of the decoder layer);
#   dedup_fraction: share of routed rows that re-use an already received token row (the rows reach the
#   experts through the dedup expand index instead of being materialised).
EXTRAS = {
    "dsv2-lite-moe": {"shared_mlp": 2816},
    "qwen3-decoder-linears-32k": {"dense_linears": [(2048, 4096), (2048, 512), (2048, 512), (4096, 2048)],
                                  "dedup_fraction": 0.25},
}


def extra_flops(extras, T, H):
    """Algorithmic GEMM FLOPs (fwd + dgrad + wgrad) of the dense parts."""
    f = 0.0
    if "shared_mlp" in extras:
        f += 3 * 6.0 * T * H * extras["shared_mlp"]
    for fin, fout in extras.get("dense_linears", []):
        f += 3 * 2.0 * T * fin * fout
    return f


def make_dedup_expand(rows, fraction, seed=0):
    """expand_idx[rows] into U = rows * (1 - fraction) unique received rows: every unique row is
    referenced at least once, the remaining references are uniform repeats."""
    import torch

    g = torch.Generator().manual_seed(seed + 1)
    U = int(round(rows * (1.0 - fraction)))
    idx = torch.cat([torch.arange(U), torch.randint(0, U, (rows - U,), generator=g)])
    return idx[torch.randperm(rows, generator=g)], U


ZIPF_BIAS_SCALE = {}  # zipf_s -> factor the popularity bias was multiplied by (reported in the bench line)


def make_routing(T, E, k, seed=0, zipf_s=None):
    """Router logits ~N(0,1) (+ an optional Zipf(s) popularity bias: log-probabilities of a seeded
    random ranking, centred) -> softmax -> top-k expert ids [T, k].  The skewed workload asks for
    routing with at least one empty expert and one above four times the mean count: the bias is
    multiplied by 1.25, 1.5, ... until the counts say so, and the factor is reported."""
    import torch

    g = torch.Generator().manual_seed(seed)
    logits = torch.randn((T, E), generator=g)
    if zipf_s is None:
        return torch.topk(logits.softmax(dim=-1), k=k, dim=-1).indices
    ranks = torch.randperm(E, generator=g).float() + 1.0
    logp = -zipf_s * ranks.log()
    bias, scale = logp - logp.mean(), 1.0
    while True:
        idx = torch.topk((logits + scale * bias).softmax(dim=-1), k=k, dim=-1).indices
        counts = torch.bincount(idx.reshape(-1), minlength=E)
        if ((counts == 0).any() and counts.max() > 4 * counts.float().mean()) or scale >= 8.0:
            break
        scale += 0.25
    ZIPF_BIAS_SCALE[zipf_s] = scale
    return idx


def gemm_flops(rows, H, I):
    """Algorithmic GEMM FLOPs of one layer, forward + dgrad + wgrad; padding rows are not counted."""
    return 3 * (2.0 * rows * H * 2 * I + 2.0 * rows * I * H)


def make_inputs(kind, H, I, E, k, T, zipf, seed=0):
    import torch

    ids = make_routing(T, E, k, seed=seed, zipf_s=zipf)
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((T, H), generator=g).bfloat16()
    dy = torch.randn((T * k, H), generator=g).bfloat16()
    r = lambda *s: (torch.randn(s, generator=g) * 0.02).bfloat16()  # noqa: E731
    if kind == "split":
        w = {"gate_proj": r(E, I, H), "up_proj": r(E, I, H), "down_proj": r(E, H, I)}
    elif kind == "fused":
        w = {"gate_up_proj": r(E, 2 * I, H), "down_proj": r(E, H, I)}
    else:
        w = {"gate_up_proj": r(E, 2 * I, H), "gate_up_proj_bias": r(E, 2 * I), "down_proj": r(E, H, I),
             "down_proj_bias": r(E, H)}
    return ids, x, dy, w


def build_module(kind, H, I, E, w):
    import torch

    from pith_train_amd.modules import experts as X

    if kind == "split":
        mod = X.Qwen3MoeExperts(H, I, E)
    elif kind == "fused":
        mod = X.Qwen35MoeExperts(H, I, E)
    else:
        mod = X.GptOssExperts(H, I, E)
    mod = mod.cuda().to(torch.bfloat16)
    with torch.no_grad():
        for n, v in w.items():
            p = getattr(mod, n)
            (p if kind == "gpt_oss" else p.weight).copy_(v.cuda())
    return mod


class GemmTimer:
    """HIP events (on the stream the kernels are launched on) around every GEMM entry point."""

    NAMES = ("pt_gemm_m_grouped_nt", "pt_gemm_m_grouped_nt_scatter", "pt_gemm_m_grouped_nt_bias",
             "pt_gemm_m_grouped_nn", "pt_gemm_m_grouped_nn_scatter",
             "pt_gemm_m_grouped_nt_scatter_bias", "pt_gemm_k_grouped_wgrad",
             "pt_gemm_k_grouped_wgrad_ld",
             "pt_gemm_nt_dense", "pt_gemm_nt_dense_splitk", "pt_gemm_nt_dense_ld", "pt_gemm_nt_dense_splitk_ld")

    def __init__(self):
        self.records = []
        self.enabled = False

    def install(self):
        import torch

        from pith_train_amd import _lib

        orig = _lib.call
        timer = self

        def call(name, *args):
            if timer.enabled and name in GemmTimer.NAMES:
                a = torch.cuda.Event(enable_timing=True)
                b = torch.cuda.Event(enable_timing=True)
                a.record()
                orig(name, *args)
                b.record()
                # rows x columns x reduction as the entry point takes them (the three int64 sizes)
                sizes = {"pt_gemm_nt_dense": args[6:9], "pt_gemm_nt_dense_splitk": args[7:10],
                         "pt_gemm_nt_dense_ld": args[8:11], "pt_gemm_nt_dense_splitk_ld": args[9:12],
                         "pt_gemm_k_grouped_wgrad": args[9:12],
                         "pt_gemm_k_grouped_wgrad_ld": args[11:14]}.get(name, args[8:11])
                timer.records.append((name, a, b, "x".join(str(int(v)) for v in sizes)))
            else:
                orig(name, *args)

        _lib.call = call
        # modules imported `_lib` (the module), so they see the patched attribute
        return self

    def install_all(self):
        """Second mode, used after the timed region only: events around every other entry point too,
        collected in ``other`` as (name, start, end, args)."""
        self.other = []
        self.all_enabled = False
        import torch

        from pith_train_amd import _lib

        inner = _lib.call
        timer = self

        def call(name, *args):
            if timer.all_enabled and name not in GemmTimer.NAMES:
                a = torch.cuda.Event(enable_timing=True)
                b = torch.cuda.Event(enable_timing=True)
                a.record()
                inner(name, *args)
                b.record()
                timer.other.append((name, a, b, args))
            else:
                inner(name, *args)

        _lib.call = call
        return self

    def in_step_report(self, steps, padded_rows, routed_rows):
        """HBM-bound entry points as they ran inside the step (after the kernels before them, with
        the caches in the state the step leaves them in): average duration of one call, and for
        the quantisers the algorithmic bytes (bf16 2 B, FP8 1 B, one fp32 scale per 128 elements,
        source rows of a gather counted once) over it.  Row counts above the padded row count are
        buffer capacities; the kernels stop at the real count, which is what is priced."""
        sc = 4.0 / 128

        def nbytes(name, a):
            rows = lambda m: min(int(m), padded_rows)  # noqa: E731
            if name == "pt_quant_rowwise_colwise":
                return rows(a[2]) * a[3] * (4 + 2 * sc)
            if name == "pt_quant_rowwise_colwise_rows":
                return (min(rows(a[2]), routed_rows) * 2 + rows(a[2]) * (2 + 2 * sc)) * a[3] + 4 * rows(a[2])
            if name in ("pt_silu_mul_quant_rowwise_colwise", "pt_clamped_swiglu_quant_rowwise_colwise"):
                return rows(a[1]) * a[2] * (4 + 2 + 2 * sc)
            if name in ("pt_silu_mul_bwd_quant_rowwise_colwise", "pt_clamped_swiglu_bwd_quant_rowwise_colwise"):
                return rows(a[4]) * a[5] * (2 + 4 + 2 * (2 + 2 * sc))
            if name == "pt_quant_blockwise_transpose_batched":
                return a[2] * a[3] * a[4] * (3 + (1 if a[9] else 0))
            if name == "pt_quant_blockwise_transpose_batched_into":
                return a[2] * a[3] * a[4] * (3 + (1 if a[11] else 0))
            if name in ("pt_quant_rowwise_transpose", "pt_quant_rowwise_transpose_ld"):
                return a[2] * a[3] * (4 + 2 * sc)
            if name in ("pt_quant_rowwise_blockwise_transpose", "pt_quant_rowwise_blockwise_transpose_ld"):
                return a[2] * a[3] * (4 + sc)
            return None

        agg = {}
        for name, a, b, args in self.other:
            d = agg.setdefault(name, [0.0, 0, 0.0])
            d[0] += a.elapsed_time(b) * 1e3
            d[1] += 1
            nb = nbytes(name, args)
            d[2] += nb if nb else 0.0
        out = []
        for name, (us, n, nb) in sorted(agg.items(), key=lambda kv: -kv[1][0]):
            row = {"entry_point": name, "calls_per_step": n / max(steps, 1), "us_per_call": round(us / n, 1),
                   "us_per_step": round(us / max(steps, 1), 1)}
            if nb:
                gbs = nb / us / 1e3
                row.update({"algorithmic_MB_per_call": round(nb / n / 1e6, 1), "GB/s": round(gbs, 0),
                            "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 3)})
            out.append(row)
        return out

    def summary(self):
        out = {}
        for name, a, b, _ in self.records:
            d = out.setdefault(name, [0.0, 0])
            d[0] += a.elapsed_time(b)
            d[1] += 1
        return {k: {"ms_total": v[0], "launches": v[1]} for k, v in out.items()}

    def by_shape(self, steps, groups, routed_rows):
        """Per (entry point, M x N x K) of a step: average duration of one launch, and the time the
        same launch needs at the MFMA peak (algorithmic FLOPs, padding rows not counted) and at the
        HBM peak (algorithmic bytes: both FP8 operands and their scales read once, the result
        written once)."""
        out = {}
        for name, a, b, shape in self.records:
            d = out.setdefault((name, shape), [0.0, 0])
            d[0] += a.elapsed_time(b)
            d[1] += 1
        rep = {}
        for (name, shape), (ms, n) in out.items():
            m, nn, k = (int(v) for v in shape.split("x"))
            if name.startswith("pt_gemm_nt_dense"):  # (the split form's slab traffic is not algorithmic)
                flop = 2.0 * m * nn * k
                byts = m * k * (1 + 4 / 128) + nn * k * (1 + 4 / 16384) + 2.0 * m * nn
            else:
                real = min(m, routed_rows)  # rows that carry tokens (the rest is per-group padding)
                flop = 2.0 * real * nn * k
                # (m may be the buffers' capacity rather than the padded row count, which then only
                # the device knows: the floor counts the rows that carry tokens)
                if name.startswith("pt_gemm_k_grouped_wgrad"):  # dW[g] = dY_g^T X_g: both twins read, [G,N,K] written
                    byts = real * (nn + k) * (1 + 4 / 128) + 2.0 * groups * nn * k
                else:
                    byts = real * k * (1 + 4 / 128) + groups * nn * k * (1 + 4 / 16384) + 2.0 * real * nn
            us = ms / n * 1e3
            rep[f"{name.replace('pt_gemm_', '')} {shape}"] = {
                "us": round(us, 1), "launches_per_step": n / max(steps, 1),
                "mfma_floor_us": round(flop / (FP8_DENSE_PEAK_TFLOPS * 1e12) * 1e6, 1),
                "hbm_floor_us": round(byts / (HBM_PEAK_GBS * 1e9) * 1e6, 1),
            }
        return rep


def hbm_kernel_report(H, I, E, rows, eidx, top_k=8, kind="fused", extras=None):
    """HIP-event timings of the HBM-bound kernels of the path at this workload's shapes, called
    through the operator layer one at a time: achieved GB/s = algorithmic bytes (2 B per bf16,
    1 B per fp8 element, 4 B per 128-element scale) / time, against the 8 TB/s HBM peak."""
    import torch

    from pith_train_amd.operators import deepgemm_quantize as Q
    from pith_train_amd.operators import fused_experts as FE
    from pith_train_amd.operators import token_scatter as TS
    from pith_train_amd.operators.silu_mul import silu_mul_halves

    def timeit(fn, iters=10):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(iters):
            fn()
        b.record()
        torch.cuda.synchronize()
        us = a.elapsed_time(b) / iters * 1e3
        if us >= 30.0:
            return us
        # A call this short is bound by the host's launch path when timed in a Python loop: record
        # 25 calls into a HIP graph and time replays, i.e. 100 back-to-back launches on the device.
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                fn()
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(25):
                    fn()
            graph.replay()
            torch.cuda.synchronize()
            a.record()
            for _ in range(4):
                graph.replay()
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) / 100 * 1e3
        except Exception:  # a call that cannot be captured keeps its host-loop time
            torch.cuda.synchronize()
            return us

    out = []

    def rep(name, us, nbytes):
        gbs = nbytes / us / 1e3
        out.append({"kernel": name, "us": round(us, 1), "algorithmic_MB": round(nbytes / 1e6, 1),
                    "GB/s": round(gbs, 0), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 3)})

    g = torch.Generator(device="cuda").manual_seed(0)
    # What this part's memory system gives a kernel that does nothing else: a device-to-device
    # copy and a fill of 512 MiB (2 x the memory-side cache), by the framework's own kernels.
    # The fractions of the kernels below are to be read against these, not against 1.0.
    ref_a = torch.randn((256 << 20,), device="cuda", generator=g).bfloat16()
    ref_b = torch.empty_like(ref_a)
    nb = ref_a.numel() * 2
    rep("reference: device-to-device copy (torch copy_), 512 MiB read + 512 MiB written", timeit(lambda: ref_b.copy_(ref_a)), 2 * nb)
    rep("reference: fill (torch zero_), 512 MiB written", timeit(lambda: ref_b.zero_()), nb)
    del ref_a, ref_b
    src = torch.randn((rows, H), device="cuda", generator=g).bfloat16()
    xp, reverse, offs, ks, ks_tensor = TS.scatter_for_grouped_gemm(src, eidx, E)
    Mp = xp.shape[0]
    _, _, _, _, src_of = TS.group_rows_with_sizes(eidx, E)
    sc = 4.0 / 128
    rep("quant_tile_kernel rowwise+colwise [Mp,H]", timeit(lambda: Q.fp8cast_rowwise_colwise_t(xp)), Mp * H * (4 + 2 * sc))
    rep("quant_tile_kernel rowwise+colwise of gathered rows [Mp,H]",
        timeit(lambda: Q.fp8cast_rowwise_colwise_t_rows(src, src_of)), (rows * 2 + Mp * (2 + 2 * sc)) * H + 4 * Mp)
    w = (torch.randn((E, 2 * I, H), device="cuda", generator=g) * 0.02).bfloat16()
    rep("quant_tile_kernel 128x128 blockwise, no transposed twin (the step's weight quantiser) [E,2I,H]",
        timeit(lambda: Q.fp8cast_blockwise_batched(w)), w.numel() * 3.0)
    rep("quant_tile_kernel 128x128 blockwise + transpose (PITHTRAIN_FP8_WEIGHT_TWIN=1) [E,2I,H]",
        timeit(lambda: Q.fp8cast_blockwise_transpose_batched(w)), w.numel() * 4.0)
    del w
    gu = torch.randn((Mp, 2 * I), device="cuda", generator=g).bfloat16()
    dh = torch.randn((Mp, I), device="cuda", generator=g).bfloat16()
    rep("quant_tile_kernel SwiGLU fwd + quant [Mp,I]", timeit(lambda: FE.silu_mul_quant(gu)), Mp * I * (4 + 2 + 2 * sc))
    rep("quant_tile_kernel SwiGLU bwd + quant [Mp,2I]", timeit(lambda: FE.silu_mul_bwd_quant(dh, gu)),
        Mp * I * (2 + 4 + 2 * (2 + 2 * sc)))
    gur = gu.clone().requires_grad_(True)
    rep("silu_mul_2d_kernel fwd [Mp,I]", timeit(lambda: silu_mul_halves(gur)), Mp * I * 6)
    o = silu_mul_halves(gur)
    rep("silu_mul_2d_kernel bwd [Mp,I]", timeit(lambda: torch.autograd.grad(o, gur, dh, retain_graph=True)), Mp * I * 10)
    del gu, dh, gur, o
    pbuf = torch.empty((src_of.shape[0], H), device="cuda", dtype=torch.bfloat16)
    rep("permute_rows_kernel alone (row copy of the scatter, indices given) [rows,H]",
        timeit(lambda: TS.permute_rows(src, src_of, pbuf, offs[E - 1:])), (rows + Mp) * H * 2 + 4 * src_of.shape[0])
    del pbuf
    rep("group_rows + permute_rows_kernel + host copy of the group sizes (scatter_for_grouped_gemm) [rows,H]",
        timeit(lambda: TS.scatter_for_grouped_gemm(src, eidx, E)), (rows + Mp) * H * 2 + 16 * rows)
    rep("gather_rows_kernel (padded_index_gather) [rows,H]", timeit(lambda: TS.padded_index_gather(xp, reverse)),
        2 * rows * H * 2 + 8 * rows)
    rep("gb_* kernels (padded_index_gather backward) [rows,H]",
        timeit(lambda: TS._PaddedIndexGather.scatter_sum(src, reverse, Mp, 1024)), (rows + Mp) * H * 2 + 12 * rows)
    # the step after the path: top-k weighted combine with the residual (forward_stage5, single rank)
    from pith_train_amd.operators.moe_combine import moe_combine

    T = rows // top_k
    tw = torch.softmax(torch.randn((T, top_k), device="cuda", generator=g), -1)
    res = torch.randn((T, H), device="cuda", generator=g).bfloat16()
    srcg = src.clone().requires_grad_(True)
    twg = tw.clone().requires_grad_(True)
    rep("moe_combine_fwd_kernel [T,k,H]", timeit(lambda: moe_combine(srcg, twg, res)), (rows + 2 * T) * H * 2 + 4 * rows)
    o = moe_combine(srcg, twg, res)
    rep("moe_combine_bwd_kernel [T,k,H]", timeit(lambda: torch.autograd.grad(o, [srcg, twg], res, retain_graph=True)),
        (2 * rows + T) * H * 2 + 8 * rows)
    # the expert-parallel branch of the same step: rows arrive in the dispatch sort's order
    from pith_train_amd.operators.moe_combine import moe_combine_ep

    local_idxs = torch.argsort(eidx, stable=True)
    rep("moe_combine_ep_fwd_kernel (+ slot index) [T,k,H]", timeit(lambda: moe_combine_ep(srcg, local_idxs, twg, res)),
        (rows + 2 * T) * H * 2 + 20 * rows)
    o = moe_combine_ep(srcg, local_idxs, twg, res)
    rep("moe_combine_bwd_kernel, rows through the slot index [T,k,H]",
        timeit(lambda: torch.autograd.grad(o, [srcg, twg], res, retain_graph=True)), (2 * rows + T) * H * 2 + 12 * rows)
    del srcg, twg, o, res, tw, local_idxs
    # the step before the path: softmax / top-k / weights of the router gate (after its logits GEMM)
    from pith_train_amd.operators.router_topk import softmax_topk, topk_softmax

    lg = (torch.randn((T, E), device="cuda", generator=g) * 2).bfloat16().requires_grad_(True)
    route = (lambda: topk_softmax(lg, top_k)) if kind == "gpt_oss" else (lambda: softmax_topk(lg, top_k, norm_topk_prob=True))
    rep("router_topk_fwd_kernel [T,E] -> [T,k]", timeit(route), T * E * 2 + T * top_k * 12)
    o = route()[1]
    rep("router_topk_bwd_kernel [T,k] -> [T,E]", timeit(lambda: torch.autograd.grad(o, lg, o.detach(), retain_graph=True)),
        2 * T * E * 2 + T * top_k * 12)
    del lg, o
    # the loss head: in-place fused cross-entropy over a 151 936-entry vocabulary (Qwen3), 4096 rows
    from pith_train_amd import _lib
    from pith_train_amd.operators.cross_entropy import cross_entropy

    Nce, Vce = 4096, 151936
    logits = (torch.randn((Nce, Vce), device="cuda", generator=g) * 2).bfloat16()
    tgt = torch.randint(0, Vce, (Nce,), device="cuda", generator=g)
    rep("ce_fwd_onchip_kernel (cross_entropy forward, in place) [N,V]", timeit(lambda: cross_entropy(logits, tgt)),
        2 * Nce * Vce * 2)
    half = torch.full((1,), 0.5, device="cuda")
    rep("ce_scale_kernel (cross_entropy backward, in place) [N,V]",
        timeit(lambda: _lib.call("pt_cross_entropy_bwd", logits.data_ptr(), Vce, _lib.dtype_code(logits.dtype), Nce, Vce,
                                 half.data_ptr(), _lib.stream_ptr(logits.device))), 2 * Nce * Vce * 2)
    del logits, tgt
    extras = extras or {}
    if kind == "gpt_oss":
        # the epilogues of the GPT-OSS experts: interleaved gate/up with biases and the clamped SwiGLU
        from pith_train_amd.operators.clamped_swiglu import clamped_swiglu
        from pith_train_amd.operators.indexed_bias_add import indexed_bias_add
        from pith_train_amd.operators.token_scatter import group_indices

        gu = torch.randn((Mp, 2 * I), device="cuda", generator=g).bfloat16().requires_grad_(True)
        bias = (torch.randn((E, 2 * I), device="cuda", generator=g) * 0.02).bfloat16().requires_grad_(True)
        gids = group_indices(offs, Mp, torch.int64)
        rep("bias_add_kernel (indexed_bias_add fwd) [Mp,2I]", timeit(lambda: indexed_bias_add(gu, bias, gids, offs)),
            Mp * 2 * I * 4 + E * 2 * I * 2)
        ob = indexed_bias_add(gu, bias, gids, offs)
        dgu = torch.randn((Mp, 2 * I), device="cuda", generator=g).bfloat16()
        rep("segment_sum_kernel (indexed_bias_add bwd: bias gradient) [Mp,2I]",
            timeit(lambda: torch.autograd.grad(ob, bias, dgu, retain_graph=True)), Mp * 2 * I * 2 + E * 2 * I * 4)
        del ob
        rep("clamped_swiglu_fwd_kernel [Mp,I]", timeit(lambda: clamped_swiglu(gu, 1.702, 7.0)), Mp * I * 6)
        oc = clamped_swiglu(gu, 1.702, 7.0)
        dhh = torch.randn((Mp, I), device="cuda", generator=g).bfloat16()
        rep("clamped_swiglu_bwd_kernel [Mp,I]", timeit(lambda: torch.autograd.grad(oc, gu, dhh, retain_graph=True)), Mp * I * 10)
        gq = gu.detach()
        rep("quant_tile_kernel clamped SwiGLU fwd + quant (the step's kernel) [Mp,I]",
            timeit(lambda: FE.clamped_swiglu_quant(gq, 1.702, 7.0)), Mp * I * (4 + 2 + 2 * sc))
        rep("quant_tile_kernel clamped SwiGLU bwd + quant + column sums (the step's kernel) [Mp,2I]",
            timeit(lambda: FE.clamped_swiglu_bwd_quant(dhh, gq, 1.702, 7.0)), Mp * I * (2 + 4 + 2 * (2 + 2 * sc)) + Mp // 128 * 2 * I * 4)
        del gu, bias, oc, dhh, dgu, gq
    if extras.get("dense_linears") or extras.get("shared_mlp"):
        # quantisation kernels of the dense FP8 linears (activation / gradient / weight flavours)
        T = rows // top_k
        fin, fout = extras["dense_linears"][0] if extras.get("dense_linears") else (H, extras["shared_mlp"])
        xa = torch.randn((T, fin), device="cuda", generator=g).bfloat16()
        ga = torch.randn((T, fout), device="cuda", generator=g).bfloat16()
        wa = (torch.randn((fout, fin), device="cuda", generator=g) * 0.02).bfloat16()
        rep(f"quant_tile_kernel rowwise + 128x128 blockwise transpose (dense activations) [{T},{fin}]",
            timeit(lambda: Q.fp8cast_rowwise_blockwise_transpose(xa)), T * fin * (4 + sc))
        rep(f"quant_tile_kernel rowwise + rowwise of the transpose (dense gradients) [{T},{fout}]",
            timeit(lambda: Q.fp8cast_rowwise_transpose(ga)), T * fout * (4 + 2 * sc))
        rep(f"quant_tile_kernel 128x128 blockwise + transpose (dense weight) [{fout},{fin}]",
            timeit(lambda: Q.fp8cast_blockwise_transpose(wa)), fout * fin * 4.0)
    if "dedup_fraction" in extras:
        # index construction of the dedup dispatch (integer only; bound by launch latency)
        from pith_train_amd.operators import ep_dispatch as EP

        T = rows // top_k
        topk = make_routing(T, E, top_k, seed=5).cuda()
        us = timeit(lambda: EP.fused_dedup_prepare_dispatch(topk, E, 8, E // 8))
        out.append({"kernel": f"dd_* kernels (fused_dedup_prepare_dispatch, ep_size 8) [{T},{top_k}]", "us": round(us, 1),
                    "algorithmic_MB": round(T * top_k * 8 * 4 / 1e6, 2), "note": "latency-bound chain of small integer kernels"})
    return out


def cpu_baseline(kind, H, I, E, k, T, zipf, budget_s=12.0):
    """The CPU oracle of the same layer on the same seeded inputs, forward + backward, on the
    threads torch takes by itself on this host (reported as ``cores``).  Two legs: the BF16
    grouped-linear semantics (the reference's pure-PyTorch path) on the whole workload, repeated
    until about ``budget_s`` seconds have been spent - the headline CPU figure -, and the FP8 leg
    (quantise -> dequantise -> fp32 matmul per group) on the rows of a few experts."""
    import torch

    from oracle import moe as OM

    cores = torch.get_num_threads()
    ids, x, dy, w = make_inputs(kind, H, I, E, k, T, zipf, seed=0)
    tokens = x.unsqueeze(1).expand(-1, k, -1).reshape(-1, H).contiguous()
    eidx = ids.reshape(-1)
    flops = OM.gemm_flops(T * k, H, I)
    OM.moe_layer_fwd_bwd(tokens[:512], eidx[:512], w, dy[:512], E, kind=kind, fp8=False)  # warm
    t0 = time.perf_counter()
    reps = 0
    while True:
        OM.moe_layer_fwd_bwd(tokens, eidx, w, dy, E, kind=kind, fp8=False)
        reps += 1
        el = time.perf_counter() - t0
        if el > budget_s or reps >= 20:
            break
    sec = el / reps
    # FP8 leg on the experts 0 .. n-1 only (their rows, their weights): the oracle's quantisers and
    # dequantised products are elementwise tensor code, an order of magnitude slower per FLOP
    n = max(1, E // 16)
    sel = (eidx < n).nonzero().flatten()
    sub_w = {name: v[:n] for name, v in w.items()}
    t1 = time.perf_counter()
    OM.moe_layer_fwd_bwd(tokens[sel], eidx[sel], sub_w, dy[sel], n, kind=kind, fp8=True, accum=torch.float32)
    sec8 = time.perf_counter() - t1
    return {
        "value": flops / sec / 1e12,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"full workload ({T * k} routed rows, {E} experts), bf16 grouped-linear oracle fwd+bwd on the host, "
                  f"{reps} rep(s), {sec:.2f} s each",
        "fp8_leg": {"value": OM.gemm_flops(int(sel.numel()), H, I) / sec8 / 1e12, "unit": "TFLOP/s", "cores": cores,
                    "sample": f"quantise -> dequantise -> fp32 matmul oracle on the {int(sel.numel())} rows of experts 0..{n - 1}, "
                              f"one pass of {sec8:.2f} s"},
    }


def gemm_shapes_report(H, I, E, k, T, zipf, data="normal", iters=20):
    """The six grouped GEMM launches of a SwiGLU expert layer's fwd + bwd, each timed alone with
    HIP events on operands that are already quantised: FP8 bytes of N(0,1) values under random
    power-of-two scales (``data="zeros"``: all-zero operands, which leave the clock at its
    maximum - the data decides the power the matrix pipes draw).  What a measurement build of the
    library (csrc/Makefile: EXTRA=-DPT_GEMM_ABLATE_...) is timed with."""
    import torch

    from pith_train_amd.operators.grouped_linear import k_grouped_fp8_wgrad, m_grouped_fp8_gemm_nn, m_grouped_fp8_gemm_nt

    ids = make_routing(T, E, k, seed=0, zipf_s=zipf).reshape(-1)
    cnt = torch.bincount(ids, minlength=E)
    ks = ((cnt + 127) // 128 * 128).to(torch.int32)
    offs = ks.cumsum(0).to(torch.int32).cuda()
    M, real = int(ks.sum()), int(cnt.sum())
    g = torch.Generator(device="cuda").manual_seed(0)

    def fp8(*shape):
        if data == "zeros":
            return torch.zeros(shape, dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn)
        return (torch.randn(shape, device="cuda", generator=g) * 100).to(torch.float8_e4m3fn)

    def sc(*shape):
        return torch.exp2(torch.randint(-8, 2, shape, device="cuda", generator=g).float())

    def timeit(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(iters):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / iters * 1e3

    out = []

    def m_grouped(name, N, K, nn):
        a = (fp8(M, K), sc(M, K // 128))
        b = (fp8(E, K, N), sc(E, K // 128, N // 128)) if nn else (fp8(E, N, K), sc(E, N // 128, K // 128))
        o = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
        fn = m_grouped_fp8_gemm_nn if nn else m_grouped_fp8_gemm_nt
        us = timeit(lambda: fn(a, b, o, offs))
        out.append({"launch": name, "shape": f"{M}x{N}x{K}", "us": round(us, 1), "TFLOP/s": round(2.0 * real * N * K / us / 1e6, 0)})

    def k_grouped(name, N, K):
        a = (fp8(N, M), sc(M // 128, N))
        b = (fp8(K, M), sc(M // 128, K))
        o = torch.empty((E, N, K), dtype=torch.bfloat16, device="cuda")
        us = timeit(lambda: k_grouped_fp8_wgrad(a, b, o, offs, False))
        out.append({"launch": name, "shape": f"{E}x{N}x{K} over {M} rows", "us": round(us, 1),
                    "TFLOP/s": round(2.0 * real * N * K / us / 1e6, 0)})

    m_grouped("forward gate_up (m-grouped NT)", 2 * I, H, False)
    m_grouped("forward down (m-grouped NT)", H, I, False)
    m_grouped("input gradient of down (m-grouped NN)", I, H, True)
    m_grouped("input gradient of gate_up (m-grouped NN)", H, 2 * I, True)
    k_grouped("weight gradient of down (k-grouped)", H, I)
    k_grouped("weight gradient of gate_up (k-grouped)", 2 * I, H)
    return {"data": data, "rows": real, "padded_rows": M, "launches": out, "total_us": round(sum(r["us"] for r in out), 1)}


def dense_reference_report(iters=20):
    """The vendor library's FP8 GEMM (``torch._scaled_mm``: one scale per tensor) and this library's
    dense entry point (1 x 128 and 128 x 128 scales) on the same random FP8 operands, three shapes."""
    import torch

    from pith_train_amd.operators.linear import _fp8_gemm_nt

    g = torch.Generator(device="cuda").manual_seed(0)
    out = []
    for M, N, K in ((8192, 4096, 4096), (32768, 4096, 2048), (65536, 1536, 2048)):
        a = (torch.randn((M, K), device="cuda", generator=g) * 100).to(torch.float8_e4m3fn)
        b = (torch.randn((N, K), device="cuda", generator=g) * 100).to(torch.float8_e4m3fn)
        sa = torch.exp2(torch.randint(-8, 2, (M, K // 128), device="cuda", generator=g).float())
        sb = torch.exp2(torch.randint(-8, 2, (N // 128, K // 128), device="cuda", generator=g).float())
        one = torch.ones((), device="cuda")

        def timeit(fn):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            x, y = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            x.record()
            for _ in range(iters):
                fn()
            y.record()
            torch.cuda.synchronize()
            return x.elapsed_time(y) / iters * 1e3

        row = {"shape": f"{M}x{N}x{K}"}
        try:
            us = timeit(lambda: torch._scaled_mm(a, b.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16))
            row["torch._scaled_mm us"] = round(us, 1)
            row["torch._scaled_mm TFLOP/s"] = round(2.0 * M * N * K / us / 1e6, 0)
        except Exception as exc:  # a build of the framework without the FP8 GEMM
            row["torch._scaled_mm"] = f"not available: {exc}"
        us = timeit(lambda: _fp8_gemm_nt(a, sa, b, sb, M, N, "cuda", torch.bfloat16))
        row["this library us"] = round(us, 1)
        row["this library TFLOP/s"] = round(2.0 * M * N * K / us / 1e6, 0)
        out.append(row)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="qwen3-30b-a3b-moe", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-cached-weights", action="store_true",
                    help="skip the extra (untimed-for-value) pass that keeps the FP8 weight cache across steps")
    ap.add_argument("--no-kernel-report", action="store_true",
                    help="skip the per-kernel GB/s table of the HBM-bound kernels (hbm_kernels in the JSON line)")
    ap.add_argument("--kernel-report-only", action="store_true",
                    help="run only the per-kernel table (what a `rocprofv3 --kernel-trace` of the HBM-bound "
                         "kernels traces) and print it as the JSON line")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="after the timed region launch gather_rows_kernel as a plain copy of 256 MiB "
                         "(identity index) three times: the known-size kernel that FETCH_SIZE / "
                         "WRITE_SIZE readings of a `rocprofv3 --pmc` run are scaled by")
    ap.add_argument("--gemm-shapes", action="store_true",
                    help="time only the six grouped GEMM launches of the workload's expert layer, each alone, on "
                         "pre-quantised synthetic operands (see gemm_shapes_report) and print the table as the JSON line")
    ap.add_argument("--gemm-data", default="normal", choices=("normal", "zeros"),
                    help="operand bytes of --gemm-shapes: FP8 of N(0,1) values, or zeros (full clock)")
    ap.add_argument("--dense-reference", action="store_true",
                    help="time torch._scaled_mm (the vendor library's FP8 GEMM) and this library's dense GEMM on "
                         "three shapes and print the table as the JSON line")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU's share of the expert path; run with --gpus 1 "
              "(no collectives or multi-GPU sharding are part of it).", file=sys.stderr)
        sys.exit(2)

    import torch

    from pith_train_amd import _lib
    from pith_train_amd.dualpipe_utils import FP8WeightCacheControl
    from pith_train_amd.modules.experts import forward_stage3

    _lib.load()  # fail loudly if the HIP library is missing
    kind, H, I, E, k, T, zipf = WORKLOADS[args.workload]
    extras = EXTRAS.get(args.workload, {})
    if args.gemm_shapes:
        print(json.dumps({"workload": args.workload, "library": _lib.LIB_PATH, "gemm_shapes": gemm_shapes_report(H, I, E, k, T, zipf, args.gemm_data)}))
        return
    if args.dense_reference:
        print(json.dumps({"dense_reference": dense_reference_report()}))
        return
    ids, x, dy, w = make_inputs(kind, H, I, E, k, T, zipf)
    mod = build_module(kind, H, I, E, w)
    params = [p for p in mod.parameters()]
    eidx = ids.reshape(-1).cuda()
    dyc = dy.cuda()
    rows = T * k
    expand_idx = None
    if "dedup_fraction" in extras:
        # the experts receive only the unique rows and re-expand them through expand_idx
        expand_cpu, U = make_dedup_expand(rows, extras["dedup_fraction"])
        g = torch.Generator().manual_seed(2)
        tokens = torch.randn((U, H), generator=g).bfloat16().cuda()
        expand_idx = expand_cpu.cuda()
    else:
        tokens = x.cuda().unsqueeze(1).expand(-1, k, -1).reshape(-1, H).contiguous()
    if args.kernel_report_only:
        print(json.dumps({"workload": args.workload, "hbm_kernels": hbm_kernel_report(H, I, E, rows, eidx, k, kind, extras)}))
        return
    flops = gemm_flops(rows, H, I) + extra_flops(extras, T, H)
    dense = []  # (module, input [T, in], upstream grad [T, out])
    if extras.get("shared_mlp") or extras.get("dense_linears"):
        from pith_train_amd.modules import training
        from pith_train_amd.modules.experts import DeepSeekV2MLP

        g = torch.Generator().manual_seed(3)
        mk = lambda *s_: torch.randn(s_, generator=g).bfloat16().cuda()  # noqa: E731
        if extras.get("shared_mlp"):
            m = DeepSeekV2MLP(H, extras["shared_mlp"]).cuda().to(torch.bfloat16)
            dense.append((m, mk(T, H), mk(T, H)))
        for fin, fout in extras.get("dense_linears", []):
            m = training.Linear(fin, fout, bias=False).cuda().to(torch.bfloat16)
            dense.append((m, mk(T, fin), mk(T, fout)))
        with torch.no_grad():
            for m, _, _ in dense:
                for p_ in m.parameters():
                    p_.copy_((torch.randn(p_.shape, generator=g) * 0.02).to(p_.dtype))
    timer = GemmTimer().install()

    def step(bump=True):
        if bump:
            FP8WeightCacheControl.step()  # re-quantise the weights: nothing carried across steps
        for p in params:
            p.grad = None
        tok = tokens.detach().requires_grad_(True)
        out = forward_stage3(mod, tok, eidx, E, expand_idx=expand_idx)
        # weight gradients are written to .grad by the wgrad GEMM itself; the token gradient is
        # taken directly (a leaf's .grad would cost a clone that no training step performs)
        (dtok,) = torch.autograd.grad(out, tok, dyc)
        for m, xin, gout in dense:
            xi = xin.detach().requires_grad_(True)
            torch.autograd.grad(m(xi), [xi] + list(m.parameters()), gout)
        return dtok

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer.enabled = True
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    timer.enabled = False
    ms = elapsed / args.steps * 1e3

    gs = timer.summary()
    gemm_ms = sum(v["ms_total"] for v in gs.values())
    gemm_launches = sum(v["launches"] for v in gs.values())
    achieved = flops * args.steps / (gemm_ms * 1e-3) / 1e12 if gemm_ms > 0 else 0.0
    per_shape = timer.by_shape(args.steps, E, rows)
    floor_ms = sum(max(v["mfma_floor_us"], v["hbm_floor_us"]) * v["launches_per_step"] for v in per_shape.values()) / 1e3

    extra = {}
    if not args.no_cached_weights:
        # secondary figure: the reference quantises weights once per optimizer step and reuses them
        # for every micro-batch; `value` above re-quantises them in every step
        for _ in range(2):
            step(bump=False)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(args.steps):
            step(bump=False)
        torch.cuda.synchronize()
        ms_c = (time.perf_counter() - t1) / args.steps * 1e3
        extra["weights_cached"] = {"ms_per_step": ms_c, "value": flops / (ms_c * 1e-3) / 1e12, "unit": "TFLOP/s",
                                   "note": "FP8 weight cache kept across steps (one quantisation per optimizer step, "
                                           "as FP8WeightCacheControl does); not the headline value"}

    padded_rows = int((-(-torch.bincount(eidx.cpu(), minlength=E) // 128) * 128).sum())
    if not args.no_kernel_report:
        # the HBM-bound kernels where they run: a few more steps with events around every entry point
        timer.install_all()
        step()
        torch.cuda.synchronize()
        timer.all_enabled = True
        n_extra = min(args.steps, 10)
        for _ in range(n_extra):
            step()
        torch.cuda.synchronize()
        timer.all_enabled = False
        extra["hbm_kernels_in_step"] = timer.in_step_report(n_extra, padded_rows, rows)

    if args.calibrate_copy:
        cr, ch = 65536, 2048  # 65536 rows x 2048 bf16 = 256 MiB read + 256 MiB written (+ 512 KiB of indices)
        csrc = torch.randn((cr, ch), device="cuda").bfloat16()
        cdst = torch.empty_like(csrc)
        cidx = torch.arange(cr, device="cuda", dtype=torch.int64)
        for _ in range(3):
            _lib.call("pt_gather_rows", csrc.data_ptr(), ch, cdst.data_ptr(), ch, cidx.data_ptr(), cr, ch, 2,
                      _lib.stream_ptr())
        torch.cuda.synchronize()
        assert torch.equal(csrc, cdst)

    result = {
        "metric": "MoE-layer fwd+bwd TFLOP/s (FP8 grouped-expert path, Qwen3-30B-A3B shape, 1 GPU)"
        if args.workload == "qwen3-30b-a3b-moe" else f"MoE-layer fwd+bwd TFLOP/s ({args.workload})",
        "value": flops / (ms * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3 (fp32 accumulate, bf16 in/out)",
        "data": "synthetic (seed 0: x~N(0,1) bf16, weights~N(0,0.02), grad~N(0,1), router logits~N(0,1) softmax top-k)",
        "config": {
            "workload": args.workload, "kind": kind, "hidden": H, "moe_intermediate": I, "experts": E,
            "top_k": k, "tokens": T, "routed_rows": rows,
            # rows of the grouped tensors: every expert's rows padded to a multiple of 128
            "padded_rows": padded_rows,
            "zipf_s": zipf,
            **({"zipf_bias": "b_e = scale * (log p_e - mean(log p)), p_e ~ rank_e^-s, ranks from a seeded permutation; "
                             "scale raised in steps of 0.25 until an expert is empty and one exceeds 4x the mean",
                "zipf_bias_scale": ZIPF_BIAS_SCALE.get(zipf)} if zipf is not None else {}),
            **extras,
            "algorithmic_gemm_tflop_per_step": flops / 1e12,
            "weight_quant_in_step": True,
        },
        "roofline": {
            "bound": "mfma",
            "kernel": "fp8_gemm_nt_rowsplit_kernel (grouped launches) / fp8_gemm_nt_pipelined_kernel (dense launches): every GEMM launch of the step, fwd, dgrad, wgrad; the library picks the main loop per mode and shape",
            "achieved": achieved,
            "peak": FP8_DENSE_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / FP8_DENSE_PEAK_TFLOPS,
            "traffic": GEMM_TRAFFIC_BYTES_PER_LAUNCH.get(args.workload),
            "algorithmic_flop_per_launch": flops / max(gemm_launches / max(args.steps, 1), 1),
            "avg_launch_ms": gemm_ms / max(gemm_launches, 1),
            "launches_per_step": gemm_launches / max(args.steps, 1),
            "gemm_ms_per_step": gemm_ms / max(args.steps, 1),
            "per_entry_point_ms_per_step": {k2: v["ms_total"] / args.steps for k2, v in gs.items()},
            "per_shape": per_shape,
            # every launch priced at the better of the two peaks: what the step's GEMMs would take on
            # a machine that reaches 5 PFLOP/s and 8 TB/s at once
            "floor_ms_per_step": floor_ms,
            "frac_of_floor": floor_ms / (gemm_ms / max(args.steps, 1)) if gemm_ms > 0 else 0.0,
        },
        **extra,
    }
    if not args.no_kernel_report:
        result["hbm_kernels"] = hbm_kernel_report(H, I, E, rows, eidx, k, kind, extras)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(kind, H, I, E, k, T, zipf)
        if extras:
            result["cpu_baseline"]["sample"] += " (routed experts only; the dense parts of this workload are not in the CPU figure)"
    print(json.dumps(result))


if __name__ == "__main__":
    main()
