"""Expert blocks of the supported model families and the stage-3 composition around them.

Mirrors the expert path of the reference's model files:
  * ``Qwen3MoeExperts``      - models/qwen3_moe.py:45-65   (gate, up, down as three grouped linears)
  * ``DeepSeekV2Experts``    - models/deepseek_v2.py:111-129
  * ``DeepSeekV2MLP``        - models/deepseek_v2.py:94-108 (dense shared expert)
  * ``Qwen35MoeExperts``     - models/qwen35_moe.py:179-200 (fused gate_up, concatenated halves)
  * ``GptOssExperts``        - models/gpt_oss.py:95-157     (fused interleaved gate_up, biases,
                                                              clamped SwiGLU)
  * ``forward_stage3``       - models/qwen3_moe.py:216-227  (expand -> scatter -> experts -> gather)

The constructors take plain sizes instead of Hugging Face config objects; everything else
(parameter names, shapes, call signatures) follows the reference so that checkpoints and callers
line up.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from ..dualpipe_utils import FP8WeightCacheControl
from ..operators import fused_experts
from ..operators.clamped_swiglu import clamped_swiglu
from ..operators.deepgemm_quantize import fp8cast_grouped_weight, fp8cast_grouped_weight_cat, weight_twin_enabled
from ..operators.grouped_linear import FP8GroupedLinear, FP8GroupedLinearFunc, GroupedLinearFunc
from ..operators.indexed_bias_add import indexed_bias_add
from ..operators.silu_mul import silu_mul, silu_mul_halves
from ..operators.token_scatter import (
    group_indices,
    group_rows_with_sizes,
    padded_index_gather,
    precompute_group_indices,
    scatter_for_grouped_gemm,
)
from . import training


class Qwen3MoeExperts(nn.Module):
    def __init__(self, hidden_size: int, moe_intermediate_size: int, num_experts: int):
        super().__init__()
        self.gate_proj = training.GroupedLinear(num_experts, hidden_size, moe_intermediate_size)
        self.up_proj = training.GroupedLinear(num_experts, hidden_size, moe_intermediate_size)
        self.down_proj = training.GroupedLinear(num_experts, moe_intermediate_size, hidden_size)
        self._gu_cache = None  # gate and up quantised into one fused operand (FP8 path)
        self._gu_version = -1

    def _fused_gate_up_quant(self):
        """gate and up weights quantised into one fused ``[G, 2I, H]`` operand; cached like the
        layers' own quantised weights (one quantisation per ``FP8WeightCacheControl`` version)."""
        parts = [self.gate_proj.weight, self.up_proj.weight]
        if torch.compiler.is_compiling():
            return fp8cast_grouped_weight_cat(parts)
        ver = FP8WeightCacheControl.version
        if self._gu_cache is None or self._gu_version != ver or (self._gu_cache[2] is not None) != weight_twin_enabled():
            self._gu_cache = fp8cast_grouped_weight_cat(parts)
            self._gu_version = ver
        return self._gu_cache

    def forward(self, x, grouped_mm_offs, ks=None, ks_tensor=None, row_map=None, fuse_activation: bool = True,
                expand_idx=None):
        """``row_map`` (extension, FP8 layers only): the scatter's int32 source-row map.  ``x`` is
        then the un-permuted ``[m, H]`` token tensor and the result comes back un-permuted; the
        permutation happens inside the first quantisation and the last GEMM's store.
        ``expand_idx`` (one-node path only): ``x`` holds deduplicated rows, see
        :func:`fused_experts.compose_row_maps`.  With
        ``fuse_activation`` (FP8 layers, intermediate size a multiple of 128) the block runs as one
        autograd node on a fused gate_up operand: the tokens are quantised once instead of once
        per projection, one GEMM serves both, and the SwiGLU and its gradient are computed inside
        the kernels that quantise them (same bits as the three-operator composition)."""
        if (fuse_activation and training.fp8 and x.shape[0] > 0 and isinstance(self.gate_proj, FP8GroupedLinear)
                and isinstance(self.up_proj, FP8GroupedLinear) and isinstance(self.down_proj, FP8GroupedLinear)
                and fused_experts.supported_split(x, self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight)):
            return fused_experts.FP8SwiGLUSplitExpertsFunc.apply(
                x, self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight, grouped_mm_offs,
                self._fused_gate_up_quant(), self.down_proj._get_quantized_weight(), row_map, expand_idx,
            )  # fmt: skip
        assert expand_idx is None, "expand_idx needs the one-node FP8 path"
        gi = precompute_group_indices(grouped_mm_offs, x.shape[0])
        kwargs = dict(grouped_mm_offs=grouped_mm_offs, ks=ks, ks_tensor=ks_tensor, group_indices=gi)
        if row_map is not None:
            g = self.gate_proj(x, in_rows=row_map, **kwargs)
            u = self.up_proj(x, in_rows=row_map, **kwargs)
            return self.down_proj(silu_mul(g, u), out_rows=row_map, out_m=x.shape[0], **kwargs)
        g = self.gate_proj(x, **kwargs)
        u = self.up_proj(x, **kwargs)
        return self.down_proj(silu_mul(g, u), **kwargs)


class DeepSeekV2Experts(Qwen3MoeExperts):
    """Same composition as the Qwen3 experts (models/deepseek_v2.py:111-129)."""


class DeepSeekV2MLP(nn.Module):
    """Dense SwiGLU MLP (the shared experts run as one of these)."""

    def __init__(self, hidden_size: int, intermediate_size: int):
        super().__init__()
        self.gate_proj = training.Linear(hidden_size, intermediate_size, bias=False)
        self.up_proj = training.Linear(hidden_size, intermediate_size, bias=False)
        self.down_proj = training.Linear(intermediate_size, hidden_size, bias=False)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.down_proj(silu_mul(self.gate_proj(x), self.up_proj(x)))


class Qwen35MoeExperts(nn.Module):
    def __init__(self, hidden_size: int, moe_intermediate_size: int, num_experts: int):
        super().__init__()
        self.num_experts = num_experts
        self.hidden_size = hidden_size
        self.moe_intermediate_size = moe_intermediate_size
        self.gate_up_proj = training.GroupedLinear(num_experts, hidden_size, 2 * moe_intermediate_size)
        self.down_proj = training.GroupedLinear(num_experts, moe_intermediate_size, hidden_size)

    def forward(self, x, grouped_mm_offs, ks=None, ks_tensor=None, row_map=None, fuse_activation: bool = True,
                expand_idx=None):
        """``row_map`` / ``expand_idx``: see :meth:`Qwen3MoeExperts.forward`.  With ``fuse_activation`` (FP8 layers)
        the block runs as one autograd node whose SwiGLU output and SwiGLU gradient are computed
        inside the kernels that quantise them (same bits as the three-operator composition)."""
        if (fuse_activation and training.fp8 and x.shape[0] > 0 and isinstance(self.gate_up_proj, FP8GroupedLinear)
                and isinstance(self.down_proj, FP8GroupedLinear)
                and fused_experts.supported(x, self.gate_up_proj.weight, self.down_proj.weight)):
            return fused_experts.FP8SwiGLUExpertsFunc.apply(
                x, self.gate_up_proj.weight, self.down_proj.weight, grouped_mm_offs, ks, ks_tensor,
                self.gate_up_proj._get_quantized_weight(), self.down_proj._get_quantized_weight(), row_map, expand_idx,
            )  # fmt: skip
        assert expand_idx is None, "expand_idx needs the one-node FP8 path"
        gi = precompute_group_indices(grouped_mm_offs, x.shape[0])
        kwargs = dict(grouped_mm_offs=grouped_mm_offs, ks=ks, ks_tensor=ks_tensor, group_indices=gi)
        if row_map is not None:
            gate_up = self.gate_up_proj(x, in_rows=row_map, **kwargs)
            return self.down_proj(silu_mul_halves(gate_up), out_rows=row_map, out_m=x.shape[0], **kwargs)
        gate_up = self.gate_up_proj(x, **kwargs)
        # the halves are read in place (same arithmetic as silu_mul on contiguous copies)
        return self.down_proj(silu_mul_halves(gate_up), **kwargs)


class GptOssExperts(nn.Module):
    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int, swiglu_limit: float = 7.0):
        super().__init__()
        self.num_experts = num_experts
        self.swiglu_limit = float(swiglu_limit)
        self.gate_up_proj = nn.Parameter(torch.empty(num_experts, 2 * intermediate_size, hidden_size))
        self.gate_up_proj_bias = nn.Parameter(torch.zeros(num_experts, 2 * intermediate_size))
        self.down_proj = nn.Parameter(torch.empty(num_experts, hidden_size, intermediate_size))
        self.down_proj_bias = nn.Parameter(torch.zeros(num_experts, hidden_size))
        self._wq_cache: dict | None = None
        self._wq_version: int = -1
        # extension: the two indexed_bias_add steps happen in the stores of the GEMMs before them
        # (same bits) wherever the shapes and dtypes allow it
        self.fuse_bias = True
        # extension (needs fuse_bias): the whole block as one autograd node whose quantisation
        # kernels compute the clamped SwiGLU and its gradient instead of reading them from memory
        self.fuse_activation = True

    def _quantized_weight(self, name: str, weight: torch.Tensor):
        if torch.compiler.is_compiling():
            return fp8cast_grouped_weight(weight)
        ver = FP8WeightCacheControl.version
        cache = self._wq_cache
        if self._wq_version != ver or cache is None:
            cache = self._wq_cache = {}
            self._wq_version = ver
        if name not in cache or (cache[name][2] is not None) != weight_twin_enabled():
            cache[name] = fp8cast_grouped_weight(weight)
        return cache[name]

    def _group_linear(self, x, weight, name, offs, ks, ks_tensor, group_indices_, in_rows=None, bias=None,
                      out_rows=None, out_m=None):
        if x.shape[0] == 0:
            return x @ weight[0].transpose(-2, -1)
        if training.fp8:
            return FP8GroupedLinearFunc.apply(
                x, weight, offs, ks, ks_tensor, self._quantized_weight(name, weight), group_indices_, in_rows,
                out_rows, out_m, bias,
            )
        assert in_rows is None, "row maps need the FP8 layers"
        return GroupedLinearFunc.apply(x, weight, offs)

    def bias_fusable(self, x) -> bool:
        """Whether the two ``indexed_bias_add`` steps happen in the stores of the GEMMs."""
        return (self.fuse_bias and training.fp8 and x.shape[0] > 0 and x.dtype == torch.bfloat16
                and self.gate_up_proj_bias.dtype == x.dtype and self.down_proj_bias.dtype == x.dtype
                and self.gate_up_proj.shape[1] % 8 == 0 and self.down_proj.shape[1] % 8 == 0)

    def one_node(self, x) -> bool:
        """Whether the block runs as one autograd node (fused biases and activation).  That node
        takes every row count from ``grouped_mm_offs`` on the device, so its ``row_map`` may be
        sized for more rows than the routing produced."""
        return self.bias_fusable(x) and self.fuse_activation and self.down_proj.shape[2] % 8 == 0

    def forward(self, x, grouped_mm_offs, ks=None, ks_tensor=None, row_map=None, scatter_output: bool = False):
        """``row_map`` (extension, FP8 only): the scatter's int32 source-row map; ``x`` is then the
        un-permuted token tensor and the first quantisation gathers its rows.  The result stays
        in the grouped layout unless ``scatter_output`` is set (with ``row_map`` and the fused
        biases): then the last GEMM stores every row, bias added, at its un-permuted place, and
        the backward sums the bias gradient over the grouped order through the same map.
        With ``self.fuse_bias`` (FP8 only) the two ``indexed_bias_add`` steps happen in the stores
        of the GEMMs before them (same bits)."""
        M = x.shape[0] if row_map is None else row_map.shape[0]
        fused = self.bias_fusable(x)
        assert not scatter_output or (fused and row_map is not None), "scatter_output needs row_map and the fused biases"
        if M % 128 == 0 and self.one_node(x):
            return fused_experts.FP8ClampedSwiGLUExpertsFunc.apply(
                x, self.gate_up_proj, self.gate_up_proj_bias, self.down_proj, self.down_proj_bias, grouped_mm_offs,
                self._quantized_weight("gate_up_proj", self.gate_up_proj), self._quantized_weight("down_proj", self.down_proj),
                1.702, self.swiglu_limit, row_map, scatter_output,
            )
        if fused:
            gate_up = self._group_linear(x, self.gate_up_proj, "gate_up_proj", grouped_mm_offs, ks, ks_tensor, None, row_map,
                                         self.gate_up_proj_bias)
            activated = clamped_swiglu(gate_up, 1.702, self.swiglu_limit)
            return self._group_linear(activated, self.down_proj, "down_proj", grouped_mm_offs, ks, ks_tensor, None, None,
                                      self.down_proj_bias, row_map if scatter_output else None,
                                      x.shape[0] if scatter_output else None)
        group_ids = group_indices(grouped_mm_offs, M, torch.int64)
        gate_up = self._group_linear(x, self.gate_up_proj, "gate_up_proj", grouped_mm_offs, ks, ks_tensor, None, row_map)
        gate_up = indexed_bias_add(gate_up, self.gate_up_proj_bias, group_ids, grouped_mm_offs)
        activated = clamped_swiglu(gate_up, 1.702, self.swiglu_limit)
        out = self._group_linear(activated, self.down_proj, "down_proj", grouped_mm_offs, ks, ks_tensor, None)
        return indexed_bias_add(out, self.down_proj_bias, group_ids, grouped_mm_offs)


def forward_stage3(experts: nn.Module, gathered_tokens, expert_idxs, experts_per_rank: int, expand_idx=None,
                   fuse_expand: bool = True, fuse_permute: bool = True, host_sizes: bool = False):
    """Expert compute between the dispatch and combine all-to-alls.

    With ``fuse_permute`` (FP8 Qwen3 / DeepSeek / Qwen3.5 experts, no ``expand_idx``) the permuted
    copy of the tokens, its inverse gather and their two backward passes are never materialised:
    only the index half of the scatter runs, the first quantisation reads rows through the
    source map and the last GEMM of forward and of backward stores rows through it.  The result
    is bit-identical to the unfused composition.  Unless ``host_sizes`` is set, this path also
    drops the scatter's device-to-host copy of the group sizes (token_scatter.py:230-243 waits for
    the GPU there on every call): buffers are sized for the largest padded row count the routing
    could produce and every kernel reads the real count from ``grouped_mm_offs``.

    ``expand_idx`` (EP > 1) re-expands the deduplicated received rows to one row per routed
    (token, expert) pair.  With ``fuse_expand`` that gather is folded into the scatter's row copy
    (each unique row is read once per use and no expanded copy is materialised); without it the
    two steps run separately as in the reference.
    """
    if (fuse_permute and training.fp8 and expert_idxs.shape[0] > 0
            and isinstance(experts, (Qwen3MoeExperts, Qwen35MoeExperts))
            and isinstance(experts.down_proj, FP8GroupedLinear)
            and experts.down_proj.out_features % 8 == 0 and experts.down_proj.in_features % 8 == 0):
        if isinstance(experts, Qwen35MoeExperts):
            fused_node = fused_experts.supported(gathered_tokens, experts.gate_up_proj.weight, experts.down_proj.weight)
        else:
            fused_node = (isinstance(experts.gate_proj, FP8GroupedLinear) and isinstance(experts.up_proj, FP8GroupedLinear)
                          and fused_experts.supported_split(gathered_tokens, experts.gate_proj.weight,
                                                            experts.up_proj.weight, experts.down_proj.weight))
        if expand_idx is None or (fused_node and fuse_expand):
            _, grouped_mm_offs, ks, ks_tensor, src_of = group_rows_with_sizes(
                expert_idxs, experts_per_rank, device=gathered_tokens.device, host_sizes=host_sizes or not fused_node)
            if expand_idx is None:
                return experts(gathered_tokens, grouped_mm_offs, ks=ks, ks_tensor=ks_tensor, row_map=src_of)
            # deduplicated rows: the first quantisation reads them through expand_idx composed with
            # the scatter's map, so neither the expanded nor the permuted copy exists
            return experts(gathered_tokens, grouped_mm_offs, ks=ks, ks_tensor=ks_tensor, row_map=src_of,
                           expand_idx=expand_idx)
    if (fuse_permute and expand_idx is None and training.fp8 and expert_idxs.shape[0] > 0
            and isinstance(experts, GptOssExperts)):
        # the one-node block needs no host-side sizes (see the SwiGLU branch above)
        reverse_shuffle_idxs, grouped_mm_offs, ks, ks_tensor, src_of = group_rows_with_sizes(
            expert_idxs, experts_per_rank, device=gathered_tokens.device,
            host_sizes=host_sizes or not experts.one_node(gathered_tokens))
        if experts.bias_fusable(gathered_tokens):
            # both sides: rows gathered by the first quantisation, stored un-permuted (bias added)
            # by the last GEMM; the bias gradients are summed through the same map
            return experts(gathered_tokens, grouped_mm_offs, ks=ks, ks_tensor=ks_tensor, row_map=src_of, scatter_output=True)
        # input side only: the unfused bias add wants the grouped layout
        outs = experts(gathered_tokens, grouped_mm_offs, ks=ks, ks_tensor=ks_tensor, row_map=src_of)
        return padded_index_gather(outs, reverse_shuffle_idxs)
    pre = None
    if expand_idx is not None:
        if fuse_expand:
            pre = expand_idx
        else:
            gathered_tokens = padded_index_gather(gathered_tokens, expand_idx)
    output_tokens, reverse_shuffle_idxs, grouped_mm_offs, ks, ks_tensor = scatter_for_grouped_gemm(
        gathered_tokens, expert_idxs, experts_per_rank, pre_index=pre
    )
    del gathered_tokens
    outs = experts(output_tokens, grouped_mm_offs, ks=ks, ks_tensor=ks_tensor)
    return padded_index_gather(outs, reverse_shuffle_idxs)
