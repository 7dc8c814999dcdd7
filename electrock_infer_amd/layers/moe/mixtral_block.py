"""The model's MoE block with the reference's class surface (electrock_infer/models/mixtral.py:19-63):
a replicated router gate (layers/linear.py:31-54) in front of ``FusedMoE``.  ``forward`` runs gate,
router, sort, both expert GEMMs and the combine through one C entry point."""
from typing import Optional

import torch
import torch.distributed as dist
import torch.nn as nn

from ..layernorm import RMSNorm
from .fused_moe import fused_experts_gated, fused_experts_normed
from .mixtral_moe import FusedMoE


class ReplicatedLinear(nn.Module):
    """``weight [output_size, input_size]`` replicated on every rank; only the MoE gate uses it
    (layers/linear.py:31-54).  No bias support is needed by that caller."""

    def __init__(self, input_size: int, output_size: int, bias: bool = False,
                 params_dtype: Optional[torch.dtype] = None):
        super().__init__()
        if bias:
            raise NotImplementedError("the router gate has no bias (models/mixtral.py:40-42)")
        self.input_size = input_size
        self.output_size = output_size
        self.weight = nn.Parameter(torch.empty(output_size, input_size, dtype=params_dtype or torch.get_default_dtype()),
                                   requires_grad=False)
        self.weight.weight_loader = self.weight_loader
        self.register_parameter("bias", None)

    def weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor):
        assert param.size() == loaded_weight.size()
        param.data.copy_(loaded_weight)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return torch.nn.functional.linear(x, self.weight, self.bias)


class MixtralMoE(nn.Module):
    """``forward(hidden_states)`` = ``experts(hidden_states, gate(hidden_states))`` of the reference
    (models/mixtral.py:53-63), with the gate computed inside the router's launch.  ``bf16_logits=True``
    (default) rounds the logits to bf16 before the selection as the reference's bf16 gate does; ``bf16_act=True``
    stores the SiLU*mul activations as bf16 instead of fp16 between the GEMMs; ``w2_dtype=torch.float16`` keeps
    ``experts.w2_weight`` as float16 (the loader's copy converts), which saves the w2 GEMM its conversions."""

    def __init__(self, num_experts: int, top_k: int, hidden_size: int, intermediate_size: int,
                 params_dtype: Optional[torch.dtype] = None, tp_size: Optional[int] = None, prefix: str = "",
                 bf16_logits: bool = True, bf16_act: bool = False, w2_dtype: Optional[torch.dtype] = None):
        super().__init__()
        self.hidden_size = hidden_size
        self.bf16_logits = bf16_logits
        self.gate = ReplicatedLinear(hidden_size, num_experts, bias=False, params_dtype=params_dtype)
        self.experts = FusedMoE(num_experts=num_experts, top_k=top_k, hidden_size=hidden_size,
                                intermediate_size=intermediate_size, params_dtype=params_dtype,
                                reduce_results=True, renormalize=True, tp_size=tp_size, bf16_act=bf16_act,
                                w2_dtype=w2_dtype)

    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        orig_shape = hidden_states.shape
        hidden_states = hidden_states.view(-1, self.hidden_size)
        e = self.experts
        out = fused_experts_gated(hidden_states, self.gate.weight, e.w13_weight, e.w2_weight, topk=e.top_k,
                                  renormalize=e.renormalize, inplace=True, bf16_logits=self.bf16_logits,
                                  bf16_act=e.bf16_act)
        if e.reduce_results and e.tp_size > 1:
            dist.all_reduce(out)
        return out.view(orig_shape)


class PostAttentionMoE(nn.Module):
    """The tail of the reference's decoder layer (models/mixtral.py:194-197) as one module and one library call:

        hidden_states, residual = post_attention_layernorm(hidden_states, residual)
        hidden_states = block_sparse_moe(hidden_states)

    ``forward(hidden_states, residual)`` returns ``(hidden_states, residual)`` like those two lines; the norm,
    the gate and the router run in one launch.  Holds the reference's sub-modules under their names."""

    def __init__(self, post_attention_layernorm: RMSNorm, block_sparse_moe: MixtralMoE):
        super().__init__()
        self.post_attention_layernorm = post_attention_layernorm
        self.block_sparse_moe = block_sparse_moe

    def forward(self, hidden_states: torch.Tensor, residual: torch.Tensor):
        norm, moe = self.post_attention_layernorm, self.block_sparse_moe
        e = moe.experts
        orig_shape = hidden_states.shape
        out, res = fused_experts_normed(hidden_states.view(-1, moe.hidden_size), residual.view(-1, moe.hidden_size),
                                        norm.weight, norm.eps, moe.gate.weight, e.w13_weight, e.w2_weight, topk=e.top_k,
                                        renormalize=e.renormalize, bf16_logits=moe.bf16_logits, bf16_act=e.bf16_act)
        if e.reduce_results and e.tp_size > 1:
            dist.all_reduce(out)
        return out.view(orig_shape), res.view(orig_shape)
