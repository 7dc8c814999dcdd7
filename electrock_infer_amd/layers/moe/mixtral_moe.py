"""FusedMoE layer with the reference's class surface
(electrock_infer/layers/moe/mixtral_moe.py:8-152): same constructor arguments,
parameter names/shapes, ``weight_loader`` and in-place ``forward``."""
from typing import Optional

import torch
import torch.distributed as dist
import torch.nn as nn

from ... import _lib
from .fused_moe import fused_experts

# the reference's largest batch (max_num_batched_tokens, config.py:9): w2 is kept as float16 only when every batch
# size up to it can be served that way
_W2_F16_MIN_TOKENS = 32768


class FusedMoE(nn.Module):
    """Mixtral block-sparse MoE experts.

    Holds ``w13_weight [E, 2*I/tp, H]`` (gate rows then up rows) and
    ``w2_weight [E, H, I/tp]``; ``forward(hidden_states, router_logits)``
    overwrites and returns ``hidden_states``.  Only the reference's tensor
    parallel sharding of ``I`` is understood by ``weight_loader``; this build
    runs on one GPU, so ``reduce_results`` only matters when a caller has
    initialised a process group with ``tp_size > 1`` itself.
    """

    def __init__(self, num_experts: int, top_k: int, hidden_size: int, intermediate_size: int,
                 tp_size: Optional[int] = None, params_dtype: Optional[torch.dtype] = None,
                 renormalize: bool = True, reduce_results: bool = False, *, bf16_act: bool = False,
                 w2_dtype: Optional[torch.dtype] = None):
        super().__init__()
        self.tp_size = tp_size if tp_size is not None else 1
        # the reference reads dist.get_rank() unconditionally (mixtral_moe.py:41);
        # without a process group there is exactly one rank
        self.tp_rank = dist.get_rank() if dist.is_available() and dist.is_initialized() else 0
        self.num_experts = num_experts
        self.top_k = top_k
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.renormalize = renormalize
        self.reduce_results = reduce_results
        # not in the reference: the SiLU*mul activations pass from the w13 to the w2 GEMM as fp16 (three more mantissa
        # bits than the reference's bf16 cache2, clamped to +-65504; a call that clamped anything says so in
        # ``get_workspace(...).saturated()``).  bf16_act=True stores them as bf16 instead: the reference's range and
        # rounding, the range-safe choice for checkpoints with very large activations.
        self.bf16_act = bf16_act
        if w2_dtype not in (None, torch.bfloat16, torch.float16):
            raise ValueError("w2_dtype must be bfloat16 or float16")
        self.params_dtype = params_dtype or torch.get_default_dtype()
        if w2_dtype is None:
            # not in the reference either: with bfloat16 parameters w2 is held as float16 (the loader's copy converts
            # the checkpoint, exactly for every weight of magnitude 2^-14 .. 65504), so that the w2 GEMM multiplies
            # the fp16 activations without converting its weight fragments (8192 tokens: -10 % on that kernel).
            # w2_dtype=torch.bfloat16 keeps the checkpoint's type; so do bf16_act and shapes that only the
            # shape-generic kernels take.
            w2_dtype = self.params_dtype
            if self.params_dtype == torch.bfloat16 and not bf16_act and intermediate_size % self.tp_size == 0 and \
                    _lib.load().em_moe_w2_f16_max_tokens(hidden_size, intermediate_size // self.tp_size, num_experts,
                                                         top_k) >= _W2_F16_MIN_TOKENS:
                w2_dtype = torch.float16
        self.w2_dtype = w2_dtype
        if self.intermediate_size % self.tp_size != 0:
            raise ValueError(f"intermediate_size ({self.intermediate_size}) must be divisible by "
                             f"tp_size ({self.tp_size})")
        self.intermediate_size_per_partition = self.intermediate_size // self.tp_size

        self.w13_weight = nn.Parameter(torch.empty(self.num_experts, 2 * self.intermediate_size_per_partition,
                                                   self.hidden_size, dtype=self.params_dtype),
                                       requires_grad=False)
        self.w2_weight = nn.Parameter(torch.empty(self.num_experts, self.hidden_size,
                                                  self.intermediate_size_per_partition,
                                                  dtype=self.w2_dtype), requires_grad=False)
        self.w13_weight.weight_loader = self.weight_loader
        self.w2_weight.weight_loader = self.weight_loader

    def forward(self, hidden_states: torch.Tensor, router_logits: torch.Tensor) -> torch.Tensor:
        final_hidden_states = fused_experts(hidden_states=hidden_states, w1=self.w13_weight,
                                            w2=self.w2_weight, gating_output=router_logits,
                                            topk=self.top_k, renormalize=self.renormalize, inplace=True,
                                            activation="silu", bf16_act=self.bf16_act)
        if self.reduce_results and self.tp_size > 1:
            dist.all_reduce(final_hidden_states)
        return final_hidden_states

    def weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor, shard_id: str,
                      expert_id: int) -> None:
        """Copy one checkpoint tensor (``experts.{e}.w1|w3|w2.weight``) into the
        stacked parameter: w1 -> w13[e, :I], w3 -> w13[e, I:], w2 -> w2[e], each
        narrowed to this rank's slice of ``I`` (mixtral_moe.py:121-152)."""
        shard = self.intermediate_size_per_partition
        param_data = param.data[expert_id]
        if shard_id in ("w1", "w3"):
            loaded_shard = loaded_weight.narrow(0, shard * self.tp_rank, shard)
            if shard_id == "w1":
                param_data[:shard, :].copy_(loaded_shard)
            else:
                param_data[shard:, :].copy_(loaded_shard)
        elif shard_id == "w2":
            param_data.copy_(loaded_weight.narrow(1, shard * self.tp_rank, shard))
        else:
            raise ValueError(f"unknown shard_id: {shard_id}")
