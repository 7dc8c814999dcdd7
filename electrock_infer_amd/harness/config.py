"""Configuration of the harness.  The reference reads the model's shape from a Hugging Face config on disk
(electrock_infer/config.py:21-24) and its engine limits from keyword arguments (config.py:8-19); no model directory
exists here, so the shape is a plain dataclass with Mixtral-8x7B's values as defaults and the weights are drawn at
random."""
from dataclasses import dataclass, field

import torch


@dataclass
class ModelConfig:
    """Shape of a Mixtral-style decoder (defaults: Mixtral-8x7B, utils/mixtral_info.txt)."""
    vocab_size: int = 32000
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    num_local_experts: int = 8
    num_experts_per_tok: int = 2
    rms_norm_eps: float = 1e-5
    rope_theta: float = 1e6
    max_position_embeddings: int = 32768
    torch_dtype: torch.dtype = torch.bfloat16

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads


@dataclass
class SamplingParams:
    """Per-request sampling controls (electrock_infer/sampling_params.py:4-8)."""
    temperature: float = 1.0
    max_tokens: int = 64
    ignore_eos: bool = False
    max_total_tokens: int = -1


@dataclass
class EngineConfig:
    """Engine limits, with the reference's names and defaults (config.py:8-19) where they apply to one GPU."""
    model: ModelConfig = field(default_factory=ModelConfig)
    max_num_batched_tokens: int = 32768
    max_num_seqs: int = 300
    max_model_len: int = 4096
    gpu_memory_utilization: float = 0.90
    eos: int = -1
    kvcache_block_size: int = 32
    num_kvcache_blocks: int = -1        # -1: sized from the free device memory (model_runner.py:92-104)
    seed: int = 0                       # of the random weights
    device: str = "cuda:0"
    fused_moe_tail: bool = True         # post-attention norm + gate + router + experts in one library call

    def __post_init__(self):
        self.max_model_len = min(self.max_model_len, self.model.max_position_embeddings)
