"""End-to-end harness around the MoE layer: a Mixtral-shaped decoder-only model with a paged KV cache, a
prefill-first batch planner with preemption, a prefix-reusing pool of KV blocks and a sampler -- this build's own
counterpart of the reference's engine (electrock_infer/engine/*, models/mixtral.py, layers/sampler.py), kept small.

It exists to run the MoE path inside a whole generation loop (the end-to-end configuration of the benchmark) and is
not part of the hot path: attention is torch's scaled_dot_product_attention over a gathered paged cache, the dense
projections are torch matmuls; only the norms and the MoE block go through this package's own kernels.
"""
from .config import EngineConfig, ModelConfig, SamplingParams  # noqa: F401
from .engine import LLMEngine  # noqa: F401

LLM = LLMEngine
