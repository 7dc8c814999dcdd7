"""Owns the model and the KV cache of one GPU and turns a scheduled batch into one forward pass and one sampled
token per sequence (counterpart of electrock_infer/engine/model_runner.py:92-236, single process: the reference's
shared-memory fan-out to tensor-parallel ranks has nothing to do on one GPU)."""
from typing import List

import torch

from ..layers.moe.fused_moe import reserve_workspace
from .config import EngineConfig
from .model import BatchContext, MixtralForCausalLM, Sampler
from .sequence import Sequence


class ModelRunner:

    def __init__(self, config: EngineConfig):
        self.config = config
        self.block_size = config.kvcache_block_size
        self.device = torch.device(config.device)
        cfg = config.model
        torch.cuda.set_device(self.device)
        with torch.device(self.device):
            self.model = MixtralForCausalLM(cfg, fused_moe_tail=config.fused_moe_tail)
        self.model.init_random_weights(config.seed)
        self.sampler = Sampler()
        # one MoE workspace for the largest batch the planner can form: no layer call allocates afterwards
        reserve_workspace(self.device, config.max_num_batched_tokens, cfg.hidden_size, cfg.intermediate_size,
                          cfg.num_local_experts, cfg.num_experts_per_tok)
        self.allocate_kv_cache()

    def allocate_kv_cache(self) -> None:
        """[2, layers, blocks, block_size, kv_heads, head_dim]; the block count comes from the configuration or from
        the device memory left under gpu_memory_utilization (model_runner.py:92-110)."""
        config, cfg = self.config, self.config.model
        block_bytes = 2 * cfg.num_hidden_layers * self.block_size * cfg.num_key_value_heads * cfg.head_dim * \
            torch.empty((), dtype=cfg.torch_dtype).element_size()
        if config.num_kvcache_blocks <= 0:
            free, total = torch.cuda.mem_get_info(self.device)
            budget = int(total * config.gpu_memory_utilization) - (total - free)
            if budget < block_bytes:
                raise RuntimeError("no device memory left for the KV cache")
            # what max_num_seqs sequences of max_model_len tokens can ever use is enough
            most = config.max_num_seqs * (-(-config.max_model_len // self.block_size))
            config.num_kvcache_blocks = min(budget // block_bytes, most)
        self.kv_cache = torch.zeros(2, cfg.num_hidden_layers, config.num_kvcache_blocks, self.block_size,
                                    cfg.num_key_value_heads, cfg.head_dim, dtype=cfg.torch_dtype, device=self.device)
        for i, layer in enumerate(self.model.model.layers):
            layer.self_attn.attn.k_cache = self.kv_cache[0, i]
            layer.self_attn.attn.v_cache = self.kv_cache[1, i]
            layer.self_attn.attn.kv_cache = self.kv_cache[:, i]

    # ---- batch preparation ----
    def _to_device(self, values, dtype) -> torch.Tensor:
        return torch.tensor(values, dtype=dtype, pin_memory=True).to(self.device, non_blocking=True)

    def _block_tables(self, seqs: List[Sequence]) -> torch.Tensor:
        width = max(len(s.block_table) for s in seqs)
        return self._to_device([s.block_table + [0] * (width - len(s.block_table)) for s in seqs], torch.int64)

    def prepare_prefill(self, seqs: List[Sequence]):
        """Feed the tokens behind every sequence's cached prefix; their cache slots follow from the block table."""
        input_ids, positions, slots, q_lens, k_lens, last = [], [], [], [], [], []
        for seq in seqs:
            n, cached = len(seq), seq.num_cached_tokens
            if cached == n:          # everything was found in the prefix cache: still feed the last token
                cached -= 1
            input_ids.extend(seq[cached:])
            positions.extend(range(cached, n))
            q_lens.append(n - cached)
            k_lens.append(n)
            for pos in range(cached, n):
                slots.append(seq.block_table[pos // self.block_size] * self.block_size + pos % self.block_size)
            last.append(len(input_ids) - 1)
        need_tables = any(k != q for q, k in zip(q_lens, k_lens))
        ctx = BatchContext(True, self._to_device(slots, torch.int64), q_lens, k_lens,
                           block_tables=self._block_tables(seqs) if need_tables else None,
                           last_token_index=self._to_device(last, torch.int64))
        return self._to_device(input_ids, torch.int64), self._to_device(positions, torch.int64), ctx

    def prepare_decode(self, seqs: List[Sequence]):
        """One token per sequence: the last one sampled, at position len - 1, into the last slot of its table."""
        input_ids = [s.last_token for s in seqs]
        positions = [len(s) - 1 for s in seqs]
        slots = [s.block_table[-1] * self.block_size + s.last_block_num_tokens - 1 for s in seqs]
        ctx = BatchContext(False, self._to_device(slots, torch.int64), [], [], block_tables=self._block_tables(seqs),
                           context_lens=self._to_device([len(s) for s in seqs], torch.int64))
        # the same for every layer of the step: key j of a sequence counts if j < its context length
        keys = ctx.block_tables.shape[1] * self.block_size
        ctx.decode_mask = (torch.arange(keys, device=self.device)[None, :] < ctx.context_lens[:, None])[:, None, None, :]
        return self._to_device(input_ids, torch.int64), self._to_device(positions, torch.int64), ctx

    # ---- one step ----
    @torch.inference_mode()
    def run_model(self, input_ids, positions, ctx: BatchContext) -> torch.Tensor:
        return self.model.compute_logits(self.model(input_ids, positions, ctx), ctx)

    def run(self, seqs: List[Sequence], is_prefill: bool, return_logits: bool = False):
        input_ids, positions, ctx = self.prepare_prefill(seqs) if is_prefill else self.prepare_decode(seqs)
        temperatures = self._to_device([s.temperature for s in seqs], torch.float32)
        logits = self.run_model(input_ids, positions, ctx)
        token_ids = self.sampler(logits, temperatures).tolist()
        return (token_ids, logits) if return_logits else token_ids
