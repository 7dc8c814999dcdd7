"""Request queue -> batch planner -> model runner -> finished completions (counterpart of
electrock_infer/engine/llm_engine.py:88-143).  Prompts are token-id lists: no tokenizer files exist offline."""
from time import perf_counter
from typing import Dict, List, Optional, Sequence as Seq, Union

from .config import EngineConfig, ModelConfig, SamplingParams
from .model_runner import ModelRunner
from .batch_planner import BatchPlanner
from .sequence import Sequence


class LLMEngine:

    def __init__(self, model: Optional[ModelConfig] = None, model_runner=None, **kwargs):
        """``model_runner``: an object with ``run(seqs, is_prefill[, return_logits])`` to use instead of the GPU model
        (host tests of the request loop); it must leave ``config.num_kvcache_blocks`` as given."""
        self.config = EngineConfig(model=model or ModelConfig(), **kwargs)
        Sequence.block_size = self.config.kvcache_block_size
        self.model_runner = model_runner if model_runner is not None else ModelRunner(self.config)  # sizes config.num_kvcache_blocks
        self.planner = BatchPlanner(self.config)
        self.stats: Dict[str, float] = {}
        self.step_hook = None          # called as hook(seqs, is_prefill, logits) after every step when set

    def add_request(self, prompt: Seq[int], sampling_params: SamplingParams) -> Sequence:
        if isinstance(prompt, str):
            raise TypeError("prompts are lists of token ids (there is no tokenizer in this harness)")
        limit = self.config.max_model_len          # <= max_position_embeddings: the rotary table ends there
        if len(prompt) + 1 > limit:
            raise ValueError("prompt longer than max_model_len")
        seq = Sequence(prompt, sampling_params)
        # no request may grow past the positions the model has: the request ends at max_model_len tokens at the latest
        # (the reference has no such cap, llm_engine.py:88-91; there a long request indexes past its rotary table)
        seq.max_total_tokens = limit if seq.max_total_tokens <= 0 else min(seq.max_total_tokens, limit)
        self.planner.submit(seq)
        return seq

    def step(self):
        """One scheduled batch through the model.  Returns the requests that finished and the batch's token count:
        positive for a prefill step (tokens in the batch), negative for a decode step (minus the sequences)."""
        plan = self.planner.plan()
        seqs, is_prefill = plan.seqs, plan.is_prefill
        if self.step_hook is not None:
            token_ids, logits = self.model_runner.run(seqs, is_prefill, return_logits=True)
            self.step_hook(seqs, is_prefill, logits)
        else:
            token_ids = self.model_runner.run(seqs, is_prefill)
        finished = [(seq.seq_id, seq.completion_token_ids) for seq in self.planner.commit(seqs, token_ids)]
        return finished, (sum(len(s) for s in seqs) if is_prefill else -len(seqs))

    def is_finished(self) -> bool:
        return self.planner.idle()

    def generate(self, prompts: List[List[int]], sampling_params: Union[SamplingParams, List[SamplingParams]]):
        """Run all requests to completion; returns ``[{"token_ids": [...]}, ...]`` in the order of the prompts and
        leaves step counts and times in ``self.stats``."""
        if not isinstance(sampling_params, list):
            sampling_params = [sampling_params] * len(prompts)
        order = [self.add_request(p, sp).seq_id for p, sp in zip(prompts, sampling_params)]
        done: Dict[int, List[int]] = {}
        stats = {"prefill_steps": 0, "decode_steps": 0, "prefill_tokens": 0, "decode_tokens": 0, "prefill_s": 0.0,
                 "decode_s": 0.0}
        while not self.is_finished():
            t0 = perf_counter()
            finished, n = self.step()           # sampling ends in a device-to-host copy: the step is complete
            dt = perf_counter() - t0
            kind = "prefill" if n > 0 else "decode"
            stats[kind + "_steps"] += 1
            stats[kind + "_tokens"] += abs(n)
            stats[kind + "_s"] += dt
            done.update(finished)
        stats["preemptions"] = self.planner.num_preemptions
        self.stats = stats
        return [{"token_ids": done[i]} for i in order]
