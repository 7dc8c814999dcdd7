"""Request queue -> scheduler -> model runner -> finished completions (counterpart of
electrock_infer/engine/llm_engine.py:88-143).  Prompts are token-id lists: no tokenizer files exist offline."""
from time import perf_counter
from typing import Dict, List, Optional, Sequence as Seq, Union

from .config import EngineConfig, ModelConfig, SamplingParams
from .model_runner import ModelRunner
from .scheduler import Scheduler
from .sequence import Sequence


class LLMEngine:

    def __init__(self, model: Optional[ModelConfig] = None, **kwargs):
        self.config = EngineConfig(model=model or ModelConfig(), **kwargs)
        Sequence.block_size = self.config.kvcache_block_size
        self.model_runner = ModelRunner(self.config)          # sizes config.num_kvcache_blocks
        self.scheduler = Scheduler(self.config)
        self.stats: Dict[str, float] = {}
        self.step_hook = None          # called as hook(seqs, is_prefill, logits) after every step when set

    def add_request(self, prompt: Seq[int], sampling_params: SamplingParams) -> Sequence:
        if isinstance(prompt, str):
            raise TypeError("prompts are lists of token ids (there is no tokenizer in this harness)")
        if len(prompt) + 1 > self.config.max_model_len:
            raise ValueError("prompt longer than max_model_len")
        seq = Sequence(prompt, sampling_params)
        self.scheduler.add(seq)
        return seq

    def step(self):
        """One scheduled batch through the model.  Returns the requests that finished and the batch's token count:
        positive for a prefill step (tokens in the batch), negative for a decode step (minus the sequences)."""
        seqs, is_prefill = self.scheduler.schedule()
        if self.step_hook is not None:
            token_ids, logits = self.model_runner.run(seqs, is_prefill, return_logits=True)
            self.step_hook(seqs, is_prefill, logits)
        else:
            token_ids = self.model_runner.run(seqs, is_prefill)
        self.scheduler.postprocess(seqs, token_ids)
        finished = [(seq.seq_id, seq.completion_token_ids) for seq in seqs if seq.is_finished]
        return finished, (sum(len(s) for s in seqs) if is_prefill else -len(seqs))

    def is_finished(self) -> bool:
        return self.scheduler.is_finished()

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
        stats["preemptions"] = self.scheduler.num_preemptions
        self.stats = stats
        return [{"token_ids": done[i]} for i in order]
