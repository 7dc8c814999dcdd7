"""Which requests run in the next step.

Policy (the reference's, electrock_infer/engine/scheduler.py:24-74): requests that wait are started first, in
arrival order, for as long as the step's token budget, its sequence budget and the free KV blocks allow; only a
step that could start none is a decode step of the running requests, oldest first, in which a request that needs
a block when none is free takes it from the youngest running request (which goes back to the head of the waiting
line and is prefilled again later, prompt and completion so far), or gives way itself when it is the last one.

Construction (this build's own): the running requests are a plain list in admission order and a step is planned
into a ``Plan`` record; the decode planner walks that list by index and evicts from its tail.
"""
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, List

from .config import EngineConfig
from .kv_pool import KVBlockPool
from .sequence import Sequence, SequenceStatus


@dataclass
class Plan:
    seqs: List[Sequence] = field(default_factory=list)
    is_prefill: bool = False
    fresh_tokens: int = 0          # prefill: tokens that are not served from the prefix cache


class BatchPlanner:

    def __init__(self, config: EngineConfig):
        self.max_seqs = config.max_num_seqs
        self.max_tokens = config.max_num_batched_tokens
        self.eos = config.eos
        self.pool = KVBlockPool(config.num_kvcache_blocks, config.kvcache_block_size)
        self.waiting: Deque[Sequence] = deque()
        self.running: List[Sequence] = []
        self.num_preemptions = 0

    def submit(self, seq: Sequence) -> None:
        self.waiting.append(seq)

    def idle(self) -> bool:
        return not self.waiting and not self.running

    # ---- planning ----
    def _plan_prefill(self) -> Plan:
        plan = Plan(is_prefill=True)
        for seq in list(self.waiting):                    # arrival order; the first one that does not fit ends the batch
            if len(plan.seqs) == self.max_seqs or plan.fresh_tokens + len(seq) > self.max_tokens or not self.pool.fits(seq):
                break
            self.pool.admit(seq)
            plan.fresh_tokens += len(seq) - seq.num_cached_tokens
            plan.seqs.append(seq)
        for seq in plan.seqs:
            self.waiting.popleft()
            seq.status = SequenceStatus.RUNNING
            self.running.append(seq)
        return plan

    def _plan_decode(self) -> Plan:
        plan = Plan(is_prefill=False)
        keep, i = self.running, 0
        while i < len(keep) and len(plan.seqs) < self.max_seqs:
            seq = keep[i]
            while not self.pool.can_grow(seq) and len(keep) > i + 1:
                self._evict(keep.pop())                   # the youngest gives its blocks
            if self.pool.can_grow(seq):
                self.pool.grow(seq)
                plan.seqs.append(seq)
                i += 1
            else:
                self._evict(keep.pop(i))                  # nobody behind it: it goes itself
        if not plan.seqs:
            raise RuntimeError("the KV cache cannot hold a single running request")
        return plan

    def plan(self) -> Plan:
        p = self._plan_prefill() if self.waiting else Plan()
        return p if p.seqs else self._plan_decode()

    def _evict(self, seq: Sequence) -> None:
        seq.status = SequenceStatus.WAITING
        self.pool.release(seq)
        self.waiting.appendleft(seq)
        self.num_preemptions += 1

    # ---- after the step ----
    def _is_done(self, seq: Sequence, token_id: int) -> bool:
        if token_id == self.eos and not seq.ignore_eos:
            return True
        return seq.num_completion_tokens == seq.max_tokens or len(seq) == seq.max_total_tokens

    def commit(self, seqs: List[Sequence], token_ids: List[int]) -> List[Sequence]:
        """Append the sampled tokens; requests that end here leave the running list and give their blocks back.
        Returns them."""
        ended = []
        for seq, token_id in zip(seqs, token_ids):
            seq.append_token(token_id)
            if self._is_done(seq, token_id):
                seq.status = SequenceStatus.FINISHED
                self.pool.release(seq)
                ended.append(seq)
        if ended:
            gone = {id(s) for s in ended}
            self.running = [s for s in self.running if id(s) not in gone]
        return ended
