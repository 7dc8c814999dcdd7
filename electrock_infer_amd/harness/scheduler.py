"""Prefill-first batch scheduler with preemption (counterpart of electrock_infer/engine/scheduler.py:24-74)."""
from collections import deque
from typing import List, Tuple

from .block_manager import BlockManager
from .config import EngineConfig
from .sequence import Sequence, SequenceStatus


class Scheduler:

    def __init__(self, config: EngineConfig):
        self.max_num_seqs = config.max_num_seqs
        self.max_num_batched_tokens = config.max_num_batched_tokens
        self.eos = config.eos
        self.block_manager = BlockManager(config.num_kvcache_blocks, config.kvcache_block_size)
        self.waiting = deque()
        self.running = deque()
        self.num_preemptions = 0

    def is_finished(self) -> bool:
        return not self.waiting and not self.running

    def add(self, seq: Sequence) -> None:
        self.waiting.append(seq)

    def schedule(self) -> Tuple[List[Sequence], bool]:
        """The next batch and whether it is a prefill batch.  Waiting requests go first, in arrival order, while the
        token budget, the sequence budget and the free KV blocks last; only when none can start does a decode step
        of the running requests follow, preempting from the back of the queue when a new block is needed and none
        is free."""
        batch, budget = [], 0
        while self.waiting and len(batch) < self.max_num_seqs:
            seq = self.waiting[0]
            if budget + len(seq) > self.max_num_batched_tokens or not self.block_manager.can_allocate(seq):
                break
            self.block_manager.allocate(seq)
            budget += len(seq) - seq.num_cached_tokens
            seq.status = SequenceStatus.RUNNING
            self.waiting.popleft()
            self.running.append(seq)
            batch.append(seq)
        if batch:
            return batch, True

        while self.running and len(batch) < self.max_num_seqs:
            seq = self.running.popleft()
            while not self.block_manager.can_append(seq):
                if self.running:
                    self.preempt(self.running.pop())
                else:
                    self.preempt(seq)
                    break
            else:
                self.block_manager.may_append(seq)
                batch.append(seq)
        if not batch:
            raise RuntimeError("the KV cache cannot hold a single running request")
        self.running.extendleft(reversed(batch))
        return batch, False

    def preempt(self, seq: Sequence) -> None:
        """Back to the front of the waiting queue; its blocks are freed and it is prefilled again later (prompt and
        the completion so far)."""
        seq.status = SequenceStatus.WAITING
        self.block_manager.deallocate(seq)
        self.waiting.appendleft(seq)
        self.num_preemptions += 1

    def postprocess(self, seqs: List[Sequence], token_ids: List[int]) -> None:
        for seq, token_id in zip(seqs, token_ids):
            seq.append_token(token_id)
            done = (not seq.ignore_eos and token_id == self.eos) or seq.num_completion_tokens == seq.max_tokens \
                or seq.max_total_tokens == len(seq)
            if done:
                seq.status = SequenceStatus.FINISHED
                self.block_manager.deallocate(seq)
                self.running.remove(seq)
