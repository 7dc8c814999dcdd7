"""One request's tokens and cache bookkeeping (counterpart of electrock_infer/engine/sequence.py:14-86)."""
import itertools
from enum import Enum

from .config import SamplingParams


class SequenceStatus(Enum):
    WAITING = 0
    RUNNING = 1
    FINISHED = 2


class Sequence:
    """Token ids of a request (prompt + completion), the ids of the KV-cache blocks that hold them, and how many of
    the leading tokens were found in the prefix cache when the blocks were allocated."""

    block_size = 32                      # tokens per KV-cache block (sequence.py:15)
    _ids = itertools.count()

    def __init__(self, token_ids, sampling_params: SamplingParams):
        if len(token_ids) == 0:
            raise ValueError("a request needs at least one prompt token")
        self.seq_id = next(Sequence._ids)
        self.status = SequenceStatus.WAITING
        self.token_ids = list(token_ids)
        self.num_prompt_tokens = len(self.token_ids)
        self.num_cached_tokens = 0
        self.block_table = []
        self.temperature = sampling_params.temperature
        self.max_tokens = sampling_params.max_tokens
        self.ignore_eos = sampling_params.ignore_eos
        self.max_total_tokens = sampling_params.max_total_tokens

    def __len__(self):
        return len(self.token_ids)

    def __getitem__(self, key):
        return self.token_ids[key]

    @property
    def last_token(self):
        return self.token_ids[-1]

    @property
    def is_finished(self):
        return self.status is SequenceStatus.FINISHED

    @property
    def num_completion_tokens(self):
        return len(self.token_ids) - self.num_prompt_tokens

    @property
    def completion_token_ids(self):
        return self.token_ids[self.num_prompt_tokens:]

    @property
    def num_blocks(self):
        return -(-len(self.token_ids) // self.block_size)

    @property
    def num_cached_blocks(self):
        return self.num_cached_tokens // self.block_size

    @property
    def last_block_num_tokens(self):
        return len(self.token_ids) - (self.num_blocks - 1) * self.block_size

    def block(self, i):
        """Token ids of logical block i."""
        if not 0 <= i < self.num_blocks:
            raise IndexError(i)
        return self.token_ids[i * self.block_size:(i + 1) * self.block_size]

    def append_token(self, token_id: int):
        self.token_ids.append(int(token_id))
