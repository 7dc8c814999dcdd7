"""KV-cache block allocator with prefix caching (counterpart of electrock_infer/engine/block_manager.py:28-120).

A full block is identified by a 64-bit hash chained over the hashes of the blocks in front of it, so two requests
that start with the same tokens share the physical blocks of their common prefix; a freed block keeps its hash until
it is handed out again, so a later request can still pick it up."""
from collections import deque

import numpy as np
import xxhash

from .sequence import Sequence


class Block:
    __slots__ = ("block_id", "ref_count", "hash", "token_ids")

    def __init__(self, block_id: int):
        self.block_id = block_id
        self.ref_count = 0
        self.hash = -1            # -1: not a complete, hashed block
        self.token_ids = []


class BlockManager:

    def __init__(self, num_blocks: int, block_size: int):
        if num_blocks <= 0:
            raise ValueError("the KV cache needs at least one block")
        self.block_size = block_size
        self.blocks = [Block(i) for i in range(num_blocks)]
        self.hash_to_block_id = {}
        self.free_block_ids = deque(range(num_blocks))
        self.used_block_ids = set()

    @staticmethod
    def compute_hash(token_ids, prefix: int = -1) -> int:
        """xxh64 over the previous block's hash (8 bytes, little endian) and the block's token ids as int64
        (block_manager.py:37-43)."""
        h = xxhash.xxh64()
        if prefix != -1:
            h.update(prefix.to_bytes(8, "little"))
        h.update(np.asarray(token_ids, dtype=np.int64).tobytes())
        return h.intdigest()

    # ---- physical blocks ----
    def _take(self, block_id: int) -> Block:
        block = self.blocks[block_id]
        assert block.ref_count == 0
        block.ref_count, block.hash, block.token_ids = 1, -1, []
        self.free_block_ids.remove(block_id)
        self.used_block_ids.add(block_id)
        return block

    def _release(self, block_id: int) -> None:
        assert self.blocks[block_id].ref_count == 0
        self.used_block_ids.remove(block_id)
        self.free_block_ids.append(block_id)

    # ---- prefill ----
    def can_allocate(self, seq: Sequence) -> bool:
        return len(self.free_block_ids) >= seq.num_blocks

    def allocate(self, seq: Sequence) -> None:
        """Give every logical block of the sequence a physical one; leading full blocks whose chained hash (and
        tokens) match a block in the table are shared instead and counted in ``seq.num_cached_tokens``."""
        assert not seq.block_table
        chain, missed = -1, False
        for i in range(seq.num_blocks):
            tokens = seq.block(i)
            chain = self.compute_hash(tokens, chain) if len(tokens) == self.block_size else -1
            hit = self.hash_to_block_id.get(chain, -1)
            if hit == -1 or self.blocks[hit].token_ids != tokens:
                missed = True                      # everything behind the first miss is new as well
            if missed:
                block = self._take(self.free_block_ids[0])
            else:
                seq.num_cached_tokens += self.block_size
                if hit in self.used_block_ids:
                    block = self.blocks[hit]
                    block.ref_count += 1
                else:                               # freed earlier, contents still intact: revive it
                    block = self._take(hit)
            if chain != -1:
                block.hash, block.token_ids = chain, tokens
                self.hash_to_block_id[chain] = block.block_id
            seq.block_table.append(block.block_id)

    def deallocate(self, seq: Sequence) -> None:
        """Give the blocks back, last block first, so that the blocks of a prefix are the last to be reused."""
        for block_id in reversed(seq.block_table):
            block = self.blocks[block_id]
            block.ref_count -= 1
            if block.ref_count == 0:
                self._release(block_id)
        seq.num_cached_tokens = 0
        seq.block_table.clear()

    # ---- decode: the sequence has just grown by one token ----
    def can_append(self, seq: Sequence) -> bool:
        return len(self.free_block_ids) >= (1 if len(seq) % self.block_size == 1 else 0)

    def may_append(self, seq: Sequence) -> None:
        table = seq.block_table
        last = self.blocks[table[-1]]
        fill = len(seq) % self.block_size
        if fill == 1:                                # the new token opens a block
            assert last.hash != -1
            table.append(self._take(self.free_block_ids[0]).block_id)
        elif fill == 0:                              # the new token completes a block: hash it for later requests
            assert last.hash == -1
            tokens = seq.block(seq.num_blocks - 1)
            prefix = self.blocks[table[-2]].hash if len(table) > 1 else -1
            last.hash, last.token_ids = self.compute_hash(tokens, prefix), tokens
            self.hash_to_block_id[last.hash] = last.block_id
        else:
            assert last.hash == -1
