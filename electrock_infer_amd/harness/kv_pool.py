"""Pool of KV-cache blocks with prefix reuse.

Policy (what the reference's engine does, electrock_infer/engine/block_manager.py:28-120): a full block of a
request is named by xxh64 over (the name of the block in front of it, its token ids as int64), so requests that
begin with the same tokens share the physical blocks of their common prefix; a block that is given back keeps its
name until it is handed out for something else and can be taken up again by a later request; free blocks are
handed out oldest first.

Construction (this build's own): the pool is a handful of numpy arrays indexed by block id -- reference count,
digest, sealed flag, a [blocks, block_size] token matrix and the two link arrays of an intrusive doubly linked
free list (so that taking a particular free block out of the middle, the "revival", is O(1)) -- and a request is
admitted in two passes: the digests of all its full blocks are chained up front and looked up to find the length
of the reusable prefix, then the prefix is shared and the rest is taken from the head of the free list.
"""
from typing import Dict, List

import numpy as np
import xxhash

from .sequence import Sequence

_NIL = -1


def block_digest(token_ids, parent: int = _NIL) -> int:
    """Name of a full block: xxh64(parent digest as 8 little-endian bytes, if any ++ token ids as int64)."""
    h = xxhash.xxh64()
    if parent != _NIL:
        h.update(int(parent).to_bytes(8, "little"))
    h.update(np.asarray(token_ids, dtype=np.int64).tobytes())
    return h.intdigest()


def chain_digests(token_ids, block_size: int) -> List[int]:
    """Digests of all full blocks of a token list, each chained to the one before."""
    out, parent = [], _NIL
    for start in range(0, len(token_ids) - block_size + 1, block_size):
        parent = block_digest(token_ids[start:start + block_size], parent)
        out.append(parent)
    return out


class KVBlockPool:

    def __init__(self, num_blocks: int, block_size: int):
        if num_blocks <= 0:
            raise ValueError("the KV cache needs at least one block")
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.refs = np.zeros(num_blocks, dtype=np.int32)
        self.sealed = np.zeros(num_blocks, dtype=bool)           # holds a full block whose digest is valid
        self.digest = np.zeros(num_blocks, dtype=np.uint64)
        self.content = np.zeros((num_blocks, block_size), dtype=np.int64)
        self.by_digest: Dict[int, int] = {}                       # digest -> the block that last took that name
        # free list, oldest first: head -> ... -> tail; a block in use has both links at _NIL and in_free False
        self._next = np.arange(1, num_blocks + 1, dtype=np.int32)
        self._prev = np.arange(-1, num_blocks - 1, dtype=np.int32)
        self._next[-1] = _NIL
        self._head, self._tail = 0, num_blocks - 1
        self.in_free = np.ones(num_blocks, dtype=bool)
        self.num_free = num_blocks

    # ---- free list ----
    def _unlink(self, b: int) -> None:
        p, n = int(self._prev[b]), int(self._next[b])
        if p == _NIL:
            self._head = n
        else:
            self._next[p] = n
        if n == _NIL:
            self._tail = p
        else:
            self._prev[n] = p
        self._prev[b] = self._next[b] = _NIL
        self.in_free[b] = False
        self.num_free -= 1

    def _push_back(self, b: int) -> None:
        self._prev[b], self._next[b] = self._tail, _NIL
        if self._tail == _NIL:
            self._head = b
        else:
            self._next[self._tail] = b
        self._tail = b
        self.in_free[b] = True
        self.num_free += 1

    def free_ids(self) -> List[int]:
        """Free block ids in the order they will be handed out."""
        out, b = [], self._head
        while b != _NIL:
            out.append(b)
            b = int(self._next[b])
        return out

    def _claim(self, b: int, keep_name: bool) -> int:
        """Take free block b into use with one reference; unless it is taken up for its old contents, its name is void."""
        assert self.in_free[b] and self.refs[b] == 0
        self._unlink(b)
        self.refs[b] = 1
        if not keep_name:
            self.sealed[b] = False
        return b

    def _seal(self, b: int, digest: int, tokens) -> None:
        self.sealed[b] = True
        self.digest[b] = digest
        self.content[b] = tokens
        self.by_digest[digest] = b

    def _lookup(self, digest: int, tokens) -> int:
        """The block that holds exactly these tokens under this name, or _NIL."""
        b = self.by_digest.get(digest, _NIL)
        if b == _NIL or not self.sealed[b] or int(self.digest[b]) != digest or not np.array_equal(self.content[b], tokens):
            return _NIL
        return b

    # ---- a request enters (prefill) ----
    def fits(self, seq: Sequence) -> bool:
        """Room for the request if nothing of it were cached (the reference's admission rule)."""
        return self.num_free >= seq.num_blocks

    def admit(self, seq: Sequence) -> None:
        """Fill ``seq.block_table``; the leading full blocks found in the pool are shared and counted in
        ``seq.num_cached_tokens``, everything behind the first miss is fresh."""
        assert not seq.block_table
        bs = self.block_size
        tokens = seq.token_ids
        names = chain_digests(tokens, bs)
        reuse = []
        for i, name in enumerate(names):
            b = self._lookup(name, tokens[i * bs:(i + 1) * bs])
            if b == _NIL:
                break
            reuse.append(b)
        for b in reuse:
            if self.in_free[b]:
                self._claim(b, keep_name=True)       # given back earlier, contents intact
            else:
                self.refs[b] += 1
        seq.num_cached_tokens = len(reuse) * bs
        table = list(reuse)
        for i in range(len(reuse), seq.num_blocks):
            b = self._claim(self._head, keep_name=False)
            if i < len(names):                        # a full block: later requests may find it
                self._seal(b, names[i], tokens[i * bs:(i + 1) * bs])
            table.append(b)
        seq.block_table.extend(int(b) for b in table)

    def release(self, seq: Sequence) -> None:
        """Drop the request's references; blocks nobody holds any more join the free list, the request's last block
        first, so that the blocks of its prefix are the last to be handed out again."""
        for b in reversed(seq.block_table):
            self.refs[b] -= 1
            if self.refs[b] == 0:
                self._push_back(b)
        seq.block_table.clear()
        seq.num_cached_tokens = 0

    # ---- a running request has grown by one token (decode) ----
    def blocks_to_grow(self, seq: Sequence) -> int:
        """1 when the newest token opens a block, else 0."""
        return 1 if len(seq) % self.block_size == 1 else 0

    def can_grow(self, seq: Sequence) -> bool:
        return self.num_free >= self.blocks_to_grow(seq)

    def grow(self, seq: Sequence) -> None:
        """Make the table cover the newest token: open a block for it, or, when it completes a block, give that block
        its name so that later requests can share it."""
        fill = len(seq) % self.block_size
        table = seq.block_table
        if fill == 1:
            table.append(int(self._claim(self._head, keep_name=False)))
        elif fill == 0:
            last = table[-1]
            assert not self.sealed[last]
            parent = int(self.digest[table[-2]]) if len(table) > 1 else _NIL
            tokens = seq.token_ids[-self.block_size:]
            self._seal(last, block_digest(tokens, parent), tokens)
