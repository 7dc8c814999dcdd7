"""Host logic of the end-to-end harness (no GPU): sequences, the prefix-reusing pool of KV blocks and the batch planner,
with the behaviours the reference's engine has (electrock_infer/engine/block_manager.py:56-120, scheduler.py:24-74)."""
import numpy as np
import pytest
import xxhash

from electrock_infer_amd.harness.batch_planner import BatchPlanner
from electrock_infer_amd.harness.config import EngineConfig, ModelConfig, SamplingParams
from electrock_infer_amd.harness.engine import LLMEngine
from electrock_infer_amd.harness.kv_pool import KVBlockPool, block_digest, chain_digests
from electrock_infer_amd.harness.sequence import Sequence, SequenceStatus

BS = 4


@pytest.fixture(autouse=True)
def small_blocks():
    old = Sequence.block_size
    Sequence.block_size = BS
    yield
    Sequence.block_size = old


def seq(tokens, **kw):
    return Sequence(tokens, SamplingParams(**kw))


def test_sequence_block_arithmetic():
    s = seq(list(range(10)))
    assert (len(s), s.num_blocks, s.last_block_num_tokens, s.block(2)) == (10, 3, 2, [8, 9])
    s.append_token(77)
    assert s.last_token == 77 and s.num_completion_tokens == 1 and s.completion_token_ids == [77]
    with pytest.raises(IndexError):
        s.block(3)


def test_block_digest_is_xxh64_chained_over_int64_tokens():
    # the definition written out: xxh64(parent digest as 8 little-endian bytes ++ token ids as int64)
    first = xxhash.xxh64(np.array([1, 2, 3, 4], dtype=np.int64).tobytes()).intdigest()
    assert block_digest([1, 2, 3, 4]) == first
    h = xxhash.xxh64()
    h.update(first.to_bytes(8, "little"))
    h.update(np.array([5, 6, 7, 8], dtype=np.int64).tobytes())
    assert block_digest([5, 6, 7, 8], first) == h.intdigest()
    assert block_digest([5, 6, 7, 8], first) != block_digest([5, 6, 7, 8])
    assert chain_digests([1, 2, 3, 4, 5, 6, 7, 8, 9], BS) == [first, h.intdigest()]      # the open block has no name
    assert chain_digests([1, 2, 3], BS) == []


def test_prefix_blocks_are_shared_and_survive_a_free():
    pool = KVBlockPool(8, BS)
    a = seq([1, 2, 3, 4, 5, 6, 7, 8, 9])          # two full blocks + one token
    pool.admit(a)
    assert a.num_cached_tokens == 0 and a.block_table == [0, 1, 2] and pool.num_free == 5    # oldest free blocks first
    b = seq([1, 2, 3, 4, 5, 6, 7, 8, 20, 21])     # same two leading blocks
    pool.admit(b)
    assert b.num_cached_tokens == 8 and b.block_table[:2] == a.block_table[:2] and b.block_table[2] != a.block_table[2]
    assert pool.refs[a.block_table[0]] == 2 and pool.num_free == 4
    c = seq([1, 2, 3, 4, 9, 9, 9, 9])             # first block shared, second differs: everything behind is new
    pool.admit(c)
    assert c.num_cached_tokens == 4 and c.block_table[0] == a.block_table[0] and c.block_table[1] not in a.block_table
    shared = a.block_table[:2]
    for s in (a, b, c):
        pool.release(s)
        assert s.block_table == [] and s.num_cached_tokens == 0
    assert pool.num_free == 8 and not pool.refs.any() and sorted(pool.free_ids()) == list(range(8))
    # behind the blocks that were never used: every request's blocks last block first, as their last holder lets go
    assert pool.free_ids() == [5, 6, 7, 2, 3, 1, 4, 0]
    d = seq([1, 2, 3, 4, 5, 6, 7, 8, 30])         # freed blocks keep their name: taken up again, out of the middle
    pool.admit(d)
    assert d.num_cached_tokens == 8 and d.block_table[:2] == shared and d.block_table[2] == 5
    assert pool.free_ids() == [6, 7, 2, 3, 4]
    # a block handed out for other contents loses its name: nobody finds the old tokens there
    e = seq(list(range(100, 120)))                # takes all five free blocks
    pool.admit(e)
    assert pool.num_free == 0 and e.num_cached_tokens == 0
    pool.release(e)
    pool.release(d)
    f = seq([1, 2, 3, 4, 9, 9, 9, 9, 1])          # c's second block [9,9,9,9] lived in block 4, overwritten by e
    pool.admit(f)
    assert f.num_cached_tokens == 4 and f.block_table[0] == shared[0]


def test_decode_appends_open_and_seal_blocks():
    pool = KVBlockPool(4, BS)
    s = seq([1, 2, 3])
    pool.admit(s)
    assert not pool.sealed[s.block_table[0]]
    s.append_token(4)                              # block complete: gets its name
    assert pool.can_grow(s) and pool.blocks_to_grow(s) == 0
    pool.grow(s)
    assert pool.sealed[s.block_table[0]] and int(pool.digest[s.block_table[0]]) == block_digest([1, 2, 3, 4])
    assert len(s.block_table) == 1
    s.append_token(5)                              # opens a second block
    assert pool.blocks_to_grow(s) == 1
    pool.grow(s)
    assert len(s.block_table) == 2
    for tok in (6, 7, 8):
        s.append_token(tok)
        pool.grow(s)
    assert int(pool.digest[s.block_table[1]]) == block_digest([5, 6, 7, 8], block_digest([1, 2, 3, 4]))   # chained
    t = seq([1, 2, 3, 4, 5, 6, 7, 8, 7])           # a later request finds both sealed blocks
    pool.admit(t)
    assert t.num_cached_tokens == 8 and t.block_table[:2] == s.block_table[:2]


def engine_config(blocks, **kw):
    return EngineConfig(model=ModelConfig(), num_kvcache_blocks=blocks, kvcache_block_size=BS, **kw)


def test_planner_prefills_first_within_budgets():
    pl = BatchPlanner(engine_config(16, max_num_batched_tokens=12, max_num_seqs=8))
    for n in (5, 6, 4):
        pl.submit(seq(list(range(100 * n, 100 * n + n)), max_tokens=2, ignore_eos=True))
    p = pl.plan()
    assert p.is_prefill and [len(s) for s in p.seqs] == [5, 6] and p.fresh_tokens == 11   # + 4 would pass the budget
    assert pl.commit(p.seqs, [1, 1]) == []
    p2 = pl.plan()
    assert p2.is_prefill and [len(s) for s in p2.seqs] == [4]        # a waiting request still goes before decode
    pl.commit(p2.seqs, [1])
    p3 = pl.plan()
    assert not p3.is_prefill and len(p3.seqs) == 3
    ended = pl.commit(p3.seqs, [1, 1, 1])                            # max_tokens = 2 reached by all three
    assert len(ended) == 3 and pl.idle() and all(s.status is SequenceStatus.FINISHED for s in p3.seqs)
    assert pl.pool.num_free == 16


def test_planner_counts_only_uncached_tokens_against_the_budget():
    """The reference's rule (scheduler.py:29-38): a request starts if the tokens started so far plus its whole length
    fit the budget; what it then adds to "so far" is its length minus what the prefix cache held."""
    pl = BatchPlanner(engine_config(16, max_num_batched_tokens=20, max_num_seqs=8))
    shared = [7, 7, 7, 7, 8, 8, 8, 8]
    pl.submit(seq(shared + [1], max_tokens=4, ignore_eos=True))
    pl.submit(seq(shared + [2, 3], max_tokens=4, ignore_eos=True))   # 9 + 10 <= 20; 8 of its tokens are cached
    pl.submit(seq([5, 5, 5, 5], max_tokens=4, ignore_eos=True))      # (9 + 2) + 4 <= 20 although 9 + 10 + 4 > 20
    pl.submit(seq([6] * 6, max_tokens=4, ignore_eos=True))           # (9 + 2 + 4) + 6 > 20: waits
    p = pl.plan()
    assert [len(s) for s in p.seqs] == [9, 10, 4] and p.seqs[1].num_cached_tokens == 8 and p.fresh_tokens == 15
    assert len(pl.waiting) == 1


def test_planner_sequence_budget_and_decode_cap():
    pl = BatchPlanner(engine_config(16, max_num_batched_tokens=64, max_num_seqs=2))
    for i in range(3):
        pl.submit(seq([10 * i + 1, 10 * i + 2], max_tokens=3, ignore_eos=True))
    p = pl.plan()
    assert p.is_prefill and len(p.seqs) == 2
    pl.commit(p.seqs, [0, 0])
    p = pl.plan()
    assert p.is_prefill and len(p.seqs) == 1
    pl.commit(p.seqs, [0])
    p = pl.plan()
    assert not p.is_prefill and p.seqs == pl.running[:2]             # the oldest two; the third waits its turn


def test_planner_preempts_the_youngest_when_blocks_run_out():
    pl = BatchPlanner(engine_config(4, max_num_batched_tokens=64, max_num_seqs=8))
    a, b = seq([1, 2, 3, 4, 5, 6, 7], max_tokens=8, ignore_eos=True), seq([9, 8, 7, 6, 5, 4, 3], max_tokens=8, ignore_eos=True)
    pl.submit(a)
    pl.submit(b)
    p = pl.plan()
    assert p.is_prefill and len(p.seqs) == 2 and pl.pool.num_free == 0           # 2 + 2 blocks: cache full
    pl.commit(p.seqs, [50, 60])                    # both now hold 8 tokens = 2 full blocks
    p = pl.plan()
    assert not p.is_prefill and len(p.seqs) == 2   # token 8 still fits the second block
    pl.commit(p.seqs, [51, 61])                    # 9 tokens each: the next step needs a third block each
    p = pl.plan()
    assert not p.is_prefill and p.seqs == [a]      # b, the youngest, was preempted to make room
    assert pl.num_preemptions == 1 and b.status is SequenceStatus.WAITING and pl.waiting[0] is b and b.block_table == []
    assert b.token_ids[-2:] == [60, 61]            # it keeps its completion and is prefilled again with it
    assert pl.running == [a]


def test_a_lone_request_that_cannot_grow_gives_way_itself():
    pl = BatchPlanner(engine_config(2, max_num_batched_tokens=64, max_num_seqs=8))
    a = seq([1, 2, 3, 4, 5, 6, 7, 8], max_tokens=8, ignore_eos=True)
    pl.submit(a)
    pl.commit(pl.plan().seqs, [9])                 # nine tokens in a pool of two blocks
    with pytest.raises(RuntimeError, match="cannot hold"):
        pl.plan()
    assert pl.num_preemptions == 1 and pl.waiting[0] is a and pl.pool.num_free == 2


def test_eos_and_length_limits_finish_a_request():
    pl = BatchPlanner(engine_config(8, eos=2))
    s1, s2, s3 = seq([5, 5], max_tokens=10), seq([6, 6], max_tokens=10, ignore_eos=True), seq([7, 7], max_tokens=1)
    for s in (s1, s2, s3):
        pl.submit(s)
    p = pl.plan()
    ended = pl.commit(p.seqs, [2, 2, 9])
    assert s1.is_finished and not s2.is_finished and s3.is_finished and ended == [s1, s3] and pl.running == [s2]


class _EchoRunner:
    """Stands in for the GPU model: every sequence gets its own length as the next token."""

    def __init__(self):
        self.longest = 0

    def run(self, seqs, is_prefill, return_logits=False):
        self.longest = max([self.longest] + [len(s) for s in seqs])
        return [len(s) for s in seqs]


def test_engine_ends_every_request_at_max_model_len():
    """No request grows past the positions the model has, whatever max_tokens asks for: the rotary table of the GPU
    model is indexed by position, so the limit is enforced on the host."""
    runner = _EchoRunner()
    eng = LLMEngine(ModelConfig(max_position_embeddings=24), model_runner=runner, num_kvcache_blocks=32,
                    kvcache_block_size=BS, max_model_len=4096, max_num_seqs=4, max_num_batched_tokens=64)
    assert eng.config.max_model_len == 24
    prompts = [list(range(20)), list(range(5)), list(range(23))]
    outs = eng.generate(prompts, [SamplingParams(max_tokens=30, ignore_eos=True), SamplingParams(max_tokens=3, ignore_eos=True),
                                  SamplingParams(max_tokens=30, ignore_eos=True, max_total_tokens=1000)])
    assert [len(o["token_ids"]) for o in outs] == [4, 3, 1]            # 20 + 4 = 24, 5 + 3, 23 + 1 = 24
    assert runner.longest == 23                                          # the model never saw position 24
    assert outs[0]["token_ids"] == [20, 21, 22, 23]
    assert eng.planner.pool.num_free == 32
    with pytest.raises(ValueError, match="max_model_len"):
        eng.add_request(list(range(24)), SamplingParams())
    with pytest.raises(TypeError):
        eng.add_request("text", SamplingParams())
