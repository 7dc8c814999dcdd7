"""Host logic of the end-to-end harness (no GPU): sequences, the prefix-caching block manager and the scheduler, with
the behaviours the reference's engine has (electrock_infer/engine/block_manager.py:56-120, scheduler.py:24-74)."""
import numpy as np
import pytest
import xxhash

from electrock_infer_amd.harness.block_manager import BlockManager
from electrock_infer_amd.harness.config import EngineConfig, ModelConfig, SamplingParams
from electrock_infer_amd.harness.scheduler import Scheduler
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


def test_block_hash_is_xxh64_chained_over_int64_tokens():
    # the definition written out: xxh64(prefix hash as 8 little-endian bytes ++ token ids as int64)
    first = xxhash.xxh64(np.array([1, 2, 3, 4], dtype=np.int64).tobytes()).intdigest()
    assert BlockManager.compute_hash([1, 2, 3, 4]) == first
    h = xxhash.xxh64()
    h.update(first.to_bytes(8, "little"))
    h.update(np.array([5, 6, 7, 8], dtype=np.int64).tobytes())
    assert BlockManager.compute_hash([5, 6, 7, 8], first) == h.intdigest()
    assert BlockManager.compute_hash([5, 6, 7, 8], first) != BlockManager.compute_hash([5, 6, 7, 8])


def test_prefix_blocks_are_shared_and_survive_a_free():
    bm = BlockManager(8, BS)
    a = seq([1, 2, 3, 4, 5, 6, 7, 8, 9])          # two full blocks + one token
    bm.allocate(a)
    assert a.num_cached_tokens == 0 and len(a.block_table) == 3 and len(bm.free_block_ids) == 5
    b = seq([1, 2, 3, 4, 5, 6, 7, 8, 20, 21])     # same two leading blocks
    bm.allocate(b)
    assert b.num_cached_tokens == 8 and b.block_table[:2] == a.block_table[:2] and b.block_table[2] != a.block_table[2]
    assert bm.blocks[a.block_table[0]].ref_count == 2 and len(bm.free_block_ids) == 4
    c = seq([1, 2, 3, 4, 9, 9, 9, 9])             # first block shared, second differs: everything behind is new
    bm.allocate(c)
    assert c.num_cached_tokens == 4 and c.block_table[0] == a.block_table[0] and c.block_table[1] not in a.block_table
    shared = a.block_table[:2]
    for s in (a, b, c):
        bm.deallocate(s)
        assert s.block_table == [] and s.num_cached_tokens == 0
    assert len(bm.free_block_ids) == 8 and not bm.used_block_ids
    d = seq([1, 2, 3, 4, 5, 6, 7, 8, 30])         # freed blocks keep their hash: picked up again
    bm.allocate(d)
    assert d.num_cached_tokens == 8 and d.block_table[:2] == shared


def test_decode_appends_open_and_seal_blocks():
    bm = BlockManager(4, BS)
    s = seq([1, 2, 3])
    bm.allocate(s)
    assert bm.blocks[s.block_table[0]].hash == -1
    s.append_token(4)                              # block complete: gets its hash
    assert bm.can_append(s)
    bm.may_append(s)
    assert bm.blocks[s.block_table[0]].hash == BlockManager.compute_hash([1, 2, 3, 4]) and len(s.block_table) == 1
    s.append_token(5)                              # opens a second block
    bm.may_append(s)
    assert len(s.block_table) == 2
    t = seq([1, 2, 3, 4, 7])                       # a later request finds the sealed block
    bm.allocate(t)
    assert t.num_cached_tokens == 4 and t.block_table[0] == s.block_table[0]


def engine_config(blocks, **kw):
    return EngineConfig(model=ModelConfig(), num_kvcache_blocks=blocks, kvcache_block_size=BS, **kw)


def test_scheduler_prefills_first_within_budgets():
    sch = Scheduler(engine_config(16, max_num_batched_tokens=12, max_num_seqs=8))
    for n in (5, 6, 4):
        sch.add(seq(list(range(100 * n, 100 * n + n)), max_tokens=2, ignore_eos=True))
    batch, is_prefill = sch.schedule()
    assert is_prefill and [len(s) for s in batch] == [5, 6]          # 5 + 6 + 4 would pass the token budget
    sch.postprocess(batch, [1, 1])
    batch2, is_prefill2 = sch.schedule()
    assert is_prefill2 and [len(s) for s in batch2] == [4]           # a waiting request still goes before decode
    sch.postprocess(batch2, [1])
    batch3, is_prefill3 = sch.schedule()
    assert not is_prefill3 and len(batch3) == 3
    sch.postprocess(batch3, [1, 1, 1])                               # max_tokens = 2 reached by all three
    assert sch.is_finished() and all(s.status is SequenceStatus.FINISHED for s in batch3)
    assert len(sch.block_manager.free_block_ids) == 16


def test_scheduler_preempts_the_youngest_when_blocks_run_out():
    sch = Scheduler(engine_config(4, max_num_batched_tokens=64, max_num_seqs=8))
    a, b = seq([1, 2, 3, 4, 5, 6, 7], max_tokens=8, ignore_eos=True), seq([9, 8, 7, 6, 5, 4, 3], max_tokens=8, ignore_eos=True)
    sch.add(a)
    sch.add(b)
    batch, is_prefill = sch.schedule()
    assert is_prefill and len(batch) == 2 and not sch.block_manager.free_block_ids     # 2 + 2 blocks: cache full
    sch.postprocess(batch, [50, 60])               # both now hold 8 tokens = 2 full blocks
    batch, is_prefill = sch.schedule()
    assert not is_prefill and len(batch) == 2      # token 8 still fits the second block
    sch.postprocess(batch, [51, 61])               # 9 tokens each: the next step needs a third block each
    batch, is_prefill = sch.schedule()
    assert not is_prefill and batch == [a]         # b, the youngest, was preempted to make room
    assert sch.num_preemptions == 1 and b.status is SequenceStatus.WAITING and sch.waiting[0] is b and b.block_table == []
    assert b.token_ids[-2:] == [60, 61]            # it keeps its completion and is prefilled again with it


def test_eos_and_length_limits_finish_a_request():
    sch = Scheduler(engine_config(8, eos=2))
    s1, s2, s3 = seq([5, 5], max_tokens=10), seq([6, 6], max_tokens=10, ignore_eos=True), seq([7, 7], max_tokens=1)
    for s in (s1, s2, s3):
        sch.add(s)
    batch, _ = sch.schedule()
    sch.postprocess(batch, [2, 2, 9])
    assert s1.is_finished and not s2.is_finished and s3.is_finished
