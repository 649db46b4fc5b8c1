"""Host layout layer: Sequence, BlockManager, Scheduler, Context.

The first block restates the reference's own CPU tests
(nano-vdllm/tests/test_sequence_spans.py, tests/test_model_runner_acache.py:26-61)
against this package's classes; the rest checks the vectorised slot-map builder
against the oracle's per-token restatement on random layouts.
"""
import random

import pytest

from acache_amd import BlockManager, Config, Scheduler, Sequence
from acache_amd.utils import get_context, reset_context, set_context
from oracle import acache_oracle as O


def _allocate_fake_blocks(seq, first_block=2):
    seq.block_table = list(range(first_block, first_block + seq.num_cache_blocks))


@pytest.mark.parametrize(
    ("tokens", "affix_start", "affix_end", "generation_start"),
    [
        ([10, 11, 12], 0, 2, None),
        ([10, 20, 21, 11], 1, 3, None),
        ([10, 99, 99, 20, 21], 3, 5, 1),
    ],
)
def test_affix_layout_maps_shared_and_private_slots(tokens, affix_start, affix_end, generation_start):
    seq = Sequence(tokens, gen_length=2, block_length=2, cache_block_size=4, mask_id=99,
                   prompt_affix_start=affix_start, prompt_affix_end=affix_end,
                   generation_start=generation_start)
    seq.enable_acache(anchor_ratio=0.5)
    anchor = affix_end - 1
    seq.set_anchor_positions([anchor])
    _allocate_fake_blocks(seq)
    seq.finalize_slot_mapping(shared_slot_offset=0)

    assert seq.recompute_positions == sorted([anchor] + seq.non_affix_positions)
    assert seq.read_slot_map[affix_start] == 0
    assert seq.read_slot_map[anchor] != anchor - affix_start
    assert all(slot >= 0 for slot in seq.read_slot_map)
    assert seq.block_query_start() == seq.recompute_positions.index(seq.generation_start)


def test_suffix_layout_generates_inside_prompt_and_preserves_right_context():
    seq = Sequence([10, 50, 51, 20, 21], gen_length=2, block_length=2, mask_id=99,
                   prompt_affix_start=3, prompt_affix_end=5, generation_start=1)
    assert seq.token_ids == [10, 99, 99, 20, 21]
    assert seq.generated_token_ids == [99, 99]
    assert seq.prompt_affix_token_ids == [20, 21]


def test_generation_and_affix_spans_must_not_overlap():
    with pytest.raises(ValueError, match="must not overlap"):
        Sequence([10, 11, 12, 13], gen_length=2, mask_id=99, prompt_affix_start=1,
                 prompt_affix_end=3, generation_start=2)


def test_span_errors():
    with pytest.raises(ValueError, match="Infill generation span"):
        Sequence([1, 2, 3], gen_length=4, generation_start=1)
    with pytest.raises(ValueError, match="Affix span must be contained"):
        Sequence([1, 2, 3], gen_length=1, prompt_affix_start=2, prompt_affix_end=9)
    seq = Sequence([1, 2, 3], gen_length=1)
    with pytest.raises(ValueError, match="ACache affix span"):
        seq.enable_acache(affix_start=1, affix_end=99)


def test_relocation_workspace_blocks_can_be_released():
    manager = BlockManager(num_blocks=8, cache_block_size=4)
    manager.reserve_prefix(5)
    manager.release_prefix_tail(2)
    assert manager.reserved_block_ids == {0, 1}
    assert manager.used_block_ids == {0, 1}
    assert set(manager.free_block_ids) == set(range(2, 8))


def test_block_manager_fifo_order_and_exhaustion():
    bm = BlockManager(num_blocks=6, cache_block_size=4)
    bm.reserve_prefix(2)
    a = Sequence(list(range(6)), gen_length=2, cache_block_size=4)      # 8 tokens -> 2 blocks
    b = Sequence(list(range(6)), gen_length=2, cache_block_size=4)
    c = Sequence(list(range(6)), gen_length=2, cache_block_size=4)
    bm.allocate(a)
    bm.allocate(b)
    assert a.block_table == [2, 3] and b.block_table == [4, 5]
    assert not bm.can_allocate(c)                       # block exhaustion -> admission stops
    bm.deallocate(a)
    assert a.block_table == [] and list(bm.free_block_ids) == [3, 2]    # returned in reverse order
    assert bm.can_allocate(c)
    bm.allocate(c)
    assert c.block_table == [3, 2]
    assert not bm.is_free(3) and bm.num_free_blocks == 0
    with pytest.raises(AssertionError):
        bm.allocate(c)                                  # a sequence that already owns blocks
    d = Sequence(list(range(6)), gen_length=2, cache_block_size=4)
    with pytest.raises(IndexError):
        bm.allocate(d)                                  # empty pool, as the reference's free_block_ids[0]
    assert d.block_table == []


def test_anchor_budget_and_private_slot_accounting():
    seq = Sequence(list(range(100)), gen_length=28, cache_block_size=16, prompt_affix_start=10, prompt_affix_end=90)
    assert seq.num_private_slots == 128 and seq.num_cache_blocks == 8
    seq.enable_acache(anchor_ratio=0.07)
    assert seq.affix_len == 80 and seq.num_anchor_tokens == O.anchor_budget(0.07, 80) == 6
    assert seq.num_private_slots == 6 + 128 - 80
    assert seq.num_cache_blocks == 4 and seq.last_cache_block_num_tokens == 6
    seq.enable_acache(anchor_ratio=1.0)
    assert seq.num_anchor_tokens == 80
    seq.enable_acache(anchor_ratio=0.0)
    assert seq.num_anchor_tokens == 0 and seq.acache_enabled


def test_vectorised_slot_maps_equal_per_token_restatement_on_random_layouts():
    rng = random.Random(0)
    for _ in range(200):
        bs = rng.choice([4, 8, 16, 256])
        A = rng.randint(1, 60)
        head = rng.randint(0, 20)
        tail = rng.randint(0, 20)
        gen = rng.randint(1, 12)
        placement = rng.choice(["prefix", "infix", "suffix"])
        if placement == "prefix":
            tokens = list(range(A + tail))
            kw = dict(prompt_affix_start=0, prompt_affix_end=A)
        elif placement == "infix":
            tokens = list(range(head + A + tail))
            kw = dict(prompt_affix_start=head, prompt_affix_end=head + A)
        else:  # generation window inside the prompt, affix after it
            tokens = list(range(head + gen + A))
            kw = dict(prompt_affix_start=head + gen, prompt_affix_end=head + gen + A, generation_start=head)
        seq = Sequence(tokens, gen_length=gen, block_length=4, cache_block_size=bs, mask_id=-7, **kw)
        ratio = rng.choice([0.0, 0.07, 0.2, 0.5, 1.0])
        seq.enable_acache(anchor_ratio=ratio)
        K = seq.num_anchor_tokens
        anchors = sorted(rng.sample(range(seq.affix_start, seq.affix_end), K))
        seq.set_anchor_positions(anchors)
        pool = list(range(3, 3 + seq.num_cache_blocks + 5))
        rng.shuffle(pool)
        seq.block_table = pool[: seq.num_cache_blocks]
        off = rng.choice([0, 0, 1000])
        seq.finalize_slot_mapping(shared_slot_offset=off)
        read, rpos, rslots = O.finalize_slot_mapping(len(seq), seq.affix_start, seq.affix_end, anchors,
                                                     seq.block_table, bs, off)
        assert seq.read_slot_map == read
        assert seq.recompute_positions == rpos
        assert seq.recompute_slot_mapping == rslots
        assert len(set(rslots)) == len(rslots)                    # every recomputed position owns one slot
        assert seq.private_slots().tolist() == O.private_slots(seq.block_table, seq.num_private_slots, bs)


def test_disabled_acache_layout_is_identity_over_private_slots():
    seq = Sequence([1, 2, 3, 4, 5], gen_length=3, cache_block_size=4)
    seq.block_table = [7, 2]
    seq.finalize_slot_mapping()
    assert seq.read_slot_map == [28, 29, 30, 31, 8, 9, 10, 11]
    assert seq.recompute_slot_mapping == seq.read_slot_map
    assert seq.recompute_positions == list(range(8))


def test_context_positional_order_matches_reference_callers():
    # model_runner.py:1380-1393 passes twelve positionals in this order
    set_context(True, "cq", "ck", "sl", 5, 9, "sm", None, True, "rsm", "skl", "sh")
    ctx = get_context()
    assert (ctx.is_caching, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.seqlens, ctx.max_seqlen_q,
            ctx.max_seqlen_k, ctx.slot_mapping, ctx.block_tables, ctx.use_acache, ctx.read_slot_mapping,
            ctx.shared_kv_lens, ctx.affix_shifts) == (True, "cq", "ck", "sl", 5, 9, "sm", None, True, "rsm", "skl", "sh")
    reset_context()
    assert get_context().use_acache is False and get_context().slot_mapping is None


def test_scheduler_admits_until_blocks_run_out():
    cfg = Config(max_num_seqs=0, num_kvcache_blocks=3, cache_block_size=4, max_num_batched_tokens=64)
    sched = Scheduler(cfg)
    seqs = [Sequence(list(range(6)), gen_length=2, cache_block_size=4) for _ in range(2)]
    for s in seqs:
        sched.add(s)
    admitted, is_new = sched.schedule()
    assert is_new and admitted == [seqs[0]] and len(sched.waiting) == 1
    running, is_new = sched.schedule()
    assert not is_new and running == [seqs[0]]
    sched.postprocess([seqs[0]], [True])
    assert seqs[0].is_finished and not sched.running
    admitted, is_new = sched.schedule()
    assert is_new and admitted == [seqs[1]]
    sched.preempt(seqs[1])
    assert list(sched.waiting) == [seqs[1]] and not sched.is_finished()
