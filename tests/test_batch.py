"""The batch builder on the CPU: the exact arrays of the reference's
tests/test_continuous_batching.py:27-39, padding, and what is refused."""

from __future__ import annotations

import pytest
import torch

from kvforge_amd.cache import CacheGroup, CacheManager
from kvforge_amd.engine.batch import (DecodeShape, MetaBuffers, Step, StepEntry, Workspace, extend_tables,
                                      fill_step)


def setup(num_blocks=16, bs=4, groups=None):
    groups = groups or [CacheGroup((0,))]
    cache = CacheManager(bs, groups, num_blocks)
    meta = MetaBuffers(64, 8, [8] * len(groups), "cpu")
    step = Step()
    step.ws, step.device = Workspace("cpu"), "cpu"
    return cache, meta, step


def test_flat_varlen_batch_reference_vector():
    cache, meta, step = setup()
    cache.allocate("a", 6)
    cache.allocate("b", 2)
    counts = fill_step(step, meta, [StepEntry("a", [1, 2, 3], 3, "last"), StepEntry("b", [9], 1, "all")],
                       cache.block_table, lambda r: -1, 4)
    assert step.token_ids.tolist() == [1, 2, 3, 9]
    assert step.positions.tolist() == [3, 4, 5, 1]
    assert step.cu_q.tolist() == [0, 3, 4]
    assert step.ctx_lens.tolist() == [6, 2]
    assert step.logits_rows.tolist() == [2, 3] and counts == [1, 1]
    assert step.seq_of_token.tolist() == [0, 0, 0, 1]
    ta, tb = cache.block_table("a"), cache.block_table("b")
    assert step.block_tables[0][0, :2].tolist() == ta and step.block_tables[0][1, :1].tolist() == tb
    assert (step.block_tables[0][0, 2:] == -1).all()
    # a slot computed as the kernels do equals the manager's
    for tok in range(4):
        s, p = int(step.seq_of_token[tok]), int(step.positions[tok])
        slot = int(step.block_tables[0][s, p // 4]) * 4 + p % 4
        assert slot == cache.slot("ab"[s], p)
    assert step.n_decode == 1 and step.decode_seq_ids.tolist() == [1] and step.prefill_seqs == [0]
    assert step.decode_shape == DecodeShape(n=1, max_ctx=2, sum_ctx=2)
    # attention's work list for the run of 3 tokens: 3 tokens x group size over items of 16 or
    # 4 rows, one item per row, the longest walk (the last item) first
    from kvforge_amd.parts.attention import prefill_work_rows
    assert prefill_work_rows(step.q_lens, step.prefill_seqs, 2, 16) == [(0, 0, -1)]
    assert prefill_work_rows(step.q_lens, step.prefill_seqs, 6, 16) == [(0, 0, -1), (0, 1, -1)]   # both end in the last token
    assert prefill_work_rows(step.q_lens, step.prefill_seqs, 6, 4) == [(0, 3, -1), (0, 4, -1), (0, 1, -1), (0, 2, -1), (0, 0, -1)]
    # several runs: by the keys an item walks, those before its run included; equal walks stay
    # in sequence order
    q_lens = [3, 3, 1]
    assert prefill_work_rows(q_lens, [0, 1], 6, 4, start_pos=[2, 1, 9]) == \
        [(0, 3, -1), (0, 4, -1), (0, 1, -1), (0, 2, -1), (1, 3, -1), (1, 4, -1), (0, 0, -1), (1, 1, -1), (1, 2, -1), (1, 0, -1)]


def test_wanted_places_and_modes():
    cache, meta, step = setup()
    cache.allocate("a", 8)
    cache.allocate("b", 2)
    counts = fill_step(step, meta, [StepEntry("a", [5, 6, 7, 8], 0, [0, 2]),
                                    StepEntry("b", [1, 2], 0, "none")],
                       cache.block_table, lambda r: -1, 4)
    assert step.logits_rows.tolist() == [0, 2] and counts == [2, 0]
    with pytest.raises(ValueError):
        StepEntry("a", [1], 0, [1]).wanted()
    with pytest.raises(ValueError):
        StepEntry("a", [1], 0, "some").wanted()


def test_pure_decode_padding_is_inert():
    cache, meta, step = setup()
    for r in "ab":
        cache.allocate(r, 5)
    fill_step(step, meta, [StepEntry("a", [3], 4), StepEntry("b", [4], 4)], cache.block_table,
              lambda r: -1, 4, pad_to=4)
    assert step.n_seqs == 4 and step.n_tokens == 4 and step.n_decode == 4
    assert step.decode_seq_ids is None
    assert step.ctx_lens.tolist() == [5, 5, 0, 0]
    assert (step.block_tables[0][2:] == -1).all()
    # a padded batch has a fixed shape: one logits row per sequence, padding included
    assert step.decode_shape == DecodeShape(n=2, max_ctx=5, sum_ctx=10) and step.n_logits == 4
    assert step.logits_rows.tolist() == [0, 1, 2, 3]
    with pytest.raises(ValueError, match="padding"):
        fill_step(step, meta, [StepEntry("a", [3], 4, "none")], cache.block_table, lambda r: -1, 4,
                  pad_to=2)


def test_tables_carry_the_pages_of_a_run_of_decode_steps():
    """``lookahead``: the tables hold the pages of positions the device will reach by itself,
    and a table that lacks them is refused; what is owed to the stream is settled on demand."""
    cache, meta, step = setup()
    cache.allocate("a", 4)                      # one page of 4 tokens, full
    with pytest.raises(ValueError, match="pages"):
        fill_step(step, meta, [StepEntry("a", [7], 3, "last")], cache.block_table, lambda r: -1, 4,
                  pad_to=2, lookahead=3)
    assert cache.can_append_all([("a", 7)])
    cache.append_slots("a", 7, 3)               # positions 4..6 of the run
    fill_step(step, meta, [StepEntry("a", [7], 3, "last")], cache.block_table, lambda r: -1, 4,
              pad_to=2, lookahead=3)
    assert step.block_tables[0][0, :2].tolist() == cache.block_table("a")
    assert step.ctx_lens.tolist() == [4, 0]
    assert not cache.can_append_all([("a", 4 * 16 + 1)])   # more pages than the pool has
    assert step.take_owed(torch.zeros(1)) is None


def test_tables_are_extended_without_touching_the_batch():
    """``extend_tables``: a batch that is on the device keeps its tokens, positions and lengths
    (the device has moved them on by itself); only its table rows grow."""
    cache, meta, step = setup()
    cache.allocate("a", 4)
    cache.allocate("b", 2)
    entries = [StepEntry("a", [7], 3, "last"), StepEntry("b", [9], 1, "last")]
    fill_step(step, meta, entries, cache.block_table, lambda r: -1, 4, pad_to=4)
    before = meta.device_buf.clone()
    meta.view("ctx_lens", 4)[:2] += 3            # what the device did meanwhile
    meta.view("token_ids", 4)[:2] = torch.tensor([55, 66], dtype=torch.int32)
    cache.append_slots("a", 11, 3)               # two more pages for a, none for b
    extend_tables(meta, entries, 4, [11, 2], cache.block_table, 4)
    assert step.block_tables[0][0, :3].tolist() == cache.block_table("a")
    assert step.block_tables[0][1, :1].tolist() == cache.block_table("b")
    assert step.block_tables[0][2:].eq(-1).all()
    assert meta.view("ctx_lens", 4).tolist() == [7, 5, 0, 0]
    assert meta.view("token_ids", 4)[:2].tolist() == [55, 66]
    first_table = meta.table_off[0]
    untouched = torch.ones(meta.total, dtype=torch.bool)
    untouched[first_table:] = False
    untouched[meta.off["ctx_lens"]:meta.off["ctx_lens"] + 2] = False
    untouched[meta.off["token_ids"]:meta.off["token_ids"] + 2] = False
    assert torch.equal(meta.device_buf[untouched], before[untouched])
    with pytest.raises(ValueError, match="pages"):
        extend_tables(meta, entries, 4, [11, 9], cache.block_table, 4)


def test_refusals():
    cache, meta, step = setup()
    cache.allocate("a", 4)
    with pytest.raises(ValueError, match="pages"):
        fill_step(step, meta, [StepEntry("a", [1, 2], 4)], cache.block_table, lambda r: -1, 4)
    with pytest.raises(ValueError, match="capacity"):
        fill_step(step, meta, [StepEntry("a", [1] * 65, 0)], cache.block_table, lambda r: -1, 4)
    with pytest.raises(ValueError):
        fill_step(step, meta, [], cache.block_table, lambda r: -1, 4)


def test_workspace_hands_out_the_same_memory_until_it_grows():
    """Scratch tensors are asked for by name, dtype and shape at every step: the same request gives
    the same view, another shape of the same name shares its memory, and when a buffer has to
    grow the views of the old one are not handed out again (graphs that were recorded with them
    keep the old memory alive through ``snapshot``)."""
    ws = Workspace("cpu")
    a = ws.buf("x", (4, 8), torch.float32)
    assert ws.buf("x", (4, 8), torch.float32) is a
    b = ws.buf("x", (2, 8), torch.float32)
    assert b.data_ptr() == a.data_ptr() and tuple(b.shape) == (2, 8)
    other = ws.buf("x", (4, 8), torch.bfloat16)
    assert other.data_ptr() != a.data_ptr()
    kept = ws.snapshot()
    big = ws.buf("x", (16, 8), torch.float32)
    assert big.data_ptr() != a.data_ptr()
    again = ws.buf("x", (4, 8), torch.float32)
    assert again is not a and again.data_ptr() == big.data_ptr()
    assert any(t.data_ptr() == a.data_ptr() for t in kept)
    z = ws.zeros("flags", (8,), torch.int32)
    assert int(z.sum()) == 0
    ws.frozen = True
    assert ws.buf("x", (4, 8), torch.float32) is again
    with pytest.raises(RuntimeError, match="grow"):
        ws.buf("x", (64, 8), torch.float32)


def test_uneven_contexts_ask_for_cuts_of_the_key_range():
    from kvforge_amd.parts.attention import PagedAttention, skew_cuts
    assert skew_cuts(600, 32 * 600, 32) == 1                     # even contexts: none
    assert skew_cuts(1800, 1800 + 31 * 100, 32) == 1             # too short to be worth a merge
    assert skew_cuts(32768, 32768 + 31 * 600, 32) == 8           # one long context among short ones
    assert skew_cuts(8192, 8192 + 31 * 600, 32) == 4
    assert skew_cuts(8192, 8192 + 63 * 600, 64) == 4
    assert skew_cuts(4352, 4352 + 31 * 300, 32) == 4
    assert skew_cuts(3000, 3000 + 3000, 2) == 1                  # twice the mean is the aim
    assert skew_cuts(2100, 2100 + 63 * 10, 64) == 4              # never cuts below 512 keys
    assert skew_cuts(40000, 40000, 1) == 1                       # one sequence: the other rule's case
    # what a captured decode step is kept by: the cell of 512 keys the longest context (or the
    # window) lies in, and the cuts that uneven contexts ask for at the cell's lower edge
    full = PagedAttention("a", 64, 4, 2, 16, None)
    windowed = PagedAttention("a", 64, 4, 2, 16, None, window=600)
    assert full.launch_key(DecodeShape(8, 640, 8 * 600)) == (1, 1)
    assert full.launch_key(DecodeShape(8, 511, 8 * 500)) == (0, 1)
    assert full.launch_key(DecodeShape(32, 32768, 32768 + 31 * 600)) == (64, 8)
    assert windowed.launch_key(DecodeShape(32, 32768, 32768 + 31 * 600)) == (1, 1)


def test_what_a_part_sends_along_with_a_step():
    """``Step.upload_ints``: on the CPU (no staging memory to go through) the values simply
    become a tensor on the step's device; a step that was never filled does the same."""
    cache, meta, step = setup()
    assert step.upload_ints([3, 1, 4]).tolist() == [3, 1, 4]
    cache.allocate("a", 6)
    fill_step(step, meta, [StepEntry("a", [1, 2, 3], 3, "last")], cache.block_table, lambda r: -1, 4)
    got = step.upload_ints([(0, 1, -1), (0, 0, 2)])
    assert got.dtype == torch.int32 and got.tolist() == [0, 1, -1, 0, 0, 2]
    assert meta.total == meta.extra_off + meta.extra_size and meta.extra_size >= 4 * 64


def test_prefill_work_rows_hold_every_item_once_longest_walk_first():
    """Random runs, group sizes and item sizes: every item of every run longer than one token
    appears once, alone in its row, and the rows never go from a shorter walk to a longer one."""
    import random
    from kvforge_amd.parts.attention import prefill_work_rows
    rng = random.Random(5)
    for _ in range(200):
        n = rng.randint(1, 6)
        q_lens = [rng.choice([1, 1, 2, 3, 17, 64, 200, 1000]) for _ in range(n)]
        start = [rng.choice([0, 0, 5, 64, 999]) for _ in range(n)]
        seqs = [b for b in range(n) if q_lens[b] > 1]
        group, per_item = rng.choice([1, 2, 3, 4, 7, 8]), rng.choice([64, 128])
        rows = prefill_work_rows(q_lens, seqs, group, per_item, start)
        assert all(second == -1 for _, _, second in rows)
        want = sorted((b, i) for b in seqs for i in range(-(-q_lens[b] * group // per_item)))
        assert sorted((b, i) for b, i, _ in rows) == want
        ends = [start[b] + min(q_lens[b], -(-(i + 1) * per_item // group)) for b, i, _ in rows]
        assert ends == sorted(ends, reverse=True)
