"""The layout of a step's batch on the host (no GPU): entries in kernel order, slots, block
tables, work lists, token checks. Runs build_context with the device "cpu"."""
import random

import numpy as np
import pytest
import torch

from pytriton_llama_amd.cache.manager import CacheManager, OutOfPages
from pytriton_llama_amd.engine.batch import StepEntry, build_context, take_pages, work_items
from pytriton_llama_amd.engine.request import Request, SamplingParams
from pytriton_llama_amd.parts.base import WorkList, paged_kv_spec

FULL = paged_kv_spec(2, 16)
WIN = paged_kv_spec(2, 16, window=100)      # a second group of pages; nothing here passes its window


def _manager(page_size=4, num_pages=64, seqs=8):
    return CacheManager([FULL, WIN], page_size=page_size, num_pages=num_pages, max_num_seqs=seqs)


def test_work_items_cover_every_block_once_longest_first():
    rng = random.Random(3)
    for _ in range(50):
        n = rng.randint(1, 5)
        q_lens = [rng.randint(1, 300) for _ in range(n)]
        ctx_lens = [q + rng.randint(0, 200) for q in q_lens]
        first = rng.randint(0, n - 1)
        rows = rng.choice([16, 64, 128])
        ws, wo = work_items(q_lens, ctx_lens, first, rows)
        assert ws.dtype == np.int32 and wo.dtype == np.int32
        want = {(s, off) for s in range(first, n) for off in range(0, q_lens[s], rows)}
        assert set(zip(ws.tolist(), wo.tolist())) == want and len(ws) == len(want)
        keys = [ctx_lens[s] - q_lens[s] + min(off + rows, q_lens[s]) for s, off in zip(ws, wo)]
        assert keys == sorted(keys, reverse=True)
    ws, wo = work_items([1, 1], [5, 9], 2, 64)          # nothing but single tokens
    assert len(ws) == 0 and len(wo) == 0


def test_context_lays_single_tokens_first_and_lists_rows_in_the_callers_order():
    m = _manager()
    for r in "abc":
        m.admit(r)
    m.append("b", 6)                                    # b has six tokens in the cache already
    entries = [StepEntry("a", [5, 6, 7, 8, 9], [4, 0]), StepEntry("b", [3], [0]),
               StepEntry("c", np.asarray([1, 2], dtype=np.int32), [])]
    lists = (WorkList(16), WorkList(64, after_decode=True), WorkList(3, after_decode=True))
    ctx, order = build_context(entries, m, "cpu", vocab_size=10, work_lists=lists)
    assert order == [1, 0, 2] and ctx.num_decode_seqs == 1
    assert ctx.token_ids.tolist() == [3, 5, 6, 7, 8, 9, 1, 2]
    assert ctx.positions.tolist() == [6, 0, 1, 2, 3, 4, 0, 1]
    assert ctx.q_start.tolist() == [0, 1, 6, 8] and ctx.ctx_len.tolist() == [7, 5, 2]
    assert ctx.logit_rows.tolist() == [5, 1, 0]         # a's places 4 and 0, then b's
    assert not ctx.logit_rows_are_identity and ctx.max_q_len == 5 and ctx.max_ctx_len == 7
    for g in range(2):
        want = m.slots("b", g, 6, 1) + m.slots("a", g, 0, 5) + m.slots("c", g, 0, 2)
        assert ctx.groups[g].slots.tolist() == want
        table = ctx.groups[g].block_table.tolist()
        assert table[0] == m.block_table("b", g) and table[1] == m.block_table("a", g)
        assert table[2] == m.block_table("c", g) + [-1]
    assert ctx.work[lists[1]][0].tolist() == [1, 2] and ctx.work[lists[1]][1].tolist() == [0, 0]
    assert ctx.work[lists[0]][0].tolist() == [0, 1, 2] and ctx.work[lists[0]][1].tolist() == [0, 0, 0]
    # blocks of three rows of the sequences behind the single token: most keys first
    assert list(zip(ctx.work[lists[2]][0].tolist(), ctx.work[lists[2]][1].tolist())) == [(1, 3), (1, 0), (2, 0)]
    assert ctx.token_ids.dtype == torch.int32


def test_slot_array_matches_the_page_table_and_refuses_what_is_not_held():
    m = _manager(page_size=4)
    m.admit("a")
    m.append("a", 11)
    table = m.block_table("a", 0)
    assert m.slots("a", 0, 2, 7) == [table[p // 4] * 4 + p % 4 for p in range(2, 9)]
    assert m.slot_array("a", 0, 10, 1).dtype == np.int32
    with pytest.raises(RuntimeError):
        m.slots("a", 0, 8, 8)                            # positions 12..15 have no page


def test_bad_entries_take_no_pages():
    m = _manager(num_pages=4)
    m.admit("a"); m.admit("b")
    free = [g.pool.num_free for g in m.paged]
    for entries, err in [([StepEntry("a", [1, 2, 99], [])], ValueError),      # token outside
                         ([StepEntry("a", [1], []), StepEntry("b", [-1], [])], ValueError),
                         ([StepEntry("a", [1, 2], [2])], ValueError),            # wanted place outside
                         ([StepEntry("a", [], [])], ValueError),
                         ([StepEntry("a", [1], []), StepEntry("a", [2], [])], ValueError),
                         ([StepEntry("a", [1] * 12, []), StepEntry("b", [1] * 8, [])], OutOfPages)]:
        with pytest.raises(err):
            build_context(entries, m, "cpu", vocab_size=50)
        assert [g.pool.num_free for g in m.paged] == free
        assert m.num_tokens["a"] == 0 and m.num_tokens["b"] == 0
    arrays = []
    assert take_pages([StepEntry("a", [4, 5, 6], [])], m, 50, arrays) == [0]
    assert arrays[0].dtype == np.int32 and arrays[0].tolist() == [4, 5, 6]


def test_request_gives_prompt_portions_as_arrays_and_the_rest_as_lists():
    r = Request("r", np.arange(10, 20), SamplingParams())
    assert isinstance(r.prompt, list) and r.prompt == list(range(10, 20))
    r.output.extend([7, 8])
    part = r.token_slice(2, 5)
    assert isinstance(part, np.ndarray) and part.dtype == np.int32 and part.tolist() == [12, 13, 14, 15, 16]
    assert r.token_slice(9, 1) == [19] and r.token_slice(10, 2) == [7, 8]
    assert r.token_slice(8, 4) == [18, 19, 7, 8]
    assert Request("s", [1, 2, 3], SamplingParams()).prompt_array.tolist() == [1, 2, 3]


def test_a_padded_layout_fills_what_the_step_leaves_with_rows_that_do_nothing():
    """The layout of a recorded step (three places for single tokens, one sequence of up to
    eight tokens): padding rows have token 0, position 0, cache slot -1, no context and the
    padding state slot; the work lists are as long as the size class can need and end in empty
    items, whose first row is not below the rows of their sequence."""
    from pytriton_llama_amd.engine.batch import SeqInput, StepLayout, StepSizes
    m = _manager(page_size=4)
    for r in "abc":
        m.admit(r)
    m.append("a", 9)
    m.append("b", 2)
    lists = (WorkList(16), WorkList(4, after_decode=True))
    sizes = StepSizes(decode_rows=3, multi_seqs=1, multi_tokens=8, table_width=6, logit_rows=4)
    lay = StepLayout(m, lists, "cpu", sizes)
    assert lay.most_work_items(lists[0], sizes) == 3 + 1 + 1 and lay.most_work_items(lists[1], sizes) == 2 + 1
    starts = [m.append("a", 1), m.append("b", 1), m.append("c", 5)]
    q_lens, ctx_lens = lay.fill([SeqInput("a", 7, starts[0]), SeqInput("b", 8, starts[1])],
                                [SeqInput("c", np.arange(20, 25, dtype=np.int32), starts[2])], [0, 1, 3 + 4])
    assert q_lens == [1, 1, 1, 5] and ctx_lens == [10, 3, 0, 5]
    lay.to_device()
    ctx = lay.context([1, 1, 1, 8], [24] * 4, False)
    assert ctx.token_ids.tolist() == [7, 8, 0] + [20, 21, 22, 23, 24] + [0, 0, 0]
    assert ctx.positions.tolist() == [9, 2, 0] + [0, 1, 2, 3, 4] + [0, 0, 0]
    assert ctx.q_start.tolist() == [0, 1, 2, 3, 8] and ctx.ctx_len.tolist() == [10, 3, 0, 5]
    assert ctx.state_slots.tolist() == [m.slot_of["a"], m.slot_of["b"], m.padding_slot, m.slot_of["c"]]
    assert ctx.logit_rows.tolist() == [0, 1, 7, 0]
    assert ctx.num_tokens == 11 and ctx.num_seqs == 4 and ctx.num_decode_seqs == 3 and ctx.max_q_len == 8
    for g in range(2):
        assert ctx.groups[g].slots.tolist() == (m.slots("a", g, 9, 1) + m.slots("b", g, 2, 1) + [-1] +
                                                m.slots("c", g, 0, 5) + [-1, -1, -1])
        table = ctx.groups[g].block_table.tolist()
        assert table[0] == m.block_table("a", g) + [-1] * 3 and table[3] == m.block_table("c", g) + [-1] * 4
    items = lambda wl: list(zip(ctx.work[wl][0].tolist(), ctx.work[wl][1].tolist()))
    # every place of a single token is a block (the padding one has no keys), then the portion
    assert items(lists[0]) == [(0, 0), (3, 0), (1, 0), (2, 0), (3, 16)]
    assert items(lists[1]) == [(3, 4), (3, 0), (3, 8)]
    for wl in lists:
        for s, off in items(wl)[-1:]:
            assert off >= q_lens[s] and off % wl.block_rows == 0          # the empty item
    # the next step of the same size class: "a" has grown by a page, "b" is gone, the portion
    # of "c" is shorter; the row of "a" is written only where it grew
    before = lay.tables_np[0][0].copy()
    starts = [m.append("a", 3), m.append("c", 2)]
    assert len(m.block_table("a", 0)) == 4
    lay.tables_np[0][0, 0] = 77                            # (would be overwritten by a full rewrite)
    lay.fill([SeqInput("a", 1, starts[0] + 2)], [SeqInput("c", np.asarray([5, 6], dtype=np.int32), starts[1])], [0])
    assert lay.tables_np[0][0].tolist() == [77] + before[1:3].tolist() + [m.block_table("a", 0)[3], -1, -1]
    assert lay.np_of["ctx_len"].tolist() == [13, 0, 0, 7] and lay.np_of["q_start"].tolist() == [0, 1, 2, 3, 5]
    assert lay.np_of["token_ids"].tolist() == [1, 0, 0, 5, 6] + [0] * 6
    assert lay.np_of["state_slots"].tolist()[1:3] == [m.padding_slot] * 2
    with pytest.raises(ValueError, match="larger than its layout"):
        lay.fill([SeqInput("a", 1, 0)] * 4, [], [])


def test_a_layout_of_single_tokens_only_writes_its_work_lists_once():
    from pytriton_llama_amd.engine.batch import SeqInput, StepLayout, StepSizes
    m = _manager(page_size=4)
    m.admit("a")
    lists = (WorkList(32), WorkList(32, after_decode=True))
    lay = StepLayout(m, lists, "cpu", StepSizes(4, 0, 0, 5, 4))
    lay.fill([SeqInput("a", 3, m.append("a", 1))], [], range(4))
    lay.to_device()
    ctx = lay.context([1] * 4, [20] * 4, True)
    assert sorted(ctx.work[lists[0]][0].tolist()) == [0, 1, 2, 3] and ctx.work[lists[0]][1].tolist() == [0] * 4
    assert ctx.work[lists[1]][0].numel() == 0 and lay.static_work
    assert ctx.logit_rows.tolist() == [0, 1, 2, 3] and ctx.logit_rows_are_identity
