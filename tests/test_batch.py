"""The layout of a step's batch on the host (no GPU): entries in kernel order, slots, block
tables, work lists, token checks. Runs build_context with the device "cpu"."""
import random

import numpy as np
import pytest
import torch

from pytriton_llama_amd.cache.manager import CacheManager, OutOfPages
from pytriton_llama_amd.engine.batch import StepEntry, build_context, take_pages, work_items
from pytriton_llama_amd.engine.request import Request, SamplingParams
from pytriton_llama_amd.parts.base import PagedKVSpec

FULL = PagedKVSpec(2, 16)
WIN = PagedKVSpec(2, 16, window=100)      # a second group of pages; nothing here passes its window


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
    ctx, order = build_context(entries, m, "cpu", vocab_size=10)
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
    assert ctx.work["multi64"][0].tolist() == [1, 2] and ctx.work["multi64"][1].tolist() == [0, 0]
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
