"""The cache manager on the CPU: no page lost, held twice or freed twice,
under random orders of requests; windows give pages back; slots."""
import random

import pytest

from pytriton_llama_amd.cache import RELEASED, CacheManager, OutOfPages, OutOfSlots, PagePool
from pytriton_llama_amd.parts import StateSpec, paged_kv_spec

FULL = paged_kv_spec(2, 16)
WIN = paged_kv_spec(2, 16, window=10)


def test_nine_pages_like_the_reference_scenarios():
    """The 9-block scenarios of the reference's tests/test_mem_manager.py:26-183
    (alloc 3; alloc 10 fails and leaves the state; release then alloc again;
    free everything), on pages."""
    m = CacheManager([FULL], page_size=1, num_pages=9, max_num_seqs=4)
    m.admit("a")
    m.append("a", 3)
    assert m.paged[0].pool.num_free == 6 and len(m.block_table("a", 0)) == 3
    m.admit("b")
    assert not m.can_append("b", 10)
    with pytest.raises(OutOfPages):
        m.append("b", 10)
    assert m.paged[0].pool.num_free == 6 and m.num_tokens["b"] == 0   # nothing was taken
    m.append("b", 4)
    held = set(m.block_table("a", 0))
    m.free("a")
    assert m.paged[0].pool.num_free == 5
    m.admit("c")
    m.append("c", 3)
    assert set(m.block_table("c", 0)) == held                           # freed pages are used again
    m.free("b")
    m.free("c")
    assert m.paged[0].pool.num_free == 9
    m.check()


def test_pages_grow_with_tokens_and_slots_address_them():
    m = CacheManager([FULL, FULL], page_size=4, num_pages=5, max_num_seqs=2)
    assert len(m.paged) == 1 and m.paged[0].layers == [0, 1]        # same needs: one group
    m.admit("a")
    assert m.append("a", 5) == 0
    assert m.pages_needed("a", 3) == [0] and m.pages_needed("a", 4) == [1]
    assert m.append("a", 3) == 5
    t = m.block_table("a", 0)
    assert len(t) == 2
    assert m.slots("a", 0, 3, 3) == [t[0] * 4 + 3, t[1] * 4 + 0, t[1] * 4 + 1]


def test_double_free_and_unknown_requests_raise():
    m = CacheManager([FULL], 4, 4, 2)
    m.admit("a")
    m.append("a", 4)
    m.free("a")
    with pytest.raises(RuntimeError):
        m.free("a")
    with pytest.raises(RuntimeError):
        m.append("zz", 1)
    pool = PagePool(3)
    p = pool.take(2)
    pool.give_back(p)
    with pytest.raises(RuntimeError):
        pool.give_back(p[:1])


def test_state_slots():
    m = CacheManager([FULL, StateSpec((3, 5)), None], 4, 4, max_num_seqs=2)
    assert m.layer_home == [("paged", 0, 0), ("state", 0, 0), None]
    s = {m.admit("a"), m.admit("b")}
    assert s == {0, 1} and m.num_free_slots == 0
    with pytest.raises(OutOfSlots):
        m.admit("c")
    with pytest.raises(RuntimeError):
        m.admit("a")
    sa = m.slot_of["a"]
    m.free("a")
    assert m.admit("c") == sa
    m.check()


def test_groups_with_different_needs_have_their_own_pages():
    m = CacheManager([FULL, WIN, FULL, WIN], page_size=4, num_pages=[8, 4], max_num_seqs=2)
    assert [g.layers for g in m.paged] == [[0, 2], [1, 3]]
    m.admit("a")
    m.append("a", 16)                       # 4 pages in both groups
    assert [g.pool.num_free for g in m.paged] == [4, 0]
    assert m.release_behind_window("a") == 1
    # a query at position 16 reads keys 7..16: page 0 (keys 0-3) is dead, page 1 (4-7) still holds key 7
    assert m.block_table("a", 1)[0] == RELEASED and m.block_table("a", 1)[1] >= 0
    assert [g.pool.num_free for g in m.paged] == [4, 1]
    assert m.can_append("a", 4) and not m.can_append("a", 5)
    m.append("a", 4)
    m.release_behind_window("a")
    assert m.block_table("a", 1)[:2] == [RELEASED, RELEASED]
    with pytest.raises(RuntimeError):
        m.slots("a", 1, 0, 1)
    m.check()
    m.free("a")
    assert [g.pool.num_free for g in m.paged] == [8, 4]


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_the_books(seed):
    rng = random.Random(seed)
    m = CacheManager([FULL, WIN, StateSpec((2,))], page_size=rng.choice([1, 4, 16]),
                     num_pages=[rng.randint(6, 30), rng.randint(6, 30)], max_num_seqs=5)
    live, n = {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.num_free_slots:
            rid = f"r{n}"
            n += 1
            m.admit(rid)
            live[rid] = 0
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            k = rng.randint(1, 20)
            before = [g.pool.num_free for g in m.paged]
            if m.can_append(rid, k):
                assert m.append(rid, k) == live[rid]
                live[rid] += k
                m.release_behind_window(rid)
            else:
                with pytest.raises(OutOfPages):
                    m.append(rid, k)
                assert [g.pool.num_free for g in m.paged] == before
        elif live:
            rid = rng.choice(list(live))
            m.free(rid)
            del live[rid]
        m.check()
        for rid, cnt in live.items():
            assert m.num_tokens[rid] == cnt
            full, win = m.block_table(rid, 0), m.block_table(rid, 1)
            assert len(full) == -(-cnt // m.page_size) and all(p >= 0 for p in full)
            first = max(0, cnt - 10 + 1) // m.page_size
            assert all((p == RELEASED) == (i < first) for i, p in enumerate(win))
    for rid in list(live):
        m.free(rid)
    m.check()
    assert all(g.pool.num_free == g.pool.num_pages for g in m.paged) and m.num_free_slots == 5


def test_cache_sizing_counts_the_fixed_state():
    """The state pools come out of the memory before the pages do."""
    import torch
    from pytriton_llama_amd.cache import CacheStorage
    from pytriton_llama_amd.engine.llm import pages_that_fit
    from pytriton_llama_amd.parts import StateSpec, paged_kv_spec
    layers = [paged_kv_spec(2, 16), StateSpec((1000,), torch.float32), StateSpec((1000,), torch.float32),
              paged_kv_spec(2, 16), StateSpec((8, 8), None)]
    m = CacheManager(layers, 16, 4, 10)
    assert m.padding_slot == 10 and m.padding_slot not in m._free_slots
    per_page = CacheStorage.bytes_per_page(m, torch.bfloat16)
    assert per_page == 2 * 2 * 2 * 16 * 16 * 2
    fixed = CacheStorage.state_bytes(m, torch.bfloat16)
    assert fixed == 2 * 11 * 1000 * 4 + 1 * 11 * 64 * 2          # every slot and the padding slot
    assert pages_that_fit(fixed + 10 * per_page + 5, per_page, fixed, 1000) == 10
    assert pages_that_fit(fixed + 10 * per_page + 5, per_page, 0, 1000) > 10
    assert pages_that_fit(10 ** 9, per_page, fixed, 7) == 7
    with pytest.raises(RuntimeError, match="fixed-size state"):
        pages_that_fit(fixed - 1, per_page, fixed, 1000)
    with pytest.raises(RuntimeError, match="no memory left"):
        pages_that_fit(fixed + per_page - 1, per_page, fixed, 1000)
    assert pages_that_fit(fixed, 0, fixed, 1000) == 1            # a model without paged layers


def test_decode_copies_are_left_out_when_they_would_not_leave_room_for_the_cache(capsys, monkeypatch):
    """The second copies of the weights take what the matrices take once more, plus the largest
    of them while it is built; they are made only if the cache's floor stays free."""
    import torch
    import pytriton_llama_amd  # noqa: F401
    from pytriton_llama_amd.config import EngineConfig, build_model
    from pytriton_llama_amd.engine import llm
    from tiny_configs import TINY_B
    assert llm.decode_copies_fit(100, 30, 200, 70) and not llm.decode_copies_fit(100, 30, 200, 71)
    model = build_model(TINY_B)
    model.dtype = torch.float32
    assert model.decode_copy_bytes() == (0, 0)                    # the decode kernels copy bfloat16 only
    model.dtype = torch.bfloat16
    copies, largest = model.decode_copy_bytes()
    H, I, V, L = 128, 320, 384, 3
    per_layer = (4 + 2 * 1) * 32 * H + H * 4 * 32 + 3 * I * H
    assert copies == 2 * (L * per_layer + 2 * V * H) and largest == 2 * max(V * H, I * H)
    made = []
    monkeypatch.setattr(model, "make_decode_copies", lambda: made.append(1) or 0)
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (copies + largest + 999, 10 ** 9))
    assert not llm.make_decode_copies_if_room(model, "cuda:0", 1000) and not made
    assert "decode_weight_copies=False" in capsys.readouterr().err
    assert llm.make_decode_copies_if_room(model, "cuda:0", 999) and made == [1]
    # what the cache must get at least, and what recorded steps are allowed
    ec = EngineConfig(dtype="bfloat16", page_size=16, max_model_len=64, max_num_seqs=4, use_graphs=False)
    per_page = 2 * L * 1 * 16 * 32 * 2
    assert llm.cache_floor_bytes(model, ec) == 4 * per_page
    ec.num_pages = 9
    assert llm.cache_floor_bytes(model, ec) == 9 * per_page
    ec.use_graphs = True
    rows = (4 + 2) * 32 + H + 2 * I + H                                  # q|k|v, o, gate|up, down
    assert model.widest_step_row_bytes() == 2 * rows * 2
    pool = llm.graph_pool_bytes(model, ec)
    assert pool == (2048 + 4) * 2 * rows * 2 + 5 * V * 4
    assert llm.cache_floor_bytes(model, ec) == 9 * per_page + pool


def test_paged_specs_name_their_tensors():
    """A paged layer keeps whatever tensors its spec names: keys and values, or one latent tensor
    a token with a dtype of its own. Equal specs share a group, the storage makes a pool for
    every tensor of a group, and a page costs what its tensors take."""
    import torch
    from pytriton_llama_amd.cache import CacheStorage
    from pytriton_llama_amd.parts import PagedSpec, PagedTensor
    latent = PagedSpec((PagedTensor("latent", (12,)), PagedTensor("gate", (3, 2), token_axis=1, dtype=torch.float32)))
    same = PagedSpec((PagedTensor("latent", (12,)), PagedTensor("gate", (3, 2), token_axis=1, dtype=torch.float32)))
    windowed = PagedSpec((PagedTensor("latent", (12,)),), window=7)
    m = CacheManager([latent, FULL, same, windowed, None], page_size=8, num_pages=[5, 6, 4], max_num_seqs=2)
    assert [len(g.layers) for g in m.paged] == [2, 1, 1]
    assert m.layer_home == [("paged", 0, 0), ("paged", 1, 0), ("paged", 0, 1), ("paged", 2, 0), None]
    s = CacheStorage(m, torch.bfloat16, "cpu")
    assert s.paged_pools[0]["latent"].shape == (2, 5, 8, 12) and s.paged_pools[0]["latent"].dtype == torch.bfloat16
    assert s.paged_pools[0]["gate"].shape == (2, 5, 3, 8, 2) and s.paged_pools[0]["gate"].dtype == torch.float32
    assert set(s.paged_pools[1]) == {"k", "v"} and s.paged_pools[1]["k"].shape == (1, 6, 2, 8, 16)
    per_page = 2 * 8 * (12 * 2 + 6 * 4) + 1 * 2 * 2 * 8 * 16 * 2 + 1 * 8 * 12 * 2
    assert CacheStorage.bytes_per_page(m, torch.bfloat16) == per_page
    view = s.view(2)
    assert view.kind == "paged" and view.group == 0 and view.latent.shape == (5, 8, 12)
    assert view.tensors["gate"].data_ptr() == s.paged_pools[0]["gate"][1].data_ptr()
    with pytest.raises(AttributeError, match="keeps no tensor"):
        view.k
    kv = s.view(1)
    assert kv.k.shape == (6, 2, 8, 16) and kv.v.shape == kv.k.shape
    with pytest.raises(ValueError, match="names of their own"):
        PagedSpec((PagedTensor("a", (2,)), PagedTensor("a", (3,))))
    with pytest.raises(ValueError):
        PagedTensor("x", (2,), token_axis=3).page_shape(4)
    with pytest.raises(TypeError, match="unknown cache spec"):
        CacheManager([("k", 2, 16)], 8, 4, 2)
