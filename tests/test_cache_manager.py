"""The cache manager on the host: pages, block tables, windows, state slots (no GPU)."""

import numpy as np
import pytest
import torch

from mini_infer_amd.cache import RELEASED, CacheManager, PagePool, StateSlots
from mini_infer_amd.exceptions import OutOfMemoryError
from mini_infer_amd.parts.base import CacheNeeds, PagedKVNeeds, StateNeeds


def _needs(window=None, layers=2):
    return [CacheNeeds(pages=PagedKVNeeds(2, 16, window)) for _ in range(layers)]


def _manager(needs=None, pages=8, page_size=4, max_requests=4, storage=False):
    return CacheManager(needs or _needs(), page_size=page_size, num_pages=pages,
                        max_requests=max_requests, allocate_storage=storage)


def test_pool_allocates_unique_pages_and_notices_double_free():
    pool = PagePool(4)
    pages = [pool.allocate() for _ in range(4)]
    assert sorted(pages) == [0, 1, 2, 3] and pool.num_free == 0
    with pytest.raises(OutOfMemoryError):
        pool.allocate()
    pool.free(pages[1])
    with pytest.raises(RuntimeError, match="twice"):
        pool.free(pages[1])
    with pytest.raises(ValueError):
        pool.free(99)
    assert pool.allocate() == pages[1]  # the page freed last is used again first
    pool.check()


def test_fresh_pool_hands_out_scattered_ids_the_same_every_time():
    """Requests that grow side by side must not end up with neighbouring pages: a fresh pool's
    ids come in a scattered order, the same one for a pool size."""
    first = PagePool(256).allocate_many(256)
    assert first == PagePool(256).allocate_many(256)
    assert sorted(first) == list(range(256))
    neighbours = sum(1 for a, b in zip(first, first[1:]) if abs(a - b) == 1)
    assert neighbours < 16


def test_allocate_many_is_all_or_nothing():
    pool = PagePool(3)
    pool.allocate()
    with pytest.raises(OutOfMemoryError):
        pool.allocate_many(3)
    assert pool.num_free == 2
    assert len(pool.allocate_many(2)) == 2


def test_growth_positions_and_slot_mapping():
    m = _manager(pages=8, page_size=4)
    m.add_request("a")
    m.reserve({"a": 6})
    index = m.build_step_index([("a", 6)])
    table = m.groups[0].tables["a"]
    assert len(table) == 2
    assert index.positions.tolist() == [0, 1, 2, 3, 4, 5]
    assert index.slot_mapping[0].tolist() == [table[0] * 4 + i for i in range(4)] + [table[1] * 4, table[1] * 4 + 1]
    assert index.seq_lens.tolist() == [6] and index.cu_seqlens_q.tolist() == [0, 6]
    m.commit({"a": 6})
    # the next portion continues where the request stands, in the partly filled page first
    m.reserve({"a": 3})
    index = m.build_step_index([("a", 3)])
    table = m.groups[0].tables["a"]
    assert len(table) == 3
    assert index.positions.tolist() == [6, 7, 8]
    assert index.slot_mapping[0].tolist() == [table[1] * 4 + 2, table[1] * 4 + 3, table[2] * 4]
    assert index.max_q_len == 3 and index.max_seq_len == 9
    m.commit({"a": 3})
    assert m.length("a") == 9
    m.check()


def test_batch_index_of_several_requests():
    m = _manager(pages=16, page_size=4)
    for rid in "abc":
        m.add_request(rid)
    m.reserve({"a": 5, "b": 1, "c": 2})
    m.commit({"a": 5, "b": 1, "c": 2})
    m.reserve({"b": 1, "c": 7, "a": 1})
    index = m.build_step_index([("b", 1), ("c", 7), ("a", 1)])
    assert index.cu_seqlens_q.tolist() == [0, 1, 8, 9]
    assert index.token_request.tolist() == [0] + [1] * 7 + [2]
    assert index.positions.tolist() == [1] + list(range(2, 9)) + [5]
    assert index.seq_lens.tolist() == [2, 9, 6]
    assert index.block_tables[0].shape == (3, 3)
    assert index.block_tables[0][0, 1] == RELEASED  # padding beyond a short table
    assert index.state_slots.tolist() == [m.state_slot("b"), m.state_slot("c"), m.state_slot("a")]


def test_reserve_is_all_or_nothing():
    m = _manager(pages=4, page_size=4)
    m.add_request("a")
    m.add_request("b")
    m.reserve({"a": 8})
    m.commit({"a": 8})
    before = {rid: list(m.groups[0].tables[rid]) for rid in "ab"}
    with pytest.raises(OutOfMemoryError):
        m.reserve({"a": 1, "b": 9})  # needs 1 + 3 pages, 2 are free
    assert {rid: m.groups[0].tables[rid] for rid in "ab"} == before
    assert m.num_free_pages() == 2
    m.check()


def test_free_gives_everything_back_and_pages_are_used_again():
    m = _manager(pages=4, page_size=4)
    m.add_request("a")
    m.reserve({"a": 16})
    m.commit({"a": 16})
    used = set(m.groups[0].tables["a"])
    assert m.num_free_pages() == 0
    m.free_request("a")
    assert m.num_free_pages() == 4
    with pytest.raises(KeyError):
        m.free_request("a")
    m.add_request("b")
    m.reserve({"b": 5})
    assert set(m.groups[0].tables["b"]) <= used
    m.check()


def test_window_group_releases_pages_the_window_has_passed():
    needs = [CacheNeeds(pages=PagedKVNeeds(2, 16, None)), CacheNeeds(pages=PagedKVNeeds(2, 16, 6))]
    m = _manager(needs, pages=8, page_size=4)
    assert len(m.groups) == 2 and m.groups[1].window == 6
    m.add_request("a")
    m.reserve({"a": 13})
    m.commit({"a": 13})
    # the next query (position 13) sees keys 8..13: pages 0 and 1 of the windowed group are dead
    assert m.groups[1].tables["a"][:2] == [RELEASED, RELEASED]
    assert all(p != RELEASED for p in m.groups[1].tables["a"][2:])
    assert all(p != RELEASED for p in m.groups[0].tables["a"])
    assert m.num_free_pages(1) == 8 - 2 and m.num_free_pages(0) == 8 - 4
    # growing further writes into live pages only
    m.reserve({"a": 4})
    index = m.build_step_index([("a", 4)])
    assert (index.slot_mapping[1] >= 0).all()
    m.commit({"a": 4})
    m.check()
    m.free_request("a")
    assert m.num_free_pages(0) == 8 and m.num_free_pages(1) == 8
    m.check()


def test_groups_are_formed_by_needs_and_calls_without_cache_have_none():
    needs = [
        CacheNeeds(pages=PagedKVNeeds(2, 16, None)),
        None,  # a call that reads another call's cache
        CacheNeeds(pages=PagedKVNeeds(1, 32, None)),
        CacheNeeds(pages=PagedKVNeeds(2, 16, None), state=StateNeeds((3,), torch.float32)),
        CacheNeeds(state=StateNeeds((2, 2), torch.float32)),
    ]
    m = CacheManager(needs, page_size=4, num_pages=8, max_requests=2, device="cpu")
    assert [g.calls for g in m.groups] == [[0, 3], [2]]
    caches = m.layer_caches()
    assert caches[0].k_pages.shape == (8, 2, 4, 16) and caches[2].k_pages.shape == (8, 1, 4, 32)
    assert caches[1].group is None and caches[1].k_pages is None
    assert caches[3].state.shape == (3, 3) and caches[4].state.shape == (3, 2, 2) and caches[4].group is None
    assert caches[0].k_pages.data_ptr() != caches[3].k_pages.data_ptr()


def test_state_slots_are_zeroed_on_reuse():
    slots = StateSlots(2, {0: StateNeeds((3,), torch.float32)}, "cpu")
    a = slots.allocate("a")
    slots.tensors[0][a] = 7.0
    slots.free(a)
    with pytest.raises(RuntimeError, match="twice"):
        slots.free(a)
    b = slots.allocate("b")
    assert b == a and torch.all(slots.tensors[0][b] == 0)
    slots.allocate("c")
    with pytest.raises(OutOfMemoryError):
        slots.allocate("d")
    slots.check()


def test_truncate_gives_back_whole_pages():
    m = _manager(pages=8, page_size=4)
    m.add_request("a")
    m.reserve({"a": 14})
    m.commit({"a": 14})
    m.truncate("a", 5)
    assert m.length("a") == 5 and len(m.groups[0].tables["a"]) == 2 and m.num_free_pages() == 6
    m.check()


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("window", [None, 7])
def test_random_orders_lose_no_page(seed, window):
    """Requests come, grow by random portions, end in random order: after every
    operation no page is lost, held twice or freed twice, and at the end all are free."""
    rng = np.random.default_rng(seed)
    m = CacheManager(_needs(window) + _needs(None, 1), page_size=4, num_pages=12, max_requests=4,
                     allocate_storage=False)
    live: dict[str, int] = {}
    next_id = 0
    reused = False
    ever_used: set[int] = set()
    for _ in range(300):
        action = rng.random()
        if action < 0.25 and len(live) < 4:
            rid = f"r{next_id}"
            next_id += 1
            m.add_request(rid)
            live[rid] = 0
        elif action < 0.85 and live:
            chosen = [r for r in live if rng.random() < 0.6] or [next(iter(live))]
            extents = {r: int(rng.integers(1, 9)) for r in chosen}
            try:
                m.reserve(extents)
            except OutOfMemoryError:
                victim = max(live, key=live.get)
                m.free_request(victim)
                del live[victim]
            else:
                index = m.build_step_index(list(extents.items()))
                for g, group in enumerate(m.groups):
                    pages = set((index.slot_mapping[g] // 4).tolist())
                    reused |= bool(pages & ever_used)
                    ever_used |= pages
                m.commit(extents)
                for r, n in extents.items():
                    live[r] += n
                    assert m.length(r) == live[r]
        elif live:
            rid = list(live)[int(rng.integers(0, len(live)))]
            m.free_request(rid)
            del live[rid]
        m.check()
    for rid in list(live):
        m.free_request(rid)
    m.check()
    assert all(m.num_free_pages(g.index) == 12 for g in m.groups)
    assert m.states.num_free == 4
    assert reused


def test_keys_and_values_are_sized_apart_and_layout_is_what_the_mixer_declared():
    needs = [
        CacheNeeds(pages=PagedKVNeeds(2, 16, v_head_dim=40)),
        CacheNeeds(pages=PagedKVNeeds(2, 16, v_head_dim=40)),
        CacheNeeds(pages=PagedKVNeeds(2, 16, v_transposed=True)),
        CacheNeeds(pages=PagedKVNeeds(1, 24, v_head_dim=0)),
    ]
    manager = CacheManager(needs, page_size=4, num_pages=6, max_requests=2, dtype=torch.float32, allocate_storage=True)
    assert [g.calls for g in manager.groups] == [[0, 1], [2], [3]]
    wide, transposed, single = manager.groups
    assert wide.k_storage.shape == (2, 6, 2, 4 * 16) and wide.v_storage.shape == (2, 6, 2, 4 * 40)
    assert single.v_storage is None
    caches = manager.layer_caches()
    assert caches[0].k_pages.shape == (6, 2, 4, 16) and caches[0].v_pages.shape == (6, 2, 4, 40)
    assert caches[2].v_pages.shape == (6, 2, 16, 4) and caches[2].v_transposed and not caches[0].v_transposed
    assert caches[3].k_pages.shape == (6, 1, 4, 24) and caches[3].v_pages is None
    # views of one call do not overlap another call's
    caches[0].v_pages.fill_(1.0)
    assert caches[1].v_pages.abs().sum() == 0 and caches[0].k_pages.abs().sum() == 0
    with pytest.raises(ValueError):
        CacheManager([CacheNeeds(pages=PagedKVNeeds(0, 16))], page_size=4, num_pages=2, max_requests=1,
                     allocate_storage=False)


def test_slot_table_row_follows_the_request():
    from mini_infer_amd import ops
    from mini_infer_amd.cache import state_slots as layout

    assert ops.SLOT_WORDS == layout.SLOT_WORDS  # the kernels and the manager agree on the row
    m = _manager(storage=True)
    m.add_request("a")
    slot = m.state_slot("a")
    assert m.states.table.shape == (4, layout.SLOT_WORDS) and m.states.table.dtype == torch.int32
    m.set_sampling("a", temperature=0.7, top_k=40, top_p=0.95, seed=(5 << 32) | 0xFFFFFFFE, draw=3)
    assert m.states.seed(slot) == (5 << 32) | 0xFFFFFFFE and m.states.draws(slot) == 3
    m.reserve({"a": 6})
    m.commit({"a": 6})
    assert m.states.position(slot) == 6
    m.truncate("a", 5)
    assert m.states.position(slot) == 5
    m.states.count_draw(slot)
    assert m.states.draws(slot) == 4
    # the device copy holds what was pushed (settings, seed, draw as set; position as truncated)
    row = m.states.table[slot].tolist()
    assert row[layout.SLOT_SEED_LO] == -2 and row[layout.SLOT_SEED_HI] == 5 and row[layout.SLOT_TOP_K] == 40
    assert row[layout.SLOT_POSITION] == 5 and row[layout.SLOT_DRAW] == 3
    m.free_request("a")
    m.add_request("b")
    assert m.state_slot("b") == slot and m.states.draws(slot) == 0 and m.states.position(slot) == 0
    assert m.states.table[slot].tolist()[:4] == [0, 0, 0, 0]


def test_cancel_reservation_gives_back_exactly_what_reserve_took():
    """A step that did not happen: a windowed group that has already released pages, a group
    that keeps everything, a request that grows and one admitted for this very step.  After
    `cancel_reservation` tables, pools and lengths are what they were, and `check()` holds."""
    needs = [CacheNeeds(pages=PagedKVNeeds(2, 16)), CacheNeeds(pages=PagedKVNeeds(2, 16, window=6))]
    m = CacheManager(needs, page_size=4, num_pages=12, max_requests=3, allocate_storage=False)
    m.add_request("old")
    m.reserve({"old": 17})
    m.commit({"old": 17})
    windowed = m.groups[1]
    assert windowed.tables["old"][:3] == [-1, -1, -1]  # the window has passed three pages
    tables_before = [list(g.tables["old"]) for g in m.groups]
    free_before = [g.pool.num_free for g in m.groups]
    m.add_request("new")
    extents = {"old": 9, "new": 6}
    m.reserve(extents)
    assert [g.pool.num_free for g in m.groups] == [f - 4 for f in free_before]
    m.cancel_reservation(extents)
    m.check()
    assert [list(g.tables["old"]) for g in m.groups] == tables_before
    assert [g.tables["new"] for g in m.groups] == [[], []]
    assert [g.pool.num_free for g in m.groups] == free_before
    assert m.length("old") == 17 and m.length("new") == 0
    m.free_request("new")
    m.free_request("old")
    m.check()
    assert [g.pool.num_free for g in m.groups] == [12, 12]


def test_several_named_state_tensors_per_call_are_zeroed_on_reuse():
    needs = [CacheNeeds(state={"tail": StateNeeds((3,), torch.bfloat16), "recurrent": StateNeeds((2, 2))}), None,
             CacheNeeds(pages=PagedKVNeeds(1, 16), state=StateNeeds((5,)))]
    m = CacheManager(needs, page_size=4, num_pages=4, max_requests=2, dtype=torch.float32, device="cpu")
    caches = m.layer_caches()
    assert set(caches[0].state) == {"tail", "recurrent"} and caches[1].state is None
    assert caches[0].state["tail"].dtype == torch.bfloat16 and caches[0].state["recurrent"].shape == (3, 2, 2)
    assert caches[2].state.shape == (3, 5) and caches[2].k_pages is not None
    slot = m.add_request("a")
    caches[0].state["tail"][slot] = 7.0
    caches[0].state["recurrent"][slot] = 3.0
    caches[2].state[slot] = 1.0
    saved = m.states.snapshot(torch.tensor([slot, -1]))
    caches[0].state["recurrent"][slot] = 9.0
    caches[0].state["recurrent"][-1] = 4.0
    m.states.restore(torch.tensor([slot, -1]), saved)
    assert caches[0].state["recurrent"][slot].flatten().tolist() == [3.0] * 4
    assert caches[0].state["recurrent"][-1].flatten().tolist() == [0.0] * 4  # nobody's row, put back too
    m.free_request("a")
    assert m.add_request("b") == slot
    for tensor in (caches[0].state["tail"], caches[0].state["recurrent"], caches[2].state):
        assert float(tensor[slot].float().abs().sum()) == 0.0
    with pytest.raises(ValueError, match="mapping of names"):
        CacheManager([CacheNeeds(state={})], page_size=4, num_pages=1, max_requests=1, allocate_storage=False)
