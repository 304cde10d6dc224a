"""The cache manager's bookkeeping: no page lost, held twice or freed twice, under random orders of requests;
windows give pages back mid-request; slots for per-request state."""

import random

import pytest
import torch

from ampere_kv_engine_amd.cache import (RELEASED, BlockTable, CacheManager, PageAllocator, PagePoolExhausted,
                                        SlotsExhausted, SlotTable)
from ampere_kv_engine_amd.parts.base import PagedKV, SlotState


def test_pool_is_a_stack_and_refuses_double_free():
    pool = PageAllocator(4)
    assert [pool.allocate() for _ in range(4)] == [0, 1, 2, 3]            # reference: block_pool.py:12-13
    with pytest.raises(PagePoolExhausted):
        pool.allocate()
    pool.free(1)
    pool.free(3)
    assert pool.allocate() == 3 and pool.allocate() == 1                      # freed pages are reused first, last in first out
    pool.free(2)
    with pytest.raises(ValueError):
        pool.free(2)
    with pytest.raises(ValueError):
        pool.free(17)


def test_block_table_appends_all_or_nothing_and_locates():
    pool = PageAllocator(3)
    table = BlockTable(pool, 4)
    assert table.append_tokens(4) == 0 and table.pages == (0,)              # length 4 needs one page of 4
    assert table.append_tokens(1) == 4 and table.pages == (0, 1)            # length 5 needs two
    assert table.locate(4) == (1, 0) and table.locate(3) == (0, 3)
    with pytest.raises(ValueError):
        table.locate(5)                                                       # beyond the registered length
    with pytest.raises(PagePoolExhausted):
        table.append_tokens(8)                                                # needs 2 more pages, 1 free: nothing taken
    assert table.length == 5 and pool.num_free == 1
    table.release()
    table.release()                                                           # harmless
    assert pool.num_free == 3 and table.length == 0


def test_window_gives_pages_back_while_the_request_lives():
    pool = PageAllocator(8)
    table = BlockTable(pool, 4, window=6)
    table.append_tokens(16)                     # a whole 16-token portion needs all its keys: 4 pages
    assert table.num_held == 4
    table.append_tokens(1)                      # query at 16 reads keys 11..16: pages 0 and 1 (keys 0..7) are passed
    assert table.pages[:2] == (RELEASED, RELEASED) and table.num_held == 3 and pool.num_free == 5
    with pytest.raises(ValueError):
        table.locate(3)
    assert table.locate(16) == (table.pages[4], 0)
    for _ in range(40):
        table.append_tokens(1)
    assert table.num_held <= 3                  # never more than the window needs
    table.release()
    assert pool.num_free == 8


def _manager(**kw):
    needs = {0: PagedKV(2, 16), 1: PagedKV(2, 16), 2: PagedKV(2, 16, window=12), 3: SlotState((3, 5)), 4: None}
    return CacheManager(needs, page_size=4, num_pages=24, max_seqs=3, dtype=torch.float32, **kw)


def test_groups_by_need_and_tensor_shapes():
    m = _manager()
    assert [g.layers for g in m.groups] == [[0, 1], [2]]
    plane = 24 * 2 * 4 * 16                      # pages x heads x page size x width
    assert m.groups[0].pages.shape == (2, 2 * plane) and m.groups[1].pages.shape == (1, 2 * plane)
    assert m.layer_cache[1].k.shape == (24, 2, 4, 16) and m.layer_cache[1].k.data_ptr() == m.groups[0].pages[1].data_ptr()
    assert m.layer_cache[1].v.shape == (24, 2, 16, 4) and m.layer_cache[1].v.data_ptr() == m.groups[0].pages[1, plane:].data_ptr()
    assert m.layer_cache[3].state.shape == (3, 3, 5) and m.layer_cache[4].group is None
    assert m.bytes_per_token() == (2 * 2 + 2 * 1) * 2 * 16 * 4


def test_keys_and_values_of_different_widths_and_keys_alone():
    """A mixer's values may be narrower (or wider) than its keys, or absent: each such need is a group of its own, its
    layers' views have the widths asked for and do not overlap, and a token's bytes count both widths."""
    needs = {0: PagedKV(2, 16), 1: PagedKV(2, 16, value_dim=8), 2: PagedKV(3, 24, value_dim=0), 3: PagedKV(2, 16, value_dim=16),
             4: PagedKV(2, 16, value_dim=8)}
    m = CacheManager(needs, page_size=4, num_pages=6, max_seqs=2, dtype=torch.float32)
    assert [g.layers for g in m.groups] == [[0], [1, 4], [2], [3]]      # (an explicit width equal to the keys' is another need)
    narrow, alone = m.layer_cache[4], m.layer_cache[2]
    assert narrow.k.shape == (6, 2, 4, 16) and narrow.v.shape == (6, 2, 8, 4)
    assert alone.k.shape == (6, 3, 4, 24) and alone.v is None
    assert m.groups[1].pages.shape == (2, 6 * 2 * 4 * (16 + 8)) and m.groups[2].pages.shape == (1, 6 * 3 * 4 * 24)
    m.groups[1].pages.zero_()
    narrow.k.fill_(1.0), narrow.v.fill_(2.0)
    assert float(m.groups[1].pages[0].abs().sum()) == 0.0                                  # the other layer of the group
    assert float(m.groups[1].pages[1].sum()) == 6 * 2 * 4 * (16 * 1.0 + 8 * 2.0)           # every element once
    assert m.bytes_per_token() == (2 * 32 + 2 * 2 * 24 + 3 * 24 + 2 * 32) * 4


def test_slots_are_zeroed_when_taken_again():
    m = _manager()
    a = m.open("a")
    m.layer_cache[3].state[a.slot] = 7.0
    m.close(a)
    b = m.open("b")
    assert b.slot == a.slot and float(m.layer_cache[3].state[b.slot].abs().sum()) == 0.0
    m.open("c"), m.open("d")
    with pytest.raises(SlotsExhausted):
        m.open("e")
    with pytest.raises(ValueError):
        m.open("c")


def test_reserve_is_all_or_nothing_across_groups():
    m = _manager()
    a, b = m.open("a"), m.open("b")
    assert m.reserve(a, 60) == 0               # 15 pages in each group
    assert m.num_free_pages == [9, 9]
    with pytest.raises(PagePoolExhausted):
        m.reserve(b, 40)                       # needs 10 pages
    assert b.length == 0 and all(t.length == 0 for t in b.tables) and m.num_free_pages == [9, 9]
    m.close(a)
    m.close(a)
    m.close(b)
    assert m.num_free_pages == [24, 24] and m.slots.num_free == 3
    with pytest.raises(ValueError):
        m.reserve(a, 1)


@pytest.mark.parametrize("seed", range(6))
def test_no_page_lost_held_twice_or_freed_twice_under_random_orders(seed):
    rng = random.Random(seed)
    m = _manager(allocate_tensors=False)
    live, counter = {}, 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and m.slots.num_free:
            counter += 1
            live[f"r{counter}"] = m.open(f"r{counter}")
        elif action < 0.85 and live:
            seq = live[rng.choice(sorted(live))]
            count = rng.choice((1, 1, 1, 2, 3, 7, 13))
            before = (seq.length, [t.pages for t in seq.tables], m.num_free_pages)
            try:
                m.reserve(seq, count)
            except PagePoolExhausted:
                assert (seq.length, [t.pages for t in seq.tables], m.num_free_pages) == before
        elif live:
            name = rng.choice(sorted(live))
            m.close(live.pop(name))
        # invariants
        for group in m.groups:
            held = [p for s in live.values() for p in s.tables[group.index].pages if p != RELEASED]
            assert len(held) == len(set(held)), "a page is held twice"
            assert len(held) + group.allocator.num_free == m.num_pages, "a page was lost"
            assert all(group.allocator.is_held(p) for p in held)
        for s in live.values():
            assert all(t.length == s.length for t in s.tables)
            assert all(tuple(t.page_array.tolist()) == t.pages and t.num_pages == len(t.pages) for t in s.tables)
            full, windowed = s.tables
            assert full.num_held == -(-s.length // 4)
            assert windowed.num_held <= -(-(12 + 13) // 4) + 1
        assert len({s.slot for s in live.values()}) == len(live) == m.max_seqs - m.slots.num_free
    for seq in live.values():
        m.close(seq)
    assert m.num_free_pages == [24, 24] and m.slots.num_free == 3


def test_slot_table():
    slots = SlotTable(2)
    a, b = slots.take(), slots.take()
    assert (a, b) == (0, 1)
    slots.give_back(a)
    with pytest.raises(ValueError):
        slots.give_back(a)
    assert slots.take() == a


def test_a_mixer_may_say_how_its_state_starts():
    """`SlotState(init=...)`: the slot of a new request is set by the mixer's own function, also when the slot was
    used before; without it the state is zeroed."""
    def ones_then_index(state):
        state.fill_(1.0)
        state[0] = 3.0
    needs = {0: SlotState((4,), torch.float32, init=ones_then_index), 1: SlotState((2,))}
    m = CacheManager(needs, page_size=4, num_pages=4, max_seqs=2, dtype=torch.float32)
    a = m.open("a")
    assert m.layer_cache[0].state[a.slot].tolist() == [3.0, 1.0, 1.0, 1.0] and m.layer_cache[1].state[a.slot].tolist() == [0.0, 0.0]
    m.layer_cache[0].state[a.slot] = -5.0
    m.layer_cache[1].state[a.slot] = -5.0
    m.close(a)
    b = m.open("b")
    assert b.slot == a.slot
    assert m.layer_cache[0].state[b.slot].tolist() == [3.0, 1.0, 1.0, 1.0] and m.layer_cache[1].state[b.slot].tolist() == [0.0, 0.0]


def test_a_step_is_checked_in_the_order_its_requests_register():
    """A windowed group: in one step a single-token request needs a new page while a portion of another request
    gives pages back.  The single token registers first, so the pages the portion frees come too late for it: the
    step must be refused as a whole, with nothing registered, and not fail half-way."""
    from ampere_kv_engine_amd.engine.batch import BatchBuilder, StepEntry
    needs = {0: PagedKV(1, 16, window=4)}
    m = CacheManager(needs, page_size=4, num_pages=5, max_seqs=2, dtype=torch.float32, device="cpu")
    builder = BatchBuilder(m, "cpu", 64, 2, 16)
    old, young = m.open("old"), m.open("young")
    builder.build([StepEntry(old, [0] * 16, [])])            # 4 pages; a later step of `old` frees 3 of them
    builder.build([StepEntry(young, [0] * 4, [])])           # 1 page (none of it passed yet): the pool is empty
    assert m.num_free_pages == [0]
    before = (old.length, young.length, old.tables[0].pages, young.tables[0].pages)
    # in caller order `old` would free 3 pages before `young` needs 1; in the step's order `young` (one token) is first
    with pytest.raises(PagePoolExhausted, match="'young'"):
        builder.build([StepEntry(old, [0, 0], []), StepEntry(young, [0], [0])])
    assert (old.length, young.length, old.tables[0].pages, young.tables[0].pages) == before
    assert m.num_free_pages == [0]
    builder.build([StepEntry(old, [0, 0], [])])              # alone it fits: pages are given back first
    builder.build([StepEntry(young, [0], [0])])
    m.close(old), m.close(young)
    assert m.num_free_pages == [5]


def test_the_kernels_and_the_host_lay_a_slot_out_alike():
    """The words of a request's slot are named once for the kernels (csrc/common.h) and once for the host
    (cache/slots.py); the library reports its layout and the kernel set refuses one that differs from the host's."""
    import ctypes
    from ampere_kv_engine_amd.cache import slots
    from ampere_kv_engine_amd.csrc.build import ensure_built
    lib = ctypes.CDLL(ensure_built())
    layout = (ctypes.c_int * 8)()
    assert lib.akv_slot_layout(layout) == 0
    assert tuple(layout) == (slots.SLOT_WORDS, slots.WORD_LENGTH, slots.WORD_LAST_TOKEN, slots.WORD_TEMPERATURE,
                             slots.WORD_SEED_LOW, slots.WORD_SEED_HIGH, slots.WORD_DRAWS, slots.WORD_TAKEN)
