"""The cache's bookkeeping on the host: no slot or page lost, held twice or freed twice (no GPU)."""
import random

import pytest
import torch

from palm_infra_amd.cache import (PAGE_TOKENS, CacheFull, CacheMisuse, FreeList, KVNeed, ModelCache, StateNeed,
                                  pages_for)


def test_free_list_hands_out_each_number_once_and_lowest_first():
    f = FreeList(4, "slot")
    assert [f.take() for _ in range(4)] == [0, 1, 2, 3]
    with pytest.raises(CacheFull):
        f.take()
    f.give_back(2)
    f.give_back(0)
    with pytest.raises(CacheMisuse, match="not held"):
        f.give_back(2)
    with pytest.raises(CacheMisuse, match="does not exist"):
        f.give_back(9)
    assert f.take() == 0 and f.take() == 2          # what was given back is used again, lowest first
    f.check()


def test_take_many_takes_nothing_if_it_cannot_take_all():
    f = FreeList(3, "page")
    f.take()
    with pytest.raises(CacheFull):
        f.take_many(3)
    assert f.free_count == 2
    f.check()


def _cache(needs=None, shares=None, max_tokens=64 * 12, max_seqs=None, max_positions=4096):
    needs = needs if needs is not None else [[KVNeed(2, 16)], [KVNeed(2, 16)]]
    shares = shares if shares is not None else [None] * len(needs)
    return ModelCache(needs, shares, max_tokens, max_seqs, max_positions, torch.float32, "cpu")


def test_pages_follow_lengths_and_come_back():
    c = _cache()
    a, b = c.open(), c.open()
    c.reserve([(a, 70), (b, 1)])
    c.commit([(a, 70), (b, 1)])
    g = c.groups_of(KVNeed)[0]
    assert g.table.slot_pages[a] == [0, 1] and g.table.slot_pages[b] == [2]
    assert c.lengths[a] == 70 and c.lengths[b] == 1
    for _ in range(58):                              # 70 -> 128: still two pages
        c.reserve([(a, 1)]); c.commit([(a, 1)])
    assert len(g.table.slot_pages[a]) == 2
    c.reserve([(a, 1)]); c.commit([(a, 1)])          # 129: a third
    assert g.table.slot_pages[a] == [0, 1, 3]
    assert g.table_dev[a, :4].tolist() == [0, 1, 3, g.pad_page]
    c.close(a)
    assert g.table.pages.free_count == 12 - 1
    c.check()
    d = c.open()
    assert d == a                                    # the slot is used again ...
    c.reserve([(d, 10)])
    assert g.table.slot_pages[d] == [0]              # ... and so is its first page, uncleared
    with pytest.raises(CacheMisuse):
        c.close(7)
    c.close(d)
    with pytest.raises(CacheMisuse):
        c.close(d)
    c.check()


def test_a_step_that_does_not_fit_takes_nothing():
    c = _cache(max_tokens=64 * 4)
    a, b = c.open(), c.open()
    c.reserve([(a, 64)]); c.commit([(a, 64)])
    free = c.groups_of(KVNeed)[0].table.pages.free_count
    with pytest.raises(CacheFull, match="more pages"):
        c.reserve([(a, 65), (b, 100)])               # 2 + 2 pages wanted, 3 free
    assert c.groups_of(KVNeed)[0].table.pages.free_count == free and c.lengths[a] == 64
    with pytest.raises(CacheFull, match="longest sequence"):
        c.reserve([(b, 64 * 4 + 1)])
    with pytest.raises(CacheFull, match="more pages"):
        c.check_room([(a, 65), (b, 100)])            # the same question without taking anything
    c.check_room([(a, 64), (b, 100)])
    assert c.groups_of(KVNeed)[0].table.pages.free_count == free and c.lengths[a] == 64 and c.lengths[b] == 0
    with pytest.raises(CacheMisuse, match="not open"):
        c.reserve([(3, 1)])
    c.check()


def test_longest_sequence_is_bounded_by_positions_and_by_the_cache():
    assert _cache(max_tokens=64 * 12, max_positions=100).max_seq_tokens == 100
    assert _cache(max_tokens=64 * 2, max_positions=4096).max_seq_tokens == 128
    assert _cache(max_tokens=64 * 5, max_positions=None).max_seq_tokens == 320      # a model without a limit of its own
    assert _cache(max_tokens=65).max_tokens == 128   # rounded up to whole pages


def test_groups_have_storage_of_their_own():
    needs = [[KVNeed(2, 16)], [KVNeed(1, 32, window=100)], [KVNeed(2, 16)], [KVNeed(1, 32, window=100), StateNeed("s", (3, 2))]]
    c = _cache(needs)
    assert len(c.groups_of(KVNeed)) == 2 and len(c.groups_of(StateNeed)) == 1
    full, win = c.groups_of(KVNeed)
    assert full.k.shape == (2, 13, 2, PAGE_TOKENS, 16) and win.k.shape == (2, 13, 1, PAGE_TOKENS, 32)
    assert full.v.shape == (2, 13, 2, 16, PAGE_TOKENS)                  # values are kept transposed
    assert full.k.data_ptr() != win.k.data_ptr() and full.table is not win.table
    lc = c.layer_caches
    assert lc[0].kv is full and lc[2].kv is full and (lc[0].kv_entry, lc[2].kv_entry) == (0, 1)
    assert lc[1].kv is win and lc[3].kv is win and lc[3].states["s"].shape == (c.max_seqs + 1, 3, 2)
    assert lc[0].k.data_ptr() != lc[2].k.data_ptr()


def test_a_window_gives_pages_back_as_the_sequence_grows():
    c = _cache([[KVNeed(1, 16, window=70)], [KVNeed(1, 16)]])
    win, full = c.groups_of(KVNeed)
    s = c.open()
    c.reserve([(s, 200)]); c.commit([(s, 200)])
    # the next query sits at 200 and reads keys 131..200: pages 0 and 1 (positions 0..127) are out of reach
    assert win.table.slot_pages[s] == [-1, -1, 2, 3] and full.table.slot_pages[s] == [0, 1, 2, 3]
    assert win.table_dev[s, :4].tolist() == [win.pad_page, win.pad_page, 2, 3]
    assert win.table.pages.free_count == 12 - 2
    c.reserve([(s, 1)]); c.commit([(s, 1)])          # 201: first key needed is 132, page 2 still is
    assert win.table.slot_pages[s][2] == 2
    c.check()
    c.close(s)
    assert win.table.pages.free_count == 12 and full.table.pages.free_count == 12


def test_state_is_zero_for_a_new_sequence():
    c = _cache([[StateNeed("h", (4,))]])
    s = c.open()
    c.groups_of(StateNeed)[0].data[0, s] = 5.0
    c.close(s)
    assert c.open() == s
    assert float(c.groups_of(StateNeed)[0].data[0, s].abs().sum()) == 0.0


def test_an_entry_can_read_another_entrys_cache():
    c = _cache([[KVNeed(2, 16)], []], shares=[None, 0])
    a, b = c.layer_caches
    assert b.kv is a.kv and b.kv_entry == a.kv_entry and a.writes and not b.writes
    assert c.groups_of(KVNeed)[0].k.shape[0] == 1


def test_random_traffic_keeps_the_books():
    rng = random.Random(0)
    c = _cache([[KVNeed(2, 16)], [KVNeed(2, 16, window=90)]], max_tokens=64 * 40, max_seqs=9)
    live = {}
    for step in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < 9:
            live[c.open()] = 0
        elif op < 0.4 and live:
            s = rng.choice(list(live))
            c.close(s)
            del live[s]
        elif live:
            batch = rng.sample(list(live), rng.randint(1, len(live)))
            growth = [(s, rng.choice([1, 1, 1, 5, 64, 130])) for s in batch]
            try:
                c.reserve(growth)
            except CacheFull:
                continue
            c.commit(growth)
            for s, n in growth:
                live[s] += n
        c.check()
        for s, n in live.items():
            assert c.lengths[s] == n
            for g in c.groups_of(KVNeed):
                pages = g.table.slot_pages[s]
                assert len(pages) >= pages_for(n)
                first = 0 if g.need.window is None else max(0, n - g.need.window + 1) // PAGE_TOKENS
                assert all(p >= 0 for p in pages[first:pages_for(n)])     # every page a query can reach is there
                assert g.table_dev[s, :len(pages)].tolist() == [p if p >= 0 else g.pad_page for p in pages]
    for s in list(live):
        c.close(s)
    c.check()
    assert all(g.table.pages.free_count == g.n_pages for g in c.groups_of(KVNeed)) and c.slots.free_count == 9


def test_rows_of_a_part_s_own_shape_grow_in_pages_beside_keys_and_values():
    from palm_infra_amd.cache import RowsGroup, RowsNeed
    needs = [[KVNeed(2, 16)], [RowsNeed("latent", (24,), dtype="float32")], [RowsNeed("latent", (24,), dtype="float32"), StateNeed("s", (3,))],
             [RowsNeed("codes", (2, 5), dtype="int32", window=70)]]
    c = _cache(needs)
    rows = [g for g in c.groups if isinstance(g, RowsGroup)]
    assert len(rows) == 2 and len(c.groups_of(KVNeed)) == 1 and len(c.paged_groups) == 3 and len(c.groups_of(StateNeed)) == 1
    latent, codes = rows
    assert latent.data.shape == (2, 13, PAGE_TOKENS, 24) and latent.data.dtype == torch.float32       # two entries share the group
    assert codes.data.shape == (1, 13, PAGE_TOKENS, 2, 5) and codes.data.dtype == torch.int32
    lc = c.layer_caches
    assert lc[1].rows["latent"].data.data_ptr() != lc[2].rows["latent"].data.data_ptr() and lc[1].kv is None
    assert lc[1].rows["latent"].table_dev is latent.table_dev and "s" in lc[2].states
    s = c.open()
    c.reserve([(s, 200)]); c.commit([(s, 200)])
    assert latent.table.slot_pages[s] == [0, 1, 2, 3] and codes.table.slot_pages[s] == [-1, -1, 2, 3]     # the window gave two back
    assert latent.table_dev[s, :4].tolist() == [0, 1, 2, 3]
    c.check()
    c.close(s)
    assert all(g.table.pages.free_count == g.n_pages for g in c.paged_groups)
    with pytest.raises(ValueError, match="twice for rows named"):
        _cache([[RowsNeed("x", (4,)), RowsNeed("x", (4,), dtype="float32")]])


def test_a_need_of_a_kind_the_cache_has_never_heard_of():
    """The cache asks a need how it is stored and asks the group how it shows itself to its part: a kind of
    storage defined here, outside the package, is grouped, opened and handed to its entries like the others."""
    from dataclasses import dataclass

    class CounterGroup:
        table = None

        def __init__(self, need, n_entries, n_slots):
            self.need, self.n_entries = need, n_entries
            self.data = torch.zeros((n_entries, n_slots + 1), dtype=torch.int64)
            self.opened = []

        def sync(self):
            pass

        def on_open(self, slot):
            self.opened.append(slot)
            self.data[:, slot] = self.need.start

        def nbytes(self):
            return self.data.numel() * 8

        def attach(self, layer_cache, entry):
            layer_cache.states = layer_cache.states or {}
            layer_cache.states["counter"] = self.data[entry]

    @dataclass(frozen=True)
    class CounterNeed:
        start: int

        def make_group(self, n_entries, n_pages, n_slots, max_pages_per_slot, dtype, device):
            return CounterGroup(self, n_entries, n_slots)

    c = _cache([[KVNeed(2, 16), CounterNeed(7)], [CounterNeed(7)], [CounterNeed(9)]])
    mine = [g for g in c.groups if isinstance(g, CounterGroup)]
    assert [g.n_entries for g in mine] == [2, 1]
    s = c.open()
    assert mine[0].opened == [s] and int(c.layer_caches[1].states["counter"][s]) == 7 and int(c.layer_caches[2].states["counter"][s]) == 9
    assert c.nbytes() >= sum(g.nbytes() for g in mine)
    c.reserve([(s, 100)]); c.commit([(s, 100)])
    c.check()
