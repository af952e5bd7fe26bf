"""The cache of a model: a slot for each live sequence, keys and values for each layer that keeps
them, and per-sequence state of fixed size beside them.

The reference has one sequence, one flat ``[kv_head, n_ctx, head_dim]`` buffer pair per layer with
the length in a 64-byte prefix (engine/engine.h:34-63, engine/model_loader.cpp:853-904), and, for
other kinds of layers, fixed-size state buffers without a length that ``reset()`` must zero
(engine/model_loader.cpp:906-939, engine/engine.cpp:270-297).  Here there are many sequences:

* Layers whose mixers ask for the same kind of storage (an equal *need*: same kv heads, head size and window;
  or rows of the same name and shape) form a *group*.  A group has storage of its own: ``k`` and ``v`` of shape
  ``[layers of the group, pages + 1, kv_heads, PAGE_TOKENS, head_dim]`` (``v`` with the last two swapped) and one page table (the pages
  of every slot), shared by the group's layers.  The last page is never handed out: rows that pad a
  batch write there.
* State groups are ``[layers of the group, slots + 1, *shape]``, zeroed when a slot is opened.
* ``lengths[slot]`` is the whole state of a sequence's progress.
"""
from __future__ import annotations

from dataclasses import dataclass

import copy

import numpy as np
import torch

from .pool import PAGE_TOKENS, CacheFull, CacheMisuse, FreeList, PageTable, pages_for


# ---- what a part may ask for ----------------------------------------------------------------------
# A need is a frozen description; run-order entries with equal needs share one group (one allocation, for
# growing storage one page table).  A need says of itself how it is stored: ``make_group`` allocates the
# group, and the group says how it shows itself to the part (``attach``).  ``ModelCache`` knows no kind of
# need by name: a mixer with storage of another shape brings a need and a group class of its own.
#
# A group has: ``need``, ``n_entries``; ``table`` (a ``PageTable`` if the storage grows with the sequence, else
# None; its ``window`` says whether pages are given back as a sequence grows); ``sync()`` (bring device copies of
# host bookkeeping up to date, without making the host wait for the device); ``on_open(slot)``; ``nbytes()``;
# ``attach(layer_cache, entry)``, which hangs what the part is to see on the entry's ``LayerCache`` under a field of
# the need's choosing (the shipped ones use ``kv``, ``rows[name]`` and ``states[name]``).  Storage in pages derives
# from ``PagedGroup``, which reads one thing of its need: ``window`` (absent or None: every position is kept).

@dataclass(frozen=True)
class KVNeed:
    """Keys and values of every position (``window`` None) or of the last ``window`` positions, in the layout
    the attention kernels read: K ``[pages, kv_heads, PAGE_TOKENS, head_dim]``, V with the last two swapped."""
    num_kv_heads: int
    head_dim: int
    window: int | None = None

    def make_group(self, n_entries, n_pages, n_slots, max_pages_per_slot, dtype, device):
        return KVGroup(self, n_entries, n_pages, n_slots, max_pages_per_slot, dtype, device)


@dataclass(frozen=True)
class RowsNeed:
    """One row of shape ``row_shape`` for every position (or for the last ``window`` positions), under a name
    of the part's choosing: storage that grows with the sequence but is not keys and values of the attention
    kernels' layout (a compressed row, keys alone, values of another width).  ``dtype`` None: the run's."""
    name: str
    row_shape: tuple[int, ...]
    dtype: str | None = None
    window: int | None = None

    def make_group(self, n_entries, n_pages, n_slots, max_pages_per_slot, dtype, device):
        return RowsGroup(self, n_entries, n_pages, n_slots, max_pages_per_slot, dtype, device)


@dataclass(frozen=True)
class StateNeed:
    """A tensor of fixed shape for each sequence, zero when the sequence starts."""
    name: str
    shape: tuple[int, ...]
    dtype: str = "float32"

    def make_group(self, n_entries, n_pages, n_slots, max_pages_per_slot, dtype, device):
        return StateGroup(self, n_entries, n_slots, device)


class PagedGroup:
    """Storage in pages of PAGE_TOKENS positions with one page table for the group's entries.  The last page
    is never handed out: rows that pad a batch write there."""

    def __init__(self, need, n_entries: int, n_pages: int, n_slots: int, max_pages_per_slot: int, device):
        self.need, self.n_entries, self.n_pages = need, n_entries, n_pages
        self.table = PageTable(n_pages, n_slots, max_pages_per_slot, getattr(need, "window", None))
        self.pad_page = n_pages
        self.table_host = torch.full((n_slots + 1, max_pages_per_slot), self.pad_page, dtype=torch.int32)
        self.table_dev = self.table_host.to(device)
        # Stale rows go to the device through pinned memory, two buffers in turn, each written again only after the
        # copy that last read it has run: the host never waits for the step that is still running (a step launched
        # ahead of its predecessor's results would otherwise stop at every page border of every sequence).
        self._pinned = torch.device(device).type == "cuda"
        self._staging: list = [None, None]           # int32 [rows, pages of a slot + 1]: a slot's pages, then its number
        self._staged: list = [None, None]
        self._turn = 0

    def sync(self) -> None:
        """Bring the device's copy of the page lists up to date: all stale rows in one indexed copy, queued on
        the stream like the step that reads them."""
        if not self.table.dirty:
            return
        slots = sorted(self.table.dirty)
        k, width = len(slots), self.table_host.shape[1]
        turn = self._turn = self._turn ^ 1
        if self._staged[turn] is not None:
            self._staged[turn].synchronize()
        buf = self._staging[turn]
        if buf is None or buf.shape[0] < k:
            buf = self._staging[turn] = torch.empty((max(k, 16), width + 1), dtype=torch.int32, pin_memory=self._pinned)
        rows = buf.numpy()[:k]
        rows[:, :width] = self.pad_page
        for i, slot in enumerate(slots):
            pages = self.table.slot_pages[slot]
            if pages:
                rows[i, :len(pages)] = np.where(np.asarray(pages, dtype=np.int32) >= 0, pages, self.pad_page)
            rows[i, width] = slot
        self.table_host[slots] = buf[:k, :width]
        up = buf[:k].to(self.table_dev.device, non_blocking=True)
        self.table_dev.index_copy_(0, up[:, width].long(), up[:, :width])
        if self._pinned:
            self._staged[turn] = torch.cuda.Event()
            self._staged[turn].record()
        self.table.dirty.clear()

    def on_open(self, slot: int) -> None:
        pass                                                    # nothing is read beyond a sequence's length


class KVGroup(PagedGroup):
    def __init__(self, need: KVNeed, n_entries: int, n_pages: int, n_slots: int, max_pages_per_slot: int,
                 dtype: torch.dtype, device):
        super().__init__(need, n_entries, n_pages, n_slots, max_pages_per_slot, device)
        # values are kept transposed (positions innermost): both products of attention then sum over an
        # index that is contiguous in memory
        self.k = torch.zeros((n_entries, n_pages + 1, need.num_kv_heads, PAGE_TOKENS, need.head_dim), dtype=dtype,
                             device=device)
        self.v = torch.zeros((n_entries, n_pages + 1, need.num_kv_heads, need.head_dim, PAGE_TOKENS), dtype=dtype,
                             device=device)

    def nbytes(self) -> int:
        return 2 * self.k.numel() * self.k.element_size()

    def attach(self, layer_cache, entry: int) -> None:
        if layer_cache.kv is not None:
            raise ValueError("a run-order entry asks for two key/value stores")
        layer_cache.kv, layer_cache.kv_entry = self, entry


@dataclass
class RowsView:
    """What a part sees of its rows: ``data [pages + 1, PAGE_TOKENS, *row_shape]`` of its own entry, and the
    group's page table on the device (``[slots + 1, pages of a slot]``, int32): position p of slot s lies at
    ``data[table_dev[s, p // PAGE_TOKENS], p % PAGE_TOKENS]``."""
    data: torch.Tensor
    group: "RowsGroup"

    @property
    def table_dev(self) -> torch.Tensor:
        return self.group.table_dev


class RowsGroup(PagedGroup):
    def __init__(self, need: RowsNeed, n_entries: int, n_pages: int, n_slots: int, max_pages_per_slot: int,
                 dtype: torch.dtype, device):
        super().__init__(need, n_entries, n_pages, n_slots, max_pages_per_slot, device)
        dt = getattr(torch, need.dtype) if need.dtype else dtype
        self.data = torch.zeros((n_entries, n_pages + 1, PAGE_TOKENS) + tuple(need.row_shape), dtype=dt, device=device)

    def nbytes(self) -> int:
        return self.data.numel() * self.data.element_size()

    def attach(self, layer_cache, entry: int) -> None:
        layer_cache.rows = layer_cache.rows or {}
        if self.need.name in layer_cache.rows:
            raise ValueError(f"a run-order entry asks twice for rows named {self.need.name!r}")
        layer_cache.rows[self.need.name] = RowsView(self.data[entry], self)


class StateGroup:
    table = None                                                # does not grow: no pages

    def __init__(self, need: StateNeed, n_entries: int, n_slots: int, device):
        self.need, self.n_entries = need, n_entries
        self.data = torch.zeros((n_entries, n_slots + 1) + tuple(need.shape), dtype=getattr(torch, need.dtype),
                                device=device)

    def sync(self) -> None:
        pass

    def on_open(self, slot: int) -> None:
        self.data[:, slot].zero_()

    def nbytes(self) -> int:
        return self.data.numel() * self.data.element_size()

    def attach(self, layer_cache, entry: int) -> None:
        layer_cache.states = layer_cache.states or {}
        layer_cache.states[self.need.name] = self.data[entry]


@dataclass
class LayerCache:
    """What one entry of the run order sees of the cache."""
    kv: KVGroup | None = None
    kv_entry: int = -1
    writes: bool = True               # False: the entry reads another entry's storage and writes none
    states: dict | None = None        # name -> tensor [slots + 1, *shape]
    rows: dict | None = None          # name -> RowsView

    @property
    def k(self) -> torch.Tensor:
        return self.kv.k[self.kv_entry]

    @property
    def v(self) -> torch.Tensor:
        return self.kv.v[self.kv_entry]


class ModelCache:
    """``needs[i]`` is the list of needs of run-order entry ``i`` (empty for an entry that reads another
    entry's cache: ``shares[i]`` is that entry's index)."""

    def __init__(self, needs: list[list], shares: list[int | None], max_tokens: int, max_seqs: int | None,
                 max_positions: int | None, dtype: torch.dtype, device):
        if max_tokens <= 0:
            raise ValueError(f"max_tokens = {max_tokens} must be positive")
        self.device, self.dtype = device, dtype
        n_pages = pages_for(max_tokens)
        self.max_seqs = int(max_seqs) if max_seqs else min(n_pages, 1024)
        self.max_tokens = n_pages * PAGE_TOKENS
        self.max_seq_tokens = min(max_positions, self.max_tokens) if max_positions else self.max_tokens
        max_pages_per_slot = pages_for(self.max_seq_tokens)
        self.pad_slot = self.max_seqs
        self.slots = FreeList(self.max_seqs, "slot")
        self.lengths = [0] * self.max_seqs

        members: dict[object, list[int]] = {}                   # need -> the entries that have it, in run order
        for i, entry_needs in enumerate(needs):
            for need in entry_needs:
                members.setdefault(need, []).append(i)
        self.groups = [need.make_group(len(m), n_pages, self.max_seqs, max_pages_per_slot, dtype, device)
                       for need, m in members.items()]
        self.paged_groups = [g for g in self.groups if g.table is not None]       # storage that grows: pages to manage

        self.layer_caches: list[LayerCache] = [LayerCache() for _ in needs]
        for group, entries in zip(self.groups, members.values()):
            for j, i in enumerate(entries):
                try:
                    group.attach(self.layer_caches[i], j)
                except ValueError as e:
                    raise ValueError(f"run-order entry {i}: {e}") from None
        for i, src in enumerate(shares):
            if src is not None:
                self.layer_caches[i] = copy.copy(self.layer_caches[src])      # whatever its groups hung on it
                self.layer_caches[i].writes = False

    def groups_of(self, need_type) -> list:
        """The groups whose need is of the given class, in the order in which the run order first asked for them."""
        return [g for g in self.groups if isinstance(g.need, need_type)]

    # ---- sequences ---------------------------------------------------------------------------
    def open(self) -> int:
        slot = self.slots.take()
        self.lengths[slot] = 0
        for g in self.groups:
            g.on_open(slot)
        return slot

    def close(self, slot: int) -> None:
        if not self.slots.is_held(slot):
            raise CacheMisuse(f"slot {slot} is closed but not open")
        for g in self.paged_groups:
            g.table.release(slot)
        self.lengths[slot] = 0
        self.slots.give_back(slot)

    def check_room(self, growth: list[tuple[int, int]], in_pieces: bool = False) -> None:
        """Raise ``CacheFull`` (or ``CacheMisuse``) if the step does not fit; take nothing.  ``in_pieces``: the
        tokens will go through in several steps, between which a windowed group gives pages back, so only the
        groups that keep every key are asked for the whole growth."""
        for slot, n_new in growth:
            if not self.slots.is_held(slot):
                raise CacheMisuse(f"slot {slot} is used but not open")
            if self.lengths[slot] + n_new > self.max_seq_tokens:
                raise CacheFull(f"slot {slot}: {self.lengths[slot]} + {n_new} tokens exceed the longest sequence "
                                f"the cache takes ({self.max_seq_tokens})")
        for g in self.paged_groups:
            if in_pieces and g.table.window:
                continue
            need = sum(g.table.pages_needed(slot, self.lengths[slot] + n) for slot, n in growth)
            if need > g.table.pages.free_count:
                raise CacheFull(f"the step needs {need} more pages of {PAGE_TOKENS} tokens; "
                                f"{g.table.pages.free_count} of {g.n_pages} are free")

    def reserve(self, growth: list[tuple[int, int]]) -> None:
        """Make room for ``n_new`` more tokens in each ``(slot, n_new)``; nothing is taken if the
        whole step does not fit."""
        self.check_room(growth)
        for g in self.paged_groups:
            for slot, n in growth:
                g.table.grow(slot, self.lengths[slot] + n)
            g.sync()

    def commit(self, growth: list[tuple[int, int]]) -> None:
        for slot, n in growth:
            self.lengths[slot] += n
            for g in self.paged_groups:
                g.table.trim(slot, self.lengths[slot])
        for g in self.paged_groups:
            g.sync()

    # ---- facts -------------------------------------------------------------------------------
    def tokens_held(self) -> int:
        return sum(pages_for(self.lengths[s]) * PAGE_TOKENS for s in range(self.max_seqs) if self.slots.is_held(s))

    def nbytes(self) -> int:
        return sum(g.nbytes() for g in self.groups)

    def check(self) -> None:
        self.slots.check()
        for g in self.paged_groups:
            g.table.check()
            for s in range(self.max_seqs):
                if not self.slots.is_held(s) and g.table.slot_pages[s]:
                    raise CacheMisuse(f"slot {s} is free but holds pages")
