"""The cache of a model: a slot for each live sequence, keys and values for each layer that keeps
them, and per-sequence state of fixed size beside them.

The reference has one sequence, one flat ``[kv_head, n_ctx, head_dim]`` buffer pair per layer with
the length in a 64-byte prefix (engine/engine.h:34-63, engine/model_loader.cpp:853-904), and, for
other kinds of layers, fixed-size state buffers without a length that ``reset()`` must zero
(engine/model_loader.cpp:906-939, engine/engine.cpp:270-297).  Here there are many sequences:

* Layers whose mixers ask for the same kind of storage (same kv heads, head size and window) form a
  *group*.  A group has storage of its own: ``k`` and ``v`` of shape
  ``[layers of the group, pages + 1, kv_heads, PAGE_TOKENS, head_dim]`` (``v`` with the last two swapped) and one page table (the pages
  of every slot), shared by the group's layers.  The last page is never handed out: rows that pad a
  batch write there.
* State groups are ``[layers of the group, slots + 1, *shape]``, zeroed when a slot is opened.
* ``lengths[slot]`` is the whole state of a sequence's progress.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .pool import PAGE_TOKENS, CacheFull, CacheMisuse, FreeList, PageTable, pages_for


@dataclass(frozen=True)
class KVNeed:
    """Keys and values of every position (``window`` None) or of the last ``window`` positions."""
    num_kv_heads: int
    head_dim: int
    window: int | None = None


@dataclass(frozen=True)
class StateNeed:
    """A tensor of fixed shape for each sequence, zero when the sequence starts."""
    name: str
    shape: tuple[int, ...]
    dtype: str = "float32"


class KVGroup:
    def __init__(self, need: KVNeed, n_entries: int, n_pages: int, n_slots: int, max_pages_per_slot: int,
                 dtype: torch.dtype, device):
        self.need, self.n_entries, self.n_pages = need, n_entries, n_pages
        self.table = PageTable(n_pages, n_slots, max_pages_per_slot, need.window)
        self.pad_page = n_pages
        # values are kept transposed (positions innermost): both products of attention then sum over an
        # index that is contiguous in memory
        self.k = torch.zeros((n_entries, n_pages + 1, need.num_kv_heads, PAGE_TOKENS, need.head_dim), dtype=dtype,
                             device=device)
        self.v = torch.zeros((n_entries, n_pages + 1, need.num_kv_heads, need.head_dim, PAGE_TOKENS), dtype=dtype,
                             device=device)
        self.table_host = torch.full((n_slots + 1, max_pages_per_slot), self.pad_page, dtype=torch.int32)
        self.table_dev = self.table_host.to(device)

    def sync(self) -> None:
        """Bring the device's copy of the page lists up to date: all stale rows in one indexed copy.
        The rows travel in fresh host tensors, so a later change on the host cannot reach a copy that
        the device has not run yet."""
        if not self.table.dirty:
            return
        slots = sorted(self.table.dirty)
        rows = torch.full((len(slots), self.table_host.shape[1]), self.pad_page, dtype=torch.int32)
        for i, slot in enumerate(slots):
            pages = self.table.slot_pages[slot]
            if pages:
                rows[i, :len(pages)] = torch.tensor([p if p >= 0 else self.pad_page for p in pages], dtype=torch.int32)
            self.table_host[slot] = rows[i]
        index = torch.tensor(slots, dtype=torch.long)
        self.table_dev.index_copy_(0, index.to(self.table_dev.device), rows.to(self.table_dev.device))
        self.table.dirty.clear()

    def nbytes(self) -> int:
        return 2 * self.k.numel() * self.k.element_size()


class StateGroup:
    def __init__(self, need: StateNeed, n_entries: int, n_slots: int, device):
        self.need, self.n_entries = need, n_entries
        self.data = torch.zeros((n_entries, n_slots + 1) + tuple(need.shape), dtype=getattr(torch, need.dtype),
                                device=device)


@dataclass
class LayerCache:
    """What one entry of the run order sees of the cache."""
    kv: KVGroup | None = None
    kv_entry: int = -1
    writes: bool = True               # False: the entry reads another entry's keys and values
    states: dict | None = None        # name -> tensor [slots + 1, *shape]

    @property
    def k(self) -> torch.Tensor:
        return self.kv.k[self.kv_entry]

    @property
    def v(self) -> torch.Tensor:
        return self.kv.v[self.kv_entry]


class ModelCache:
    """``needs[i]`` is the list of KVNeed/StateNeed of run-order entry ``i`` (empty for an entry that
    reads another entry's cache: ``shares[i]`` is that entry's index)."""

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

        kv_members: dict[KVNeed, list[int]] = {}
        state_members: dict[StateNeed, list[int]] = {}
        for i, entry_needs in enumerate(needs):
            for need in entry_needs:
                (kv_members if isinstance(need, KVNeed) else state_members).setdefault(need, []).append(i)
        self.kv_groups = [KVGroup(need, len(m), n_pages, self.max_seqs, max_pages_per_slot, dtype, device)
                          for need, m in kv_members.items()]
        self.state_groups = [StateGroup(need, len(m), self.max_seqs, device) for need, m in state_members.items()]

        self.layer_caches: list[LayerCache] = [LayerCache() for _ in needs]
        for group, members in zip(self.kv_groups, kv_members.values()):
            for j, i in enumerate(members):
                if self.layer_caches[i].kv is not None:
                    raise ValueError(f"run-order entry {i} asks for two key/value stores")
                self.layer_caches[i].kv, self.layer_caches[i].kv_entry = group, j
        for group, members in zip(self.state_groups, state_members.values()):
            for j, i in enumerate(members):
                lc = self.layer_caches[i]
                lc.states = lc.states or {}
                lc.states[group.need.name] = group.data[j]
        for i, src in enumerate(shares):
            if src is not None:
                s = self.layer_caches[src]
                self.layer_caches[i] = LayerCache(kv=s.kv, kv_entry=s.kv_entry, writes=False, states=s.states)

    # ---- sequences ---------------------------------------------------------------------------
    def open(self) -> int:
        slot = self.slots.take()
        self.lengths[slot] = 0
        for g in self.state_groups:
            g.data[:, slot].zero_()
        return slot

    def close(self, slot: int) -> None:
        if not self.slots.is_held(slot):
            raise CacheMisuse(f"slot {slot} is closed but not open")
        for g in self.kv_groups:
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
        for g in self.kv_groups:
            if in_pieces and g.need.window:
                continue
            need = sum(g.table.pages_needed(slot, self.lengths[slot] + n) for slot, n in growth)
            if need > g.table.pages.free_count:
                raise CacheFull(f"the step needs {need} more pages of {PAGE_TOKENS} tokens; "
                                f"{g.table.pages.free_count} of {g.n_pages} are free")

    def reserve(self, growth: list[tuple[int, int]]) -> None:
        """Make room for ``n_new`` more tokens in each ``(slot, n_new)``; nothing is taken if the
        whole step does not fit."""
        self.check_room(growth)
        for g in self.kv_groups:
            for slot, n in growth:
                g.table.grow(slot, self.lengths[slot] + n)
            g.sync()

    def commit(self, growth: list[tuple[int, int]]) -> None:
        for slot, n in growth:
            self.lengths[slot] += n
            for g in self.kv_groups:
                g.table.trim(slot, self.lengths[slot])
        for g in self.kv_groups:
            g.sync()

    # ---- facts -------------------------------------------------------------------------------
    def tokens_held(self) -> int:
        return sum(pages_for(self.lengths[s]) * PAGE_TOKENS for s in range(self.max_seqs) if self.slots.is_held(s))

    def nbytes(self) -> int:
        return sum(g.nbytes() for g in self.kv_groups) + sum(
            g.data.numel() * g.data.element_size() for g in self.state_groups)

    def check(self) -> None:
        self.slots.check()
        for g in self.kv_groups:
            g.table.check()
            for s in range(self.max_seqs):
                if not self.slots.is_held(s) and g.table.slot_pages[s]:
                    raise CacheMisuse(f"slot {s} is free but holds pages")
