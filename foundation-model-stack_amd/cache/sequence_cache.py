"""The cache of a model: a slot per live sequence, keys and values per layer
in pages, and a fixed-size state area per slot.

* A *slot* stands for one sequence: its length, its pages in every group, its
  row in every state tensor.  Slots are handed out when a batch starts and
  given back when a sequence ends; the next batch uses them again.
* A *group* collects the schedule entries whose mixers need the same kind of
  storage (same kv heads, head size and window).  Every group has storage and
  a page pool of its own: a windowed group gives pages back as soon as no
  later query can see them, a full group keeps them to the end.
* *State* is per-sequence memory of fixed size that a mixer declares (the
  reference's example is the convolution and scan state of its SSM mixer,
  fms/modules/ssm.py:98-139).  It is zeroed when a slot is handed out.

Storage layout of a group, for the kernels (csrc/rope.hip):
  keys   [entry][page][kv head][token in page][head_dim]
  values [entry][page][kv head][head_dim][token in page]
"""

from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .pages import PAGE_TOKENS, CacheFull, PagePool, pages_for


@dataclasses.dataclass(frozen=True)
class KVNeed:
    """What an attention-like mixer asks of the cache."""

    kv_heads: int
    head_dim: int
    window: int = 0  # 0: all keys; w > 0: the last w keys


@dataclasses.dataclass(frozen=True)
class StateNeed:
    """Fixed-size memory per sequence: name -> (shape, dtype name)."""

    tensors: Tuple[Tuple[str, Tuple[int, ...], str], ...]


class KVGroup:
    def __init__(self, need: KVNeed, entries: List[int], n_pages: int):
        self.need = need
        self.entries = list(entries)
        self.pool = PagePool(n_pages)
        self.keys: Optional[torch.Tensor] = None
        self.values: Optional[torch.Tensor] = None
        # slot -> logical page list; -1 marks a page given back because the window has passed it
        self.pages: Dict[int, List[int]] = {}
        # slot -> index of the slot's first page that has not been given back (everything before it is -1): a
        # window's releases are looked for from there, not from the sequence's start, at every step
        self.first_held: Dict[int, int] = {}

    def allocate_storage(self, dtype: torch.dtype, device) -> None:
        n, K, D = self.pool.n_pages, self.need.kv_heads, self.need.head_dim
        # zero-filled: the attention kernels multiply masked-out positions by zero
        self.keys = torch.zeros(len(self.entries), n, K, PAGE_TOKENS, D, dtype=dtype, device=device)
        self.values = torch.zeros(len(self.entries), n, K, D, PAGE_TOKENS, dtype=dtype, device=device)

    def bytes_per_token(self, itemsize: int) -> int:
        return 2 * len(self.entries) * self.need.kv_heads * self.need.head_dim * itemsize


class SequenceCache:
    def __init__(
        self,
        kv_needs: Sequence[Tuple[int, KVNeed]],
        state_needs: Sequence[Tuple[int, StateNeed]],
        max_tokens: int,
        max_slots: int,
        max_seq_len: int,
        dtype: torch.dtype = torch.float32,
        device=None,
    ):
        """kv_needs / state_needs: (schedule entry, need) pairs of the entries that own storage.

        max_tokens: the most tokens live sequences hold at any time, each sequence's count
        rounded up to a page.  device None keeps the bookkeeping only (no storage).
        """
        if max_tokens <= 0 or max_slots <= 0:
            raise ValueError("a cache needs room for at least one token and one slot")
        self.max_tokens = pages_for(max_tokens) * PAGE_TOKENS
        self.max_slots = max_slots
        self.max_seq_len = max_seq_len
        self.dtype, self.device = dtype, device
        n_pages = pages_for(max_tokens)

        self.groups: List[KVGroup] = []
        self.group_of_entry: Dict[int, Tuple[int, int]] = {}  # entry -> (group index, index inside the group)
        by_need: Dict[KVNeed, KVGroup] = {}
        for entry, need in kv_needs:
            group = by_need.get(need)
            if group is None:
                group = by_need[need] = KVGroup(need, [], n_pages)
                self.groups.append(group)
            self.group_of_entry[entry] = (self.groups.index(group), len(group.entries))
            group.entries.append(entry)

        self.state: Dict[int, Dict[str, torch.Tensor]] = {}
        self._state_needs = list(state_needs)

        self._free_slots: List[int] = list(range(max_slots - 1, -1, -1))
        self._live: Dict[int, int] = {}  # slot -> length
        self._clock = 0
        self._stamp: Dict[int, int] = {}  # slot -> value of the clock at its last change
        if device is not None:
            for group in self.groups:
                group.allocate_storage(dtype, device)
            for entry, need in self._state_needs:
                self.state[entry] = {
                    name: torch.zeros((max_slots, *shape), dtype=getattr(torch, dt), device=device)
                    for name, shape, dt in need.tensors
                }

    # ---- slots -----------------------------------------------------------
    def alloc_slot(self) -> int:
        if not self._free_slots:
            raise CacheFull(f"all {self.max_slots} sequence slots are in use")
        slot = self._free_slots.pop()
        if slot in self._live:
            raise AssertionError(f"slot {slot} was free while live")
        self._live[slot] = 0
        self._clock += 1
        self._stamp[slot] = self._clock
        for group in self.groups:
            group.pages[slot] = []
            group.first_held[slot] = 0
        for tensors in self.state.values():
            for t in tensors.values():
                t[slot].zero_()
        return slot

    def free_slot(self, slot: int) -> None:
        if slot not in self._live:
            raise ValueError(f"slot {slot} is not live (freed twice, or never handed out)")
        for group in self.groups:
            for page in group.pages.pop(slot):
                if page >= 0:
                    group.pool.free(page)
            group.first_held.pop(slot, None)
        del self._live[slot]
        del self._stamp[slot]
        self._free_slots.append(slot)

    def live_slots(self) -> List[int]:
        return sorted(self._live)

    def length(self, slot: int) -> int:
        return self._live[slot]

    @property
    def n_free_slots(self) -> int:
        return len(self._free_slots)

    # ---- pages -----------------------------------------------------------
    def pages_needed(self, slot: int, new_tokens: int) -> int:
        """Pages that `new_tokens` more tokens of `slot` take from the pools (the most of any group), counting
        the pages a windowed group gives back first."""
        need = 0
        for _, release, want in self._plan(slot, new_tokens):
            need = max(need, want - len(release))
        return max(need, 0)

    def _plan(self, slot: int, new_tokens: int):
        """For every group: (group, indices of the slot's pages that no query of the step can see any more,
        pages to take).  Changes nothing."""
        if slot not in self._live:
            raise ValueError(f"slot {slot} is not live")
        if new_tokens < 0:
            raise ValueError("a sequence cannot shrink")
        start = self._live[slot]
        new_len = start + new_tokens
        if new_len > self.max_seq_len:
            raise IndexError(f"sequence in slot {slot} would reach {new_len} tokens; the model has {self.max_seq_len} positions")
        plans = []
        for group in self.groups:
            pages = group.pages[slot]
            release = []
            if group.need.window > 0:
                first_visible = max(0, start - group.need.window + 1)
                release = list(range(group.first_held[slot], min(first_visible // PAGE_TOKENS, len(pages))))
            plans.append((group, release, max(0, pages_for(new_len) - len(pages))))
        return plans

    def extend_many(self, slots: Sequence[int], new_tokens: Sequence[int]) -> List[int]:
        """Make room for `new_tokens[b]` more tokens of `slots[b]`, for all of them or for none: the positions
        of each sequence's first new token.  Windowed groups first give back the pages that no query of the
        step can see.  If a sequence would pass the model's positions (IndexError) or a pool runs out
        (CacheFull), no length and no page has changed."""
        if len(set(slots)) != len(slots):
            raise ValueError("a sequence appears twice in one step")
        plans = [self._plan(slot, n) for slot, n in zip(slots, new_tokens)]
        for g, group in enumerate(self.groups):
            want = sum(p[g][2] for p in plans)
            freed = sum(len(p[g][1]) for p in plans)
            if want > group.pool.n_free + freed:
                raise CacheFull(
                    f"the step needs {want} more cache pages of group {g}, {group.pool.n_free + freed} are free "
                    f"of {group.pool.n_pages}")
        starts = []
        for slot, n, plan in zip(slots, new_tokens, plans):
            for group, release, _ in plan:
                pages = group.pages[slot]
                for i in release:
                    group.pool.free(pages[i])
                    pages[i] = -1
                if release:
                    group.first_held[slot] = release[-1] + 1
        for slot, n, plan in zip(slots, new_tokens, plans):
            for group, _, want in plan:
                pages = group.pages[slot]
                for _ in range(want):
                    pages.append(group.pool.alloc())
            starts.append(self._live[slot])
            self._live[slot] += n
            self._clock += 1
            self._stamp[slot] = self._clock
        return starts

    def extend(self, slot: int, new_tokens: int) -> int:
        """Make room for `new_tokens` more tokens of `slot`; returns the position of the first of them.
        Nothing changes if the room cannot be made."""
        return self.extend_many([slot], [new_tokens])[0]

    def stamp(self, slot: int) -> int:
        """A number that changes whenever the slot is handed out or its sequence grows, and never comes back:
        who remembers it can tell whether the sequence is still as they left it."""
        if slot not in self._stamp:
            raise ValueError(f"slot {slot} is not live")
        return self._stamp[slot]

    def pages_held(self, slot: int) -> int:
        """How many pages the slot holds over all groups: it changes when the sequence gets a page and when a
        window gives one back, so whoever keeps a copy of the block tables knows when to read them again."""
        return sum(len(group.pages[slot]) - group.first_held[slot] for group in self.groups)

    def block_table(self, group_index: int, slots: Sequence[int], n_columns: Optional[int] = None) -> torch.Tensor:
        """int32 [len(slots), n_columns] page numbers on the host (unused entries and released pages: -1)."""
        group = self.groups[group_index]
        width = max([len(group.pages[s]) for s in slots] + [1])
        if n_columns is not None:
            if n_columns < width:
                raise ValueError("block table narrower than the longest sequence")
            width = n_columns
        table = torch.full((len(slots), width), -1, dtype=torch.int32)
        for row, slot in enumerate(slots):
            pages = group.pages[slot]
            if pages:
                table[row, : len(pages)] = torch.tensor(pages, dtype=torch.int32)
        return table

    # ---- storage views -----------------------------------------------------
    def kv_of_entry(self, entry: int) -> Tuple[int, torch.Tensor, torch.Tensor]:
        """(group index, keys [pages, K, 64, D], values [pages, K, D, 64]) of a schedule entry."""
        g, i = self.group_of_entry[entry]
        group = self.groups[g]
        return g, group.keys[i], group.values[i]

    def state_of_entry(self, entry: int) -> Dict[str, torch.Tensor]:
        return self.state.get(entry, {})

    def check(self) -> None:
        """Raise if a slot or a page is lost, held twice or free twice."""
        if len(set(self._free_slots)) != len(self._free_slots):
            raise AssertionError("a slot is free twice")
        if set(self._free_slots) & set(self._live):
            raise AssertionError("a slot is both free and live")
        if len(self._free_slots) + len(self._live) != self.max_slots:
            raise AssertionError("a slot is lost")
        for group in self.groups:
            group.pool.check()
            held = [p for pages in group.pages.values() for p in pages if p >= 0]
            if len(held) != len(set(held)):
                raise AssertionError("a page belongs to two sequences")
            if len(held) != group.pool.n_held:
                raise AssertionError("pages held by sequences and by the pool differ")
            if set(group.pages) != set(self._live):
                raise AssertionError("page lists and live slots differ")
            for slot, pages in group.pages.items():
                first = group.first_held[slot]
                if any(p >= 0 for p in pages[:first]) or any(p < 0 for p in pages[first:]):
                    raise AssertionError("released pages are not exactly the pages before the first held one")
