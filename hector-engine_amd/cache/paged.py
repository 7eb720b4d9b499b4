"""The cache on the device.

Keys and values live in pages of 64 tokens. Layers are partitioned into groups
by what they keep (kv heads, key and value widths, all keys or a window of them); each
group has pools of its own, [runs][pages][kv_heads][elements of a page] for K and for
V, a page as large as the group's mixers ask for (KVNeed.k_elems, KVNeed.v_elems: the order
inside a page is theirs), and one page table [slots][blocks]
shared by its runs. A sequence holds a
slot: its row of every page table, its length, and its row of the fixed-size
state area. Slots and pages go back to the free lists when a sequence ends and
are handed out again, lowest first; nothing is cleared, because attention only
reads positions a sequence has written (the reference argues the same for its
rewind: src/kv_cache.hpp:93-96). The reference's cache is one
[layers][batch][max_seq][kv_heads][head_dim] block with a single position
(src/kv_cache.hpp:161-203); slots, pages and groups are this engine's own.
"""
from __future__ import annotations

import dataclasses

import numpy as np
import torch

from ..parts.base import KVNeed, LayerCache
from .pages import PAGE_TOKENS, CacheError, CacheFull, GroupPages, SlotBook, blocks_for  # noqa: F401


@dataclasses.dataclass
class RunPlan:
    """What one run of the schedule needs from the cache."""

    kv: KVNeed | None          # keys/values it writes (None: none, or it reads another run's)
    cache_from: int | None     # run whose keys/values it reads
    state_bytes: int = 0


class _Group:
    def __init__(self, need: KVNeed, runs: list[int], num_pages: int, max_slots: int,
                 max_blocks: int, dtype, device):
        self.need = need
        self.runs = runs
        # zero-filled once (as the reference's cache is: src/kv_cache.hpp:161-203): a masked
        # key still enters the matrix products with weight 0, so it must never be NaN
        # a page is as large as the mixers of the group say; what lies where inside it is theirs
        self.kpool = torch.zeros((len(runs), num_pages, need.kv_heads, need.k_elems), dtype=dtype, device=device)
        self.vpool = torch.zeros((len(runs), num_pages, need.kv_heads, need.v_elems), dtype=dtype, device=device)
        self.page_table = torch.full((max_slots, max_blocks), -1, dtype=torch.int32, device=device)
        # the same table on the host: a step can take its sequences' rows along with its metadata
        self.host_table = np.full((max_slots, max_blocks), -1, dtype=np.int32)


class PagedCache:
    def __init__(self, plans: list[RunPlan], *, max_tokens: int, max_slots: int,
                 max_seq_len: int, dtype: torch.dtype, device):
        if max_tokens < PAGE_TOKENS:
            raise CacheError(f"max_tokens {max_tokens} is below one page of {PAGE_TOKENS} tokens")
        self.device = device
        self.dtype = dtype
        self.num_pages = max_tokens // PAGE_TOKENS
        self.max_slots = max(1, min(max_slots, self.num_pages))
        self.max_blocks = max(1, min(blocks_for(max_seq_len), self.num_pages))
        self.max_seq_len = self.max_blocks * PAGE_TOKENS
        self.plans = plans

        # group runs by what they keep
        keys: list[KVNeed] = []
        members: list[list[int]] = []
        self.run_group: dict[int, tuple[int, int]] = {}
        for r, plan in enumerate(plans):
            if plan.kv is None:
                continue
            if plan.kv not in keys:
                keys.append(plan.kv)
                members.append([])
            gi = keys.index(plan.kv)
            self.run_group[r] = (gi, len(members[gi]))
            members[gi].append(r)
        for r, plan in enumerate(plans):
            if plan.cache_from is not None:
                if plan.cache_from not in self.run_group or plan.cache_from >= r:
                    raise CacheError(f"run {r} reads the cache of run {plan.cache_from}, "
                                     "which is not an earlier run with a cache of its own")
        self.groups = [_Group(k, m, self.num_pages, self.max_slots, self.max_blocks, dtype, device)
                       for k, m in zip(keys, members)]
        self.book = SlotBook(self.max_slots, self.max_blocks,
                             [GroupPages(self.num_pages, k.window, f"{i}") for i, k in enumerate(keys)])

        # fixed-size per-sequence state: one row per slot, one span per run
        self.state_offsets: list[int] = []
        off = 0
        for plan in plans:
            self.state_offsets.append(off)
            off += (plan.state_bytes + 255) // 256 * 256
        self.state_bytes_per_slot = off
        self.state = torch.zeros((self.max_slots, off), dtype=torch.uint8, device=device) if off else None

    # -- slots --------------------------------------------------------------
    def acquire(self) -> int:
        slot = self.book.acquire()
        if self.state is not None:
            self.state[slot].zero_()
        return slot

    def release(self, slot: int) -> None:
        self._clear(self.book.release(slot))

    def truncate(self, slot: int, new_length: int) -> None:
        """Keeps the first new_length tokens of the slot and gives back the pages beyond
        (cache/pages.py: SlotBook.truncate). A model that keeps fixed-size state per
        sequence cannot be rewound: the state has seen the dropped tokens."""
        if self.state is not None and new_length < self.length(slot):
            raise CacheError(f"slot {slot}: a model with per-sequence state cannot be truncated")
        self._clear(self.book.truncate(slot, new_length))

    def length(self, slot: int) -> int:
        try:
            return self.book.length[slot]
        except KeyError:
            raise CacheError(f"slot {slot} is not held") from None

    @property
    def free_pages(self) -> int:
        return min((g.pool.available for g in self.book.groups), default=self.num_pages)

    # -- pages --------------------------------------------------------------
    def reserve(self, growth: list[tuple[int, int]]) -> None:
        """growth: (slot, new length) for every sequence of a step. Either all get
        their pages or none does."""
        for s, n in growth:            # every check before any page is taken
            if blocks_for(n) > self.max_blocks:
                raise CacheFull(f"slot {s}: {n} tokens exceed the longest sequence the cache was "
                                f"built for ({self.max_seq_len})")
        need = sum(self.book.pages_needed(s, n) for s, n in growth)
        for g in self.book.groups:
            if need > g.pool.available:
                raise CacheFull(f"the step needs {need} more pages of {PAGE_TOKENS} tokens per "
                                f"group, {g.pool.available} are free")
        if need == 0:       # most one-token steps: every new position already has its page
            for s, n in growth:
                if n < self.book.length[s]:
                    raise CacheError(f"slot {s}: cannot shrink from {self.book.length[s]} to {n}")
            return
        added = []
        for s, n in growth:
            added += self.book.reserve(s, n)
        self._write(added)

    def commit(self, growth: list[tuple[int, int]]) -> None:
        cleared = []
        for s, n in growth:
            cleared += self.book.commit(s, n)
        self._clear(cleared)

    def _write(self, entries) -> None:
        by_group: dict[int, tuple[list, list]] = {}
        for gi, slot, block, page in entries:
            idx, val = by_group.setdefault(gi, ([], []))
            idx.append(slot * self.max_blocks + block)
            val.append(page)
        for gi, (idx, val) in by_group.items():
            self.groups[gi].host_table.reshape(-1)[idx] = val
            packed = torch.tensor([idx, val], dtype=torch.int64).to(self.device)
            self.groups[gi].page_table.view(-1).index_copy_(0, packed[0], packed[1].to(torch.int32))

    def _clear(self, entries) -> None:
        self._write([(gi, slot, block, -1) for gi, slot, block in entries])

    def rows_of_tables(self, slots: list[int], out: np.ndarray) -> None:
        """out[g, r, :] = the page table row of slots[r] in group g (int32 [groups, rows or more,
        max_blocks]; rows beyond the slots keep what they hold)."""
        for gi, g in enumerate(self.groups):
            out[gi, :len(slots)] = g.host_table[slots]

    # -- views for the layers -----------------------------------------------
    def layer_cache(self, run: int) -> LayerCache:
        plan = self.plans[run]
        src = run if plan.kv is not None else plan.cache_from
        state = None
        if plan.state_bytes:
            o = self.state_offsets[run]
            state = self.state[:, o:o + plan.state_bytes]
        if src is None:
            return LayerCache(None, None, None, False, state)
        gi, pi = self.run_group[src]
        g = self.groups[gi]
        return LayerCache(g.kpool[pi], g.vpool[pi], g.page_table, plan.kv is not None, state)

    def bytes_per_token(self) -> int:
        es = torch.empty((), dtype=self.dtype).element_size()
        return sum(len(g.runs) * g.need.kv_heads * es * (g.need.k_elems + g.need.v_elems) // PAGE_TOKENS
                   for g in self.groups)
