"""The cache manager: pages of keys and values, block tables, and state slots.

Layers are put into *groups* by what they need (``KVNeed``: heads, head size, all
keys or a window of them).  Every group has its own page pool, its own K and V
storage and its own block table per request; one page id of a group covers all the
layers of that group.  The reference has one such group, for attention
(include/celeg/runtime/cache/page_layout.hpp:14-142;
src/backend/cuda/memory/paged_kv.cu:10-130), and keeps the short convolution's
state per lane (include/celeg/detail/model/layer_state.hpp:180-187); here state of
fixed size per request lives in *slots*: one row of one buffer per request, zeroed
when the request starts, with a region for every layer that declared a need.

Storage of a group: K ``[pages + 1, layers, kv_heads, page_tokens, head_dim]`` and V
``[pages + 1, layers, kv_heads, head_dim, page_tokens]`` (transposed inside a page: the
layout the matrix-core attention kernel reads without shuffling).  The extra last page is never handed out: rows that pad a batch to a
fixed size write there.  Likewise the last slot (``null_slot``) is never given to a
request.

Pages are given back when a request closes, and, in a window group, as soon as
every position of a page lies before the window of the next token.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..parts.base import KVNeed, StateNeed
from .pages import PageError, PagePool


@dataclass
class CacheLayout:
    """What a model's run order needs.  ``kv_of_step[i] = (group, layer_in_group,
    writes)`` for the entries of the run order whose mixer uses keys and values;
    ``states`` lists (run-order entry, need)."""
    kv_groups: List[KVNeed] = field(default_factory=list)
    group_layers: List[int] = field(default_factory=list)
    kv_of_step: Dict[int, Tuple[int, int, bool]] = field(default_factory=dict)
    states: List[Tuple[int, StateNeed]] = field(default_factory=list)

    def kv_bytes_per_token(self, itemsize: int) -> int:
        return sum(2 * n * g.kv_heads * g.head_dim * itemsize
                   for g, n in zip(self.kv_groups, self.group_layers))


class KVView:
    """What a mixer's kernels need to reach one layer's keys and values."""
    __slots__ = ("k", "v", "layer", "n_layers", "table", "page_tokens", "kv_heads",
                 "head_dim", "group")

    def __init__(self, k, v, layer, n_layers, table, page_tokens, kv_heads, head_dim, group):
        self.k, self.v, self.layer, self.n_layers = k, v, layer, n_layers
        self.table, self.page_tokens = table, page_tokens
        self.kv_heads, self.head_dim, self.group = kv_heads, head_dim, group


class LayerCache:
    """The cache of one entry of the run order."""
    __slots__ = ("kv", "writes_kv", "states")

    def __init__(self, kv: Optional[KVView], writes_kv: bool, states: Dict[str, torch.Tensor]):
        self.kv, self.writes_kv, self.states = kv, writes_kv, states


class _Group:
    def __init__(self, need: KVNeed, n_layers: int, n_pages: int, page_tokens: int,
                 n_slots: int, max_pages_per_request: int, device, dtype):
        self.need = need
        self.n_layers = n_layers
        self.pool = PagePool(n_pages, page_tokens)
        self.k = torch.zeros((n_pages + 1, n_layers, need.kv_heads, page_tokens, need.head_dim),
                             dtype=dtype, device=device)
        self.v = torch.zeros((n_pages + 1, n_layers, need.kv_heads, need.head_dim, page_tokens),
                             dtype=dtype, device=device)
        self.trash_page = n_pages
        # block tables: row = slot, column = logical page (position // page_tokens)
        self.table_host = np.full((n_slots + 1, max_pages_per_request), -1, dtype=np.int32)
        self.table_host[n_slots, :] = self.trash_page
        self.table = torch.from_numpy(self.table_host.copy()).to(device)
        # per slot: physical page of each logical page (None once given back)
        self.pages: List[List[Optional[int]]] = [[] for _ in range(n_slots)]
        self.first_live: List[int] = [0] * n_slots
        self.updates: Dict[Tuple[int, int], int] = {}


class CacheManager:
    def __init__(self, layout: CacheLayout, *, page_tokens: int, n_pages,
                 max_requests: int, max_context: int, device, dtype):
        if page_tokens <= 0 or max_requests <= 0 or max_context <= 0:
            raise ValueError("cache manager: page_tokens, max_requests and max_context "
                             "must be positive")
        self.layout = layout
        self.page_tokens = page_tokens
        self.max_requests = max_requests
        self.max_context = max_context
        self.null_slot = max_requests
        self.device = device
        self.dtype = dtype
        self.max_pages_per_request = (max_context + page_tokens - 1) // page_tokens
        if isinstance(n_pages, int):
            n_pages = [n_pages] * len(layout.kv_groups)
        if len(n_pages) != len(layout.kv_groups):
            raise ValueError("cache manager: one page count per group is needed")
        self.groups = [
            _Group(need, layers, pages, page_tokens, max_requests,
                   self.max_pages_per_request, device, dtype)
            for need, layers, pages in zip(layout.kv_groups, layout.group_layers, n_pages)]
        # state slots: one row of bytes per request (+ the null slot)
        self._state_regions: Dict[Tuple[int, str], Tuple[int, StateNeed]] = {}
        offset = 0
        for step, need in layout.states:
            if (step, need.name) in self._state_regions:
                raise ValueError(f"run-order entry {step} declares state '{need.name}' twice")
            itemsize = torch.empty((), dtype=need.dtype).element_size()
            count = int(np.prod(need.shape)) if need.shape else 1
            self._state_regions[(step, need.name)] = (offset, need)
            offset += (count * itemsize + 15) // 16 * 16
        self.slot_bytes = offset
        self.state_buffer = torch.zeros((max_requests + 1, max(offset, 16)),
                                        dtype=torch.uint8, device=device)
        self._state_views: Dict[Tuple[int, str], torch.Tensor] = {}
        for key, (off, need) in self._state_regions.items():
            itemsize = torch.empty((), dtype=need.dtype).element_size()
            count = int(np.prod(need.shape)) if need.shape else 1
            flat = self.state_buffer[:, off:off + count * itemsize].view(need.dtype)
            self._state_views[key] = flat.view((max_requests + 1,) + tuple(need.shape))
        self._free_slots: List[int] = list(range(max_requests - 1, -1, -1))
        self._open: Dict[int, int] = {}  # slot -> tokens covered by pages so far

    # ------------------------------------------------------------------ requests
    @property
    def n_free_slots(self) -> int:
        return len(self._free_slots)

    def open_slots(self) -> List[int]:
        return sorted(self._open)

    def open(self) -> Optional[int]:
        """A slot for a new request, its state zeroed; None if every slot is taken."""
        if not self._free_slots:
            return None
        slot = self._free_slots.pop()
        self._open[slot] = 0
        if self.slot_bytes:
            self.state_buffer[slot].zero_()
        return slot

    def close(self, slot: int) -> None:
        """Give back everything the request holds."""
        if slot not in self._open:
            raise PageError(f"slot {slot} is not open")
        for g in self.groups:
            live = [p for p in g.pages[slot] if p is not None]
            g.pool.release(live)
            for idx, p in enumerate(g.pages[slot]):
                if p is not None:
                    g.table_host[slot, idx] = -1
            g.pages[slot] = []
            g.first_live[slot] = 0
        del self._open[slot]
        self._free_slots.append(slot)

    def pages_needed(self, slot: int, start_pos: int, n_new: int) -> List[int]:
        """New pages each group would need for positions [start_pos, start_pos + n_new)."""
        top = (start_pos + n_new - 1) // self.page_tokens
        return [max(0, top + 1 - len(g.pages[slot])) for g in self.groups]

    def prepare(self, slot: int, start_pos: int, n_new: int) -> bool:
        """Make the request's pages cover positions [start_pos, start_pos + n_new), after
        giving back the pages that no later token can see (window groups).  False, with
        no page taken, if some pool has too few free pages."""
        if slot not in self._open:
            raise PageError(f"slot {slot} is not open")
        if n_new <= 0 or start_pos < 0:
            raise ValueError("prepare: n_new must be positive and start_pos >= 0")
        if start_pos + n_new > self.max_context:
            raise ValueError(f"context limit reached: {start_pos + n_new} > {self.max_context}")
        for g in self.groups:
            if g.need.window is not None:
                self._release_passed(g, slot, start_pos)
        need = self.pages_needed(slot, start_pos, n_new)
        if any(n > g.pool.n_free for n, g in zip(need, self.groups)):
            return False
        for n, g in zip(need, self.groups):
            new_pages = g.pool.allocate(n)
            for p in new_pages:
                idx = len(g.pages[slot])
                g.pages[slot].append(p)
                g.table_host[slot, idx] = p
                g.updates[(slot, idx)] = p
        self._open[slot] = max(self._open[slot], start_pos + n_new)
        return True

    def _release_passed(self, g: _Group, slot: int, next_pos: int) -> None:
        lowest_needed = max(0, next_pos - g.need.window + 1)
        first_needed_page = lowest_needed // self.page_tokens
        pages = g.pages[slot]
        for idx in range(g.first_live[slot], min(first_needed_page, len(pages))):
            if pages[idx] is not None:
                g.pool.release([pages[idx]])
                pages[idx] = None
                g.table_host[slot, idx] = -1
        g.first_live[slot] = max(g.first_live[slot], min(first_needed_page, len(pages)))

    def covers(self, slot: int, start_pos: int, n_new: int) -> bool:
        """Whether every position a step over [start_pos, start_pos+n_new) reads or writes
        has a page in every group."""
        if slot not in self._open:
            return False
        top = (start_pos + n_new - 1) // self.page_tokens
        for g in self.groups:
            pages = g.pages[slot]
            if top >= len(pages):
                return False
            low = 0 if g.need.window is None else max(0, start_pos - g.need.window + 1)
            for idx in range(low // self.page_tokens, top + 1):
                if pages[idx] is None:
                    return False
        return True

    def pages_held(self, slot: int) -> List[List[int]]:
        return [[p for p in g.pages[slot] if p is not None] for g in self.groups]

    def free_pages(self) -> List[int]:
        return [g.pool.n_free for g in self.groups]

    # ------------------------------------------------------------------ device side
    def drain_table_updates(self) -> List[List[Tuple[int, int, int]]]:
        """Pages added to the block tables since the last call, per group, in order:
        (slot, logical page, physical page), at most one per table entry.  The step function ships them to the device
        with the step's other metadata.  Entries of pages that were given back are not
        cleared on the device: no kernel reads a table beyond the positions of its rows
        (the host copy ``table_host`` does show -1 there)."""
        out = []
        for g in self.groups:
            out.append([(slot, idx, page) for (slot, idx), page in g.updates.items()])
            g.updates = {}
        return out

    def requeue_table_updates(self, updates: Sequence[Sequence[Tuple[int, int, int]]]) -> None:
        """Put drained updates back (the step they were to travel with was refused).  A newer
        update of the same table entry wins."""
        for g, drained in zip(self.groups, updates):
            fresh = g.updates
            g.updates = {(slot, idx): page for slot, idx, page in drained}
            g.updates.update(fresh)

    def layer_cache(self, step: int) -> LayerCache:
        kv = None
        writes = False
        if step in self.layout.kv_of_step:
            gi, layer, writes = self.layout.kv_of_step[step]
            g = self.groups[gi]
            kv = KVView(g.k, g.v, layer, g.n_layers, g.table, self.page_tokens,
                        g.need.kv_heads, g.need.head_dim, gi)
        states = {name: view for (s, name), view in self._state_views.items() if s == step}
        return LayerCache(kv, writes, states)

    # ------------------------------------------------------------------ checks
    def check(self) -> None:
        """No page lost, none held twice; slots free or open, never both."""
        for g in self.groups:
            g.pool.check()
            seen = {}
            for slot in range(self.max_requests):
                for p in g.pages[slot]:
                    if p is None:
                        continue
                    if slot not in self._open:
                        raise PageError(f"closed slot {slot} still holds page {p}")
                    if p in seen:
                        raise PageError(f"page {p} is held by slots {seen[p]} and {slot}")
                    seen[p] = slot
            for p in range(g.pool.n_pages):
                if (g.pool.holders(p) > 0) != (p in seen):
                    raise PageError(f"page {p}: pool and block tables disagree")
        if set(self._free_slots) & set(self._open):
            raise PageError("a slot is both free and open")
        if len(set(self._free_slots)) != len(self._free_slots):
            raise PageError("a slot is free twice")
        if len(self._free_slots) + len(self._open) != self.max_requests:
            raise PageError("a slot is lost")

    def memory_bytes(self) -> Dict[str, int]:
        kv = sum(g.k.numel() * g.k.element_size() * 2 for g in self.groups)
        return {"kv_cache": kv, "state": self.state_buffer.numel(),
                "block_tables": sum(g.table.numel() * 4 for g in self.groups)}
