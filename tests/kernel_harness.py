"""What the tests of single kernels stand on: a cache (the library's cache manager for the
bookkeeping, torch tensors for the pages, block tables and state slots) and a step's batch (the
library's batch builder for the layout, torch tensors for the arrays), so that a kernel is
called through ``HipOps`` with the same arrays the engine gives it."""
from types import SimpleNamespace

import numpy as np
import torch

from celeg_amd.cache import CacheManager, cache_layout
from celeg_amd.native import HostObject

DEV = "cuda:0"


class HarnessCache:
    def __init__(self, kv_heads, head_dim, n_layers, dtype, n_pages=64, page_tokens=16, slots=4,
                 states=(), max_context=512, window=None):
        groups = [(kv_heads, head_dim, window, n_layers)] if kv_heads else []
        uses = {i: (0, i, True) for i in range(n_layers)} if kv_heads else {}
        self.manager = CacheManager(cache_layout(groups, uses, [(s, name, shape) for s, name, shape in states]),
                                    page_tokens=page_tokens, n_pages=n_pages, max_requests=slots,
                                    max_context=max_context)
        self.page_tokens, self.null_slot, self.n_groups = page_tokens, slots, len(groups)
        self.pages_per_request = (max_context + page_tokens - 1) // page_tokens
        self.kv = None
        if kv_heads:
            k = torch.zeros(n_pages + 1, n_layers, kv_heads, page_tokens, head_dim, dtype=dtype, device=DEV)
            v = torch.zeros(n_pages + 1, n_layers, kv_heads, head_dim, page_tokens, dtype=dtype, device=DEV)
            table = torch.full((slots + 1, self.pages_per_request), -1, dtype=torch.int32, device=DEV)
            table[slots] = n_pages                        # the null slot's row names the spare page
            self.kv = dict(k=k, v=v, table=table, n_layers=n_layers, page_tokens=page_tokens,
                           kv_heads=kv_heads, head_dim=head_dim, group=0)
        self.states = {(s, name): torch.zeros((slots + 1,) + tuple(shape), device=DEV) for s, name, shape in states}

    # the bookkeeping is the library's
    def open(self):
        slot = self.manager.open()
        for (s, name), t in self.states.items():
            t[slot].zero_()
        return slot

    def close(self, slot):
        self.manager.close(slot)

    def prepare(self, slot, start, n):
        return self.manager.prepare(slot, start, n)

    def pages_held(self, slot):
        return self.manager.pages_held(slot)

    def table_host(self, slot, logical, group=0):
        return self.manager.table(group, slot, logical)

    def layer_cache(self, step):
        kv = SimpleNamespace(layer=step, **self.kv) if self.kv is not None and step < self.kv["n_layers"] else None
        return SimpleNamespace(kv=kv, writes_kv=kv is not None,
                               states={name: t for (s, name), t in self.states.items() if s == step})

    def apply_updates(self):
        for g, updates in enumerate(self.manager.drain_table_updates()):
            for slot, logical, page in updates:
                self.kv["table"][slot, logical] = page


def make_cache(kv_heads, head_dim, n_layers, dtype, **kw):
    return HarnessCache(kv_heads, head_dim, n_layers, dtype, **kw)


def build_batch(ops, cache, entries):
    """The step's arrays on the device, laid out by the library's batch builder; the block-table
    updates since the last step are applied."""
    builder = HostObject("batch", capacity=1 << 16, n_groups=1)
    out = builder.call("build", [{"slot": e.slot, "start_pos": e.start_pos, "tokens": list(e.tokens),
                                  "want": list(e.want)} for e in entries], [[]], {"null_slot": cache.null_slot})
    cache.apply_updates()
    b = SimpleNamespace(**{k: v for k, v in out.items() if not isinstance(v, list)})
    for name in ("token_ids", "positions", "token_seq", "token_slot", "cu_seqlens", "seq_slot", "seq_start",
                 "logit_rows"):
        setattr(b, name, torch.tensor(out[name], dtype=torch.int32, device=DEV))
    b.entry_order = out["entry_order"]
    b.context_bound = 0
    return b, builder
