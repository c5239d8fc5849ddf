"""The library's page pool and cache manager by themselves, without a GPU: the bookkeeping
(which pages are free, who holds which, block tables, state slots), for tests and tools.  The
objects live in the library (``csrc/host/cache.cpp``); these are handles to them."""
from __future__ import annotations

from typing import Any, Dict, List, Optional, Sequence

from ..native import HostError, HostObject


class PageError(RuntimeError):
    pass


def _translate(err: HostError):
    if err.kind == "PageError":
        return PageError(str(err))
    if err.kind in ("ConfigError", "StepError"):
        return ValueError(str(err))
    return RuntimeError(str(err))


class _Host:
    def __init__(self, kind: str, **args):
        try:
            self._obj = HostObject(kind, **args)
        except HostError as err:
            raise _translate(err) from None

    def _call(self, method: str, *args):
        try:
            return self._obj.call(method, *args)
        except HostError as err:
            raise _translate(err) from None


class PagePool(_Host):
    def __init__(self, n_pages: int, page_tokens: int):
        super().__init__("pool", n_pages=n_pages, page_tokens=page_tokens)
        self.n_pages, self.page_tokens = n_pages, page_tokens

    @property
    def n_free(self) -> int:
        return self._call("state")["n_free"]

    @property
    def n_used(self) -> int:
        return self._call("state")["n_used"]

    def allocate(self, count: int) -> Optional[List[int]]:
        return self._call("allocate", count)

    def allocate_tokens(self, n_tokens: int) -> Optional[List[int]]:
        return self._call("allocate_tokens", n_tokens)

    def retain(self, pages: Sequence[int]) -> None:
        self._call("retain", list(pages))

    def release(self, pages: Sequence[int]) -> None:
        self._call("release", list(pages))

    def holders(self, page: int) -> int:
        return self._call("state")["holders"][page]

    def check(self) -> None:
        self._call("check")


def cache_layout(kv_groups=(), kv_of_step=None, states=()) -> Dict[str, Any]:
    """A cache layout as the library reads it.  ``kv_groups``: (kv_heads, head_dim, window or None,
    layers); ``kv_of_step``: {run-order entry: (group, layer in group, writes)}; ``states``:
    (run-order entry, name, shape[, dtype])."""
    return {"kv_groups": [{"kv_heads": g[0], "head_dim": g[1], "window": g[2], "layers": g[3]} for g in kv_groups],
            "kv_of_step": [{"step": s, "group": u[0], "layer": u[1], "writes": u[2]}
                           for s, u in (kv_of_step or {}).items()],
            "states": [{"step": s[0], "name": s[1], "shape": list(s[2]), "dtype": s[3] if len(s) > 3 else "float32"}
                       for s in states]}


class CacheManager(_Host):
    """The bookkeeping of the cache manager (no device memory)."""

    def __init__(self, layout: Dict[str, Any], *, page_tokens: int, n_pages, max_requests: int, max_context: int):
        super().__init__("cache", layout=layout, page_tokens=page_tokens, n_pages=n_pages,
                         max_requests=max_requests, max_context=max_context)
        self.page_tokens, self.max_requests, self.max_context = page_tokens, max_requests, max_context
        self.null_slot = max_requests

    @property
    def handle(self) -> int:
        return self._obj.handle

    def state(self) -> Dict[str, Any]:
        return self._call("state")

    @property
    def n_free_slots(self) -> int:
        return self.state()["free_slots"]

    def open_slots(self) -> List[int]:
        return self.state()["open_slots"]

    def free_pages(self) -> List[int]:
        return self.state()["free_pages"]

    def open(self) -> Optional[int]:
        slot = self._call("open")
        return None if slot < 0 else slot

    def close(self, slot: int) -> None:
        self._call("close", slot)

    def prepare(self, slot: int, start_pos: int, n_new: int) -> bool:
        return self._call("prepare", slot, start_pos, n_new)

    def covers(self, slot: int, start_pos: int, n_new: int) -> bool:
        return self._call("covers", slot, start_pos, n_new)

    def pages_needed(self, slot: int, start_pos: int, n_new: int) -> List[int]:
        return self._call("pages_needed", slot, start_pos, n_new)

    def pages_held(self, slot: int) -> List[List[int]]:
        return self._call("pages_held", slot)

    def table(self, group: int, slot: int, logical: int) -> int:
        return self._call("table", group, slot, logical)

    def drain_table_updates(self):
        return [[tuple(u) for u in g] for g in self._call("drain")]

    def requeue_table_updates(self, updates) -> None:
        self._call("requeue", [[list(u) for u in g] for g in updates])

    def check(self) -> None:
        self._call("check")


__all__ = ["PagePool", "PageError", "CacheManager", "cache_layout"]
