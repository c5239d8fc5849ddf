"""The step function: runs one batch of (request, its next tokens) through the model,
from the cache, and returns the logits at the wanted places.

The reference runs prompt portions and decode tokens in separate passes
(src/backend/cuda/runtime/engine_control.cpp:4-23;
src/backend/cuda/packed/execution.cu:141-224 and 234-384); here one function takes
both in one batch.  Positions are the caller's to keep: ``start_pos`` is an input,
so the scheduler and the trace replay drive the same function.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import time

import torch

from ..cache.manager import CacheManager
from ..parts.base import Runtime
from .batch import TOKEN_FROM_DEVICE, BatchBuilder, StepBatch, StepEntry, packed_layout
from .model import Model


class Workspace:
    """Reusable buffers by name, sized for the largest use so far.  ``generation``
    changes whenever a buffer moves, which invalidates captured graphs."""

    def __init__(self, device):
        self.device = device
        self._flat: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}
        self.generation = 0
        self.frozen = False

    def buf(self, name: str, shape, dtype) -> torch.Tensor:
        count = 1
        for s in shape:
            count *= int(s)
        key = (name, dtype)
        flat = self._flat.get(key)
        if flat is None or flat.numel() < count:
            if self.frozen:
                raise RuntimeError(f"workspace buffer '{name}' would move while a graph is "
                                   "being captured")
            flat = torch.empty(max(count, 1), dtype=dtype, device=self.device)
            self._flat[key] = flat
            self.generation += 1
        return flat[:count].view(tuple(int(s) for s in shape))

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self._flat.values())


class ModelRunner:
    def __init__(self, model: Model, cache: CacheManager, rt: Runtime, *,
                 max_batched_tokens: int):
        self.model = model
        self.cache = cache
        self.rt = rt
        self.max_batched_tokens = max_batched_tokens
        model.bind_cache(cache)
        n_groups = len(cache.groups)
        S = cache.max_requests
        # room for the largest step, with as many table updates as rows plus requests
        self._update_room = max_batched_tokens // cache.page_tokens + 2 * S + 8
        _, ints = packed_layout(max_batched_tokens, S, max_batched_tokens,
                                [self._update_room] * n_groups)
        self.builder = BatchBuilder(rt.device, ints, n_groups,
                                    pin=torch.device(rt.device).type == "cuda")
        self.steps_run = 0
        self.use_graphs = True
        self._graphs: Dict[tuple, tuple] = {}
        self._portion_graphs: Dict[tuple, tuple] = {}
        self._mixed_graphs: Dict[tuple, tuple] = {}
        self.captures = 0              # recordings made, and the time they took
        self._weights = None           # number of weights, counted at first need
        self.capture_seconds = 0.0
        self._portion_seen: Dict[tuple, int] = {}
        self._token_source: Optional[torch.Tensor] = None
        self._buckets = sorted({min(1 << i, S) for i in range(0, 12)})
        self.last_batch: Optional[StepBatch] = None

    # ------------------------------------------------------------------ checks
    def _validate(self, entries: Sequence[StepEntry]) -> None:
        if not entries:
            raise ValueError("step: no entries")
        if len(entries) > self.cache.max_requests:
            raise ValueError(f"step: {len(entries)} requests exceed max_requests "
                             f"{self.cache.max_requests}")
        seen = set()
        total = 0
        vocab = self.model.spec.vocab_size
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise ValueError("step: an entry has no tokens")
            if e.slot in seen:
                raise ValueError(f"step: slot {e.slot} appears twice in one step")
            seen.add(e.slot)
            if e.start_pos < 0 or e.start_pos + n > self.cache.max_context:
                raise ValueError(f"context limit reached: position {e.start_pos + n} exceeds "
                                 f"{self.cache.max_context}")
            if n == 1:
                in_range = 0 <= e.tokens[0] < vocab or \
                    (e.tokens[0] == TOKEN_FROM_DEVICE and self._token_source is not None)
            else:
                toks = np.asarray(e.tokens)
                in_range = toks.min() >= 0 and toks.max() < vocab
            if not in_range:
                raise ValueError(f"step: token id out of range [0, {vocab})")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise ValueError(f"wanted place {w} is outside the entry's {n} tokens")
            if not self.cache.covers(e.slot, e.start_pos, n):
                raise ValueError(f"step: the pages of slot {e.slot} do not cover positions "
                                 f"[{e.start_pos}, {e.start_pos + n})")
            total += n
        if total > self.max_batched_tokens:
            raise ValueError(f"step: {total} tokens exceed max_batched_tokens "
                             f"{self.max_batched_tokens}")

    # ------------------------------------------------------------------ the step
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Logits, 32-bit [number of wanted places, vocab], in the order of the entries
        and of each entry's ``want``.  The tensor is a view of a reused buffer: it holds
        until the next step."""
        self._validate(entries)
        if self._graph_applies(entries):
            return self._step_from_graph(entries)
        portion = self._portion_shape(entries)
        if portion is not None:
            return self._portion_from_graph(entries, portion)
        mixed = self._mixed_shape(entries)
        if mixed is not None:
            return self._mixed_from_graph(entries, mixed)
        updates = self._drain_updates([self._update_room] * len(self.cache.groups))
        batch = self._build(entries, updates, null_slot=self.cache.null_slot)
        self._begin_step(batch)
        self.last_batch = batch
        logits = self.model.forward(batch, self.rt)
        self.steps_run += 1
        return logits

    # ------------------------------------------------------------------ captured decode steps
    # A step in which every request brings one token and wants its logits is launch-bound:
    # it is captured once per batch-size bucket as a HIP graph and replayed (the reference
    # captures its decode step likewise, src/backend/cuda/model/execution.cu:168-246).
    # Rows that pad the batch to the bucket use the null slot and the spare page, so they
    # touch no request's cache.  Capture and its warm-up run on such padding rows only:
    # a request's state is never advanced twice.
    def _graph_applies(self, entries: Sequence[StepEntry]) -> bool:
        if not self.use_graphs or torch.device(self.rt.device).type != "cuda" \
                or not self.model.graph_safe:
            return False
        if len(entries) > self._buckets[-1]:
            return False
        return all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries)

    # A recorded step's launches are fixed, and the attention over few requests sizes its grid
    # by the context: a graph is therefore good up to a bound on the context, and there is one
    # per (batch-size bucket, bound).
    CONTEXT_BOUNDS = (4096, 16384, 65536)

    def _context_bound(self, entries: Sequence[StepEntry]) -> int:
        longest = max(e.start_pos + len(e.tokens) for e in entries)
        for bound in self.CONTEXT_BOUNDS:
            if longest <= bound:
                return min(bound, self.cache.max_context)
        return self.cache.max_context

    def _step_from_graph(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        S = len(entries)
        bucket = next(b for b in self._buckets if b >= S)
        bound = self._context_bound(entries)
        caps = [bucket + 8] * len(self.cache.groups)
        captured = self._graphs.get((bucket, bound))
        if captured is None or captured[2] != self.rt.ws.generation:
            captured = self._capture(bucket, caps, bound)
        updates = self._drain_updates(caps)
        batch = self._build(entries, updates, pad_to=bucket,
                            null_slot=self.cache.null_slot, update_caps=caps)
        self.last_batch = batch
        captured[0].replay()
        self.steps_run += 1
        return captured[1][:S]

    def _capture(self, bucket: int, caps, bound: int):
        empty = [[] for _ in self.cache.groups]

        def make_batch():
            batch = self.builder.build([], empty, pad_to=bucket, null_slot=self.cache.null_slot,
                                       update_caps=caps)
            batch.context_bound = bound
            return batch
        captured = self._capture_batch(make_batch)
        self._graphs[(bucket, bound)] = captured
        return captured

    # ------------------------------------------------------------------ captured portions
    # A step that is one portion of one prompt launches some 150 kernels and is bound by
    # the host's launches at this model size.  Portions of a size that has come before (the
    # token budget makes long prompts arrive in equal portions) are replayed from a graph
    # captured for that size, on the null slot like the decode graphs.
    PORTION_GRAPHS = 8          # sizes kept
    PORTION_MIN_TOKENS = 32
    LONG_CONTEXT = 4096

    def _portion_shape(self, entries: Sequence[StepEntry]):
        if not self.use_graphs or torch.device(self.rt.device).type != "cuda" \
                or not self.model.graph_safe or len(entries) != 1:
            return None
        e = entries[0]
        n = len(e.tokens)
        if n < self.PORTION_MIN_TOKENS:
            return None
        want = list(e.want)
        if want not in ([], [n - 1]):
            return None
        # (the attention over a portion's rows chooses its tiles by the context too: a long one or not)
        shape = (n, len(want), e.start_pos + n >= self.LONG_CONTEXT)
        if shape not in self._portion_graphs:
            seen = self._portion_seen.get(shape, 0) + 1
            self._portion_seen[shape] = seen
            if seen < 2 or len(self._portion_graphs) >= self.PORTION_GRAPHS:
                return None
        return shape

    def _portion_from_graph(self, entries: Sequence[StepEntry], shape) -> torch.Tensor:
        n, n_want, long_context = shape
        caps = [n // self.cache.page_tokens + 10] * len(self.cache.groups)
        captured = self._portion_graphs.get(shape)
        if captured is None or captured[2] != self.rt.ws.generation:
            null = [StepEntry(self.cache.null_slot, 0, [0] * n, [n - 1] if n_want else [])]

            def make_batch():
                batch = self.builder.build(null, [[] for _ in self.cache.groups],
                                           null_slot=self.cache.null_slot, update_caps=caps)
                batch.context_bound = 2 * self.LONG_CONTEXT if long_context else 0
                return batch
            captured = self._capture_batch(make_batch)
            self._portion_graphs[shape] = captured
        updates = self._drain_updates(caps)
        batch = self._build(entries, updates, null_slot=self.cache.null_slot, update_caps=caps)
        self.last_batch = batch
        captured[0].replay()
        self.steps_run += 1
        return captured[1]

    # ------------------------------------------------------------------ captured mixed steps
    # Under a token budget the steady state of serving is a step of a few portions of prompts
    # (of the portion size) beside the single tokens of the decoding requests: some 150
    # launches again, several times the GPU's time for them at small model sizes.  Such steps
    # are replayed from a graph per (bucket of single rows, sizes of the portions in their
    # order, bound on the context); single rows are padded to the bucket with null-slot rows,
    # which lie between the real single rows and the portions.  Recording costs several
    # steps' time, so the shapes are kept few: coarse buckets (a padding row costs little
    # beside a portion), and every portion's last row gets logits, wanted or not.
    MIXED_GRAPHS = 16
    MIXED_MAX_PORTIONS = 4
    MIXED_BUCKETS = (4, 16, 64, 256)
    MIXED_SEEN_BEFORE_RECORDING = 8      # shapes of a passing phase are not worth a recording
    # A recording costs several steps' time and only pays where the host's launches, not the
    # GPU, bound the step: where the step's products (two operations per row and weight, at
    # the rate the library reaches on so few rows) take less time than its launches (some ten
    # a layer).  Measured at the 350M shape: 480 rows 2.4 ms a step eager, 1.8 replayed;
    # 2,048 rows are bound by the GPU either way, and so are 544 rows at the 2.6B shape.
    HOST_SECONDS_PER_LAUNCH = 14e-6
    LAUNCHES_PER_LAYER = 10
    FEW_ROWS_FLOPS_PER_SECOND = 400e12

    def _bound_by_launches(self, rows: int) -> bool:
        if self._weights is None:
            self._weights = sum(int(np.prod(w.shape)) for w in self.model.expected_tensors().values())
        gpu = 2.0 * rows * self._weights / self.FEW_ROWS_FLOPS_PER_SECOND
        host = self.HOST_SECONDS_PER_LAUNCH * self.LAUNCHES_PER_LAYER * len(self.model.spec.order)
        return gpu < host

    def _mixed_shape(self, entries: Sequence[StepEntry]):
        if not self.use_graphs or torch.device(self.rt.device).type != "cuda" \
                or not self.model.graph_safe or len(entries) < 2:
            return None
        portions = []
        n_single = 0
        for e in entries:
            n = len(e.tokens)
            want = list(e.want)
            if n == 1:
                if want != [0]:
                    return None
                n_single += 1
            else:
                if n < self.PORTION_MIN_TOKENS or want not in ([], [n - 1]):
                    return None
                portions.append(n)
        limit = self._buckets[-1]
        if not portions or len(portions) > self.MIXED_MAX_PORTIONS or n_single > limit \
                or not self._bound_by_launches(n_single + sum(portions)):
            return None
        bucket = next((min(b, limit) for b in self.MIXED_BUCKETS if b >= n_single), limit)
        shape = (bucket, tuple(portions), self._context_bound(entries))
        if shape not in self._mixed_graphs:
            seen = self._portion_seen.get(shape, 0) + 1
            self._portion_seen[shape] = seen
            if seen < self.MIXED_SEEN_BEFORE_RECORDING or len(self._mixed_graphs) >= self.MIXED_GRAPHS:
                return None
        return shape

    def _mixed_from_graph(self, entries: Sequence[StepEntry], shape) -> torch.Tensor:
        bucket, portions, bound = shape
        room = bucket + 8 + sum(n // self.cache.page_tokens + 10 for n in portions)
        caps = [room] * len(self.cache.groups)
        captured = self._mixed_graphs.get(shape)
        if captured is None or captured[2] != self.rt.ws.generation:
            null = [StepEntry(self.cache.null_slot, 0, [0] * n, [n - 1]) for n in portions]

            def make_batch():
                batch = self.builder.build(null, [[] for _ in self.cache.groups],
                                           null_slot=self.cache.null_slot, update_caps=caps,
                                           pad_singles_to=bucket)
                batch.context_bound = bound
                return batch
            captured = self._capture_batch(make_batch)
            self._mixed_graphs[shape] = captured
        updates = self._drain_updates(caps)
        # every portion's last row gets logits, as in the recording; those nobody wants lie
        # behind the wanted ones
        batch = self._build(entries, updates, null_slot=self.cache.null_slot, update_caps=caps,
                            pad_singles_to=bucket, last_rows_too=True)
        self.last_batch = batch
        captured[0].replay()
        self.steps_run += 1
        return captured[1][:sum(len(e.want) for e in entries)]

    def _capture_batch(self, make_batch):
        """Warm-up run and capture of the model's forward over the batch ``make_batch()``
        builds (of null-slot rows only): (graph, logits, workspace generation)."""
        started = time.perf_counter()
        self.captures += 1
        batch = make_batch()
        self._begin_step(batch)
        self.model.forward(batch, self.rt)          # warm-up: buffers, libraries, heuristics
        torch.cuda.synchronize(self.rt.device)
        graph = torch.cuda.CUDAGraph()
        self.rt.ws.frozen = True
        try:
            with torch.cuda.graph(graph):
                self._begin_step(batch)
                logits = self.model.forward(batch, self.rt)
        finally:
            self.rt.ws.frozen = False
        torch.cuda.synchronize(self.rt.device)
        self.capture_seconds += time.perf_counter() - started
        return (graph, logits, self.rt.ws.generation)

    # ------------------------------------------------------------------ tokens from the device
    @property
    def token_source(self) -> Optional[torch.Tensor]:
        """int32 [slots]: the token every slot sampled last, on the device.  With it set, an
        entry may bring ``[TOKEN_FROM_DEVICE]`` instead of a token, and the step can be
        launched before the host has read the previous step's tokens."""
        return self._token_source

    @token_source.setter
    def token_source(self, tensor: Optional[torch.Tensor]) -> None:
        if tensor is not None and (tensor.dtype != torch.int32 or tensor.numel() <= self.cache.null_slot):
            raise ValueError("token_source must be int32 with an entry for every slot and the null slot")
        if tensor is not self._token_source:
            self._graphs.clear()            # recorded steps do or do not hold the lookup
            self._portion_graphs.clear()
            self._mixed_graphs.clear()
        self._token_source = tensor

    def _resolve_tokens(self, batch: StepBatch) -> None:
        if self._token_source is not None:
            self.rt.ops.resolve_tokens(batch.token_ids, batch.token_slot, self._token_source,
                                       batch.n_tokens)

    def _drain_updates(self, caps):
        """The block-table updates since the last step, per group.  A group with more of them
        than the step's metadata has room for (a large reservation made at once) has them
        shipped on their own, ahead of the step."""
        updates = self.cache.drain_table_updates()
        for g, u in enumerate(updates):
            if len(u) > caps[g]:
                self._ship_table_updates(g, u)
                updates[g] = []
        return updates

    def _build(self, entries, updates, **how) -> StepBatch:
        """``builder.build``; if it refuses the step, the drained updates go back to the cache
        manager, so that the device's block tables still get them with the next step."""
        try:
            return self.builder.build(entries, updates, **how)
        except Exception:
            self.cache.requeue_table_updates(updates)
            raise

    def _ship_table_updates(self, group: int, updates) -> None:
        flat = torch.tensor([len(updates)] + [v for u in updates for v in u], dtype=torch.int32)
        self.rt.ops.apply_table_updates(self.cache.groups[group].table, flat.to(self.rt.device),
                                        len(updates))

    def _begin_step(self, batch: StepBatch) -> None:
        """The block-table updates the step brings and the tokens it takes from the device: one
        launch where there is one cache group and the kernels have that form."""
        caps = batch.table_update_caps
        if len(caps) == 1 and caps[0] > 0 and hasattr(self.rt.ops, "step_prologue"):
            self.rt.ops.step_prologue(self.cache.groups[0].table, batch.table_updates[0], caps[0],
                                      batch.token_ids, batch.token_slot, self._token_source,
                                      batch.n_tokens)
            return
        self._apply_table_updates(batch)
        self._resolve_tokens(batch)

    def _apply_table_updates(self, batch: StepBatch) -> None:
        for g, (upd, cap) in enumerate(zip(batch.table_updates, batch.table_update_caps)):
            if cap > 0:
                self.rt.ops.apply_table_updates(self.cache.groups[g].table, upd, cap)
