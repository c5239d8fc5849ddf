"""The scheduler: admits requests, cuts prompts into portions under a token budget,
lets every decoding request take one token per step, finishes and frees.

What it mirrors of the reference: submission checks
(src/backend/cuda/runtime/request_lifecycle.cpp:10-32), the queue order priority
descending then id ascending (src/runtime/concurrency/batch_planner.cpp:14-50),
admission that stops at the first request whose pages cannot be had (the request
stays queued, request_lifecycle.cpp:103-198), the token budget
``max_batched_tokens - #decoding`` and portions of at most ``prefill_chunk_tokens``
(src/backend/cuda/runtime/prefill_scheduler.cpp:4-186), the two reservation policies
(decode_scheduler.cpp:23-66), finishing on an end token (which is emitted) or on
``max_new_tokens`` (decode_scheduler.cpp:68-99), and the states Queued, Prefill,
Decoding, Finished, Cancelled, Failed (include/celeg/runtime/concurrency/policy.hpp:10-25).

What differs: portions and decode tokens go into ONE step; logits are sampled after
the step that produced them, so a request that finishes is not fed again.

When pages run out: a queued request waits; a decoding request whose next token needs
a page that is not free is left out of the step and tried again later (the reference
does the same); a prompt portion is cut to what the free pages hold.  If no running
request can take a single token, the youngest running request is preempted: it gives
back its pages and slot and goes back to the head of the queue, to be recomputed
from its prompt plus what it has generated (its output so far is kept).  A request
that cannot fit the pool even alone fails.

A request is one growing sequence, prompt + generated; ``fed`` counts how many of its
tokens are in the cache.  A step feeds ``seq[fed:fed+n]``; when that reaches the end of
the sequence the last row's logits are sampled.  Decoding is the case n = 1.
"""
from __future__ import annotations

import enum
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Sequence, Tuple

from ..sampling.sampler import GenerationConfig


class RequestStatus(enum.Enum):
    QUEUED = "queued"
    PREFILL = "prefill"
    DECODING = "decoding"
    FINISHED = "finished"
    CANCELLED = "cancelled"
    FAILED = "failed"

    @property
    def done(self) -> bool:
        return self in (RequestStatus.FINISHED, RequestStatus.CANCELLED, RequestStatus.FAILED)


@dataclass
class RequestOptions:
    """Defaults as include/celeg/runtime/request_types.hpp:16-26, except that the end
    tokens default to the model's own (None here)."""
    max_new_tokens: int = 128
    eos_token_ids: Optional[Sequence[int]] = None
    priority: int = 0
    generation: GenerationConfig = field(default_factory=GenerationConfig)


@dataclass
class SchedulerOptions:
    """Defaults as include/celeg/backend/cuda/concurrency.hpp:18-32."""
    max_active_requests: int = 8
    max_batched_tokens: int = 512
    prefill_chunk_tokens: int = 256
    policy: str = "max_utilization"      # or "guaranteed_no_evict"
    # 1: a portion that the step's budget cuts short is cut exactly at the budget, as the
    # reference does (src/backend/cuda/runtime/prefill_scheduler.cpp:4-186).  More: such a
    # portion (not one that the prompt's end or the portion size cuts) is shortened further to
    # a multiple of this, or left for the next step; the steps of a steady load then repeat a
    # few shapes, which the runner replays from recorded graphs, instead of a new shape for
    # every number of decoding requests, at the price of somewhat more steps (measured at the
    # 350M shape, 64 requests, portions of 256 under a budget of 512: 549 steps against 530).
    portion_granule: int = 1

    def validate(self) -> None:
        if self.max_active_requests <= 0 or self.max_batched_tokens <= 0 \
                or self.prefill_chunk_tokens <= 0 or self.portion_granule <= 0:
            raise ValueError("scheduler options must be positive")
        if self.policy not in ("max_utilization", "guaranteed_no_evict"):
            raise ValueError("policy must be max_utilization or guaranteed_no_evict")


@dataclass
class Request:
    id: int
    prompt: List[int]
    options: RequestOptions
    eos: Tuple[int, ...]
    status: RequestStatus = RequestStatus.QUEUED
    slot: Optional[int] = None
    fed: int = 0
    generated: List[int] = field(default_factory=list)
    pending: Deque[int] = field(default_factory=deque)   # generated, not yet polled
    error: str = ""
    cancel_requested: bool = False
    preemptions: int = 0
    order: int = 0            # admission order, for "youngest"

    @property
    def sequence_length(self) -> int:
        return len(self.prompt) + len(self.generated)

    def tokens(self, begin: int, count: int) -> List[int]:
        p = len(self.prompt)
        out = []
        for i in range(begin, begin + count):
            out.append(self.prompt[i] if i < p else self.generated[i - p])
        return out


@dataclass
class PlannedEntry:
    request: Request
    start: int
    count: int
    samples: bool     # the portion reaches the end of the sequence: sample from its last row


class Scheduler:
    def __init__(self, cache, options: SchedulerOptions, *, max_context: int,
                 default_eos: Sequence[int] = ()):
        options.validate()
        self.cache = cache
        self.options = options
        self.max_context = max_context
        self.default_eos = tuple(default_eos)
        self.requests: Dict[int, Request] = {}
        self.queue: List[Request] = []
        self.active: List[Request] = []
        self._next_id = 0
        self._admitted = 0
        self.new_slots: List[Tuple[int, Request]] = []
        self.released_slots: List[int] = []
        self.stats = {"steps": 0, "preemptions": 0, "stalled_decodes": 0, "prefill_tokens": 0,
                      "decode_tokens": 0}

    # ------------------------------------------------------------------ submission
    def submit(self, prompt: Sequence[int], options: Optional[RequestOptions] = None) -> int:
        options = options or RequestOptions()
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise ValueError("request prompt is empty")
        if len(prompt) > self.max_context:
            raise ValueError("request prompt exceeds max_context")
        if options.max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive")
        if len(prompt) + options.max_new_tokens > self.max_context:
            raise ValueError("prompt plus max_new_tokens exceeds max_context")
        options.generation.validate()
        eos = tuple(options.eos_token_ids) if options.eos_token_ids is not None else self.default_eos
        req = Request(self._next_id, prompt, options, eos)
        self._next_id += 1
        self.requests[req.id] = req
        self.queue.append(req)
        return req.id

    def cancel(self, request_id: int) -> None:
        req = self.requests[request_id]
        if not req.status.done:
            req.cancel_requested = True

    def has_work(self) -> bool:
        return bool(self.queue or self.active)

    # ------------------------------------------------------------------ planning
    def _best_queued(self) -> Request:
        return min(self.queue, key=lambda r: (-r.options.priority, r.id))

    def _release(self, req: Request, status: RequestStatus, error: str = "") -> None:
        if req.slot is not None:
            self.cache.close(req.slot)
            self.released_slots.append(req.slot)
            req.slot = None
        if req in self.active:
            self.active.remove(req)
        if req in self.queue:
            self.queue.remove(req)
        req.status = status
        req.error = error

    def _affordable(self, req: Request, start: int, want: int) -> int:
        """The largest n <= want such that the pages for positions [start, start+n) can be
        had now (0 if not even one token can)."""
        P = self.cache.page_tokens
        n = want
        while n > 0:
            need = self.cache.pages_needed(req.slot, start, n)
            if all(k <= f for k, f in zip(need, self.cache.free_pages())):
                return n
            # shrink to the end of the previous page
            end = start + n
            n = ((end - 1) // P) * P - start
        return 0

    def _admit(self, budget: int) -> None:
        while self.queue and len(self.active) < self.options.max_active_requests \
                and self.cache.n_free_slots > 0 and budget > 0:
            req = self._best_queued()
            slot = self.cache.open()
            if slot is None:
                return
            req.slot = slot
            total = req.sequence_length
            if self.options.policy == "guaranteed_no_evict":
                reserve = len(req.prompt) + req.options.max_new_tokens
                ok = self.cache.prepare(slot, 0, reserve)
            else:
                first = min(total, self.options.prefill_chunk_tokens, budget)
                ok = self._affordable(req, 0, first) > 0
            if not ok:
                self.cache.close(slot)
                req.slot = None
                if not self.active:
                    # nothing is running and it still does not fit: it never will
                    self._release(req, RequestStatus.FAILED,
                                  "request needs more cache pages than the pool holds")
                    continue
                return            # stays queued; admission stops here
            self.queue.remove(req)
            req.status = RequestStatus.PREFILL
            req.fed = 0
            req.order = self._admitted
            self._admitted += 1
            self.active.append(req)
            self.new_slots.append((slot, req))
            budget -= min(total, self.options.prefill_chunk_tokens)

    def plan(self) -> List[PlannedEntry]:
        """Decide this step's entries.  Pages for them are taken here."""
        for req in list(self.requests.values()):
            if req.cancel_requested and not req.status.done:
                self._release(req, RequestStatus.CANCELLED)
        while True:
            entries = self._plan_once()
            if entries or not self.active:
                return entries
            self._preempt_youngest()

    def _plan_once(self) -> List[PlannedEntry]:
        entries: List[PlannedEntry] = []
        decoding = [r for r in self.active if r.sequence_length - r.fed == 1
                    and r.status == RequestStatus.DECODING]
        budget = self.options.max_batched_tokens
        for req in decoding:
            if budget <= 0:
                break
            if self.cache.prepare(req.slot, req.fed, 1):
                entries.append(PlannedEntry(req, req.fed, 1, True))
                budget -= 1
            else:
                self.stats["stalled_decodes"] += 1
        self._admit(budget)
        for req in self.active:
            if req.status != RequestStatus.PREFILL or budget <= 0:
                continue
            remaining = req.sequence_length - req.fed
            count = min(remaining, self.options.prefill_chunk_tokens, budget)
            if count == budget and count < min(remaining, self.options.prefill_chunk_tokens):
                rounded = count - count % self.options.portion_granule
                if rounded > 0 or entries:
                    count = rounded
            count = self._affordable(req, req.fed, count)
            if count <= 0:
                continue
            if not self.cache.prepare(req.slot, req.fed, count):
                continue
            entries.append(PlannedEntry(req, req.fed, count, req.fed + count == req.sequence_length))
            budget -= count
        return entries

    def _preempt_youngest(self) -> None:
        victim = max(self.active, key=lambda r: r.order)
        if len(self.active) == 1:
            self._release(victim, RequestStatus.FAILED,
                          "request needs more cache pages than the pool holds")
            return
        self.cache.close(victim.slot)
        self.released_slots.append(victim.slot)
        victim.slot = None
        victim.fed = 0
        victim.status = RequestStatus.QUEUED
        victim.preemptions += 1
        self.stats["preemptions"] += 1
        self.active.remove(victim)
        self.queue.insert(0, victim)

    def drain_slot_events(self):
        """(slots released, (slot, request) pairs newly bound) since the last call, in that
        order of effect: the caller drops and starts per-slot sampling state with them."""
        released, new = self.released_slots, self.new_slots
        self.released_slots, self.new_slots = [], []
        return released, new

    # ------------------------------------------------------------------ after the step
    def accept(self, entries: Sequence[PlannedEntry], sampled: Sequence[int]) -> None:
        """``sampled``: one token for every entry with ``samples``, in order."""
        self.stats["steps"] += 1
        it = iter(sampled)
        for e in entries:
            req = e.request
            req.fed = e.start + e.count
            if e.count == 1 and req.status == RequestStatus.DECODING:
                self.stats["decode_tokens"] += 1
            else:
                self.stats["prefill_tokens"] += e.count
            if not e.samples:
                continue
            token = int(next(it))
            req.generated.append(token)
            req.pending.append(token)
            req.status = RequestStatus.DECODING
            if token in req.eos or len(req.generated) >= req.options.max_new_tokens \
                    or req.sequence_length >= self.max_context:
                self._release(req, RequestStatus.FINISHED)

    def poll(self, request_id: int) -> Tuple[RequestStatus, List[int], str]:
        """Drain the tokens generated since the last poll
        (src/backend/cuda/runtime/request_lifecycle.cpp:57-73)."""
        req = self.requests[request_id]
        tokens = list(req.pending)
        req.pending.clear()
        return req.status, tokens, req.error
