"""The Python entry point: submit / step / poll / cancel, and ``generate``.

Shaped after the reference's concurrent engine and its C API
(include/celeg/backend/cuda/concurrency.hpp:36-70; include/celeg/api.h:19-183:
``celeg_engine_create/submit/poll/status/cancel/step``): one ``step()`` admits, runs
ONE batch through the step function, samples on the returned logits and frees what
finished.
"""
from __future__ import annotations

import time
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..sampling.sampler import GenerationConfig, Sampler, XorShift64Star
from .batch import TOKEN_FROM_DEVICE, StepEntry
from .loading import LoadedModel, load_model
from .scheduler import (PlannedEntry, Request, RequestOptions, RequestStatus, Scheduler,
                        SchedulerOptions)


class Engine:
    def __init__(self, loaded: LoadedModel, options: Optional[SchedulerOptions] = None,
                 sampler: Optional[Sampler] = None):
        self.loaded = loaded
        self.options = options or SchedulerOptions(
            max_active_requests=loaded.cache.max_requests,
            max_batched_tokens=loaded.runner.max_batched_tokens)
        if self.options.max_batched_tokens > loaded.runner.max_batched_tokens:
            raise ValueError("max_batched_tokens exceeds what the step function was sized for")
        if self.options.max_active_requests > loaded.cache.max_requests:
            raise ValueError("max_active_requests exceeds the cache manager's slots")
        self.scheduler = Scheduler(loaded.cache, self.options,
                                   max_context=loaded.cache.max_context,
                                   default_eos=loaded.spec.eos_token_ids)
        self.sampler = sampler or Sampler(loaded.rt.ops, loaded.rt.device,
                                          loaded.spec.vocab_size, loaded.cache.max_requests)
        self._rng: Dict[int, XorShift64Star] = {}
        # ``generate`` launches decode steps one ahead of their tokens (see _plan_ahead)
        self.run_ahead = torch.device(loaded.rt.device).type == "cuda"
        if self.run_ahead:
            loaded.runner.token_source = self.sampler.last_tokens
        self.last_logits: Optional[torch.Tensor] = None
        self.metrics = {"steps": 0, "steps_ahead": 0, "step_seconds": 0.0}

    @classmethod
    def from_folder(cls, model_dir: str, *, dtype="bfloat16", device="cuda:0",
                    page_tokens: int = 16, n_pages: Optional[int] = None,
                    max_active_requests: int = 8, max_batched_tokens: int = 2048,
                    prefill_chunk_tokens: int = 1024, context: Optional[int] = None,
                    policy: str = "max_utilization", ops=None,
                    gemm_backend: str = "library", portion_granule: int = 1) -> "Engine":
        # (Steps of 2,048 tokens and portions of 1,024: on an MI355X a step of a few hundred
        # rows leaves most of the chip idle.  64 requests of 2,048 + 256 tokens at the 350M
        # shape take 0.50 s with portions of 2,048 and 0.91 s with the reference's 512 / 256,
        # include/celeg/backend/cuda/concurrency.hpp:18-32, which ``SchedulerOptions`` keeps.)
        loaded = load_model(model_dir, dtype=dtype, device=device, page_tokens=page_tokens,
                            n_pages=n_pages, max_requests=max_active_requests,
                            max_context=context, max_batched_tokens=max_batched_tokens, ops=ops,
                            gemm_backend=gemm_backend)
        return cls(loaded, SchedulerOptions(max_active_requests, max_batched_tokens,
                                            prefill_chunk_tokens, policy, portion_granule))

    # ------------------------------------------------------------------ requests
    def submit(self, prompt: Sequence[int], options: Optional[RequestOptions] = None) -> int:
        vocab = self.loaded.spec.vocab_size
        for t in prompt:
            if not 0 <= int(t) < vocab:
                raise ValueError(f"token id {t} out of range [0, {vocab})")
        return self.scheduler.submit(prompt, options)

    def cancel(self, request_id: int) -> None:
        self.scheduler.cancel(request_id)

    def status(self, request_id: int) -> RequestStatus:
        return self.scheduler.requests[request_id].status

    def poll(self, request_id: int) -> Tuple[RequestStatus, List[int], str]:
        return self.scheduler.poll(request_id)

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    # ------------------------------------------------------------------ one step
    def _sync_slots(self) -> None:
        released, new = self.scheduler.drain_slot_events()
        for slot in released:
            self.sampler.end(slot)
        for slot, req in new:
            rng = self._rng.setdefault(req.id, XorShift64Star(req.options.generation.seed))
            self.sampler.begin(slot, req.options.generation, rng=rng)

    def step(self) -> int:
        """Runs one batch; returns the number of tokens it fed (0 if there was nothing)."""
        plan = self.scheduler.plan()
        self._sync_slots()
        if not plan:
            return 0
        return self._complete(self._launch(plan))

    # A step in two halves, so that ``generate`` can launch the next step before it reads
    # this one's tokens.
    def _launch(self, plan: List[PlannedEntry], device_tokens: bool = False):
        start = time.perf_counter()
        entries = [StepEntry(e.request.slot, e.start,
                             [TOKEN_FROM_DEVICE] if device_tokens else e.request.tokens(e.start, e.count),
                             [e.count - 1] if e.samples else []) for e in plan]
        logits = self.loaded.runner.step(entries)
        self.last_logits = logits
        self.metrics["steps_ahead"] += int(device_tokens)
        slots = [e.request.slot for e in plan if e.samples]
        if self.sampler.uses_seen():
            self.sampler.mark_seen(self.loaded.runner.last_batch)
        if slots:
            self.sampler.launch(logits, slots)
        return plan, bool(slots), start

    def _complete(self, launched) -> int:
        plan, sampled_rows, start = launched
        sampled = self.sampler.fetch() if sampled_rows else []
        # a request that ended while this step was already under way: its row is dropped
        it = iter(sampled)
        entries, tokens = [], []
        for e in plan:
            token = next(it) if e.samples else None
            if e.request.status.done:
                continue
            entries.append(e)
            if e.samples:
                tokens.append(token)
        self.scheduler.accept(entries, tokens)
        self._sync_slots()
        for req in [e.request for e in plan if e.request.status.done]:
            self._rng.pop(req.id, None)
        self.metrics["steps"] += 1
        self.metrics["step_seconds"] += time.perf_counter() - start
        return sum(e.count for e in entries)

    def _plan_ahead(self, plan: List[PlannedEntry]) -> Optional[List[PlannedEntry]]:
        """The step after ``plan``, decided before ``plan``'s tokens are known: possible when
        every active request is decoding (nothing waits, nothing is being prefilled), for the
        requests that this step's token cannot end by count or context.  A request that the
        token does end (an end token) rides along for one row that is dropped afterwards;
        what it writes lies in its own pages and state, which are only handed on by later
        steps on the same stream."""
        sched = self.scheduler
        if not self.run_ahead or self.loaded.runner.token_source is None or sched.queue \
                or len(plan) != len(sched.active):
            return None
        ahead = []
        for e in plan:
            req = e.request
            if e.count != 1 or not e.samples or req.status != RequestStatus.DECODING or req.cancel_requested:
                return None
            if len(req.generated) + 1 >= req.options.max_new_tokens \
                    or e.start + 2 >= sched.max_context:
                continue
            ahead.append(PlannedEntry(req, e.start + 1, 1, True))
        if not ahead:
            return None
        cache = self.loaded.cache
        need = [0] * len(cache.groups)
        for e in ahead:
            for g, n in enumerate(cache.pages_needed(e.request.slot, e.start, 1)):
                need[g] += n
        if any(n > free for n, free in zip(need, cache.free_pages())):
            return None              # let the ordinary step decide what to do without pages
        for e in ahead:
            if not cache.prepare(e.request.slot, e.start, 1):
                return None
        return ahead

    # ------------------------------------------------------------------ convenience
    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int = 128,
                 generation: Optional[GenerationConfig] = None,
                 eos_token_ids: Optional[Sequence[int]] = None,
                 generations: Optional[Sequence[GenerationConfig]] = None) -> List[List[int]]:
        """Generate for every prompt (all submitted at once, batched by the scheduler) and
        return the generated tokens, the end token included if one was met."""
        ids = []
        for i, prompt in enumerate(prompts):
            g = generations[i] if generations is not None else (generation or GenerationConfig())
            ids.append(self.submit(prompt, RequestOptions(max_new_tokens=max_new_tokens,
                                                          eos_token_ids=eos_token_ids,
                                                          generation=g)))
        launched = None
        while launched is not None or self.has_work():
            if launched is None:
                plan = self.scheduler.plan()
                self._sync_slots()
                if not plan:
                    continue
                launched = self._launch(plan)
            ahead = self._plan_ahead(launched[0])
            following = self._launch(ahead, device_tokens=True) if ahead else None
            self._complete(launched)
            launched = following
        out = []
        for rid in ids:
            req = self.scheduler.requests[rid]
            if req.status == RequestStatus.FAILED:
                raise RuntimeError(f"request {rid} failed: {req.error}")
            req.pending.clear()
            out.append(list(req.generated))
        return out
