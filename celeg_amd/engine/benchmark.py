"""Timing of the step function and of the engine: prefill of one prompt, and decode steps at a
batch size.

The reference times with device events around the loop after discarded warm-up steps
(src/backend/cuda/model/execution.cu:248-299; ``--benchmark-warmup`` 8,
src/app/cuda/main.cpp:38-95) on synthetic tokens (``--benchmark-prefill-tokens``,
main.cpp:368-376).  Here the decode steps are the engine's own (scheduler, step function replayed
from its recorded graph, greedy sampling on the device, one step launched ahead of the tokens of
the one before), timed on the host between two waits for the device.
"""
from __future__ import annotations

import time
from typing import Dict, List

import numpy as np

from ..sampling import GREEDY
from .engine import Engine, LoadedModel, RequestOptions, RequestStatus, StepEntry


def random_prompt(vocab: int, n: int, seed: int) -> List[int]:
    return np.random.RandomState(seed).randint(0, vocab, size=n).tolist()


def measure_prefill(lm: LoadedModel, n_tokens: int, repeats: int = 5, warmup: int = 2,
                    seed: int = 0, offset: int = 0) -> Dict[str, float]:
    """One prompt of ``n_tokens`` in one step, logits for the last row (brought to the host);
    median of ``repeats`` after ``warmup`` runs.  With ``offset`` the step is a later portion of
    a long prompt: the ``offset`` tokens before it are fed first, in portions of ``n_tokens``,
    outside the timing."""
    prompt = random_prompt(lm.spec.vocab_size, offset + n_tokens, seed)
    times = []
    for i in range(warmup + repeats):
        slot = lm.cache.open()
        if slot is None:
            raise RuntimeError("measure_prefill: no free request slot")
        for at in range(0, offset, n_tokens):
            n = min(n_tokens, offset - at)
            if not lm.cache.prepare(slot, at, n):
                raise RuntimeError("measure_prefill: the cache pool is too small for the prompt")
            lm.runner.step([StepEntry(slot, at, prompt[at:at + n], [])])
        if not lm.cache.prepare(slot, offset, n_tokens):
            raise RuntimeError("measure_prefill: the cache pool is too small for the prompt")
        lm.native.synchronize()
        start = time.perf_counter()
        lm.runner.step([StepEntry(slot, offset, prompt[offset:], [n_tokens - 1])])     # returns when the logits are on the host
        elapsed = time.perf_counter() - start
        lm.cache.close(slot)
        if i >= warmup:
            times.append(elapsed)
    times.sort()
    median = times[len(times) // 2]
    return {"tokens": n_tokens, "ms": median * 1e3, "tokens_per_second": n_tokens / median}


class DecodeBench:
    """``batch`` requests, each with a prompt of ``context`` tokens, decoding greedily through
    the engine.  The prompts are fed first (a request that has its first token decodes along
    while the others' prompts are fed, so the contexts differ by up to ``batch`` tokens)."""

    def __init__(self, engine: Engine, batch: int, context: int, new_tokens: int, seed: int = 0):
        self.engine = engine
        self.batch = batch
        self.context = context
        vocab = engine.loaded.spec.vocab_size
        self.ids = [engine.submit(random_prompt(vocab, context, seed * 1000 + b),
                                  RequestOptions(max_new_tokens=new_tokens, eos_token_ids=[], generation=GREEDY))
                    for b in range(batch)]
        while any(engine.status(r) in (RequestStatus.QUEUED, RequestStatus.PREFILL) for r in self.ids):
            if engine.step() == 0 and not engine.has_work():
                break
        failed = [r for r in self.ids if engine.status(r) == RequestStatus.FAILED]
        if failed:
            raise RuntimeError(f"decode benchmark: {engine.poll(failed[0])[2]}")

    def generated(self) -> List[int]:
        return [self.engine.request_metrics(r)["generated_tokens"] for r in self.ids]

    def run(self, steps: int, warmup: int) -> Dict[str, float]:
        engine = self.engine
        engine.native.run_steps(warmup)
        engine.loaded.native.synchronize()
        before = self.generated()
        start = time.perf_counter()
        done = engine.native.run_steps(steps)
        engine.loaded.native.synchronize()
        elapsed = time.perf_counter() - start
        after = self.generated()
        tokens = sum(after) - sum(before)
        if tokens != done * self.batch:
            raise RuntimeError(f"decode benchmark: {done} steps of {self.batch} requests gave {tokens} tokens "
                               "(a request ended or waited for pages inside the timed steps)")
        mean_context = self.context + (sum(before) + sum(after)) / (2.0 * self.batch)
        return {"steps": done, "batch": self.batch, "ms_per_step": elapsed / max(done, 1) * 1e3,
                "tokens_per_second": tokens / elapsed, "tokens": tokens, "mean_context": mean_context}

    def close(self) -> None:
        for r in self.ids:
            self.engine.cancel(r)
        self.engine.step()
