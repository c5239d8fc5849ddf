"""Timing of the step function: prefill of one prompt, and decode steps at a batch size.

The reference times with device events around the loop after discarded warm-up steps
(src/backend/cuda/model/execution.cu:248-299; ``--benchmark-warmup`` 8,
src/app/cuda/main.cpp:38-95) on synthetic tokens
(``--benchmark-prefill-tokens``, main.cpp:368-376).  Sampling (greedy, on the device)
is inside the timed decode step, as it is inside the reference's.
"""
from __future__ import annotations

import time
from typing import Dict, List, Optional

import torch

from ..sampling.sampler import GREEDY, Sampler
from .batch import TOKEN_FROM_DEVICE, StepEntry
from .loading import LoadedModel


def _sync(device) -> None:
    if torch.device(device).type == "cuda":
        torch.cuda.synchronize(device)


def random_prompt(vocab: int, n: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def measure_prefill(lm: LoadedModel, n_tokens: int, repeats: int = 5, warmup: int = 2,
                    seed: int = 0) -> Dict[str, float]:
    """One prompt of ``n_tokens`` in one step, logits for the last row; median of
    ``repeats`` after ``warmup`` runs."""
    prompt = random_prompt(lm.spec.vocab_size, n_tokens, seed)
    times = []
    for i in range(warmup + repeats):
        slot = lm.cache.open()
        if slot is None or not lm.cache.prepare(slot, 0, n_tokens):
            raise RuntimeError("measure_prefill: the cache pool is too small for the prompt")
        _sync(lm.rt.device)
        start = time.perf_counter()
        lm.runner.step([StepEntry(slot, 0, prompt, [n_tokens - 1])])
        _sync(lm.rt.device)
        elapsed = time.perf_counter() - start
        lm.cache.close(slot)
        if i >= warmup:
            times.append(elapsed)
    times.sort()
    median = times[len(times) // 2]
    return {"tokens": n_tokens, "ms": median * 1e3, "tokens_per_second": n_tokens / median}


class DecodeBench:
    """``batch`` requests, each with ``context`` tokens in the cache, decoding greedily."""

    def __init__(self, lm: LoadedModel, batch: int, context: int, seed: int = 0,
                 prefill_chunk: int = 2048):
        self.lm = lm
        self.batch = batch
        self.sampler = Sampler(lm.rt.ops, lm.rt.device, lm.spec.vocab_size, lm.cache.max_requests)
        self.slots: List[int] = []
        self.pos: List[int] = []
        self.next_tokens: List[int] = []
        self.generated: List[List[int]] = []      # the tokens of every step, per request
        vocab = lm.spec.vocab_size
        for b in range(batch):
            slot = lm.cache.open()
            if slot is None:
                raise RuntimeError("decode benchmark: not enough request slots")
            self.sampler.begin(slot, GREEDY)
            prompt = random_prompt(vocab, context, seed * 1000 + b)
            pos = 0
            logits = None
            while pos < context:
                n = min(prefill_chunk, lm.runner.max_batched_tokens, context - pos)
                if not lm.cache.prepare(slot, pos, n):
                    raise RuntimeError("decode benchmark: the cache pool is too small")
                last = pos + n == context
                logits = lm.runner.step([StepEntry(slot, pos, prompt[pos:pos + n],
                                                   [n - 1] if last else [])])
                pos += n
            self.slots.append(slot)
            self.pos.append(context)
            self.next_tokens.append(self.sampler.sample(logits, [slot])[0])

    def step(self) -> None:
        """One decode step, the host waiting for its tokens before it goes on."""
        lm = self.lm
        entries = []
        for b, slot in enumerate(self.slots):
            if not lm.cache.prepare(slot, self.pos[b], 1):
                raise RuntimeError("decode benchmark: out of cache pages")
            entries.append(StepEntry(slot, self.pos[b], [self.next_tokens[b]], [0]))
        logits = lm.runner.step(entries)
        self.next_tokens = self.sampler.sample(logits, self.slots)
        self.generated.append(self.next_tokens)
        for b in range(self.batch):
            self.pos[b] += 1

    def steps_pipelined(self, steps: int) -> None:
        """``steps`` decode steps with the host one step ahead of the device: a step takes
        its input tokens on the device from what the previous step sampled
        (``TOKEN_FROM_DEVICE``), so it is launched before those tokens have reached the host;
        the host reads a step's tokens while the next step runs."""
        lm = self.lm
        lm.runner.token_source = self.sampler.last_tokens
        open_fetches = 0
        for k in range(steps):
            entries = []
            for b, slot in enumerate(self.slots):
                if not lm.cache.prepare(slot, self.pos[b], 1):
                    raise RuntimeError("decode benchmark: out of cache pages")
                token = self.next_tokens[b] if k == 0 else TOKEN_FROM_DEVICE
                entries.append(StepEntry(slot, self.pos[b], [token], [0]))
            logits = lm.runner.step(entries)
            self.sampler.launch(logits, self.slots)
            open_fetches += 1
            for b in range(self.batch):
                self.pos[b] += 1
            if open_fetches == 2:           # the tokens of the step before this one
                self.generated.append(self.sampler.fetch())
                open_fetches -= 1
        while open_fetches:
            self.generated.append(self.sampler.fetch())
            open_fetches -= 1
        self.next_tokens = self.generated[-1]

    def run(self, steps: int, warmup: int, pipelined: bool = True) -> Dict[str, float]:
        if pipelined:
            self.steps_pipelined(warmup)
        else:
            for _ in range(warmup):
                self.step()
        _sync(self.lm.rt.device)
        start = time.perf_counter()
        if pipelined:
            self.steps_pipelined(steps)
        else:
            for _ in range(steps):
                self.step()
        _sync(self.lm.rt.device)
        elapsed = time.perf_counter() - start
        return {"steps": steps, "batch": self.batch, "ms_per_step": elapsed / steps * 1e3,
                "tokens_per_second": self.batch * steps / elapsed,
                "context_end": self.pos[0] if self.pos else 0}

    def close(self) -> None:
        for slot in self.slots:
            self.sampler.end(slot)
            self.lm.cache.close(slot)
        self.slots = []
