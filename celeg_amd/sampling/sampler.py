"""Generation options and the sampler that turns rows of logits into tokens.

Names, meanings, defaults and limits are the reference's ``GenerationConfig``
(include/celeg/model/runtime_types.hpp:98-108; validation
src/model/execution/runtime_types.cpp:20-37): greedy when ``temperature <= 0`` or
``top_k == 1``; ``top_k`` in [1, 128]; ``top_p`` in (0, 1]; ``repetition_penalty`` >= 1;
a non-zero ``seed``.  Each request owns one xorshift64* state
(src/backend/cpu/sampler.cpp:10-22), kept on the host and seeded with its ``seed``, so
a request's draws do not depend on its batch mates.  The selection itself runs on
the GPU, one workgroup per row.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

MAX_TOP_K = 128
_MASK64 = (1 << 64) - 1


@dataclass(frozen=True)
class GenerationConfig:
    temperature: float = 0.1
    top_k: int = 50
    top_p: float = 1.0
    repetition_penalty: float = 1.05
    seed: int = 1

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0.0 or self.top_k == 1

    def validate(self) -> None:
        if not math.isfinite(self.temperature) or self.temperature < 0.0:
            raise ValueError("temperature must be finite and non-negative")
        if self.top_k <= 0 or self.top_k > MAX_TOP_K:
            raise ValueError(f"top_k must be between 1 and {MAX_TOP_K}")
        if not math.isfinite(self.top_p) or self.top_p <= 0.0 or self.top_p > 1.0:
            raise ValueError("top_p must be in (0, 1]")
        if not math.isfinite(self.repetition_penalty) or self.repetition_penalty < 1.0:
            raise ValueError("repetition_penalty must be finite and at least 1")
        if self.seed == 0 or not 0 < self.seed <= _MASK64:
            raise ValueError("seed must be non-zero")


GREEDY = GenerationConfig(temperature=0.0, top_k=1, top_p=1.0, repetition_penalty=1.0, seed=1)


class XorShift64Star:
    """s ^= s>>12; s ^= s<<25; s ^= s>>27; bits = s * 2685821657736338717;
    unit = float(((bits >> 11) + 0.5) / 2^53)  (src/backend/cpu/sampler.cpp:10-22)."""

    def __init__(self, seed: int):
        if seed == 0:
            raise ValueError("seed must be non-zero")
        self.state = seed & _MASK64

    def next_unit(self) -> float:
        s = self.state
        s ^= s >> 12
        s ^= (s << 25) & _MASK64
        s ^= s >> 27
        self.state = s
        bits = (s * 2685821657736338717) & _MASK64
        return float(np.float32((float(bits >> 11) + 0.5) * (1.0 / 9007199254740992.0)))


class Sampler:
    """Per-slot sampling state (generator, seen tokens) and the device call."""

    def __init__(self, ops, device, vocab: int, max_requests: int):
        self.ops = ops
        self.device = device
        self.vocab = vocab
        self.max_requests = max_requests
        self._configs: Dict[int, GenerationConfig] = {}
        self._rng: Dict[int, XorShift64Star] = {}
        self._seen: Optional[torch.Tensor] = None   # [max_requests, vocab] uint8, made on need
        cap = max_requests
        pin = torch.device(device).type == "cuda"
        # one staging buffer and one device buffer for a step's parameters: 4 floats a row,
        # then 3 ints a row (the same bytes seen as 32-bit floats and as 32-bit ints)
        # (two staging buffers take turns, like the buffers the tokens come back through)
        self._params = [torch.zeros(cap * 7, dtype=torch.float32, pin_memory=pin) for _ in range(2)]
        self._params_dev = torch.zeros(cap * 7, dtype=torch.float32, device=device)
        self._fparams_dev = self._params_dev[:cap * 4]
        self._iparams_dev = self._params_dev[cap * 4:].view(torch.int32)
        self._uploaded = None      # what the device buffer holds: a copy of the staged values
        self._tokens_dev = torch.empty(cap, dtype=torch.int32, device=device)
        # the token every slot sampled last, on the device: a following step can take its
        # input from here (``ModelRunner.token_source``) before the host has read it
        self.last_tokens = torch.zeros(cap + 1, dtype=torch.int32, device=device)
        # sampled tokens come back through two pinned buffers that take turns, so that one
        # step's tokens can still be on their way while the next step is launched
        self._tokens_host = [torch.zeros(cap, dtype=torch.int32, pin_memory=pin) for _ in range(2)]
        self._events = [torch.cuda.Event() if pin else None for _ in range(2)]
        self._pending = []         # launched and not fetched yet: (turn, rows)
        self._turn = 0

    def begin(self, slot: int, config: GenerationConfig, rng: Optional[XorShift64Star] = None) -> None:
        """Bind a request to ``slot``.  ``rng`` continues an existing generator (a request
        that was preempted and comes back); by default a fresh one is seeded."""
        config.validate()
        self._configs[slot] = config
        self._rng[slot] = rng if rng is not None else XorShift64Star(config.seed)
        if config.repetition_penalty > 1.0 and self._seen is None:
            self._seen = torch.zeros((self.max_requests, self.vocab), dtype=torch.uint8,
                                     device=self.device)
        elif self._seen is not None:
            self._seen[slot].zero_()

    def end(self, slot: int) -> None:
        self._configs.pop(slot, None)
        self._rng.pop(slot, None)

    def uses_seen(self) -> bool:
        return self._seen is not None and any(c.repetition_penalty > 1.0
                                              for c in self._configs.values())

    def mark_seen(self, batch) -> None:
        """Every token a step feeds (prompt portions and decoded tokens) counts as seen by
        its request."""
        if self.uses_seen():
            self.ops.mark_seen(self._seen, batch.token_ids, batch.token_slot, batch.n_tokens)

    def sample(self, logits: torch.Tensor, slots: Sequence[int]) -> List[int]:
        """One token per row of ``logits``; row i belongs to the request in ``slots[i]``."""
        if len(slots) == 0:
            return []
        self.launch(logits, slots)
        return self.fetch()

    def launch(self, logits: torch.Tensor, slots: Sequence[int]) -> None:
        """Starts the sampling of one token per row without waiting for it; ``fetch``
        returns the tokens of the oldest launch not fetched yet (at most two may be open)."""
        R = len(slots)
        if logits.shape[0] != R or logits.shape[1] != self.vocab:
            raise ValueError("sample: one row of logits per slot is needed")
        if R > self.max_requests:
            raise ValueError("sample: more rows than requests")
        if len(self._pending) >= 2:
            raise RuntimeError("sample: two launches are open; fetch one first")
        turn = self._turn          # its previous launch has been fetched: its buffers are free
        self._turn ^= 1
        cap = self.max_requests
        staged = self._params[turn].numpy()
        f, i = staged[:cap * 4], staged[cap * 4:].view(np.int32)
        for r, slot in enumerate(slots):
            c = self._configs[slot]
            f[4 * r: 4 * r + 4] = (c.temperature, c.top_p, c.repetition_penalty,
                                   0.0 if c.greedy else self._rng[slot].next_unit())
            i[3 * r] = c.top_k
            i[3 * r + 1] = slot if (c.repetition_penalty > 1.0 and self._seen is not None) else -1
            i[3 * r + 2] = slot
        # greedy rows have nothing that changes from step to step: ship only what differs
        # from what the device holds
        used = np.concatenate([f[:4 * R].view(np.int32), i[:3 * R]])
        if self._uploaded is None or not np.array_equal(used, self._uploaded):
            self._params_dev.copy_(self._params[turn], non_blocking=True)
            self._uploaded = used
        all_greedy = all(self._configs[slot].greedy for slot in slots)
        self.ops.sample(logits, self._fparams_dev, self._iparams_dev, self._seen,
                        self._tokens_dev[:R], last_tokens=self.last_tokens, **({"all_greedy": True} if all_greedy else {}))
        self._tokens_host[turn][:R].copy_(self._tokens_dev[:R], non_blocking=True)
        if self._events[turn] is not None:
            self._events[turn].record()
        self._pending.append((turn, R))

    def _sync(self, turn: int) -> None:
        if self._events[turn] is not None:
            self._events[turn].synchronize()

    def fetch(self) -> List[int]:
        """The tokens of the oldest open launch (waits for them)."""
        if not self._pending:
            return []
        turn, R = self._pending.pop(0)
        self._sync(turn)
        return self._tokens_host[turn][:R].tolist()
