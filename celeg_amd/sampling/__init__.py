"""Generation options: names, meanings, defaults and limits of the reference's ``GenerationConfig``
(include/celeg/model/runtime_types.hpp:98-108; validation
src/model/execution/runtime_types.cpp:20-37).  The sampler itself (a xorshift64* state per
request on the host, the selection on the GPU) is the library's (``csrc/host/sampler.cpp``,
``csrc/sampling.hip``)."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Tuple

MAX_TOP_K = 128
_MASK64 = (1 << 64) - 1


@dataclass(frozen=True)
class GenerationConfig:
    temperature: float = 0.1
    top_k: int = 50
    top_p: float = 1.0
    repetition_penalty: float = 1.05
    seed: int = 1
    # given out as the request's first generated tokens instead of sampled ones; the generator is
    # not advanced for them (ForcedTokenPrefix, include/celeg/model/runtime_types.hpp:93-104;
    # src/backend/cpu/sampler.cpp:31-34)
    forced_prefix: Tuple[int, ...] = ()

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0.0 or self.top_k == 1

    def validate(self) -> None:
        """The checks the library makes at submission, for callers that want them earlier."""
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
        if any(int(t) < 0 for t in self.forced_prefix):
            raise ValueError("forced_prefix holds a negative token id")


GREEDY = GenerationConfig(temperature=0.0, top_k=1, top_p=1.0, repetition_penalty=1.0, seed=1)

__all__ = ["GenerationConfig", "GREEDY", "MAX_TOP_K"]
