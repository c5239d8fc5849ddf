"""The description of a model as data: which parts, with which sizes, in which order.

An architecture turns its typed configuration into a ``ModelSpec``; everything
below (weights, cache manager, step function) reads only the spec and never asks
which architecture it came from.  The reference keeps the same separation: a
``LayerSpec`` is a mixer variant plus a feed-forward variant plus norms
(include/celeg/model/graph.hpp:431-438) and back ends consume the compiled
program, never names (src/model/program_builder.cpp:112-164).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """One part: its registered kind, its sizes and constants, and the checkpoint
    tensor that fills each of its roles (role -> tensor name)."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    tensors: Dict[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """A block: how the parts are arranged, and the parts themselves."""
    mixer: PartSpec
    mixer_norm: PartSpec
    ffn: PartSpec
    ffn_norm: PartSpec
    arrangement: str = "pre_norm"


@dataclass(frozen=True)
class RunStep:
    """One entry of the run order.  ``layer`` indexes ``ModelSpec.layers`` (a layer
    may be named more than once: its weights are shared, its cache is not).
    ``kv_from`` is the index of an EARLIER entry of the run order whose keys and
    values this entry's mixer reads instead of writing its own."""
    layer: int
    kv_from: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_context: int
    embedding: PartSpec
    layers: Tuple[LayerSpec, ...]
    order: Tuple[RunStep, ...]
    final_norm: PartSpec
    head: PartSpec
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None

    def validate(self) -> None:
        if self.vocab_size <= 0 or self.hidden_size <= 0 or self.max_context <= 0:
            raise ValueError("vocab_size, hidden_size and max_context must be positive")
        if not self.order:
            raise ValueError("the run order is empty")
        for i, step in enumerate(self.order):
            if not 0 <= step.layer < len(self.layers):
                raise ValueError(f"run order entry {i} names layer {step.layer}, "
                                 f"but the model has {len(self.layers)} layers")
            if step.kv_from is not None and not 0 <= step.kv_from < i:
                raise ValueError(f"run order entry {i} reads the cache of entry "
                                 f"{step.kv_from}, which does not run before it")

    def tensor_names(self) -> List[str]:
        names: List[str] = []
        for part in self.all_parts():
            names.extend(part.tensors.values())
        return names

    def all_parts(self) -> List[PartSpec]:
        parts = [self.embedding]
        for layer in self.layers:
            parts += [layer.mixer_norm, layer.mixer, layer.ffn_norm, layer.ffn]
        parts += [self.final_norm, self.head]
        return parts
