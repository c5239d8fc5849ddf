"""Interfaces of the parts a model is put together from, and their registries.

A part is built from a ``PartSpec`` (kind, sizes and constants, tensor names).  It
never learns which model it is in: it declares the tensors it wants and the cache
it needs, receives them, and maps rows to rows.

Kinds of part and what each must provide:

* every part: ``weight_specs()`` (role -> ``WeightSpec``) and ``load(tensors, rt)``;
* norm: ``forward(x, out, rt, delta=None, rows=None)``: normalises rows of the
  32-bit residual stream, optionally after adding ``delta`` to it in place, optionally
  only the rows listed in ``rows``;
* mixer: ``kv_need()`` (keys and values that grow with the sequence, in pages) and
  ``state_needs()`` (state of fixed size per request), and ``forward(x, batch, cache,
  rt)`` that gives the same rows however the sequence was cut into steps;
* feed-forward: ``forward(x, batch, rt)``;
* position encoding: ``tables(rt)``, what the mixer's kernels need to turn a row's
  position into its encoding;
* embedding and head: ``forward``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Tuple

import torch

from ..config.spec import PartSpec


@dataclass(frozen=True)
class WeightSpec:
    """A tensor a part wants.  ``kind``: "matrix" follows the engine's dtype, "vector"
    is always held in 32-bit (norm scales, biases, filter taps).  ``init`` picks the
    distribution of the random-weights mode: "normal" is N(0, std), "around_one" is
    1 + N(0, std).  ``also`` lists other shapes of the same tensor that are accepted."""
    shape: Tuple[int, ...]
    kind: str = "matrix"
    init: str = "normal"
    also: Tuple[Tuple[int, ...], ...] = ()


@dataclass(frozen=True)
class KVNeed:
    """Keys and values of every position, or of a trailing window of positions."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """State of fixed size per request, zero when the request starts."""
    name: str
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class Runtime:
    """What every part computes with: the device, the activation dtype, the kernels
    and a workspace of reusable buffers."""

    def __init__(self, device, dtype, ops, workspace):
        self.device = device
        self.dtype = dtype
        self.ops = ops
        self.ws = workspace


class Part:
    # True if ``forward`` only enqueues device work whose arguments do not depend on the
    # step's contents (every per-step number is read from the batch's device arrays), so
    # that a recorded step can be replayed from a HIP graph.  A part that plans on the
    # host (reads ``batch.host``, loops over requests in Python) must leave this False;
    # a model with such a part is never replayed from a graph.
    graph_safe = False

    def __init__(self, spec: PartSpec):
        self.spec = spec
        self.params = dict(spec.params)

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        pass


class Norm(Part):
    def forward(self, x, out, rt, delta=None, rows=None):
        raise NotImplementedError


class Mixer(Part):
    def kv_need(self) -> Optional[KVNeed]:
        return None

    def state_needs(self) -> List[StateNeed]:
        return []

    def set_reads_foreign_kv(self) -> None:
        """Called when a run-order entry makes this mixer read the keys and values
        another entry wrote; a mixer that cannot do that refuses."""
        raise ValueError(f"mixer '{self.spec.kind}' cannot read another layer's cache")

    def forward(self, x, batch, cache, rt):
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x, batch, rt):
        raise NotImplementedError


class PositionEncoding(Part):
    pass


class Embedding(Part):
    def forward(self, token_ids, out, rt, batch=None):
        raise NotImplementedError


class Head(Part):
    def forward(self, x, out, rt, embedding=None):
        raise NotImplementedError


# ------------------------------------------------------------------------ registries

_REGISTRIES: Dict[str, Dict[str, Callable[[PartSpec], Part]]] = {
    "norm": {}, "mixer": {}, "ffn": {}, "position": {}, "embedding": {}, "head": {},
    "block": {},
}


def register_part(role: str, kind: str, factory: Callable, replace: bool = False) -> None:
    """Add a part.  ``role`` is one of norm, mixer, ffn, position, embedding, head,
    block; ``kind`` is the name a ``PartSpec`` uses; ``factory(spec)`` builds it."""
    if role not in _REGISTRIES:
        raise ValueError(f"unknown role '{role}'; roles: {sorted(_REGISTRIES)}")
    if kind in _REGISTRIES[role] and not replace:
        raise ValueError(f"{role} '{kind}' is already registered")
    _REGISTRIES[role][kind] = factory


def build_part(role: str, spec: PartSpec):
    table = _REGISTRIES[role]
    if spec.kind not in table:
        raise ValueError(f"no {role} of kind '{spec.kind}' is registered; "
                         f"registered: {sorted(table)}")
    return table[spec.kind](spec)


def build_block(layer_spec):
    """The block arrangement a ``LayerSpec`` names, built with its parts."""
    table = _REGISTRIES["block"]
    if layer_spec.arrangement not in table:
        raise ValueError(f"no block arrangement '{layer_spec.arrangement}' is registered; "
                         f"registered: {sorted(table)}")
    return table[layer_spec.arrangement](layer_spec)


def registered_parts(role: str) -> List[str]:
    return sorted(_REGISTRIES[role])
