"""The description of a model as data, on the Python side: which parts, with which sizes, in
which order.  It mirrors the library's own description (``csrc/host/spec.hpp``) and travels to
and from it as JSON; an architecture written in Python builds one of these.

The reference keeps the same separation: a ``LayerSpec`` is a mixer variant plus a feed-forward
variant plus norms (include/celeg/model/graph.hpp:431-438) and back ends consume the compiled
program, never names (src/model/program_builder.cpp:112-164).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """One part: its registered kind, its sizes and constants (a value may itself be a part), and
    the checkpoint tensor that fills each of its roles (role -> tensor name)."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    tensors: Dict[str, str] = field(default_factory=dict)

    def to_json(self) -> Dict[str, Any]:
        params = {k: (v.to_json() if isinstance(v, PartSpec) else v) for k, v in self.params.items()}
        return {"kind": self.kind, "params": params, "tensors": dict(self.tensors)}

    @classmethod
    def from_json(cls, j: Dict[str, Any]) -> "PartSpec":
        params = {k: (cls.from_json(v) if isinstance(v, dict) and isinstance(v.get("kind"), str) else v)
                  for k, v in (j.get("params") or {}).items()}
        return cls(j["kind"], params, dict(j.get("tensors") or {}))


@dataclass(frozen=True)
class LayerSpec:
    """A block: how the parts are arranged, and the parts themselves."""
    mixer: PartSpec
    mixer_norm: PartSpec
    ffn: PartSpec
    ffn_norm: PartSpec
    arrangement: str = "pre_norm"

    def to_json(self) -> Dict[str, Any]:
        return {"mixer": self.mixer.to_json(), "mixer_norm": self.mixer_norm.to_json(),
                "ffn": self.ffn.to_json(), "ffn_norm": self.ffn_norm.to_json(),
                "arrangement": self.arrangement}


@dataclass(frozen=True)
class RunStep:
    """One entry of the run order.  ``layer`` indexes ``ModelSpec.layers`` (a layer may be named
    more than once: its weights are shared, its cache is not).  ``kv_from`` is the index of an
    EARLIER entry of the run order whose keys and values this entry's mixer reads instead of
    writing its own."""
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

    def to_json(self) -> Dict[str, Any]:
        return {"architecture": self.architecture, "vocab_size": self.vocab_size,
                "hidden_size": self.hidden_size, "max_context": self.max_context,
                "embedding": self.embedding.to_json(), "layers": [l.to_json() for l in self.layers],
                "order": [{"layer": s.layer, "kv_from": s.kv_from} for s in self.order],
                "final_norm": self.final_norm.to_json(), "head": self.head.to_json(),
                "eos_token_ids": list(self.eos_token_ids), "bos_token_id": self.bos_token_id}

    @classmethod
    def from_json(cls, j: Dict[str, Any]) -> "ModelSpec":
        layers = tuple(LayerSpec(PartSpec.from_json(l["mixer"]), PartSpec.from_json(l["mixer_norm"]),
                                 PartSpec.from_json(l["ffn"]), PartSpec.from_json(l["ffn_norm"]),
                                 l.get("arrangement", "pre_norm")) for l in j["layers"])
        order = tuple(RunStep(s["layer"], s.get("kv_from")) for s in j["order"])
        return cls(j["architecture"], j["vocab_size"], j["hidden_size"], j["max_context"],
                   PartSpec.from_json(j["embedding"]), layers, order, PartSpec.from_json(j["final_norm"]),
                   PartSpec.from_json(j["head"]), tuple(j.get("eos_token_ids") or ()), j.get("bos_token_id"))

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
