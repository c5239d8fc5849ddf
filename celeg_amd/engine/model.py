"""A model put together from a ``ModelSpec``: parts, their tensors, their cache needs,
and the forward pass over one step's rows.

The reference compiles a resolved model into a program whose layers declare their
tensors and their state layout (src/model/weight_plan.cpp:278-326;
include/celeg/model/program.hpp:118-177) and runs it layer by layer
(src/backend/cuda/packed/layer_executor.cu:93-217).  Here the run order is a list
that may name a layer twice (shared weights, separate cache) or let an entry read
the keys and values of an earlier entry.
"""
from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from ..cache.manager import CacheLayout, CacheManager
from ..config.spec import ModelSpec
from ..parts.base import Mixer, Part, Runtime, WeightSpec, build_block, build_part


class Model:
    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.embedding = build_part("embedding", spec.embedding)
        self.blocks = [build_block(layer) for layer in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm)
        self.head = build_part("head", spec.head)
        self._resolve_cache_sharing()
        self._caches = None

    # ------------------------------------------------------------------ structure
    def _mixer(self, layer: int) -> Mixer:
        return self.blocks[layer].parts()["mixer"]

    def _resolve_cache_sharing(self) -> None:
        order = self.spec.order
        writes_somewhere = set()
        for step in order:
            if step.kv_from is None:
                writes_somewhere.add(step.layer)
        for i, step in enumerate(order):
            if step.kv_from is None:
                continue
            mine = self._mixer(step.layer).kv_need()
            source_step = order[step.kv_from]
            if source_step.kv_from is not None:
                raise ValueError(f"run order entry {i} reads the cache of entry {step.kv_from}, "
                                 "which has none of its own")
            theirs = self._mixer(source_step.layer).kv_need()
            if mine is None or theirs is None:
                raise ValueError(f"run order entry {i}: only a mixer with keys and values can "
                                 "read another entry's cache, and only from such a mixer")
            if (mine.kv_heads, mine.head_dim) != (theirs.kv_heads, theirs.head_dim):
                raise ValueError(f"run order entry {i}: its mixer and the one of entry "
                                 f"{step.kv_from} differ in kv_heads or head_dim")
        for layer in range(len(self.blocks)):
            used = any(s.layer == layer for s in order)
            if used and layer not in writes_somewhere and self._mixer(layer).kv_need() is not None:
                self._mixer(layer).set_reads_foreign_kv()

    @property
    def graph_safe(self) -> bool:
        """Whether a recorded step of this model may be replayed from a HIP graph."""
        safe = self.__dict__.get("_graph_safe")
        if safe is None:      # the parts are fixed once the model is built
            safe = self.__dict__["_graph_safe"] = all(part.graph_safe for _, part in self.named_parts())
        return safe

    def named_parts(self) -> List[Tuple[str, Part]]:
        out = [("embedding", self.embedding)]
        for i, block in enumerate(self.blocks):
            for name, part in block.parts().items():
                out.append((f"layers.{i}.{name}", part))
        out += [("final_norm", self.final_norm), ("head", self.head)]
        return out

    def expected_tensors(self) -> Dict[str, WeightSpec]:
        """Checkpoint tensor name -> what is expected of it."""
        expected: Dict[str, WeightSpec] = {}
        for label, part in self.named_parts():
            for role, wspec in part.weight_specs().items():
                if role not in part.spec.tensors:
                    raise ValueError(f"{label} ({part.spec.kind}) wants a tensor for role "
                                     f"'{role}', but the model description names none")
                name = part.spec.tensors[role]
                if name in expected and expected[name].shape != wspec.shape:
                    raise ValueError(f"tensor {name} is wanted with shapes "
                                     f"{expected[name].shape} and {wspec.shape}")
                expected[name] = wspec
        return expected

    def cache_layout(self) -> CacheLayout:
        layout = CacheLayout()
        index_of_group = {}
        for i, step in enumerate(self.spec.order):
            mixer = self._mixer(step.layer)
            need = mixer.kv_need()
            if need is not None:
                if step.kv_from is not None:
                    g, layer, _ = layout.kv_of_step[step.kv_from]
                    layout.kv_of_step[i] = (g, layer, False)
                else:
                    if need not in index_of_group:
                        index_of_group[need] = len(layout.kv_groups)
                        layout.kv_groups.append(need)
                        layout.group_layers.append(0)
                    g = index_of_group[need]
                    layout.kv_of_step[i] = (g, layout.group_layers[g], True)
                    layout.group_layers[g] += 1
            for state in mixer.state_needs():
                layout.states.append((i, state))
        return layout

    # ------------------------------------------------------------------ weights
    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        """``tensors``: checkpoint name -> device tensor, already checked and converted."""
        for _, part in self.named_parts():
            mine = {role: tensors[part.spec.tensors[role]] for role in part.weight_specs()}
            part.load(mine, rt)

    # ------------------------------------------------------------------ forward
    def bind_cache(self, cache: CacheManager) -> None:
        self._caches = [cache.layer_cache(i) for i in range(len(self.spec.order))]

    def forward(self, batch, rt: Runtime) -> torch.Tensor:
        """Runs the rows of ``batch`` through every entry of the run order and returns
        32-bit logits [batch.n_logit_rows, vocab]."""
        if self._caches is None:
            raise RuntimeError("model: bind_cache() has not been called")
        T, R = batch.n_tokens, batch.n_logit_rows
        width, vocab = self.spec.hidden_size, self.spec.vocab_size
        h = rt.ws.buf("hidden", (T, width), torch.float32)
        rt.stream_stat_blocks = 0
        self.embedding.forward(batch.token_ids, h, rt, batch=batch)
        delta = None
        for i, step in enumerate(self.spec.order):
            delta = self.blocks[step.layer].forward(h, delta, batch, self._caches[i], rt)
        logits = rt.ws.buf("logits", (R, vocab), torch.float32)
        if R == 0:
            return logits
        if delta is None and hasattr(self.head, "forward_fused") and \
                self.head.forward_fused(h, self.final_norm, batch, logits, rt, self.embedding):
            return logits
        normed = rt.ws.buf("final_normed", (R, width), rt.dtype)
        self.final_norm.forward(h, normed, rt, delta=delta, rows=batch.logit_rows)
        self.head.forward(normed, logits, rt, embedding=self.embedding)
        return logits
