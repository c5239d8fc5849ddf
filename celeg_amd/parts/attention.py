"""Grouped-query attention over the paged cache.

Order of work (src/backend/cpu/model_forward_token.cpp:100-120;
src/backend/cuda/model/prefill_batched/attention/regular.cpp:23-131):
q, k, v projections; RMSNorm of every q and k head over head_dim with one weight
[head_dim] for all heads (src/backend/cpu/kernels/rope.cpp:84-94); position
encoding of q and k; k and v of ALL rows of the step are written into the pages
before any row attends (src/backend/cpu/model_forward_chunk.cpp:440-520);
scores (q.k)/sqrt(head_dim) over the keys at positions <= the row's position (and
inside the window, if there is one), softmax in 32-bit, weighted sum of values,
output projection.  The scale is applied once
(include/celeg/backend/cuda/attention_norm.hpp:13-23).
"""
from __future__ import annotations

import math

import torch

from ..config.spec import PartSpec
from .base import KVNeed, Mixer, WeightSpec, build_part, register_part
from .fused import fused_rows_ok, linear_into_stream, norm_linear


class GqaAttention(Mixer):
    graph_safe = True

    def __init__(self, spec):
        super().__init__(spec)
        p = self.params
        self.width = int(p["width"])
        self.heads = int(p["heads"])
        self.kv_heads = int(p.get("kv_heads", self.heads))
        self.head_dim = int(p["head_dim"])
        self.qk_norm = bool(p.get("qk_norm", False))
        self.eps = float(p.get("eps", 1e-6))
        self.window = p.get("window")
        if self.window is not None:
            self.window = int(self.window)
            if self.window <= 0:
                raise ValueError("gqa_attention: window must be positive")
        self.scale = float(p["scale"]) if p.get("scale") is not None \
            else 1.0 / math.sqrt(self.head_dim)
        if self.heads <= 0 or self.kv_heads <= 0 or self.heads % self.kv_heads:
            raise ValueError("gqa_attention: heads must be a positive multiple of kv_heads")
        if self.head_dim <= 0 or self.head_dim % 2:
            raise ValueError("gqa_attention: head_dim must be even")
        self.position = build_part("position", p["position"]) if p.get("position") is not None \
            else build_part("position", PartSpec("none"))
        self.own_kv = True
        self.w_qkv = self.w_q = self.w_o = self.q_norm = self.k_norm = None

    # -- declarations
    def set_reads_foreign_kv(self):
        self.own_kv = False

    def kv_need(self):
        return KVNeed(self.kv_heads, self.head_dim, self.window)

    def weight_specs(self):
        q_width, kv_width = self.heads * self.head_dim, self.kv_heads * self.head_dim
        specs = {"q_proj": WeightSpec((q_width, self.width)),
                 "out_proj": WeightSpec((self.width, q_width))}
        if self.own_kv:
            specs["k_proj"] = WeightSpec((kv_width, self.width))
            specs["v_proj"] = WeightSpec((kv_width, self.width))
        if self.qk_norm:
            specs["q_norm"] = WeightSpec((self.head_dim,), kind="vector", init="around_one")
            if self.own_kv:
                specs["k_norm"] = WeightSpec((self.head_dim,), kind="vector", init="around_one")
        return specs

    def load(self, tensors, rt):
        # q, k and v projections run as one matrix product
        # (the reference's fused_projections, src/backend/cuda/execution_plan.cpp:113).
        if self.own_kv:
            self.w_qkv = torch.cat([tensors["q_proj"], tensors["k_proj"], tensors["v_proj"]],
                                   dim=0).contiguous()
            self.w_q = self.w_qkv[: self.heads * self.head_dim]
        else:
            self.w_q = tensors["q_proj"].contiguous()
        self.w_o = tensors["out_proj"].contiguous()
        self.q_norm = tensors.get("q_norm")
        self.k_norm = tensors.get("k_norm")

    # -- work
    def forward(self, x, batch, cache, rt):
        attended = self._project_and_attend(x, None, batch, cache, rt)
        out = rt.ws.buf("mixer_out", (x.shape[0], self.width), rt.dtype)
        rt.ops.linear(attended, self.w_o, out)
        return out

    def forward_fused(self, h, norm, batch, cache, rt) -> bool:
        """h += mixer(norm(h)) with the norm folded into the q/k/v product and the residual
        addition into the output product.  False if the step cannot take the fused path."""
        q_width = self.heads * self.head_dim
        w_in = self.w_qkv if cache.writes_kv else self.w_q
        if not fused_rows_ok(rt, batch, self.width, q_width) \
                or (w_in.dtype, self.w_o.dtype) != (rt.dtype,) * 2:
            return False
        attended = self._project_and_attend(h, norm, batch, cache, rt)
        linear_into_stream(rt, attended, self.w_o, h)
        return True

    def _project_and_attend(self, x, norm, batch, cache, rt):
        """``norm`` None: ``x`` are normalised rows; else ``x`` is the residual stream and the
        norm is applied inside the product."""
        T = x.shape[0]
        q_width, kv_width = self.heads * self.head_dim, self.kv_heads * self.head_dim
        writes = cache.writes_kv
        if writes and not self.own_kv:
            raise RuntimeError("gqa_attention: built without key/value projections but asked "
                               "to write a cache")

        def project(w, out):
            if norm is None:
                rt.ops.linear(x, w, out)
            else:
                norm_linear(rt, x, norm, w, out)
        if writes:
            qkv = rt.ws.buf("attn_qkv", (T, q_width + 2 * kv_width), rt.dtype)
            project(self.w_qkv, qkv)
            q = qkv[:, :q_width]
            k = qkv[:, q_width:q_width + kv_width]
            v = qkv[:, q_width + kv_width:]
        else:
            q = rt.ws.buf("attn_q", (T, q_width), rt.dtype)
            project(self.w_q, q)
            k = v = None
        tables = self.position.tables(rt)
        rt.ops.qk_norm_rope_store(
            q, k, v, self.q_norm, self.k_norm, self.eps,
            tables["inv_freq"], tables["rotary_dim"],
            self.heads, self.kv_heads, self.head_dim, batch, cache.kv)
        attended = rt.ws.buf("attn_out", (T, q_width), rt.dtype)
        rt.ops.paged_attention(q, attended, self.heads, self.kv_heads, self.head_dim,
                               self.scale, self.window, batch, cache.kv)
        return attended


register_part("mixer", "gqa_attention", GqaAttention)
