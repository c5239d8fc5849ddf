"""The arrangement of a layer's parts.

``pre_norm``: h += mixer(norm1(h)); h += ffn(norm2(h))
(src/backend/cpu/model_forward_token.cpp:93-172).  The residual stream ``h`` is
32-bit in every mode and each sum into it is made in 32-bit; an addition is carried
forward as ``delta`` and made by the next norm's kernel, which reads ``h`` anyway.

A block arrangement is a class with ``__init__(layer_spec)`` that builds its parts,
``parts()`` (name -> part, for weights and cache needs), and
``forward(h, delta, batch, cache, rt) -> delta``.
"""
from __future__ import annotations

from .base import build_part, register_part
from .norm import RmsNorm


class PreNormBlock:
    def __init__(self, layer_spec):
        self.spec = layer_spec
        self.mixer_norm = build_part("norm", layer_spec.mixer_norm)
        self.mixer = build_part("mixer", layer_spec.mixer)
        self.ffn_norm = build_part("norm", layer_spec.ffn_norm)
        self.ffn = build_part("ffn", layer_spec.ffn)

    def parts(self):
        return {"mixer_norm": self.mixer_norm, "mixer": self.mixer,
                "ffn_norm": self.ffn_norm, "ffn": self.ffn}

    def forward(self, h, delta, batch, cache, rt):
        """``h`` [T, width] 32-bit, ``delta`` an addition to ``h`` not made yet (or None).
        Returns the feed-forward's output, which the caller's next norm adds."""
        T, width = h.shape
        normed = rt.ws.buf("normed", (T, width), rt.dtype)
        # Few rows: parts that can, take the norm in front of them and the addition behind
        # them into their own products and write the stream themselves.
        fusable = isinstance(self.mixer_norm, RmsNorm) and isinstance(self.ffn_norm, RmsNorm)
        mixed = delta
        if not (fusable and delta is None and hasattr(self.mixer, "forward_fused")
                and self.mixer.forward_fused(h, self.mixer_norm, batch, cache, rt)):
            rt.stream_stat_blocks = 0
            self.mixer_norm.forward(h, normed, rt, delta=delta)
            mixed = self.mixer.forward(normed, batch, cache, rt)
        else:
            mixed = None
        if fusable and mixed is None and hasattr(self.ffn, "forward_fused") \
                and self.ffn.forward_fused(h, self.ffn_norm, batch, rt):
            return None
        rt.stream_stat_blocks = 0
        self.ffn_norm.forward(h, normed, rt, delta=mixed)
        return self.ffn.forward(normed, batch, rt)


register_part("block", "pre_norm", PreNormBlock)
