"""Position encodings used inside a mixer.

``rope``: rotary encoding with split-half pairing: for i < rotary_dim/2 the pair
(x[i], x[i + rotary_dim/2]) is rotated by the angle position * theta^(-2i/rotary_dim)
(src/backend/cpu/kernels/rope.cpp:30-36, 95-108).  The frequencies are computed on
the host in double (include/celeg/model/position.hpp:77-78) and handed to the
kernel as a 32-bit table; the angle is the 32-bit product float(position) * frequency.

``none``: no encoding.

A position encoding hands the mixer ``tables(rt)``: a dictionary with
``inv_freq`` (a device table of rotary_dim/2 frequencies, or None) and
``rotary_dim``.
"""
from __future__ import annotations

import math

import torch

from .base import PositionEncoding, register_part


class Rope(PositionEncoding):
    graph_safe = True

    def __init__(self, spec):
        super().__init__(spec)
        self.theta = float(self.params["theta"])
        self.head_dim = int(self.params["head_dim"])
        self.rotary_dim = int(self.params.get("rotary_dim", self.head_dim))
        if not self.theta > 0:
            raise ValueError("rope: theta must be positive")
        if self.rotary_dim <= 0 or self.rotary_dim % 2 or self.rotary_dim > self.head_dim:
            raise ValueError("rope: rotary_dim must be even, positive and at most head_dim")
        self._table = None

    def inverse_frequencies(self):
        half = self.rotary_dim // 2
        return [math.pow(self.theta, -2.0 * i / self.rotary_dim) for i in range(half)]

    def tables(self, rt):
        if self._table is None or self._table.device != torch.device(rt.device):
            self._table = torch.tensor(self.inverse_frequencies(), dtype=torch.float64) \
                .to(torch.float32).to(rt.device)
        return {"inv_freq": self._table, "rotary_dim": self.rotary_dim}


class NoPosition(PositionEncoding):
    graph_safe = True

    def tables(self, rt):
        return {"inv_freq": None, "rotary_dim": 0}


register_part("position", "rope", Rope)
register_part("position", "none", NoPosition)
