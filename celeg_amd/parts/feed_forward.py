"""SwiGLU feed-forward: (silu(x W1^T) * (x W3^T)) W2^T, silu(g) = g / (1 + exp(-g))
(src/backend/cpu/model_forward_token.cpp:163-172; kernels/elementwise.cpp:101-119).
Gate and up projections run as one matrix product on the concatenation [W1; W3]
(rows [0,ff) gate, [ff,2ff) up), as the reference's w13
(src/backend/cuda/model/weight_setup.cpp:289-306)."""
from __future__ import annotations

import torch

from .base import FeedForward, WeightSpec, register_part
from .fused import fused_rows_ok, linear_into_stream, norm_linear, operand_rows


class SwiGlu(FeedForward):
    graph_safe = True

    def __init__(self, spec):
        super().__init__(spec)
        self.width = int(self.params["width"])
        self.ff = int(self.params["ff"])
        if self.width <= 0 or self.ff <= 0:
            raise ValueError("swiglu: width and ff must be positive")
        self.w_gate_up = self.w_down = None

    def weight_specs(self):
        return {"gate": WeightSpec((self.ff, self.width)),
                "up": WeightSpec((self.ff, self.width)),
                "down": WeightSpec((self.width, self.ff))}

    def load(self, tensors, rt):
        gate, up = tensors["gate"], tensors["up"]
        if gate.dtype != up.dtype:
            gate, up = gate.float(), up.float()
        self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = tensors["down"].contiguous()

    def forward(self, x, batch, rt):
        T = x.shape[0]
        gate_up = rt.ws.buf("ffn_gate_up", (T, 2 * self.ff), rt.dtype)
        rt.ops.linear(x, self.w_gate_up, gate_up)
        act = rt.ws.buf("ffn_act", (T, self.ff), rt.dtype)
        rt.ops.swiglu(gate_up, act)
        out = rt.ws.buf("ffn_out", (T, self.width), rt.dtype)
        rt.ops.linear(act, self.w_down, out)
        return out


    def forward_fused(self, h, norm, batch, rt) -> bool:
        """h += ffn(norm(h)): the norm and the SwiGLU folded into the first product, the
        residual addition into the second.  False if the step cannot take the fused path."""
        if not fused_rows_ok(rt, batch, self.width, self.ff) \
                or (self.w_gate_up.dtype, self.w_down.dtype) != (rt.dtype,) * 2:
            return False
        act = operand_rows(rt, "ffn_act_fused", batch.n_tokens, self.ff, self.width)
        norm_linear(rt, h, norm, self.w_gate_up, act, epilogue="swiglu")
        linear_into_stream(rt, act, self.w_down, h)
        return True


register_part("ffn", "swiglu", SwiGlu)
