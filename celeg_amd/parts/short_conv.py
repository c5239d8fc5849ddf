"""Double-gated short causal convolution.

bcx = x W_in^T splits into B = [0,H), C = [H,2H), x = [2H,3H)
(src/backend/cpu/kernels/convolution.cpp:16-18); bx = B*x;
conv[t,ch] = sum_tap w[ch,tap] * bx[t-(L-1-tap), ch], zero before position 0, so the
last tap multiplies the current token (convolution.cpp:19-26); y = C*conv;
out = y W_out^T (src/backend/cpu/operators/recurrent.cpp:212-240).  A step continues
from the request's saved state wherever the previous step stopped, as the
reference's ragged kernel does (src/backend/cuda/kernels/shortconv.cuh:34-64).

State per request: the last L values of bx, [L, H] in 32-bit, entry j holding
position (tokens seen so far) - L + j; every row of a step reads the old state,
then the state is replaced.

With ``bias`` (the reference's ShortConvolutionSpec.bias is never true,
include/celeg/model/graph.hpp:316-320): in_proj bias [3H] is added to bcx, the
convolution bias [H] to conv before the C gate, out_proj bias [H] to the output.
"""
from __future__ import annotations

import torch

from .base import Mixer, StateNeed, WeightSpec, register_part
from .fused import fused_rows_ok, linear_into_stream, norm_linear, operand_rows, tiled_step


class ShortConv(Mixer):
    graph_safe = True

    def __init__(self, spec):
        super().__init__(spec)
        self.width = int(self.params["width"])
        self.taps = int(self.params["taps"])
        self.bias = bool(self.params.get("bias", False))
        if self.width <= 0 or self.taps <= 0:
            raise ValueError("short_conv: width and taps must be positive")
        self.w_in = self.w_conv = self.w_out = None
        self.b_in = self.b_conv = self.b_out = None

    def state_needs(self):
        return [StateNeed("bx", (self.taps, self.width), torch.float32)]

    def weight_specs(self):
        H, L = self.width, self.taps
        specs = {"in_proj": WeightSpec((3 * H, H)),
                 "conv": WeightSpec((H, 1, L), kind="vector", also=((H, L),)),
                 "out_proj": WeightSpec((H, H))}
        if self.bias:
            specs["in_proj_bias"] = WeightSpec((3 * H,), kind="vector")
            specs["conv_bias"] = WeightSpec((H,), kind="vector")
            specs["out_proj_bias"] = WeightSpec((H,), kind="vector")
        return specs

    def load(self, tensors, rt):
        self.w_in = tensors["in_proj"].contiguous()
        self.w_conv = tensors["conv"].reshape(self.width, self.taps).contiguous()
        self.w_out = tensors["out_proj"].contiguous()
        if self.bias:
            self.b_in = tensors["in_proj_bias"]
            self.b_conv = tensors["conv_bias"]
            self.b_out = tensors["out_proj_bias"]

    def forward(self, x, batch, cache, rt):
        T, H = x.shape[0], self.width
        bcx = rt.ws.buf("conv_bcx", (T, 3 * H), rt.dtype)
        rt.ops.linear(x, self.w_in, bcx, bias=self.b_in)
        y = rt.ws.buf("conv_y", (T, H), rt.dtype)
        rt.ops.short_conv(bcx, self.w_conv, self.b_conv, cache.states["bx"], y, batch)
        out = rt.ws.buf("mixer_out", (T, H), rt.dtype)
        rt.ops.linear(y, self.w_out, out, bias=self.b_out)
        return out


    def forward_fused(self, h, norm, batch, cache, rt) -> bool:
        """h += mixer(norm(h)) with the norm, the convolution (for one new token per
        request) and the residual addition folded into the two products.  False if this
        step cannot take the fused path (nothing is done then)."""
        H = self.width
        if not fused_rows_ok(rt, batch, H) or (self.w_in.dtype, self.w_out.dtype) != (rt.dtype,) * 2:
            return False
        T = batch.n_tokens
        if batch.decode_only and batch.n_seqs == T and self.taps <= 8 and not tiled_step(rt, T):   # the fused form holds 8 taps
            y = operand_rows(rt, "conv_y_fused", T, H, H)
            norm_linear(rt, h, norm, self.w_in, y, epilogue="conv", bias=self.b_in,
                        conv=(self.w_conv, self.b_conv, cache.states["bx"], batch.seq_slot))
        else:
            y = rt.ws.buf("conv_y", (T, H), rt.dtype)
            bcx = rt.ws.buf("conv_bcx", (T, 3 * H), rt.dtype)
            norm_linear(rt, h, norm, self.w_in, bcx, bias=self.b_in)
            rt.ops.short_conv(bcx, self.w_conv, self.b_conv, cache.states["bx"], y, batch)
        linear_into_stream(rt, y, self.w_out, h, bias=self.b_out)
        return True


register_part("mixer", "short_conv", ShortConv)
