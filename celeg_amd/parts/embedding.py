"""Token embedding and the output head.

h0[t] = E[token[t]], nothing added and no scaling
(src/backend/cpu/model_forward_token.cpp:28-60); logits = x E_out^T with
E_out = E when the head is tied, else lm_head
(src/backend/cpu/model_forward_token.cpp:213-218;
src/model/inference/layer_bindings.cpp:24-95).  Logits leave in 32-bit."""
from __future__ import annotations

import torch

from .base import Embedding, Head, WeightSpec, register_part
from .fused import _sliced, fused_rows_ok, norm_linear, stream_bf16, stream_stats, tiled_step
from .norm import RmsNorm


class TokenEmbedding(Embedding):
    graph_safe = True

    def __init__(self, spec):
        super().__init__(spec)
        self.vocab = int(self.params["vocab"])
        self.width = int(self.params["width"])
        self.table = None

    def weight_specs(self):
        return {"table": WeightSpec((self.vocab, self.width))}

    def load(self, tensors, rt):
        self.table = tensors["table"].contiguous()

    def forward(self, token_ids, out, rt, batch=None):
        if batch is not None and self.table.dtype == torch.bfloat16 \
                and fused_rows_ok(rt, batch, self.width):
            # few rows: leave every row's sum of squares (and the bfloat16 copy of the
            # stream) for the first norm
            if _sliced(rt, out.shape[0], self.width) or tiled_step(rt, out.shape[0]):
                rt.ops.embed_stream(self.table, token_ids, out,
                                    stream_bf16(rt, out.shape[0], self.width),
                                    stream_stats(rt, self.width, out.shape[0]))
                rt.stream_has_bf16 = True
            else:
                rt.ops.embed_stats(self.table, token_ids, out, stream_stats(rt, self.width))
                rt.stream_has_bf16 = False
            rt.stream_stat_blocks = 1
        else:
            rt.ops.embed(self.table, token_ids, out)
        return out


class TiedHead(Head):
    """Uses the embedding table; wants no tensor of its own."""
    graph_safe = True

    def __init__(self, spec):
        super().__init__(spec)
        self.vocab = int(self.params["vocab"])

    def forward(self, x, out, rt, embedding=None):
        rt.ops.linear(x, embedding.table, out)
        return out

    def forward_fused(self, h, norm, batch, out, rt, embedding=None) -> bool:
        return _head_fused(h, norm, batch, out, rt, embedding.table)


class LinearHead(Head):
    graph_safe = True

    def __init__(self, spec):
        super().__init__(spec)
        self.vocab = int(self.params["vocab"])
        self.width = int(self.params["width"])
        self.weight = None

    def weight_specs(self):
        return {"weight": WeightSpec((self.vocab, self.width))}

    def load(self, tensors, rt):
        self.weight = tensors["weight"].contiguous()

    def forward(self, x, out, rt, embedding=None):
        rt.ops.linear(x, self.weight, out)
        return out

    def forward_fused(self, h, norm, batch, out, rt, embedding=None) -> bool:
        return _head_fused(h, norm, batch, out, rt, self.weight)


def _head_fused(h, norm, batch, out, rt, weight) -> bool:
    """Final norm and output product in one kernel for few wanted rows, 32-bit logits."""
    R = batch.n_logit_rows
    if not (isinstance(norm, RmsNorm) and weight.dtype == torch.bfloat16
            and fused_rows_ok(rt, batch, h.shape[1]) and 0 < R <= 64
            and not tiled_step(rt, batch.n_tokens)):
        return False
    norm_linear(rt, h, norm, weight, out, epilogue="store_f32", rows=batch.logit_rows, n_rows=R)
    return True


register_part("embedding", "embedding", TokenEmbedding)
register_part("head", "tied_head", TiedHead)
register_part("head", "linear_head", LinearHead)
