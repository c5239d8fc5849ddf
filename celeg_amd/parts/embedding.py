"""Token embedding and the output head.

h0[t] = E[token[t]], nothing added and no scaling
(src/backend/cpu/model_forward_token.cpp:28-60); logits = x E_out^T with
E_out = E when the head is tied, else lm_head
(src/backend/cpu/model_forward_token.cpp:213-218;
src/model/inference/layer_bindings.cpp:24-95).  Logits leave in 32-bit."""
from __future__ import annotations

from .base import Embedding, Head, WeightSpec, register_part


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

    def forward(self, token_ids, out, rt):
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


register_part("embedding", "embedding", TokenEmbedding)
register_part("head", "tied_head", TiedHead)
register_part("head", "linear_head", LinearHead)
