"""The two ends of a model: token ids in, logits out.

``token_table`` (crates/spite-models/src/llama/llama4.rs:118-119): row ``id`` of the table as
the residual stream's first value, in fp32.
``linear_head`` (llama4.rs:277-279): logits = W . (normed last hidden state), W ``[V, d]``;
tied, it reads the embedding's table.  Another architecture's embedding scale, logit cap or
bias is another kind registered under these categories, not a change to the model class.
"""
from __future__ import annotations

from .base import Embedding, Head, ParamSpec, register
from .linear import linear, Weight
from ..csrc import hipops


@register("embedding", "token_table")
class TokenTable(Embedding):
    graph_safe = True

    def __init__(self, env, vocab_size: int, width: int):
        self.V, self.d = int(vocab_size), int(width)
        self.table = None

    def params(self):
        return {"weight": ParamSpec((self.V, self.d))}

    def load(self, tensors):
        self.table = tensors["weight"].contiguous()

    def forward(self, token_ids, h, ctx):
        hipops.embed(token_ids, self.table, h)


@register("head", "linear_head")
class LinearHead(Head):
    graph_safe = True

    def __init__(self, env, vocab_size: int, width: int, tied: bool = False):
        self.V, self.d, self.tied = int(vocab_size), int(width), bool(tied)
        self.weight = None

    def params(self):
        return {} if self.tied else {"weight": ParamSpec((self.V, self.d))}

    def load(self, tensors):
        if not self.tied:
            self.weight = Weight(tensors["weight"])

    def tie(self, embedding):
        """Tied: the table stays row-major (the embedding reads its rows) and serves as W."""
        if self.tied:
            self.weight = embedding.table

    def slow_paths(self, page_size):
        return self.weight.slow_reason("output matrix") if isinstance(self.weight, Weight) else []

    def forward(self, x, logits, ctx):
        linear(x, self.weight, logits, ws=ctx.ws)
