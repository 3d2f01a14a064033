"""The two ends of a model: token embedding and the output head.

Embedding: x[t] = E[ids[t]] (engine/model.py:65).  Head: tied, logits = x E^T over
the embedding's own storage (engine/nn/layers.py:14-30); untied, x W^T without bias
(HF lm_head has none; the reference's default-bias nn.Linear,
engine/models/_builder.py:96, is not copied).  Logits leave in float32.
"""

from __future__ import annotations

import torch

from tokensprint_amd.kernels.stream import fused_rmsnorm_of
from tokensprint_amd.parts.base import (EMBEDDINGS, HEADS, OutputHead, TensorDecl,
                                        TokenEmbedding, register)


@register(EMBEDDINGS, "embedding")
class Embedding(TokenEmbedding):
    """params: weight (checkpoint name), vocab_size."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.name = params["weight"]
        self.vocab = int(params["vocab_size"])
        self.table = None

    def tensors(self):
        return {self.name: TensorDecl((self.vocab, self.ctx.width))}

    def load(self, get):
        self.table = get(self.name)

    def forward(self, token_ids):
        return self.ops.embed(self.table, token_ids)

    def step_read_tensors(self):
        return []          # a step reads the rows of its tokens, not the table


@register(HEADS, "head")
class Head(OutputHead):
    """params: weight (name), vocab_size, tied (bool: `weight` is the embedding's)."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.name = params["weight"]
        self.vocab = int(params["vocab_size"])
        self.tied = bool(params.get("tied", False))
        self.ignored = params.get("ignored")      # a tied file's redundant copy
        self.weight = None

    def tensors(self):
        t = {self.name: TensorDecl((self.vocab, self.ctx.width))}
        if self.ignored:
            t[self.ignored] = TensorDecl((self.vocab, self.ctx.width), optional=True)
        return t

    def load(self, get):
        self.weight = get(self.name)

    def forward(self, h):
        return self.ops.linear(h, self.weight, torch.float32)

    def forward_from_stream(self, resid, delta, norm):
        """Logits of the rows of the residual stream (resid float32, delta the last
        sub-layer's output not yet added, or None) behind `norm`; the add and the norm go
        into the product where the norm and the kernel provider allow it."""
        fused = fused_rmsnorm_of(norm)
        if fused is not None:
            return self.ops.norm_linear(resid, delta, fused[0], fused[1], self.weight,
                                        torch.float32)[0]
        h = norm.forward(resid) if delta is None else norm.add_forward(resid, delta)
        return self.forward(h)
