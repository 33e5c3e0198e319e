"""Token embedding: the residual stream starts as the table's rows."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Embedding, ParamSpec, register_embedding


class TokenEmbedding(Embedding):
    """x[n] = table[token_ids[n]] * scale, widened to float32 (reference:
    shrike/models/qwen.py:156,161, which has no scale: the spec's default of 1)."""

    launches_follow_shape = True

    def params(self):
        return [ParamSpec(self.tensor_name("weight"), (self.spec.vocab_size, self.width), init="embedding")]

    def load(self, tensors, runtime):
        self.table = tensors[self.tensor_name("weight")]
        self.scale = float(getattr(self.spec, "scale", 1.0))

    def forward(self, ctx, into: str = "resid") -> torch.Tensor:
        """Into the workspace buffer `into`; a model that needs the embedding's output
        again later asks for it a second time under another name."""
        resid = ctx.buffer(into, (ctx.num_tokens, self.width), torch.float32)
        ops.embed(self.table, ctx.token_ids, resid, self.scale)
        return resid


register_embedding("token_lookup", TokenEmbedding)
