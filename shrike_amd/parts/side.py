"""A per-layer token input: a second embedding, gated by the stream."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import HiddenState, ParamSpec, SideInput, register_side


class TokenSide(SideInput):
    """e = table[token][index * dim : (index + 1) * dim];  g = act(W_gate x) * e;
    y = W_proj g;  the stream gains y * rsqrt(mean(y^2) + eps) * weight.

    The table [vocab, slices * dim] is one tensor for all layers (its full name is
    in the spec); a layer reads its own slice of the token's row, whichever pass of
    a loop it runs in.  The two products are ordinary products of the runtime (both
    may come as partial sums of shares of k); the activation and the gather are one
    kernel, which adds the first product's shares up (the gates reach it in float32,
    split or not: a gate that is rounded to 8 bits first loses more where gelu is
    steep, and the norm below does not damp what a tiny y has lost); y stays pending with its norm, and
    the norm that follows (the next layer's, or the final one) forms
    resid + normed(y) and its own output in one pass over the row."""

    launches_follow_shape = True

    def params(self):
        s = self.spec
        return [
            ParamSpec(s.table_name, (s.vocab_size, s.slices * s.dim), init="embedding"),
            ParamSpec(self.tensor_name("gate"), (s.dim, self.width)),
            ParamSpec(self.tensor_name("proj"), (self.width, s.dim)),
            ParamSpec(self.tensor_name("norm"), (self.width,), init="norm", keep_float32=True),
        ]

    def check(self, runtime):
        s = self.spec
        ops.activation_code(s.activation)
        if not 0 <= s.index < s.slices or s.dim < 1:
            raise ValueError(f"{self.name}: slice {s.index} of {s.slices} slices of {s.dim} does not exist")

    def load(self, tensors, runtime):
        s = self.spec
        self.table = tensors[s.table_name]
        self.w_gate = runtime.weight(tensors[self.tensor_name("gate")])
        self.w_proj = runtime.weight(tensors[self.tensor_name("proj")])
        self.weight = tensors[self.tensor_name("norm")]
        self.eps = float(s.eps)
        self.linear_deferred = runtime.linear_deferred

    def forward(self, ctx, hidden: HiddenState, x: torch.Tensor) -> None:
        s = self.spec
        n = x.shape[0]
        gate = self.linear_deferred(ctx, "side_gate", x, self.w_gate, reader="rows", keep_float32=True)
        gated = ctx.buffer("side_gated", (n, s.dim), ctx.dtype)
        ops.act_mul_rows(gate, self.table, ctx.token_ids, s.index * s.dim, gated, s.activation)
        hidden.pending = self.linear_deferred(ctx, "side_out", gated, self.w_proj)
        hidden.pending_norm = (self.weight, self.eps)


register_side("token_side", TokenSide)
