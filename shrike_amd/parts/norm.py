"""RMSNorm fused with the residual add that precedes it."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import HiddenState, Norm, ParamSpec, register_norm


class RMSNorm(Norm):
    """y = x * rsqrt(mean(x^2) + eps) * (offset + weight) in float32, one cast at the
    end (reference: shrike/models/qwen.py:70-74, where the offset is 0).  A weight that
    is stored around zero (offset 1) gets its offset when it is loaded, in float32."""

    launches_follow_shape = True

    def params(self):
        offset = float(getattr(self.spec, "offset", 0.0))
        return [ParamSpec(self.tensor_name("weight"), (self.width,), init="norm" if offset == 0.0 else "norm_zero",
                          keep_float32=True)]

    def load(self, tensors, runtime):
        self.weight = tensors[self.tensor_name("weight")]
        offset = float(getattr(self.spec, "offset", 0.0))
        if offset != 0.0:
            self.weight = (self.weight.to(torch.float32) + offset).contiguous()
        self.eps = float(self.spec.eps)

    def forward(self, ctx, hidden: HiddenState, rows=None, write_resid=True) -> torch.Tensor:
        n = hidden.resid.shape[0] if rows is None else rows.shape[0]
        out = ctx.buffer(f"normed", (n, self.width), ctx.dtype)
        if hidden.pending is not None and hidden.pending_norm is not None:
            dweight, deps = hidden.pending_norm
            ops.add_normed_rmsnorm(hidden.resid, hidden.pending, dweight, deps, self.weight, self.eps, out,
                                   rows, write_resid)
        else:
            ops.add_rmsnorm(hidden.resid, hidden.pending, self.weight, self.eps, out, rows, write_resid)
        if write_resid:
            hidden.pending = hidden.pending_norm = None
        return out


register_norm("rmsnorm", RMSNorm)
