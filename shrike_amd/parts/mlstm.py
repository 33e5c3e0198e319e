"""The matrix memory of xLSTM (mLSTM) as a mixer with a state slot per request."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Mixer, ParamSpec, StateSpec, register_mixer


class MatrixLSTM(Mixer):
    """One product yields every projection of a token in float32: queries, keys, values,
    the output gate, and the two recurrence gates' pre-activations.  The scan kernel
    carries S, n and m per head in the request's state slot (float32), token by token,
    whether the tokens come as a prompt's portion or one at a time; the readout is
    normed per head, weighted, gated and projected.

    Everything that enters the recurrence is float32: the projections leave their
    product unrounded, the gates' tanh, logsigmoid and exponentials, the decay and the
    state are float32 in the kernel."""

    launches_follow_shape = True
    state_graph_safe = True  # the state is reached through ctx.state_slots on the device

    def _t(self, role: str) -> str:
        return self.tensor_name(role)

    def params(self):
        s, h = self.spec, self.width
        qk, v = s.num_heads * s.head_dim, s.num_heads * s.value_dim
        return [
            ParamSpec(self._t("q"), (qk, h)), ParamSpec(self._t("k"), (qk, h)), ParamSpec(self._t("v"), (v, h)),
            ParamSpec(self._t("g"), (v, h)), ParamSpec(self._t("o"), (h, v)),
            ParamSpec(self._t("norm"), (v,), init="norm", keep_float32=True),
            ParamSpec(self._t("i"), (s.num_heads, h)), ParamSpec(self._t("i.b"), (s.num_heads,), init="bias", keep_float32=True),
            ParamSpec(self._t("f"), (s.num_heads, h)), ParamSpec(self._t("f.b"), (s.num_heads,), init="bias", keep_float32=True),
        ]

    def state_floats(self) -> int:
        """Per head and tile of 4 value columns: the tile's columns of S as the scan's lanes
        hold them (rows padded to 64, 128 or 256), then n and m (every tile keeps its own
        copy of n and m; csrc/mlstm.hip)."""
        s = self.spec
        tiles = -(-s.value_dim // 4)
        rpt = 4 if s.head_dim <= 64 else 8 if s.head_dim <= 128 else 16
        return s.num_heads * tiles * (64 * rpt + 16 * rpt + 1)

    def cache_spec(self):
        return StateSpec((self.state_floats(),), "float32")

    def check(self, runtime):
        s = self.spec
        if min(s.num_heads, s.head_dim, s.value_dim) < 1:
            raise ValueError(f"{self.name}: heads, head_dim and value_dim must be positive")
        if s.head_dim > 256:
            raise ValueError(f"{self.name}: head_dim {s.head_dim} is more than the 256 the scan kernel holds")
        if not s.gate_cap > 0:
            raise ValueError(f"{self.name}: gate_cap must be positive, got {s.gate_cap}")
        if ops.mlstm_state_floats(s.num_heads, s.head_dim, s.value_dim) != self.state_floats():
            raise RuntimeError(f"{self.name}: the kernel's state layout and the cache's size disagree")

    def load(self, tensors, runtime):
        s = self.spec
        roles = ("q", "k", "v", "g", "i", "f")
        self.w_in = runtime.weight(torch.cat([tensors[self._t(r)] for r in roles], dim=0))
        qk, v = s.num_heads * s.head_dim, s.num_heads * s.value_dim
        self.offsets = {"q": 0, "k": qk, "v": 2 * qk, "g": 2 * qk + v, "i": 2 * qk + 2 * v,
                        "f": 2 * qk + 2 * v + s.num_heads}
        self.in_width = 2 * qk + 2 * v + 2 * s.num_heads
        self.i_bias, self.f_bias = tensors[self._t("i.b")], tensors[self._t("f.b")]
        self.norm_weight = tensors[self._t("norm")]
        self.w_o = runtime.weight(tensors[self._t("o")])
        self.linear = runtime.linear
        self.linear_deferred = runtime.linear_deferred

    def forward(self, ctx, x: torch.Tensor, cache) -> torch.Tensor:
        s, off = self.spec, self.offsets
        n = x.shape[0]
        proj = ctx.buffer("mlstm_proj", (n, self.in_width), torch.float32)
        self.linear(x, self.w_in, proj)
        read = ctx.buffer("mlstm_read", (n, s.num_heads * s.value_dim), torch.float32)
        # the view with the spare slot: padding rows of a fixed-size batch write there
        state = cache.state_padded if cache.state_padded is not None else cache.state
        ops.mlstm_scan(proj, off["q"], off["k"], off["v"], off["i"], off["f"], self.i_bias, self.f_bias,
                       s.gate_cap, float(s.head_dim) ** -0.5, ctx.num_seqs, s.num_heads, s.head_dim, s.value_dim,
                       ctx.positions, ctx.cu_q, ctx.state_slots, state, read)
        gated = ctx.buffer("mlstm_gated", (n, s.num_heads * s.value_dim), ctx.dtype)
        ops.headnorm_gate(read, proj[:, off["g"]:], self.norm_weight, s.eps, gated, s.num_heads, s.value_dim)
        return self.linear_deferred(ctx, "mlstm_out", gated, self.w_o)


register_mixer("mlstm", MatrixLSTM)
