"""A plain, slow form of the Mofarax decoder, one function per mechanism, written
from the design's equations with torch on the CPU.  It shares nothing with the
package: it takes the raw config dictionary and a dictionary of tensors by their
names in the weight file, runs one whole sequence at a time, keeps no cache, and
returns float32 (or float64) logits for every position.

Notation: W[.] are matrices stored [out, in]; x is the residual stream
[tokens, width]; positions count from 0.
"""

from __future__ import annotations

import math

import torch


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps), the eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def zero_centred_norm(x, w, eps):
    """RMS norm whose weight is stored around zero."""
    return unit_rms(x, eps) * (1.0 + w)


def plain_weight_norm(x, w, eps):
    return unit_rms(x, eps) * w


def embed(tokens, table, scale):
    return table[tokens] * scale


def rotate_interleaved(x, positions, base: float, dims: int, angle_dtype=None):
    """x [tokens, heads, dim].  Elements 2i and 2i+1 (i < dims/2) form a pair that
    turns by positions * base**(-2i/dims); elements from `dims` on stay.  The design
    forms positions and angles in 32-bit: with angle_dtype=torch.float32 the rates are
    rounded to it and the product is formed in it (thousands of radians are then known
    to about 1e-4), otherwise everything has x's precision."""
    out = x.clone()
    if dims == 0:
        return out
    i = torch.arange(dims // 2, dtype=torch.float64)
    rate = (base ** (-2.0 * i / dims)).to(angle_dtype or x.dtype)
    angle = (positions.to(rate.dtype)[:, None] * rate[None, :]).to(x.dtype)  # [tokens, dims/2]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def chunk_mask(n: int, size: int) -> torch.Tensor:
    """visible[i, j]: j <= i and both in the same block of `size` positions counted from 0."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (j <= i) & (i // size == j // size)


def attention_mixer(h, positions, w, prefix: str, m: dict):
    """Grouped-query attention whose values are the keys as projected (before the
    rotation); rotation of part of each head; block-local causal mask."""
    n = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w[prefix + ".q"].T).view(n, H, D)
    k = (h @ w[prefix + ".k"].T).view(n, G, D)
    v = k
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = rotate_interleaved(q, positions, float(rot["base"]), int(rot["dims"]))
    kr = rotate_interleaved(k, positions, float(rot["base"]), int(rot["dims"]))
    visible = chunk_mask(n, int(m["mask"]["size"]))
    out = torch.zeros(n, H, D, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ kr[:, g].T) * m["scale"]
        s = s.masked_fill(~visible, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, head] = p @ v[:, g]
    return out.reshape(n, H * D) @ w[prefix + ".o"].T


def dense_ff(h, w, prefix: str):
    return (gelu_tanh(h @ w[prefix + ".gate"].T) * (h @ w[prefix + ".up"].T)) @ w[prefix + ".down"].T


def token_side(x, tokens, w, layer: int, dim: int, eps: float):
    """The per-layer token input: a slice of a second embedding, gated by the stream."""
    e = w["side.embed"][tokens][:, layer * dim : (layer + 1) * dim]
    g = gelu_tanh(x @ w[f"l{layer}.side.gate"].T) * e
    y = g @ w[f"l{layer}.side.proj"].T
    return x + plain_weight_norm(y, w[f"l{layer}.side.norm"], eps)


def layer_forward(x, tokens, positions, w, cfg, layer: int):
    spec = cfg["layers"][layer]
    eps = cfg["norm"]["eps"]
    if spec["type"] != "attention":
        raise ValueError(f"unknown mixer {spec['type']!r}")
    h = zero_centred_norm(x, w[f"l{layer}.norm1"], eps)
    y = attention_mixer(h, positions, w, f"l{layer}.mix", spec["mixer"])
    if spec.get("mlp") is not None:
        if spec["mlp"]["kind"] != "dense":
            raise ValueError(f"unknown feed-forward {spec['mlp']['kind']!r}")
        y = y + dense_ff(h, w, f"l{layer}.mlp")
    x = x + y
    side = cfg.get("token_side")
    if side:
        x = token_side(x, tokens, w, layer, int(side["dim"]), eps)
    return x


def layer_runs(cfg) -> list[tuple[int, int | None]]:
    """(layer, pass number if this run opens a pass of the loop) in running order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, None) for i in range(start)]
    for t in range(times):
        for i in range(start, stop):
            runs.append((i, t if i == start else None))
    return runs + [(i, None) for i in range(stop, n)]


def forward(cfg: dict, weights: dict, tokens, dtype=torch.float32, return_layers: bool = False):
    """Logits [tokens, vocab] of one sequence; with return_layers also the stream
    after every layer run."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.numel())
    x0 = embed(tokens, w["embed"], cfg["embedding"]["scale"])
    x = x0
    after = []
    for layer, opens in layer_runs(cfg):
        if opens is not None:
            if opens > 0:
                x = x + x0
            x = x + w["loop.step"][opens]
        x = layer_forward(x, tokens, positions, w, cfg, layer)
        after.append(x)
    logits = zero_centred_norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].T
    if return_layers:
        return logits, torch.stack(after)
    return logits


def block_local_attention(q, k, v, scale: float, size: int, first: int = 0, window: int | None = None):
    """q [n, heads, dim] at positions first .. first + n - 1 over keys and values
    [ctx, groups, dim] at positions 0 .. ctx - 1: query i reads key j <= i of its own
    block of `size` positions (and, with a window, only the last `window` keys up to
    i).  One query and one head at a time, written out."""
    n, heads, dim = q.shape
    groups = k.shape[1]
    out = torch.zeros(n, heads, v.shape[2], dtype=q.dtype)
    for r in range(n):
        i = first + r
        lo = i // size * size
        if window is not None:
            lo = max(lo, i - window + 1)
        for head in range(heads):
            g = head // (heads // groups)
            s = (k[lo : i + 1, g] @ q[r, head]) * scale
            p = torch.softmax(s, dim=0)
            out[r, head] = p @ v[lo : i + 1, g]
    return out


class PlainMofarax:
    """A model folder read once; `logits(ids)` and greedy generation over it."""

    def __init__(self, model_dir, dtype=torch.float64):
        import json
        from pathlib import Path

        from safetensors.torch import load_file

        self.cfg = json.loads((Path(model_dir) / "config.json").read_text())
        self.weights = load_file(str(Path(model_dir) / "model.safetensors"))
        self.dtype = dtype

    def logits(self, token_ids, rows=None) -> torch.Tensor:
        out = forward(self.cfg, self.weights, list(token_ids), self.dtype)
        return out if rows is None else out[torch.tensor(list(rows), dtype=torch.long)]

    def layers(self, token_ids) -> torch.Tensor:
        return forward(self.cfg, self.weights, list(token_ids), self.dtype, return_layers=True)[1]

    def greedy(self, prompt, max_new_tokens: int) -> list[int]:
        seq, out = list(prompt), []
        for _ in range(max_new_tokens):
            tok = int(torch.argmax(self.logits(seq)[-1]))
            out.append(tok)
            seq.append(tok)
        return out
