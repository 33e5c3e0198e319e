"""A plain, slow form of the Minilorn decoder, one function per mechanism, written
from the design's equations with torch on the CPU.  It shares nothing with the
package: it takes the raw config dictionary and a dictionary of tensors by their
names in the weight file, runs one whole sequence at a time, keeps no cache, and
returns logits for every position (in the precision of the tensors it is given).

Notation: W[.] are matrices stored [out, in]; x is the residual stream
[tokens, width]; positions count from 0.
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps), the eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def weighted_norm(x, w, eps):
    return unit_rms(x, eps) * w


def bigram_rows(tokens: torch.Tensor, buckets: int, mul_prev: int, mul_cur: int) -> torch.Tensor:
    """Row of the pair table for every position: a hash of (previous token, token);
    the first position, which has no previous token, takes the table's last row."""
    rows = torch.full_like(tokens, buckets)
    rows[1:] = (tokens[:-1] * mul_prev + tokens[1:] * mul_cur) % buckets
    return rows


def embed(tokens, w, cfg):
    x = w["embed"][tokens]
    b = (cfg.get("embedding") or {}).get("bigram")
    if b:
        x = x + w["bigram"][bigram_rows(tokens, int(b["buckets"]), int(b["mul_prev"]), int(b["mul_cur"]))]
    return x


def causal_mask(n: int, window: int | None = None) -> torch.Tensor:
    """visible[i, j]: j <= i, and with a window also i - j < window."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    vis = j <= i
    if window is not None:
        vis = vis & (i - j < window)
    return vis


def query_temperature(positions: torch.Tensor, coef: float, every: int, dtype) -> torch.Tensor:
    """1 + coef * ln(floor((p + 1) / every) + 1) per position."""
    steps = torch.div(positions + 1, every, rounding_mode="floor")
    return (1.0 + coef * torch.log(steps.to(torch.float64) + 1.0)).to(dtype)


def attention_mixer(h, positions, w, prefix: str, m: dict, eps: float):
    """Grouped-query attention without rotation: queries scaled by a slowly growing
    function of the position, values of unit root mean square per head, capped
    scores, and a learned sink in the softmax's denominator."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[prefix + ".q"].T).view(n, H, D)
    k = (h @ w[prefix + ".k"].T).view(n, G, D)
    v = (h @ w[prefix + ".v"].T).view(n, G, V)
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(positions, float(qt["coef"]), int(qt["every"]), q.dtype)[:, None, None]
    v = unit_rms(v, eps)
    cap = m.get("softcap")
    sink = w.get(prefix + ".sink")
    visible = causal_mask(n)
    out = torch.zeros(n, H, V, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * float(m["scale"])
        if cap:
            s = float(cap) * torch.tanh(s / float(cap))
        s = s.masked_fill(~visible, -math.inf)
        if sink is not None:
            # one more term in the denominator: exp(sink), with no value behind it
            big = torch.maximum(s.max(dim=-1, keepdim=True).values, sink[head].to(s.dtype))
            e = torch.exp(s - big)
            p = e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink[head].to(s.dtype) - big))
        else:
            p = torch.softmax(s, dim=-1)
        out[:, head] = p @ v[:, g]
    return out.reshape(n, H * V) @ w[prefix + ".o"].T


def rotate_interleaved(x, positions, base: float, dims: int, angle_dtype=None):
    """x [tokens, heads, dim].  Elements 2i and 2i+1 (i < dims/2) turn by positions *
    base**(-2i/dims).  The design forms positions and angles in 32-bit: with
    angle_dtype=torch.float32 the rates are rounded to it and the product is formed in it
    (thousands of radians are then known to about 1e-4); otherwise in float64."""
    out = x.clone()
    if dims == 0:
        return out
    i = torch.arange(dims // 2, dtype=torch.float64)
    rate = (base ** (-2.0 * i / dims)).to(angle_dtype or torch.float64)
    angle = (positions.to(rate.dtype)[:, None] * rate[None, :]).to(torch.float64).to(x.dtype)
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def latent_attention_mixer(h, positions, w, prefix: str, m: dict, eps: float):
    """Attention whose queries, keys and values come through low-rank latents; each
    head has an unrotated part from the latent and a rotated part; the rotated key
    part is one vector shared by all heads; sliding window."""
    n = h.shape[0]
    H, D, R, V, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = weighted_norm(h @ w[prefix + ".dq"].T, w[prefix + ".dq.norm"], eps)
    q = (cq @ w[prefix + ".uq"].T).view(n, H, D + R)
    q_plain, q_rot = q[..., :D], q[..., D:]
    dkv = h @ w[prefix + ".dkv"].T
    c = weighted_norm(dkv[:, :C], w[prefix + ".dkv.norm"], eps)
    k_rot = dkv[:, C:].view(n, 1, R)
    k_plain = (c @ w[prefix + ".uk"].T).view(n, H, D)
    v = (c @ w[prefix + ".uv"].T).view(n, H, V)
    rot = m["rot"]
    q_rot = rotate_interleaved(q_rot, positions, float(rot["base"]), int(rot["dims"]))
    k_rot = rotate_interleaved(k_rot, positions, float(rot["base"]), int(rot["dims"]))
    window = (m.get("mask") or {}).get("size")
    visible = causal_mask(n, None if window is None else int(window))
    out = torch.zeros(n, H, V, dtype=h.dtype)
    for head in range(H):
        s = (q_plain[:, head] @ k_plain[:, head].T + q_rot[:, head] @ k_rot[:, 0].T) * float(m["scale"])
        s = s.masked_fill(~visible, -math.inf)
        out[:, head] = torch.softmax(s, dim=-1) @ v[:, head]
    return out.reshape(n, H * V) @ w[prefix + ".o"].T


def mlstm_mixer(h, w, prefix: str, m: dict, eps: float, state=None):
    """Matrix memory with exponential gates, token by token.  `state` (S, n, m per
    head) carries over from an earlier call; None starts from zeros (m = 0)."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    cap = float(m["gate_cap"])
    q = (h @ w[prefix + ".q"].T).view(T, H, D) * D**-0.5
    k = (h @ w[prefix + ".k"].T).view(T, H, D)
    v = (h @ w[prefix + ".v"].T).view(T, H, V)
    i_pre = h @ w[prefix + ".i"].T + w[prefix + ".i.b"]
    f_pre = h @ w[prefix + ".f"].T + w[prefix + ".f.b"]
    i_log = cap * torch.tanh(i_pre / cap)
    f_log = F.logsigmoid(cap * torch.tanh(f_pre / cap))
    if state is None:
        S = torch.zeros(H, D, V, dtype=h.dtype)
        nv = torch.zeros(H, D, dtype=h.dtype)
        mx = torch.zeros(H, dtype=h.dtype)
    else:
        S, nv, mx = (t.clone() for t in state)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for t in range(T):
        m_new = torch.maximum(f_log[t] + mx, i_log[t])
        keep = torch.exp(f_log[t] + mx - m_new)
        take = torch.exp(i_log[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * (k[t][:, :, None] * v[t][:, None, :])
        nv = keep[:, None] * nv + take[:, None] * k[t]
        mx = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((nv * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        out[t] = num / den[:, None]
    y = unit_rms(out, eps).reshape(T, H * V) * w[prefix + ".norm"]
    y = y * torch.sigmoid(h @ w[prefix + ".g"].T)
    return y @ w[prefix + ".o"].T, (S, nv, mx)


def xielu(z, p, q):
    """z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2."""
    ap = F.softplus(p)
    an = 0.5 + F.softplus(q)
    return torch.where(z > 0, ap * z * z + 0.5 * z, an * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z)


def dense_ffn(h, w, prefix: str):
    a = w[prefix + ".act"]
    return xielu(h @ w[prefix + ".up"].T, a[0], a[1]) @ w[prefix + ".down"].T


def mixer(kind: str, h, positions, w, prefix, m, eps):
    if kind == "attention":
        return attention_mixer(h, positions, w, prefix, m, eps)
    if kind == "latent_attention":
        return latent_attention_mixer(h, positions, w, prefix, m, eps)
    if kind == "mlstm":
        return mlstm_mixer(h, w, prefix, m, eps)[0]
    raise ValueError(f"unknown mixer {kind!r}")


def forward(cfg: dict, w: dict, tokens, return_layers: bool = False):
    """Logits [tokens, vocab] of one sequence from its first token on; with
    return_layers also the residual stream after every layer."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.shape[0])
    eps = float(cfg["norm"]["eps"])
    x = embed(tokens, w, cfg)
    layers = []
    for i, layer in enumerate(cfg["layers"]):
        name = f"l{i}"
        x = x + mixer(layer["type"], weighted_norm(x, w[name + ".norm1"], eps), positions, w, name + ".mix",
                      layer["mixer"], eps)
        if layer.get("mlp") is not None:
            x = x + dense_ffn(weighted_norm(x, w[name + ".norm2"], eps), w, name + ".mlp")
        layers.append(x)
    logits = weighted_norm(x, w["final.norm"], eps) @ w["head"].T
    return (logits, torch.stack(layers)) if return_layers else logits


class PlainMinilorn:
    """A model folder read once; `logits(ids)`, the stream after every layer, and greedy
    generation over it, in float64 unless told otherwise."""

    def __init__(self, model_dir, dtype=torch.float64):
        import json
        from pathlib import Path

        from safetensors.torch import load_file

        self.cfg = json.loads((Path(model_dir) / "config.json").read_text())
        raw = load_file(str(Path(model_dir) / "model.safetensors"))
        self.weights = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in raw.items()}

    def logits(self, token_ids, rows=None) -> torch.Tensor:
        out = forward(self.cfg, self.weights, list(token_ids))
        return out if rows is None else out[torch.tensor(list(rows), dtype=torch.long)]

    def layers(self, token_ids) -> torch.Tensor:
        return forward(self.cfg, self.weights, list(token_ids), return_layers=True)[1]

    def greedy(self, prompt, max_new_tokens: int) -> list[int]:
        seq, out = list(prompt), []
        for _ in range(max_new_tokens):
            tok = int(torch.argmax(self.logits(seq)[-1]))
            out.append(tok)
            seq.append(tok)
        return out
