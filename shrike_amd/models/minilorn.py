"""Minilorn: a pre-norm decoder whose layers each pick one of three mixers, with a
token embedding that adds a hashed embedding of the (previous token, token) pair.

config.json (every size and every constant that can differ between models):

    architecture   "Minilorn"
    vocab, width
    embedding      {bigram: {buckets, mul_prev, mul_cur}}   absent: the plain lookup
    norm           {eps}                                    all norms, plain weights
    layers[i]      {type, mixer: {...}, mlp: {kind: "dense", ff} | null}

    type "attention"          mixer {heads, kv_heads, dim, vdim, scale, softcap,
                                     q_temp: {coef, every}}
        grouped-query attention without rotation; queries grow with the logarithm of the
        position in steps of `every`; values of unit root mean square; capped scores; a
        learned sink per head in the softmax's denominator
    type "latent_attention"   mixer {heads, dim, rot_dim, vdim, q_rank, kv_rank, scale,
                                     rot: {base, dims}, mask: {size}}
        queries, keys and values through low-rank latents; a rotated key part shared by
        the heads; sliding window
    type "mlstm"              mixer {heads, dim, vdim, gate_cap}
        matrix memory with exponential gates, state per request

Tensors: embed, bigram, head, final.norm, and per layer l<i>.norm1, l<i>.norm2,
l<i>.mix.* (by mixer), l<i>.mlp.{up,down,act}.  A layer is x += mixer(norm1(x)); x +=
mlp(norm2(x)); the feed-forward is down(xielu(up(h))) with the layer's two numbers in
mlp.act; a layer whose mlp is null has neither it nor norm2.
"""

from __future__ import annotations

from dataclasses import dataclass

from ..config.engine_config import canonical_dtype
from ..config.registry import ConfigError, register_architecture
from ..config.specs import (
    AttentionSpec,
    BlockSpec,
    DenseFFNSpec,
    LatentAttentionSpec,
    LinearHeadSpec,
    MLSTMSpec,
    ModelSpec,
    PairHashEmbeddingSpec,
    RMSNormSpec,
    TokenEmbeddingSpec,
)

ARCHITECTURE = "Minilorn"
MIXERS = ("attention", "latent_attention", "mlstm")


def _get(raw, key: str, kind, where: str = "config.json"):
    if not isinstance(raw, dict) or key not in raw or raw[key] is None:
        raise ConfigError(f"{where} lacks the key {key!r}, which {ARCHITECTURE} needs")
    value = raw[key]
    if kind is int:
        if isinstance(value, bool) or not isinstance(value, int):
            raise ConfigError(f"{where}: {key} must be an integer, got {value!r}")
    elif kind is float:
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(f"{where}: {key} must be a number, got {value!r}")
        value = float(value)
    elif kind is dict and not isinstance(value, dict):
        raise ConfigError(f"{where}: {key} must be an object, got {value!r}")
    return value


def _positive(where: str, **values) -> None:
    for name, value in values.items():
        if not value > 0:
            raise ConfigError(f"{where}: {name} must be positive, got {value}")


@dataclass(frozen=True)
class SinkAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float | None
    q_temp: tuple | None  # (coef, every)

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "SinkAttention":
        dim = _get(raw, "dim", int, where)
        qt = raw.get("q_temp")
        if qt is not None:
            qt = (_get(qt, "coef", float, where + ".q_temp"), _get(qt, "every", int, where + ".q_temp"))
            _positive(where + ".q_temp", every=qt[1])
        cap = raw.get("softcap")
        out = cls(heads=_get(raw, "heads", int, where), kv_heads=_get(raw, "kv_heads", int, where), dim=dim,
                  vdim=_get(raw, "vdim", int, where) if raw.get("vdim") is not None else dim,
                  scale=_get(raw, "scale", float, where),
                  softcap=None if cap is None else _get(raw, "softcap", float, where), q_temp=qt)
        _positive(where, heads=out.heads, kv_heads=out.kv_heads, dim=out.dim, vdim=out.vdim)
        if out.softcap is not None:
            _positive(where, softcap=out.softcap)
        if out.heads % out.kv_heads:
            raise ConfigError(f"{where}: {out.heads} heads are not a multiple of {out.kv_heads} kv_heads")
        return out

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.softcap is not None:
            out["softcap"] = self.softcap
        if self.q_temp is not None:
            out["q_temp"] = {"coef": self.q_temp[0], "every": self.q_temp[1]}
        return out


@dataclass(frozen=True)
class LatentAttention:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float
    window: int | None
    rot_dims: int  # how many elements of the rotated part turn (the design says: all of it)

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "LatentAttention":
        rot = raw.get("rot") or {}
        rot_dim = _get(raw, "rot_dim", int, where)
        dims = rot_dim
        if rot_dim and rot.get("dims") is not None:
            dims = _get(rot, "dims", int, where + ".rot")
            if dims < 0 or dims % 2 or dims > rot_dim:
                raise ConfigError(f"{where}: rot.dims ({dims}) must be even and at most rot_dim ({rot_dim})")
        mask = raw.get("mask")
        out = cls(heads=_get(raw, "heads", int, where), dim=_get(raw, "dim", int, where), rot_dim=rot_dim,
                  vdim=_get(raw, "vdim", int, where), q_rank=_get(raw, "q_rank", int, where),
                  kv_rank=_get(raw, "kv_rank", int, where), scale=_get(raw, "scale", float, where),
                  rot_base=_get(rot, "base", float, where + ".rot") if dims else 1.0,
                  window=None if mask is None else _get(mask, "size", int, where + ".mask"), rot_dims=dims)
        _positive(where, heads=out.heads, dim=out.dim, vdim=out.vdim, q_rank=out.q_rank, kv_rank=out.kv_rank,
                  rot_base=out.rot_base)
        if out.rot_dim < 0 or out.rot_dim % 2:
            raise ConfigError(f"{where}: rot_dim must be even and not negative, got {out.rot_dim}")
        if out.window is not None:
            _positive(where + ".mask", size=out.window)
        return out

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
               "q_rank": self.q_rank, "kv_rank": self.kv_rank, "scale": self.scale,
               "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out


@dataclass(frozen=True)
class MatrixMemory:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "MatrixMemory":
        out = cls(heads=_get(raw, "heads", int, where), dim=_get(raw, "dim", int, where),
                  vdim=_get(raw, "vdim", int, where), gate_cap=_get(raw, "gate_cap", float, where))
        _positive(where, heads=out.heads, dim=out.dim, vdim=out.vdim, gate_cap=out.gate_cap)
        return out

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


_MIXER_CONFIGS = {"attention": SinkAttention, "latent_attention": LatentAttention, "mlstm": MatrixMemory}


@dataclass(frozen=True)
class MinilornLayer:
    type: str
    mixer: object
    ff: int | None  # width of the dense feed-forward; None: the layer has none

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


@dataclass(frozen=True)
class MinilornConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: tuple[MinilornLayer, ...]
    bigram: tuple | None = None  # (buckets, mul_prev, mul_cur)
    torch_dtype: str = "bfloat16"

    def __post_init__(self):
        if self.vocab < 1 or self.width < 1 or not self.layers:
            raise ConfigError("config.json: vocab, width and the number of layers must be positive")
        if not self.norm_eps > 0:
            raise ConfigError(f"config.json: norm.eps must be > 0, got {self.norm_eps}")
        if self.bigram is not None and self.bigram[0] < 1:
            raise ConfigError(f"config.json: embedding.bigram.buckets must be positive, got {self.bigram[0]}")

    @classmethod
    def from_dict(cls, raw: dict) -> "MinilornConfig":
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: layers must be a non-empty list")
        layers = []
        for i, entry in enumerate(listed):
            where = f"config.json layers[{i}]"
            kind = _get(entry, "type", str, where)
            if kind not in _MIXER_CONFIGS:
                raise ConfigError(f"{where}: unknown mixer type {kind!r} (known: {', '.join(MIXERS)})")
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"{where}: unknown feed-forward kind {mlp.get('kind')!r} (known: dense)")
                ff = _get(mlp, "ff", int, where + ".mlp")
                _positive(where + ".mlp", ff=ff)
            mixer = _MIXER_CONFIGS[kind].from_dict(_get(entry, "mixer", dict, where), where + ".mixer")
            layers.append(MinilornLayer(kind, mixer, ff))
        bigram = (raw.get("embedding") or {}).get("bigram")
        if bigram is not None:
            where = "config.json embedding.bigram"
            bigram = (_get(bigram, "buckets", int, where), _get(bigram, "mul_prev", int, where),
                      _get(bigram, "mul_cur", int, where))
        dtype = raw.get("torch_dtype") or "bfloat16"
        try:
            dtype = canonical_dtype(dtype)
        except ValueError as e:
            raise ConfigError(f"config.json: {e}") from None
        return cls(vocab=_get(raw, "vocab", int), width=_get(raw, "width", int),
                   norm_eps=_get(_get(raw, "norm", dict), "eps", float, "config.json norm"),
                   layers=tuple(layers), bigram=bigram, torch_dtype=dtype)

    def to_dict(self) -> dict:
        """A config.json that `from_dict` reads back to the same configuration."""
        out = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width,
               "norm": {"eps": self.norm_eps}, "layers": [layer.to_dict() for layer in self.layers],
               "torch_dtype": self.torch_dtype}
        if self.bigram is not None:
            out["embedding"] = {"bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), self.bigram))}
        return out


def mixer_spec(layer: MinilornLayer, eps: float):
    m = layer.mixer
    if layer.type == "attention":
        return AttentionSpec(
            num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, qkv_bias=False, out_bias=False,
            scale=m.scale, value_dim=m.vdim, softcap=m.softcap, sinks=True, query_temperature=m.q_temp,
            value_norm_eps=eps, names=(("q", "q"), ("k", "k"), ("v", "v"), ("o", "o"), ("sink", "sink")))
    if layer.type == "latent_attention":
        return LatentAttentionSpec(
            num_heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim, value_dim=m.vdim, q_rank=m.q_rank,
            kv_rank=m.kv_rank, scale=m.scale, eps=eps, rot_theta=m.rot_base, window=m.window, rotated=m.rot_dims)
    return MLSTMSpec(num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim, gate_cap=m.gate_cap, eps=eps)


def build_spec(cfg: MinilornConfig) -> ModelSpec:
    norm = RMSNormSpec(eps=cfg.norm_eps, names=(("weight", ""),))
    blocks = []
    for i, layer in enumerate(cfg.layers):
        ffn = None
        if layer.ff is not None:
            ffn = DenseFFNSpec(intermediate_size=layer.ff, activation="xielu",
                               names=(("up", "up"), ("down", "down"), ("act", "act")))
        blocks.append(BlockSpec(name=f"l{i}", mixer=mixer_spec(layer, cfg.norm_eps), ffn=ffn, mixer_norm=norm,
                                ffn_norm=norm, mixer_name="mix", ffn_name="mlp", mixer_norm_name="norm1",
                                ffn_norm_name="norm2"))
    if cfg.bigram is not None:
        embedding = PairHashEmbeddingSpec(cfg.vocab, buckets=cfg.bigram[0], mul_prev=cfg.bigram[1],
                                          mul_cur=cfg.bigram[2], pair_name="bigram", names=(("weight", ""),))
    else:
        embedding = TokenEmbeddingSpec(cfg.vocab, names=(("weight", ""),))
    return ModelSpec(
        architecture=ARCHITECTURE,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        blocks=tuple(blocks),
        final_norm=norm,
        tie_word_embeddings=False,
        embed_name="embed",
        final_norm_name="final.norm",
        head_name="head",
        stored_dtype=cfg.torch_dtype,
        embedding=embedding,
        head=LinearHeadSpec(cfg.vocab, names=(("weight", ""),)),
    )


register_architecture(ARCHITECTURE, MinilornConfig, build_spec)
