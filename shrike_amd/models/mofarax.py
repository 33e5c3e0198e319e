"""Mofarax: a decoder whose layers run mixer and feed-forward side by side on one
norm, whose attention takes its values from its keys and looks only inside a block
of positions, whose layers each add a gated slice of a second token embedding, and
of which a run of layers is repeated, every pass with a cache of its own.

config.json (every size and every constant that can differ between models):

    architecture   "Mofarax"
    vocab, width
    embedding      {scale}                     x = embed[token] * scale
    norm           {eps}                       all norms; weights stored around zero
    token_side     {dim}                       per-layer token input (absent: none)
    loop           {start, stop, times}        layers start..stop-1 run `times` times
    layers[i]      {type: "attention",
                    mixer: {heads, kv_heads, dim, vdim, scale, mask: {size},
                            rot: {base, dims}},
                    mlp: {kind: "dense", ff} | null}

Tensors: embed, head, final.norm, loop.step [times, width], side.embed [vocab,
layers * token_side.dim], and per layer l<i>.norm1, l<i>.mix.{q,k,o},
l<i>.mlp.{gate,up,down}, l<i>.side.{gate,proj,norm}.

Before every pass of the loop but the first the embedding's output is added to
the stream, and before every pass row t of loop.step (t the pass number); both are
schedule entries' additions, and each pass is a run of schedule positions that own
their caches.
"""

from __future__ import annotations

from dataclasses import dataclass

from ..config.engine_config import canonical_dtype
from ..config.registry import ConfigError, register_architecture
from ..config.specs import (
    AttentionSpec,
    LinearHeadSpec,
    ModelSpec,
    ParallelBlockSpec,
    RMSNormSpec,
    RotaryAdjacentSpec,
    ScheduleEntry,
    SwiGLUSpec,
    TokenEmbeddingSpec,
    TokenSideSpec,
)

ARCHITECTURE = "Mofarax"


def _get(raw: dict, key: str, kind, where: str = "config.json"):
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


@dataclass(frozen=True)
class MofaraxAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    mask_size: int
    rot_base: float
    rot_dims: int

    def __post_init__(self):
        for name in ("heads", "kv_heads", "dim", "mask_size"):
            if getattr(self, name) < 1:
                raise ConfigError(f"config.json: mixer {name} must be positive, got {getattr(self, name)}")
        if self.heads % self.kv_heads:
            raise ConfigError(f"config.json: {self.heads} heads are not a multiple of {self.kv_heads} kv_heads")
        if self.vdim != self.dim:
            raise ConfigError(f"config.json: the values are the keys, so vdim ({self.vdim}) must equal dim ({self.dim})")
        if self.rot_dims < 0 or self.rot_dims % 2 or self.rot_dims > self.dim:
            raise ConfigError(f"config.json: rot.dims must be even and at most dim, got {self.rot_dims}")
        if self.rot_dims and not self.rot_base > 0:
            raise ConfigError(f"config.json: rot.base must be > 0, got {self.rot_base}")

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "MofaraxAttention":
        rot = raw.get("rot") or {"dims": 0, "base": 1.0}
        dim = _get(raw, "dim", int, where)
        return cls(
            heads=_get(raw, "heads", int, where),
            kv_heads=_get(raw, "kv_heads", int, where),
            dim=dim,
            vdim=int(raw.get("vdim", dim)),
            scale=_get(raw, "scale", float, where),
            mask_size=_get(_get(raw, "mask", dict, where), "size", int, where + ".mask"),
            rot_base=_get(rot, "base", float, where + ".rot") if rot.get("dims") else 1.0,
            rot_dims=_get(rot, "dims", int, where + ".rot"),
        )

    def to_dict(self) -> dict:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                "scale": self.scale, "mask": {"size": self.mask_size},
                "rot": {"base": self.rot_base, "dims": self.rot_dims}}


@dataclass(frozen=True)
class MofaraxLayer:
    mixer: MofaraxAttention
    ff: int | None  # width of the dense feed-forward; None: the layer has none

    def to_dict(self) -> dict:
        return {"type": "attention", "mixer": self.mixer.to_dict(),
                "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


@dataclass(frozen=True)
class MofaraxConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: tuple[MofaraxLayer, ...]
    side_dim: int | None = None
    loop: tuple[int, int, int] | None = None  # (start, stop, times)
    torch_dtype: str = "bfloat16"

    def __post_init__(self):
        if self.vocab < 1 or self.width < 1 or not self.layers:
            raise ConfigError("config.json: vocab, width and the number of layers must be positive")
        if not self.norm_eps > 0:
            raise ConfigError(f"config.json: norm.eps must be > 0, got {self.norm_eps}")
        if self.side_dim is not None and self.side_dim < 1:
            raise ConfigError(f"config.json: token_side.dim must be positive, got {self.side_dim}")
        if self.loop is not None:
            start, stop, times = self.loop
            if not (0 <= start < stop <= len(self.layers)) or times < 1:
                raise ConfigError(f"config.json: loop {self.loop} does not fit {len(self.layers)} layers")

    @classmethod
    def from_dict(cls, raw: dict) -> "MofaraxConfig":
        layers = []
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: layers must be a non-empty list")
        for i, entry in enumerate(listed):
            where = f"config.json layers[{i}]"
            kind = _get(entry, "type", str, where)
            if kind != "attention":
                raise ConfigError(f"{where}: unknown mixer type {kind!r} (known: attention)")
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"{where}: unknown feed-forward kind {mlp.get('kind')!r} (known: dense)")
                ff = _get(mlp, "ff", int, where + ".mlp")
                if ff < 1:
                    raise ConfigError(f"{where}: mlp.ff must be positive, got {ff}")
            layers.append(MofaraxLayer(MofaraxAttention.from_dict(_get(entry, "mixer", dict, where), where + ".mixer"), ff))
        loop = raw.get("loop")
        if loop is not None:
            loop = (_get(loop, "start", int, "config.json loop"), _get(loop, "stop", int, "config.json loop"),
                    _get(loop, "times", int, "config.json loop"))
        side = raw.get("token_side")
        dtype = raw.get("torch_dtype") or "bfloat16"
        try:
            dtype = canonical_dtype(dtype)
        except ValueError as e:
            raise ConfigError(f"config.json: {e}") from None
        return cls(
            vocab=_get(raw, "vocab", int),
            width=_get(raw, "width", int),
            embedding_scale=float((raw.get("embedding") or {}).get("scale", 1.0)),
            norm_eps=_get(_get(raw, "norm", dict), "eps", float, "config.json norm"),
            layers=tuple(layers),
            side_dim=None if side is None else _get(side, "dim", int, "config.json token_side"),
            loop=loop,
            torch_dtype=dtype,
        )

    def to_dict(self) -> dict:
        """A config.json that `from_dict` reads back to the same configuration."""
        out = {
            "architecture": ARCHITECTURE,
            "vocab": self.vocab,
            "width": self.width,
            "embedding": {"scale": self.embedding_scale},
            "norm": {"eps": self.norm_eps},
            "layers": [layer.to_dict() for layer in self.layers],
            "torch_dtype": self.torch_dtype,
        }
        if self.side_dim is not None:
            out["token_side"] = {"dim": self.side_dim}
        if self.loop is not None:
            out["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        return out


LOOP_VECTORS = "loop.step"


def layer_schedule(num_layers: int, loop) -> tuple[ScheduleEntry, ...]:
    """The runs of the layers in order.  The first run of every pass of the loop adds
    that pass's row of the loop's vectors to the stream, and from the second pass on
    the embedding's output before it."""
    if loop is None:
        return tuple(ScheduleEntry(i) for i in range(num_layers))
    start, stop, times = loop
    runs = [ScheduleEntry(i) for i in range(start)]
    for t in range(times):
        for i in range(start, stop):
            first = i == start
            runs.append(ScheduleEntry(i, add_embedding=first and t > 0,
                                      add_vector=(LOOP_VECTORS, t) if first else None))
    return tuple(runs + [ScheduleEntry(i) for i in range(stop, num_layers)])


def build_spec(cfg: MofaraxConfig) -> ModelSpec:
    norm = RMSNormSpec(eps=cfg.norm_eps, offset=1.0, names=(("weight", ""),))
    blocks = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        mixer = AttentionSpec(
            num_heads=m.heads,
            num_kv_heads=m.kv_heads,
            head_dim=m.dim,
            qkv_bias=False,
            out_bias=False,
            scale=m.scale,
            position=RotaryAdjacentSpec(theta=m.rot_base, rotary_dim=m.rot_dims) if m.rot_dims else None,
            chunk=m.mask_size,
            values_from_keys=True,
            names=(("q", "q"), ("k", "k"), ("o", "o")),
        )
        ffn = None
        if layer.ff is not None:
            ffn = SwiGLUSpec(intermediate_size=layer.ff, activation="gelu_tanh",
                             names=(("gate", "gate"), ("up", "up"), ("down", "down")))
        side = None
        if cfg.side_dim is not None:
            side = TokenSideSpec(vocab_size=cfg.vocab, dim=cfg.side_dim, index=i, slices=len(cfg.layers),
                                 eps=cfg.norm_eps, activation="gelu_tanh", table_name="side.embed")
        blocks.append(ParallelBlockSpec(name=f"l{i}", norm=norm, mixer=mixer, ffn=ffn, side=side))
    return ModelSpec(
        architecture=ARCHITECTURE,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        blocks=tuple(blocks),
        final_norm=norm,
        tie_word_embeddings=False,
        schedule=layer_schedule(len(cfg.layers), cfg.loop),
        embed_name="embed",
        final_norm_name="final.norm",
        head_name="head",
        stored_dtype=cfg.torch_dtype,
        embedding=TokenEmbeddingSpec(cfg.vocab, scale=cfg.embedding_scale, names=(("weight", ""),)),
        head=LinearHeadSpec(cfg.vocab, names=(("weight", ""),)),
        stream_vectors=((LOOP_VECTORS, cfg.loop[2]),) if cfg.loop is not None else (),
    )


register_architecture(ARCHITECTURE, MofaraxConfig, build_spec)
