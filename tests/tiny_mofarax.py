"""Tiny Mofarax configurations for tests.  They differ from each other in every
size and option: grouped and ungrouped heads, head sizes that the
matrix-instruction attention kernels take (32, 64, 96) and one they do not (24),
heads rotated whole, in part and not at all, blocks of positions smaller than a
page, beside a page's edge, just over 32 and larger than any test sequence,
layers without a feed-forward, layers that differ within one model (two page
groups), loops that start after the first layer, run once, twice or three
times, or are absent, a side input of odd width or none; one model whose sizes are
multiples of nothing, with blocks of a single position in one layer."""

from __future__ import annotations

import tempfile
from pathlib import Path


def _mixer(heads, kv_heads, dim, size, rot_dims, base=10000.0, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
            "scale": dim**-0.5 if scale is None else scale, "mask": {"size": size},
            "rot": {"base": base, "dims": rot_dims}}


def _layer(mixer, ff):
    return {"type": "attention", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


MOF_P = {
    "architecture": "Mofarax", "vocab": 199, "width": 64,
    "embedding": {"scale": 3.5}, "norm": {"eps": 1e-6}, "token_side": {"dim": 8},
    "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        _layer(_mixer(4, 2, 32, 24, 32, scale=0.2), 96),
        _layer(_mixer(4, 2, 32, 24, 16, base=500.0, scale=0.2), None),
        _layer(_mixer(2, 1, 64, 40, 64), 72),
    ],
}

MOF_Q = {
    "architecture": "Mofarax", "vocab": 311, "width": 96,
    "embedding": {"scale": 1.0}, "norm": {"eps": 1e-5}, "token_side": {"dim": 5},
    "loop": {"start": 0, "stop": 1, "times": 2},
    "layers": [_layer(_mixer(6, 6, 24, 7, 12, base=777.0), 200) for _ in range(4)],
}

MOF_R = {
    "architecture": "Mofarax", "vocab": 257, "width": 128,
    "embedding": {"scale": 11.0}, "norm": {"eps": 3e-6},
    "layers": [_layer(_mixer(8, 1, 64, 1000, 0, scale=0.11), 256), _layer(_mixer(8, 1, 64, 1000, 64, scale=0.11), 256)],
}

MOF_S = {
    "architecture": "Mofarax", "vocab": 401, "width": 160,
    "embedding": {"scale": 0.75}, "norm": {"eps": 2e-5}, "token_side": {"dim": 32},
    "loop": {"start": 0, "stop": 3, "times": 1},
    "layers": [_layer(_mixer(2, 1, 96, 33, 96, base=2.0e5), 296), _layer(_mixer(2, 1, 96, 33, 48, base=2.0e5), 296),
               _layer(_mixer(2, 1, 96, 33, 96, base=2.0e5), None)],
}

# sizes that are multiples of nothing: rows that no vector load takes, a head of 10
MOF_T = {
    "architecture": "Mofarax", "vocab": 97, "width": 100,
    "embedding": {"scale": 2.25}, "norm": {"eps": 1e-4}, "token_side": {"dim": 3},
    "loop": {"start": 1, "stop": 2, "times": 2},
    "layers": [_layer(_mixer(2, 2, 10, 5, 6, base=90.0, scale=0.4), 52), _layer(_mixer(6, 2, 10, 1, 10, base=90.0), 30),
               _layer(_mixer(2, 1, 10, 11, 2, base=4.0), None)],
}

CONFIGS = {"P": MOF_P, "Q": MOF_Q, "R": MOF_R, "S": MOF_S, "T": MOF_T}
SEEDS = {"P": 5, "Q": 17, "R": 29, "S": 43, "T": 59}
PAGE_SIZES = {"P": 16, "Q": 4, "R": 32, "S": 16, "T": 8}


def make_model_dir(name: str, root=None, dtype: str = "float32", mode: str = "unit") -> Path:
    """Writes the tiny model `name` with seeded random weights (stored in `dtype`)
    into `root` (or a fresh temporary folder) and returns the folder."""
    from shrike_amd.weights import write_model_folder

    if root is None:
        root = tempfile.mkdtemp(prefix="shrike_tiny_")
    path = Path(root) / f"mofarax_{name}_{dtype}_{mode}"
    if not (path / "model.safetensors").is_file():
        write_model_folder(dict(CONFIGS[name]), path, seed=SEEDS[name], dtype=dtype, mode=mode)
    return path
