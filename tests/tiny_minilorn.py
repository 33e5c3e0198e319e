"""Tiny Minilorn configurations for tests.  They differ from each other in every size
and option: the three mixers in several orders and more than once, grouped, ungrouped
and single key/value heads, values smaller than, equal to and larger than keys, a
query temperature that steps every position, every 5 and every 64 positions, score caps
from 3 to 30, windows of 1, 9, 40 and 1,000 positions (smaller than a page, across page
edges, larger than any test sequence), rotated parts that turn whole or in part, latents
wider than 256, matrix memories whose heads take each of the scan kernel's register
forms and whose value sizes are no multiples of 16, layers without a feed-forward, a
model without the pair embedding, widths that are multiples of nothing."""

from __future__ import annotations

import tempfile
from pathlib import Path


def _attn(heads, kv_heads, dim, vdim, scale=None, softcap=10.0, coef=0.4, every=5):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                      "scale": dim**-0.5 if scale is None else scale, "softcap": softcap,
                      "q_temp": {"coef": coef, "every": every}}}


def _latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, size, base=10000.0, scale=None, dims=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank,
                      "kv_rank": kv_rank, "scale": (dim + rot_dim) ** -0.5 if scale is None else scale,
                      "rot": {"base": base, "dims": rot_dim if dims is None else dims}, "mask": {"size": size}}}


def _mlstm(heads, dim, vdim, cap=8.0):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


def _with(layer, ff):
    return {**layer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _bigram(buckets, mul_prev, mul_cur):
    return {"bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}


MIN_A = {
    "architecture": "Minilorn", "vocab": 211, "width": 64, "embedding": _bigram(97, 7, 13), "norm": {"eps": 1e-6},
    "layers": [
        _with(_attn(4, 2, 32, 16, softcap=8.0, coef=0.3, every=5), 96),
        _with(_latent(2, 16, 8, 24, 24, 40, 9, base=500.0), 80),
        _with(_mlstm(2, 16, 20, cap=6.0), None),
        _with(_attn(2, 2, 16, 48, softcap=3.0, coef=1.0, every=1), 64),
    ],
}

MIN_B = {
    "architecture": "Minilorn", "vocab": 97, "width": 100, "embedding": _bigram(1, 3, 5), "norm": {"eps": 1e-4},
    "layers": [
        _with(_mlstm(1, 40, 16, cap=20.0), 52),
        _with(_latent(3, 10, 6, 10, 36, 72, 40, base=90.0, dims=4), None),
        _with(_attn(6, 1, 24, 24, softcap=30.0, coef=0.1, every=64), 30),
        _with(_mlstm(3, 12, 50, cap=4.0), 44),
        _with(_latent(1, 24, 2, 8, 20, 30, 1, base=3.0), 60),
    ],
}

MIN_C = {
    "architecture": "Minilorn", "vocab": 300, "width": 128, "norm": {"eps": 2e-5},
    "layers": [
        _with(_latent(4, 32, 16, 32, 48, 272, 1000, base=2.0e5), 256),
        _with(_attn(4, 4, 64, 128, softcap=15.0, coef=0.25, every=16), 200),
        _with(_mlstm(2, 128, 48, cap=10.0), 128),
    ],
}

MIN_D = {
    "architecture": "Minilorn", "vocab": 150, "width": 48, "embedding": _bigram(1500, 1000003, 999983),
    "norm": {"eps": 1e-5},
    "layers": [
        _with(_attn(3, 3, 8, 5, softcap=5.0, coef=2.0, every=3), 40),
        _with(_mlstm(2, 200, 7, cap=12.0), None),
        _with(_latent(5, 6, 4, 7, 9, 11, 17, base=40.0), 33),
    ],
}

# head sizes that the matrix-instruction attention kernels take (values as large as keys, 64
# and 128, grouped and ungrouped), for prompts long enough that keys are shared among workgroups
MIN_E = {
    "architecture": "Minilorn", "vocab": 180, "width": 96, "embedding": _bigram(50, 11, 29), "norm": {"eps": 1e-5},
    "layers": [
        _with(_attn(8, 2, 64, 64, softcap=6.0, coef=0.3, every=50), 128),
        _with(_mlstm(1, 24, 32, cap=9.0), None),
        _with(_attn(4, 4, 128, 128, softcap=20.0, coef=0.2, every=300), 72),
        _with(_latent(2, 12, 4, 16, 20, 28, 100, base=1000.0), 64),
    ],
}

CONFIGS = {"A": MIN_A, "B": MIN_B, "C": MIN_C, "D": MIN_D, "E": MIN_E}
SEEDS = {"A": 3, "B": 11, "C": 23, "D": 41, "E": 53}
PAGE_SIZES = {"A": 16, "B": 4, "C": 32, "D": 8, "E": 16}


def make_model_dir(name: str, root=None, dtype: str = "float32", mode: str = "unit") -> Path:
    """Writes the tiny model `name` with seeded random weights (stored in `dtype`) into
    `root` (or a fresh temporary folder) and returns the folder."""
    from shrike_amd.weights import write_model_folder

    if root is None:
        root = tempfile.mkdtemp(prefix="shrike_tiny_")
    path = Path(root) / f"minilorn_{name}_{dtype}_{mode}"
    if not (path / "model.safetensors").is_file():
        write_model_folder(dict(CONFIGS[name]), path, seed=SEEDS[name], dtype=dtype, mode=mode)
    return path
