"""Mofarax configurations drawn at random (sizes, head counts and sizes, rotated part,
blocks of positions, layers with and without a feed-forward, loops, side widths),
each replayed in four cuttings with prompts of several hundred tokens, in float32,
against the plain implementation.  The seeds are fixed: the test is the same every time."""

import random

import numpy as np
import pytest

from .plain.mofarax import PlainMofarax
from .traces import TraceBuilder, changing_portions, last_one_by_one, mixed, run_trace, whole

pytestmark = pytest.mark.gpu


def draw_mixer(rng):
    dim = rng.choice([16, 24, 32, 40, 64, 80, 128, 160, 256])
    kv = rng.choice([1, 2, 3, 4])
    group = rng.choice([1, 2, 4, 8, 20])
    if dim * kv * group > 2048:
        group = 1
    return {"heads": kv * group, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": rng.choice([dim**-0.5, 0.07, 0.2]),
            "mask": {"size": rng.choice([1, 5, 16, 31, 32, 33, 64, 100, 256, 500, 5000])},
            "rot": {"base": rng.choice([100.0, 1e4, 1e6]), "dims": rng.choice([0, dim, dim, dim // 4 * 2, 2])}}


def draw_config(seed: int) -> dict:
    rng = random.Random(seed)
    width = rng.choice([48, 72, 128, 320, 1000])
    n = rng.choice([2, 3, 4])
    shared = draw_mixer(rng) if rng.random() < 0.5 else None
    layers = []
    for _ in range(n):
        ff = None if rng.random() < 0.2 else rng.choice([64, 100, 384])
        layers.append({"type": "attention", "mixer": shared or draw_mixer(rng),
                       "mlp": None if ff is None else {"kind": "dense", "ff": ff}})
    cfg = {"architecture": "Mofarax", "vocab": rng.choice([97, 2000]), "width": width,
           "embedding": {"scale": rng.choice([1.0, 5.5])}, "norm": {"eps": rng.choice([1e-5, 1e-6])}, "layers": layers}
    if rng.random() < 0.8:
        cfg["token_side"] = {"dim": rng.choice([16, 32, 64])}
    if rng.random() < 0.85:
        start = rng.randrange(0, n)
        cfg["loop"] = {"start": start, "stop": rng.randrange(start + 1, n + 1), "times": rng.choice([1, 2, 3])}
    return cfg


@pytest.mark.parametrize("seed", [101, 102, 103, 104])
def test_a_random_configuration_in_four_cuttings(seed, tmp_path):
    from shrike_amd.weights import write_model_folder

    cfg = draw_config(seed)
    rng = random.Random(seed + 1)
    lengths = [rng.choice([1, 2]), rng.randrange(20, 120), rng.randrange(300, 520), rng.randrange(130, 260)]
    seqs = {f"r{i}": [rng.randrange(cfg["vocab"]) for _ in range(n)] for i, n in enumerate(lengths)}
    model_dir = write_model_folder(dict(cfg), tmp_path / "model", seed=seed, dtype="float32", mode="unit")
    plain = PlainMofarax(model_dir)
    want = {rid: plain.logits(ids).numpy() for rid, ids in seqs.items()}
    tb = TraceBuilder()
    budget = max(-(-len(ids) // 64) * 64 for ids in seqs.values())
    whole(tb, "w_", seqs)
    last_one_by_one(tb, "d_", seqs, tail=40)
    changing_portions(tb, "p_", seqs, sizes=(64, 2, 48, 3, 200, 16, 1, 96, 2, 31))
    mixed(tb, "m_", seqs, budget + 128, seed=seed)
    outputs = run_trace(model_dir, "float32", tb.steps, budget + 128, tmp_path / "out", cfg["vocab"], poison=True)
    got = tb.collect(outputs)
    for (rid, pos), row in got.items():
        name = rid.split("_", 1)[1]
        assert np.isfinite(row).all(), f"{rid} position {pos} read a page that nobody holds"
        err = np.abs(row.astype(np.float64) - want[name][pos]).max() / np.abs(want[name]).max()
        assert err <= 1e-4, f"seed {seed} ({cfg}): {rid} position {pos}: rel err {err:.3e}"
