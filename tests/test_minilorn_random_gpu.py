"""Minilorn configurations drawn at random (width, vocabulary, the layers' mixers in any order and
number, head counts and sizes, values smaller and larger than keys, temperatures, caps, latent ranks,
rotated parts, windows, matrix memories of every register form, layers without a feed-forward, with
and without the pair embedding), each replayed in four cuttings with prompts of up to some hundred
tokens, in float32 and in bfloat16, against the plain implementation.  The seeds are fixed: the test
is the same every time."""

import random

import numpy as np
import pytest

from .plain.minilorn import PlainMinilorn
from .traces import TraceBuilder, changing_portions, last_one_by_one, mixed, run_trace, whole

pytestmark = pytest.mark.gpu


def draw_attention(rng):
    dim = rng.choice([8, 16, 24, 32, 40, 64, 96, 128])
    vdim = rng.choice([dim, dim, 8, 20, 48, 64, 112, 128])
    kv = rng.choice([1, 2, 3, 4])
    group = rng.choice([1, 2, 4, 5])
    return {"type": "attention",
            "mixer": {"heads": kv * group, "kv_heads": kv, "dim": dim, "vdim": vdim,
                      "scale": rng.choice([dim**-0.5, 0.09, 0.3]), "softcap": rng.choice([2.0, 7.5, 30.0, 50.0]),
                      "q_temp": {"coef": rng.choice([0.1, 0.5, 1.5]), "every": rng.choice([1, 7, 32, 100, 1000])}}}


def draw_latent(rng):
    dim = rng.choice([8, 12, 16, 32, 64])
    rot = rng.choice([2, 4, 8, 16, 32])
    kv_rank = rng.choice([8, 24, 30, 64, 120, 160, 288])
    return {"type": "latent_attention",
            "mixer": {"heads": rng.choice([1, 2, 3, 4, 8, 20]), "dim": dim, "rot_dim": rot, "vdim": rng.choice([8, 16, 24, 40]),
                      "q_rank": rng.choice([8, 20, 48, 96]), "kv_rank": kv_rank,
                      "scale": rng.choice([(dim + rot) ** -0.5, 0.11]),
                      "rot": {"base": rng.choice([50.0, 1e4, 5e5]), "dims": rot},
                      "mask": {"size": rng.choice([1, 2, 15, 16, 17, 33, 64, 100, 257, 4000])}}}


def draw_memory(rng):
    return {"type": "mlstm",
            "mixer": {"heads": rng.choice([1, 2, 3, 5]), "dim": rng.choice([4, 16, 30, 64, 72, 128, 130, 256]),
                      "vdim": rng.choice([3, 4, 16, 33, 64, 100]), "gate_cap": rng.choice([2.0, 10.0, 15.0, 40.0])}}


def draw_config(seed: int) -> dict:
    rng = random.Random(seed)
    width = rng.choice([40, 72, 128, 200, 320])
    layers = []
    for _ in range(rng.choice([2, 3, 4, 5])):
        layer = rng.choice([draw_attention, draw_latent, draw_memory])(rng)
        ff = None if rng.random() < 0.2 else rng.choice([48, 100, 256])
        layers.append({**layer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}})
    cfg = {"architecture": "Minilorn", "vocab": rng.choice([61, 97, 700, 3000]), "width": width,
           "norm": {"eps": rng.choice([1e-5, 1e-6, 1e-3])}, "layers": layers}
    if rng.random() < 0.8:
        cfg["embedding"] = {"bigram": {"buckets": rng.choice([1, 13, 509, 20011]), "mul_prev": rng.choice([1, 31, 7919]),
                                       "mul_cur": rng.choice([1, 17, 104729])}}
    return cfg


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [201, 202, 203, 204, 205, 206, 207, 208])
def test_a_random_configuration_in_four_cuttings(seed, dtype, tmp_path):
    from shrike_amd.weights import write_model_folder

    cfg = draw_config(seed)
    rng = random.Random(seed + 1)
    lengths = [rng.choice([1, 2]), rng.randrange(20, 120), rng.randrange(300, 420), rng.randrange(130, 260), rng.randrange(2, 70)]
    seqs = {f"r{i}": [rng.randrange(cfg["vocab"]) for _ in range(n)] for i, n in enumerate(lengths)}
    model_dir = write_model_folder(dict(cfg), tmp_path / "model", seed=seed, dtype=dtype, mode="unit")
    plain = PlainMinilorn(model_dir)
    want = {rid: plain.logits(ids).numpy() for rid, ids in seqs.items()}
    tb = TraceBuilder()
    budget = max(-(-len(ids) // 64) * 64 for ids in seqs.values())
    whole(tb, "w_", seqs)
    last_one_by_one(tb, "d_", seqs, tail=40)
    changing_portions(tb, "p_", seqs, sizes=(64, 2, 48, 3, 200, 16, 1, 96, 2, 31))
    mixed(tb, "m_", seqs, budget + 128, seed=seed)
    outputs = run_trace(model_dir, dtype, tb.steps, budget + 128, tmp_path / "out", cfg["vocab"], poison=True)
    got = tb.collect(outputs)
    over = []
    for (rid, pos), row in got.items():
        name = rid.split("_", 1)[1]
        assert np.isfinite(row).all(), f"{rid} position {pos} read a page that nobody holds"
        err = np.abs(row.astype(np.float64) - want[name][pos]).max() / np.abs(want[name]).max()
        if dtype == "float32":
            assert err <= 1e-4, f"seed {seed} ({cfg}): {rid} position {pos}: rel err {err:.3e}"
            # every float32 kernel sums in one order whatever else is in the step: the same bits in every cutting
            assert np.array_equal(row, got[(f"w_{name}", pos)]), f"seed {seed}: {rid} position {pos} depends on the cutting"
        elif err > 1.5e-2:
            over.append((name, pos, err))
    # bfloat16: a few positions where a memory's readout is nearly nothing or capped scores are steep
    # double what rounding does elsewhere, in every cutting alike; none is far off
    places = {(name, pos) for name, pos, _ in over}
    assert len(places) <= 0.03 * sum(lengths) and all(e <= 0.1 for _, _, e in over), (seed, cfg, over[:5])
