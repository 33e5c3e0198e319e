"""Mofarax without a GPU: its configuration reader, the parts and schedule it is
laid out as, what the cache manager gives back as blocks of positions pass, and the
pins of the plain implementation that the GPU tests compare with."""

import copy
import math

import pytest
import torch
import torch.nn.functional as F

from shrike_amd.cache import CacheManager
from shrike_amd.config import registry  # (names through the modules: another test reloads them)
from shrike_amd.models import DecoderModel
from shrike_amd.models import mofarax as mof

from .plain import mofarax as plain
from .tiny_mofarax import CONFIGS, MOF_P, MOF_R


# ------------------------------------------------------------------ configuration

@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_config_reads_back(name):
    raw = CONFIGS[name]
    assert registry.architecture_name(raw) == "Mofarax"
    arch = registry.get_architecture("Mofarax")
    cfg = arch.config_cls.from_dict(raw)
    assert arch.config_cls.from_dict(cfg.to_dict()) == cfg
    assert len(cfg.layers) == len(raw["layers"])
    assert cfg.layers[0].mixer.mask_size == raw["layers"][0]["mixer"]["mask"]["size"]
    assert cfg.embedding_scale == raw["embedding"]["scale"]


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="recurrent"), "unknown mixer type"),
    (lambda c: c["layers"][0]["mixer"].update(vdim=48), "vdim"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "multiple"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "feed-forward kind"),
    (lambda c: c["loop"].update(stop=9), "loop"),
    (lambda c: c["loop"].update(times=0), "loop"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0]["mixer"].pop("mask"), "mask"),
    (lambda c: c["norm"].update(eps=0.0), "eps"),
])
def test_config_refuses_what_it_cannot_run(change, message):
    raw = copy.deepcopy(MOF_P)
    change(raw)
    with pytest.raises(registry.ConfigError, match=message):
        mof.MofaraxConfig.from_dict(raw)


def test_tensors_the_model_declares():
    model = DecoderModel(mof.build_spec(mof.MofaraxConfig.from_dict(MOF_P)))
    shapes = {p.name: tuple(p.shape) for p in model.params()}
    assert shapes["embed"] == (199, 64) and shapes["head"] == (199, 64) and shapes["final.norm"] == (64,)
    assert shapes["loop.step"] == (3, 64)
    assert shapes["side.embed"] == (199, 3 * 8)
    assert shapes["l0.mix.q"] == (128, 64) and shapes["l0.mix.k"] == (64, 64) and shapes["l0.mix.o"] == (64, 128)
    assert shapes["l2.mix.q"] == (128, 64) and shapes["l2.mix.k"] == (64, 64)
    assert shapes["l0.mlp.gate"] == (96, 64) and shapes["l0.mlp.down"] == (64, 96)
    assert not any(n.startswith("l1.mlp") for n in shapes)  # a layer without a feed-forward
    assert not any(".v" in n for n in shapes)  # no value projection anywhere
    assert shapes["l1.side.gate"] == (8, 64) and shapes["l1.side.proj"] == (64, 8) and shapes["l1.side.norm"] == (64,)
    plain_model = DecoderModel(mof.build_spec(mof.MofaraxConfig.from_dict(MOF_R)))
    names = {p.name for p in plain_model.params()}
    assert "loop.step" not in names and "side.embed" not in names and not any(".side." in n for n in names)


def test_schedule_of_a_loop():
    runs = mof.layer_schedule(5, (1, 3, 3))
    assert [e.block for e in runs] == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    assert [e.add_embedding for e in runs] == [False, False, False, True, False, True, False, False, False]
    assert [e.add_vector for e in runs] == [None, ("loop.step", 0), None, ("loop.step", 1), None, ("loop.step", 2),
                                            None, None, None]
    assert all(e.cache_of is None for e in runs)  # every pass has caches of its own
    once = mof.layer_schedule(3, (0, 3, 1))
    assert [e.add_vector for e in once] == [("loop.step", 0), None, None] and not any(e.add_embedding for e in once)
    assert [(e.block, e.add_vector) for e in mof.layer_schedule(2, None)] == [(0, None), (1, None)]
    assert plain.layer_runs({"layers": [0] * 5, "loop": {"start": 1, "stop": 3, "times": 3}}) == [
        (0, None), (1, 0), (2, None), (1, 1), (2, None), (1, 2), (2, None), (3, None), (4, None)]


# ------------------------------------------------------------------ cache manager

def test_pages_behind_the_current_block_are_given_back():
    model = DecoderModel(mof.build_spec(mof.MofaraxConfig.from_dict(MOF_P)))
    specs = model.cache_specs()
    assert len(specs) == 1 + 2 * 3 and all(s is not None for s in specs)
    cache = CacheManager(specs, 8, 40, enable_prefix_caching=False)
    assert len(cache.groups) == 2  # blocks of 24 with heads of 32; blocks of 40 with heads of 64
    assert sorted(g.spec.chunk for g in cache.groups) == [24, 40]
    assert sorted(len(g.layers) for g in cache.groups) == [3, 4]
    assert not cache.enable_prefix_caching
    seq = cache.new_sequence()
    held = {}
    for p in range(130):
        cache.append(seq, p, 1)
        cache.trim(seq, p + 1)
        for g, table in zip(cache.groups, seq.tables):
            first = (p + 1) // g.spec.chunk * g.spec.chunk  # the next query's first key
            assert all((page >= 0) == ((i + 1) * 8 > first) for i, page in enumerate(table)), (p, table)
            held[g.spec.chunk] = max(held.get(g.spec.chunk, 0), sum(page >= 0 for page in table))
    assert held == {24: 3, 40: 5}  # a block of either size is whole pages here
    cache.free(seq)
    cache.check([])
    assert cache.num_free == 40


def test_a_portion_that_crosses_a_block_edge_keeps_what_its_first_query_reads():
    from shrike_amd.parts import kv_cache_spec

    cache = CacheManager([kv_cache_spec(1, 32, None, 10)], 4, 16, enable_prefix_caching=False)
    seq = cache.new_sequence()
    cache.append(seq, 0, 7)
    assert cache.trim(seq, 7) == 0
    cache.append(seq, 7, 9)  # positions 7..15: the query at 7 still reads keys 0..7
    assert all(p >= 0 for p in seq.tables[0])
    assert cache.trim(seq, 16) == 2  # the next query, at 16, reads from 10 on: pages 0 and 1 are done
    assert [p >= 0 for p in seq.tables[0]] == [False, False, True, True]


# ------------------------------------------------------------------ pins of the plain implementation

def test_plain_gelu_and_norms():
    z = torch.linspace(-6, 6, 101, dtype=torch.float64)
    assert torch.allclose(plain.gelu_tanh(z), F.gelu(z, approximate="tanh"), atol=1e-12)
    x = torch.randn(5, 48, dtype=torch.float64)
    w = torch.randn(48, dtype=torch.float64)
    assert torch.allclose(plain.plain_weight_norm(x, w, 1e-5), F.rms_norm(x, (48,), w, 1e-5), atol=1e-12)
    assert torch.allclose(plain.zero_centred_norm(x, w, 1e-5), F.rms_norm(x, (48,), 1 + w, 1e-5), atol=1e-12)
    # eps sits inside the root: a row of zeros stays zero, a tiny row is damped
    assert float(plain.unit_rms(torch.full((1, 4), 1e-4, dtype=torch.float64), 1e-2).abs().max()) < 2e-3


def test_plain_rotation_is_a_complex_turn_of_neighbours():
    torch.manual_seed(0)
    x = torch.randn(6, 2, 10, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 50, 51, 1000])
    out = plain.rotate_interleaved(x, pos, 100.0, 6)
    assert torch.equal(out[..., 6:], x[..., 6:])  # elements behind the rotated part
    assert torch.equal(out[0], x[0])  # position 0 turns nothing
    rates = [1.0, 100.0 ** (-2 / 6), 100.0 ** (-4 / 6)]
    for i, rate in enumerate(rates):
        z = torch.complex(x[..., 2 * i], x[..., 2 * i + 1]) * torch.polar(torch.ones(6, dtype=torch.float64),
                                                                        pos.double() * rate)[:, None]
        assert torch.allclose(out[..., 2 * i], z.real, atol=1e-12) and torch.allclose(out[..., 2 * i + 1], z.imag, atol=1e-12)
    # scores depend on the distance between positions only
    q, k = torch.randn(1, 1, 8, dtype=torch.float64), torch.randn(1, 1, 8, dtype=torch.float64)
    def score(a, b):
        return float((plain.rotate_interleaved(q, torch.tensor([a]), 30.0, 8) *
                      plain.rotate_interleaved(k, torch.tensor([b]), 30.0, 8)).sum())
    assert math.isclose(score(9, 4), score(205, 200), rel_tol=1e-9)
    assert not math.isclose(score(9, 4), score(9, 5), rel_tol=1e-3)


def test_plain_block_mask_written_out():
    m = plain.chunk_mask(7, 3)
    want = [[1, 0, 0, 0, 0, 0, 0],
            [1, 1, 0, 0, 0, 0, 0],
            [1, 1, 1, 0, 0, 0, 0],
            [0, 0, 0, 1, 0, 0, 0],
            [0, 0, 0, 1, 1, 0, 0],
            [0, 0, 0, 1, 1, 1, 0],
            [0, 0, 0, 0, 0, 0, 1]]
    assert m.int().tolist() == want
    assert plain.chunk_mask(5, 100).int().tolist() == torch.tril(torch.ones(5, 5)).int().tolist()


def test_plain_attention_for_one_token_and_against_the_library():
    """One token: every head returns its group's key as projected (the value), whatever
    the rotation.  Several tokens in one block, heads rotated: the library's attention
    on rotated queries and keys with the unrotated keys as values."""
    torch.manual_seed(1)
    m = {"heads": 4, "kv_heads": 2, "dim": 6, "scale": 0.3, "mask": {"size": 50}, "rot": {"base": 40.0, "dims": 4}}
    w = {"a.q": torch.randn(24, 10, dtype=torch.float64), "a.k": torch.randn(12, 10, dtype=torch.float64),
         "a.o": torch.randn(10, 24, dtype=torch.float64)}
    h = torch.randn(1, 10, dtype=torch.float64)
    k = (h @ w["a.k"].T).view(1, 2, 6)
    want = k.repeat_interleave(2, dim=1).reshape(1, 24) @ w["a.o"].T
    assert torch.allclose(plain.attention_mixer(h, torch.tensor([7]), w, "a", m), want, atol=1e-12)
    h = torch.randn(9, 10, dtype=torch.float64)
    pos = torch.arange(9)
    q = plain.rotate_interleaved((h @ w["a.q"].T).view(9, 4, 6), pos, 40.0, 4)
    k_in = (h @ w["a.k"].T).view(9, 2, 6)
    kr = plain.rotate_interleaved(k_in, pos, 40.0, 4)
    o = F.scaled_dot_product_attention(q.transpose(0, 1), kr.repeat_interleave(2, 1).transpose(0, 1),
                                       k_in.repeat_interleave(2, 1).transpose(0, 1), is_causal=True, scale=0.3)
    want = o.transpose(0, 1).reshape(9, 24) @ w["a.o"].T
    assert torch.allclose(plain.attention_mixer(h, pos, w, "a", m), want, atol=1e-10)
    # block_local_attention, the kernels' oracle, says the same as the masked form
    got = plain.block_local_attention(q, kr, k_in, 0.3, 4)
    mask = plain.chunk_mask(9, 4)
    for head in range(4):
        s = (q[:, head] @ kr[:, head // 2].T * 0.3).masked_fill(~mask, float("-inf"))
        assert torch.allclose(got[:, head], torch.softmax(s, -1) @ k_in[:, head // 2], atol=1e-12)


def test_plain_model_is_causal_and_blocks_do_not_see_each_other():
    """Changing a token changes no earlier logits, and none in later blocks when every
    layer's block ends before them, except through the token itself."""
    import json
    import tempfile

    from .tiny_mofarax import make_model_dir

    path = make_model_dir("Q", tempfile.mkdtemp(), dtype="float32")
    model = plain.PlainMofarax(path)
    ids = list(range(3, 31))
    base = model.logits(ids)
    other = list(ids)
    other[9] = 200
    changed = model.logits(other)
    assert torch.equal(base[:9], changed[:9])
    assert not torch.allclose(base[9], changed[9])
    assert not torch.allclose(base[13], changed[13])  # same block of 7 (positions 7..13)
    assert torch.equal(base[14:], changed[14:])  # later blocks never see position 9
    assert json.loads((path / "config.json").read_text())["layers"][0]["mixer"]["mask"]["size"] == 7
