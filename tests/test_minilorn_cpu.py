"""What pins the plain form of Minilorn (tests/plain/minilorn.py), and the configuration
reader, without a GPU: each mechanism against a second, independent way of writing it."""

import copy
import math

import pytest
import torch

import shrike_amd.models  # noqa: F401  (registers the architectures)
from shrike_amd.config import registry  # (names through the module: another test reloads it)
from shrike_amd.models import DecoderModel
from shrike_amd.parts import PagedSpec, StateSpec

from .plain import minilorn as plain
from .tiny_minilorn import CONFIGS

D = torch.float64


def test_config_reads_back_and_picks_the_parts():
    arch = registry.get_architecture("Minilorn")
    for name, raw in CONFIGS.items():
        cfg = arch.config_cls.from_dict(raw)
        again = arch.config_cls.from_dict(cfg.to_dict())
        assert again == cfg, name
        spec = arch.build_spec(cfg)
        kinds = [b.mixer.kind for b in spec.blocks]
        want = {"attention": "paged_attention", "latent_attention": "latent_attention", "mlstm": "mlstm"}
        assert kinds == [want[layer["type"]] for layer in raw["layers"]]
        assert [b.ffn is None for b in spec.blocks] == [layer["mlp"] is None for layer in raw["layers"]]
        model = DecoderModel(spec)
        specs = model.cache_specs()
        has_pairs = "embedding" in raw
        assert len(specs) == len(raw["layers"]) + has_pairs
        for layer, s in zip(raw["layers"], specs):
            assert isinstance(s, StateSpec if layer["type"] == "mlstm" else PagedSpec)
            if layer["type"] == "latent_attention":
                assert s.window == layer["mixer"]["mask"]["size"]
                assert s.tensors[0].dims[-1] == layer["mixer"]["kv_rank"] + layer["mixer"]["rot_dim"]
        if has_pairs:
            assert specs[-1] == StateSpec((1,), "int32")
        names = {p.name for p in model.params()}
        assert ("bigram" in names) == has_pairs
        for i, layer in enumerate(raw["layers"]):
            assert (f"l{i}.norm2" in names) == (layer["mlp"] is not None)


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].__setitem__("type", "conv"), "unknown mixer type"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 3), "not a multiple"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("rot_dim", 7), "even"),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 10), "at most rot_dim"),
    (lambda c: c["layers"][2]["mixer"].__delitem__("gate_cap"), "gate_cap"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "routed"), "feed-forward kind"),
    (lambda c: c["norm"].__setitem__("eps", 0), "eps"),
    (lambda c: c["embedding"]["bigram"].__setitem__("buckets", 0), "buckets"),
    (lambda c: c["layers"][0]["mixer"]["q_temp"].__setitem__("every", 0), "every"),
])
def test_config_errors_name_the_key(change, message):
    raw = copy.deepcopy(CONFIGS["A"])
    change(raw)
    with pytest.raises(registry.ConfigError, match=message):
        registry.get_architecture("Minilorn").config_cls.from_dict(raw)


def test_pair_rows_by_hand():
    rows = plain.bigram_rows(torch.tensor([4, 9, 9, 0]), buckets=7, mul_prev=3, mul_cur=5)
    assert rows.tolist() == [7, (4 * 3 + 9 * 5) % 7, (9 * 3 + 9 * 5) % 7, (9 * 3) % 7]


def test_query_temperature_steps():
    t = plain.query_temperature(torch.arange(0, 12), 0.5, 4, D)
    assert t[:3].tolist() == [1.0, 1.0, 1.0]  # floor((p + 1) / 4) = 0 up to position 2
    assert float(t[3]) == pytest.approx(1 + 0.5 * math.log(2)) and float(t[6]) == float(t[3])
    assert float(t[11]) == pytest.approx(1 + 0.5 * math.log(4))


def test_xielu_is_continuous_with_slope_one_half_at_zero_and_matches_its_formula():
    p, q = torch.tensor(0.2, dtype=D), torch.tensor(-1.0, dtype=D)
    z = torch.tensor([-2.0, -1e-6, 0.0, 1e-6, 3.0], dtype=D)
    y = plain.xielu(z, p, q)
    ap, an = math.log1p(math.exp(0.2)), 0.5 + math.log1p(math.exp(-1.0))
    assert float(y[4]) == pytest.approx(ap * 9 + 1.5)
    assert float(y[0]) == pytest.approx(an * (math.exp(-2.0) - 1 + 2.0) - 1.0)
    assert float(y[2]) == 0.0
    assert float((y[3] - y[1]) / 2e-6) == pytest.approx(0.5, abs=1e-5)


def _attention_weights(H, G, dim, vdim, width, sink):
    g = torch.Generator().manual_seed(1)
    w = {"a.q": torch.randn(H * dim, width, generator=g, dtype=D), "a.k": torch.randn(G * dim, width, generator=g, dtype=D),
         "a.v": torch.randn(G * vdim, width, generator=g, dtype=D), "a.o": torch.eye(H * vdim, dtype=D)}
    if sink is not None:
        w["a.sink"] = sink
    return w


def test_a_sink_is_a_key_with_a_zero_value_and_a_fixed_score():
    """Softmax with a sink = ordinary softmax over the keys plus one more entry of score
    `sink`, whose value is zero."""
    torch.manual_seed(0)
    n, width, H, G, dim, vdim = 6, 10, 2, 1, 4, 3
    sink = torch.tensor([0.7, -2.0], dtype=D)
    w = _attention_weights(H, G, dim, vdim, width, sink)
    h = torch.randn(n, width, dtype=D)
    m = {"heads": H, "kv_heads": G, "dim": dim, "vdim": vdim, "scale": 0.5, "softcap": 4.0, "q_temp": {"coef": 0.5, "every": 2}}
    got = plain.attention_mixer(h, torch.arange(n), w, "a", m, 1e-6).view(n, H, vdim)
    q = (h @ w["a.q"].T).view(n, H, dim) * plain.query_temperature(torch.arange(n), 0.5, 2, D)[:, None, None]
    k = (h @ w["a.k"].T).view(n, G, dim)
    v = (h @ w["a.v"].T).view(n, G, vdim)
    v = v / torch.sqrt((v * v).mean(-1, keepdim=True) + 1e-6)
    for i in range(n):
        for head in range(H):
            s = 4.0 * torch.tanh((k[: i + 1, 0] @ q[i, head]) * 0.5 / 4.0)
            p = torch.softmax(torch.cat([s, sink[head : head + 1]]), dim=0)
            assert torch.allclose(got[i, head], p[:-1] @ v[: i + 1, 0], atol=1e-12)
    # capped scores never exceed the cap
    assert float(s.abs().max()) <= 4.0


def _latent_weights(H, dim, rot, vdim, q_rank, kv_rank, width):
    g = torch.Generator().manual_seed(2)
    r = lambda *s: torch.randn(*s, generator=g, dtype=D)  # noqa: E731
    return {"l.dq": r(q_rank, width), "l.dq.norm": 1 + 0.1 * r(q_rank), "l.uq": r(H * (dim + rot), q_rank),
            "l.dkv": r(kv_rank + rot, width), "l.dkv.norm": 1 + 0.1 * r(kv_rank), "l.uk": r(H * dim, kv_rank),
            "l.uv": r(H * vdim, kv_rank), "l.o": torch.eye(H * vdim, dtype=D)}


def test_latent_attention_through_folded_matrices_and_a_window_written_out():
    """The same attention computed the other way round: queries mapped into the latent's
    space, one shared row per token, values taken from the latents and mapped afterwards."""
    torch.manual_seed(0)
    n, width, H, dim, rot, vdim, q_rank, kv_rank, window = 9, 12, 2, 4, 4, 3, 5, 6, 4
    w = _latent_weights(H, dim, rot, vdim, q_rank, kv_rank, width)
    m = {"heads": H, "dim": dim, "rot_dim": rot, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": 0.3,
         "rot": {"base": 100.0, "dims": rot}, "mask": {"size": window}}
    h = torch.randn(n, width, dtype=D)
    pos = torch.arange(n)
    got = plain.latent_attention_mixer(h, pos, w, "l", m, 1e-6).view(n, H, vdim)
    cq = plain.weighted_norm(h @ w["l.dq"].T, w["l.dq.norm"], 1e-6)
    q = (cq @ w["l.uq"].T).view(n, H, dim + rot)
    dkv = h @ w["l.dkv"].T
    c = plain.weighted_norm(dkv[:, :kv_rank], w["l.dkv.norm"], 1e-6)
    # rotation as a complex turn of the pair (2i, 2i + 1)
    def turn(x, p):
        z = torch.view_as_complex(x.reshape(-1, rot // 2, 2).contiguous())
        rate = 100.0 ** (-2.0 * torch.arange(rot // 2, dtype=D) / rot)
        return torch.view_as_real(z * torch.polar(torch.ones_like(rate), p * rate)).reshape(x.shape)
    uk, uv = w["l.uk"].view(H, dim, kv_rank), w["l.uv"].view(H, vdim, kv_rank)
    for i in range(n):
        for head in range(H):
            folded = torch.cat([uk[head].T @ q[i, head, :dim], turn(q[i, head, dim:], float(i))])
            lo = max(0, i - window + 1)
            rows = torch.stack([torch.cat([c[j], turn(dkv[j, kv_rank:], float(j))]) for j in range(lo, i + 1)])
            p = torch.softmax(rows @ folded * 0.3, dim=0)
            assert torch.allclose(got[i, head], uv[head] @ (p @ rows[:, :kv_rank]), atol=1e-10)
    # a token outside every later window changes nothing later
    h2 = h.clone()
    h2[0] += 1.0
    again = plain.latent_attention_mixer(h2, pos, w, "l", m, 1e-6).view(n, H, vdim)
    assert torch.equal(again[window:], got[window:]) and not torch.equal(again[window - 1], got[window - 1])


def _mlstm_weights(H, dim, vdim, width):
    g = torch.Generator().manual_seed(3)
    r = lambda *s: torch.randn(*s, generator=g, dtype=D)  # noqa: E731
    return {"m.q": r(H * dim, width), "m.k": r(H * dim, width), "m.v": r(H * vdim, width), "m.g": r(H * vdim, width),
            "m.o": torch.eye(H * vdim, dtype=D), "m.norm": torch.ones(H * vdim, dtype=D), "m.i": r(H, width),
            "m.i.b": r(H), "m.f": r(H, width), "m.f.b": r(H)}


def test_matrix_memory_carries_its_state_and_equals_the_unstabilised_sum():
    torch.manual_seed(0)
    n, width, H, dim, vdim, cap = 12, 7, 2, 3, 4, 5.0
    w = _mlstm_weights(H, dim, vdim, width)
    m = {"heads": H, "dim": dim, "vdim": vdim, "gate_cap": cap}
    h = torch.randn(n, width, dtype=D)
    whole, _ = plain.mlstm_mixer(h, w, "m", m, 1e-6)
    first, state = plain.mlstm_mixer(h[:5], w, "m", m, 1e-6)
    second, _ = plain.mlstm_mixer(h[5:], w, "m", m, 1e-6, state=state)
    assert torch.allclose(torch.cat([first, second]), whole, atol=1e-12)
    # without the running maximum: S_t = sum_j exp(i_j + sum_{l > j} f_l) k_j v_j^T, and the
    # readout's denominator max(|n . q|, exp(-m_t)) is scaled by exp(m_t), m_t = max(m_0 + F_t, max_j (i_j + F_t - F_j))
    q = (h @ w["m.q"].T).view(n, H, dim) * dim**-0.5
    k = (h @ w["m.k"].T).view(n, H, dim)
    v = (h @ w["m.v"].T).view(n, H, vdim)
    i_log = cap * torch.tanh((h @ w["m.i"].T + w["m.i.b"]) / cap)
    f_log = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ w["m.f"].T + w["m.f.b"]) / cap))
    t, head = n - 1, 1
    F = f_log[:, head].cumsum(0)
    wts = torch.exp(i_log[: t + 1, head] + F[t] - F[: t + 1])
    S = torch.einsum("j,jd,jv->dv", wts, k[: t + 1, head], v[: t + 1, head])
    nv = (wts[:, None] * k[: t + 1, head]).sum(0)
    m_t = max(float(F[t]), float((i_log[: t + 1, head] + F[t] - F[: t + 1]).max()))
    o = (S.T @ q[t, head]) / (max(abs(float(nv @ q[t, head])), 1.0) + 1e-6 * math.exp(m_t))
    o = o / torch.sqrt((o * o).mean() + 1e-6) * torch.sigmoid(h[t] @ w["m.g"].T)[head * vdim : (head + 1) * vdim]
    assert torch.allclose(whole[t, head * vdim : (head + 1) * vdim], o, atol=1e-9)


@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_the_whole_model_is_causal_and_its_first_token_stands_alone(name):
    from shrike_amd.weights.random_init import random_tensor

    arch = registry.get_architecture("Minilorn")
    spec = arch.build_spec(arch.config_cls.from_dict(CONFIGS[name]))
    w = {p.name: random_tensor(p, 1, torch.float32, mode="unit").double() for p in DecoderModel(spec).params()}
    vocab = CONFIGS[name]["vocab"]
    g = torch.Generator().manual_seed(4)
    ids = torch.randint(vocab, (40,), generator=g)
    full = plain.forward(CONFIGS[name], w, ids)
    assert torch.allclose(plain.forward(CONFIGS[name], w, ids[:17]), full[:17], atol=1e-9)
    assert torch.allclose(plain.forward(CONFIGS[name], w, ids[:1]), full[:1], atol=1e-9)
    other = ids.clone()
    other[30] = (other[30] + 1) % vocab
    changed = plain.forward(CONFIGS[name], w, other)
    assert torch.equal(changed[:30], full[:30]) and not torch.allclose(changed[30:], full[30:])
    if "embedding" in CONFIGS[name] and CONFIGS[name]["embedding"]["bigram"]["buckets"] > 1:
        # the token after a changed one sees it through the pair embedding even where no mixer looks back
        x, y = plain.embed(ids, w, CONFIGS[name]), plain.embed(other, w, CONFIGS[name])
        assert not torch.equal(x[31], y[31]) and torch.equal(x[32:], y[32:])
