"""The kernels that the Minilorn decoder brought, each alone against a plain computation
(tests/plain/minilorn.py): the pair embedding with the previous token kept per state
slot; the cache write with a query temperature and normed values of their own size;
attention with capped scores and a sink, one far key made to stand out; the latent
attention's preparation, rotation and attention with one key just inside and just
outside the window, in portions and single tokens, at page borders; the batched
product; the matrix memory's scan in pieces against the whole and against the plain
recurrence, in slots that are used again; the per-head norm with its gate; xIELU."""

import math

import pytest
import torch

from .plain import minilorn as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 2e-5, torch.bfloat16: 1.6e-2}


@pytest.fixture(scope="module")
def ops():
    from shrike_amd.kernels import ops

    return ops


def dev(t, dtype=None):
    return t.to("cuda", dtype).contiguous() if dtype else t.to("cuda").contiguous()


def i32(x):
    return torch.as_tensor(x, dtype=torch.int32).to("cuda")


def close(got, want, dtype, what=""):
    want = want.double().cpu()
    err = float((got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err <= TOL[dtype], f"{what} rel err {err:.3e} > {TOL[dtype]}"


def step_arrays(starts, lens):
    """positions, token_seq, cu_q of a step whose sequence s brings lens[s] tokens from starts[s]."""
    positions = torch.cat([torch.arange(s, s + l) for s, l in zip(starts, lens)])
    token_seq = torch.cat([torch.full((l,), i) for i, l in enumerate(lens)])
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)))
    return i32(positions), i32(token_seq), i32(cu)


def tables_for(ctx_lens, page_size, num_pages, seed=0):
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(num_pages, generator=g).tolist()
    width = max(-(-n // page_size) for n in ctx_lens)
    rows = []
    for n in ctx_lens:
        need = -(-n // page_size)
        rows.append([perm.pop() for _ in range(need)] + [0] * (width - need))
    return torch.tensor(rows, dtype=torch.int32)


# ------------------------------------------------------------------ pair embedding

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("buckets, mul_prev, mul_cur", [(13, 5, 3), (1, 1, 1), (5000, 1000003, 999983)])
def test_pair_embedding_keeps_the_previous_token_per_slot(ops, dtype, buckets, mul_prev, mul_cur):
    torch.manual_seed(1)
    vocab, hidden, slots = 50, 24, 3
    table, pairs = torch.randn(vocab, hidden).to(dtype), torch.randn(buckets + 1, hidden).to(dtype)
    cfg = {"embedding": {"bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}}
    w = {"embed": table.double(), "bigram": pairs.double()}
    seqs = {0: torch.randint(vocab, (23,)), 2: torch.randint(vocab, (9,)), 1: torch.randint(vocab, (1,))}
    want = {s: plain.embed(ids, w, cfg) for s, ids in seqs.items()}
    last = torch.full((slots + 1,), 7, dtype=torch.int32, device="cuda")  # what earlier holders left behind
    done = {s: 0 for s in seqs}
    # steps: (slot, tokens) pairs; portions of several sizes beside single tokens, a sequence left out of a step
    plan = [[(0, 5), (2, 1)], [(0, 1), (2, 2), (1, 1)], [(0, 2)], [(2, 6), (0, 15)]]
    for step in plan:
        starts = [done[s] for s, _ in step]
        lens = [n for _, n in step]
        ids = torch.cat([seqs[s][done[s] : done[s] + n] for s, n in step])
        positions, token_seq, cu = step_arrays(starts, lens)
        out = torch.empty(sum(lens), hidden, device="cuda")
        ops.embed_pairs(dev(table), dev(pairs), i32(ids), positions, token_seq, cu, i32([s for s, _ in step]), last,
                        out, buckets, mul_prev, mul_cur)
        row = 0
        for s, n in step:
            close(out[row : row + n], want[s][done[s] : done[s] + n], torch.float32, f"slot {s} from {done[s]}")
            row, done[s] = row + n, done[s] + n
    assert done == {s: len(ids) for s, ids in seqs.items()}
    # a new request in slot 0 starts at position 0: what the slot holds is not read
    fresh = torch.randint(vocab, (4,))
    positions, token_seq, cu = step_arrays([0], [4])
    out = torch.empty(4, hidden, device="cuda")
    ops.embed_pairs(dev(table), dev(pairs), i32(fresh), positions, token_seq, cu, i32([0]), last, out, buckets,
                    mul_prev, mul_cur)
    close(out, plain.embed(fresh, w, cfg), torch.float32)
    assert int(last[0]) == int(fresh[-1])


# ------------------------------------------------------------------ attention with a sink

def plain_sink_attention(q, k, v, pos_q, scale, cap, sink):
    """One head: q [n, d] at positions pos_q over keys/values [ctx, .]; causal."""
    out = torch.zeros(q.shape[0], v.shape[1], dtype=torch.float64)
    for r in range(q.shape[0]):
        s = (k[: pos_q[r] + 1] @ q[r]) * scale
        if cap:
            s = cap * torch.tanh(s / cap)
        big = max(float(s.max()), float(sink))
        e = torch.exp(s - big)
        out[r] = (e / (e.sum() + math.exp(float(sink) - big))) @ v[: pos_q[r] + 1]
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, page_size, cap",
                         [(6, 2, 40, 72, 16, 45.0), (3, 3, 32, 32, 8, 4.0), (6, 1, 24, 7, 4, 0.0), (2, 2, 64, 128, 16, 9.0)])
def test_attention_with_a_sink_capped_scores_and_values_of_their_own_size(ops, dtype, heads, kv_heads, dim, vdim,
                                                                         page_size, cap):
    """A portion of a prompt beside single tokens, 700 keys; in every sequence one key far
    back is made to stand out for the last query (its score would be 20 uncapped); the sink
    of head 0 is large enough to halve that head's weights, that of the last head small."""
    torch.manual_seed(2)
    ctx = [700, 333, 1]
    lens = [1, 1, 1] if dim == 24 else [37, 1, 1]
    order = sorted(range(3), key=lambda i: lens[i] != 1)
    ctx, lens = [ctx[i] for i in order], [lens[i] for i in order]
    starts = [c - l for c, l in zip(ctx, lens)]
    scale = dim**-0.5
    tables = tables_for(ctx, page_size, 300, seed=dim)
    slab = 32 if dim % 32 == 0 else dim
    k_pool = torch.full((300, kv_heads, dim // slab, page_size, slab), float("nan"), dtype=dtype, device="cuda")
    v_pool = torch.full((300, kv_heads, vdim, page_size), float("nan"), dtype=dtype, device="cuda")
    keys = [torch.randn(c, kv_heads, dim) * 0.3 for c in ctx]
    values = [torch.randn(c, kv_heads, vdim) for c in ctx]
    n = sum(lens)
    q = torch.randn(n, heads, dim) * 0.3
    row = 0
    for s, (c, l) in enumerate(zip(ctx, lens)):
        far = 3  # the far key: position 3 of a long sequence; the one-token sequence keeps its random query
        last = row + l - 1
        for h in range(heads if c > 300 else 0):
            g = h // (heads // kv_heads)
            unit = keys[s][far, g] / keys[s][far, g].norm()
            q[last, h] = unit * 20.0 / scale / float(keys[s][far, g].norm())
        row += l
    sinks = torch.randn(heads)
    sinks[0], sinks[-1] = 4.0, -6.0
    q, keys, values = q.to(dtype), [k.to(dtype) for k in keys], [v.to(dtype) for v in values]
    for s, c in enumerate(ctx):
        for first in range(0, c, page_size):
            page, m = int(tables[s, first // page_size]), min(page_size, c - first)
            kk = keys[s][first : first + m].to("cuda")
            k_pool[page, :, :, :m, :] = kk.view(m, kv_heads, dim // slab, slab).permute(1, 2, 0, 3)
            v_pool[page, :, :, :m] = values[s][first : first + m].to("cuda").permute(1, 2, 0)
    positions, token_seq, _ = step_arrays(starts, lens)
    out = torch.empty(n, heads * vdim, dtype=dtype, device="cuda")
    ops.attention(dev(q.reshape(n, heads * dim)), out, heads, kv_heads, dim, positions, token_seq, dev(tables), k_pool,
                  v_pool, page_size, None, scale, v_dim=vdim, softcap=cap or None, sinks=dev(sinks))
    want = torch.zeros(n, heads, vdim, dtype=torch.float64)
    row = 0
    for s, (c, l) in enumerate(zip(ctx, lens)):
        pos_q = list(range(c - l, c))
        for h in range(heads):
            g = h // (heads // kv_heads)
            want[row : row + l, h] = plain_sink_attention(q[row : row + l, h].double(), keys[s][:, g].double(),
                                                          values[s][:, g].double(), pos_q, scale, cap, sinks[h])
        row += l
    close(out.view(n, heads, vdim), want, dtype)
    # head 0's sink takes most of the weight where no key stands out: leaving it out would show
    s1 = ctx.index(1)
    r1 = sum(lens[:s1])
    without = plain_sink_attention(q[r1 : r1 + 1, 0].double(), keys[s1][:, 0].double(), values[s1][:, 0].double(),
                                   [0], scale, cap, -1e30)
    assert float((without[0] - want[r1, 0]).abs().max()) > 10 * TOL[dtype] * float(want.abs().max())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, page_size, every", [(6, 2, 40, 72, 16, 100), (3, 3, 8, 5, 4, 3),
                                                                          (2, 1, 64, 64, 8, 1)])
def test_cache_write_with_a_query_temperature_and_normed_values(ops, dtype, heads, kv_heads, dim, vdim, page_size, every):
    torch.manual_seed(3)
    coef, eps = 0.7, 1e-5
    starts = [every - 2 if every > 2 else 0, 2 * every - 1, 1000]  # just before a step of the temperature, on one, far out
    lens = [4, 1, 3]
    ctx = [s + l for s, l in zip(starts, lens)]
    n = sum(lens)
    tables = tables_for(ctx, page_size, 400, seed=every)
    slab = 32 if dim % 32 == 0 else dim
    k_pool = torch.zeros((400, kv_heads, dim // slab, page_size, slab), dtype=dtype, device="cuda")
    v_pool = torch.zeros((400, kv_heads, vdim, page_size), dtype=dtype, device="cuda")
    qkv = (torch.randn(n, heads * dim + kv_heads * (dim + vdim)) * 3).to(dtype)
    positions, token_seq, _ = step_arrays(starts, lens)
    got = dev(qkv.clone())
    ops.qkv_store(got, heads, kv_heads, dim, vdim, positions, token_seq, dev(tables), k_pool, v_pool, page_size,
                  q_temperature=(coef, every), v_norm_eps=eps)
    pos = positions.cpu().long()
    factor = plain.query_temperature(pos, coef, every, torch.float64)
    assert float(factor[0]) == 1.0 or every <= 2
    x = qkv.double()
    close(got[:, : heads * dim], x[:, : heads * dim] * factor[:, None], dtype, "queries")
    assert torch.equal(got[:, heads * dim :].cpu(), qkv[:, heads * dim :]), "keys and values stay as they are in the row"
    k = x[:, heads * dim : (heads + kv_heads) * dim].view(n, kv_heads, dim)
    v = plain.unit_rms(x[:, (heads + kv_heads) * dim :].view(n, kv_heads, vdim), eps)
    for t in range(n):
        s = int(token_seq[t])
        page, slot = int(tables[s, int(pos[t]) // page_size]), int(pos[t]) % page_size
        got_k = k_pool[page, :, :, slot, :].reshape(kv_heads, dim)
        assert torch.equal(got_k.cpu().double(), k[t]), "keys are stored as projected"
        close(v_pool[page, :, :, slot], v[t], dtype, "values")


# ------------------------------------------------------------------ latent attention

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("q_rank, kv_rank, rot_dim, page_size, base", [(96, 160, 32, 16, 5e4), (9, 11, 4, 4, 40.0),
                                                                      (300, 272, 32, 8, 1e6), (5, 7, 0, 16, 1.0)])
def test_latent_preparation_norms_rotates_and_writes_the_row(ops, dtype, q_rank, kv_rank, rot_dim, page_size, base):
    torch.manual_seed(4)
    eps = 1e-5
    starts, lens = [0, 77, 5000], [5, 1, 3]
    ctx = [s + l for s, l in zip(starts, lens)]
    n = sum(lens)
    tables = tables_for(ctx, page_size, 1400, seed=3)
    pool = torch.zeros(1400, page_size, kv_rank + rot_dim, dtype=dtype, device="cuda")
    down = (torch.randn(n, q_rank + kv_rank + rot_dim) * 2).to(dtype)
    wq, wkv = 1 + 0.1 * torch.randn(q_rank), 1 + 0.1 * torch.randn(kv_rank)
    inv_freq = (base ** (-torch.arange(0, rot_dim, 2, dtype=torch.float64) / max(rot_dim, 1))).float()
    positions, token_seq, _ = step_arrays(starts, lens)
    c_q = torch.empty(n, q_rank, dtype=dtype, device="cuda")
    ops.latent_prepare(dev(down), q_rank, kv_rank, rot_dim, dev(wq), dev(wkv), eps, dev(inv_freq) if rot_dim else None,
                       positions, token_seq, dev(tables), c_q, pool, page_size)
    x = down.double()
    close(c_q, plain.weighted_norm(x[:, :q_rank], wq.double(), eps), dtype, "query latent")
    c = plain.weighted_norm(x[:, q_rank : q_rank + kv_rank], wkv.double(), eps)
    pos = positions.cpu().long()
    k_rot = plain.rotate_interleaved(x[:, q_rank + kv_rank :].view(n, 1, rot_dim), pos, base, rot_dim,
                                     angle_dtype=torch.float32).view(n, rot_dim)
    want = torch.cat([c, k_rot], dim=1)
    for t in range(n):
        page, slot = int(tables[int(token_seq[t]), int(pos[t]) // page_size]), int(pos[t]) % page_size
        close(pool[page, slot], want[t], dtype, f"row of token {t}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_rotation_of_a_slice_of_every_head(ops, dtype):
    torch.manual_seed(5)
    n, heads, src_head, dst_head, rot = 9, 3, 20, 30, 8
    src = torch.randn(n, heads * src_head).to(dtype)
    dst = torch.zeros(n, heads * dst_head, dtype=dtype, device="cuda")
    positions = i32([0, 1, 2, 3000, 3001, 17, 18, 19, 65000])
    inv_freq = (777.0 ** (-torch.arange(0, rot, 2, dtype=torch.float64) / rot)).float()
    ops.rotate_heads(dev(src), src_head, 12, dst, dst_head, 22, heads, rot, dev(inv_freq), positions)
    want = plain.rotate_interleaved(src.double().view(n, heads, src_head)[..., 12:], positions.cpu().long(), 777.0, rot,
                                    angle_dtype=torch.float32)
    close(dst.view(n, heads, dst_head)[..., 22:], want, dtype)
    assert float(dst.view(n, heads, dst_head)[..., :22].abs().max()) == 0.0, "only the slice is written"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, key_dim, v_dim, window, page_size", [(6, 176, 160, 56, 16), (3, 15, 11, 9, 4), (2, 304, 272, 40, 8),
                                                                      (1, 32, 30, 1, 16), (4, 48, 40, 1000, 16), (28, 512, 448, 100, 16),
                                                                      (20, 576, 512, 33, 16), (17, 640, 640, 64, 32)])
def test_latent_attention_at_the_windows_edges(ops, dtype, heads, key_dim, v_dim, window, page_size):
    """Rows of a portion and single tokens.  For chosen queries one key is made to stand out:
    the oldest key inside the window (its row must dominate) or the newest outside it (it
    must not be seen at all), far back behind several pages; among random scores near zero."""
    torch.manual_seed(6)
    ctx, lens = [300, 131, 260], [1, 1, 70]
    starts = [c - l for c, l in zip(ctx, lens)]
    n, scale = sum(lens), 0.25
    tables = tables_for(ctx, page_size, 260, seed=window)
    pool = torch.full((260, page_size, key_dim), float("nan"), dtype=dtype, device="cuda")
    rows = [torch.randn(c, key_dim) * 0.2 for c in ctx]
    q = torch.randn(n, heads, key_dim) * 0.2
    positions, token_seq, _ = step_arrays(starts, lens)
    pos = positions.cpu().long()
    marks = []  # (token row, inside?)
    for t in ([0, 1] + list(range(2, n, 7)) + [n - 1]):
        s, p = int(token_seq[t]), int(pos[t])
        inside = (t % 2 == 0)
        j = p - window + 1 if inside else p - window
        if j < 0:
            continue
        for h in range(heads):
            q[t, h] = rows[s][j] / rows[s][j].norm() ** 2 * 25.0 / scale
        marks.append((t, inside))
    q, rows = q.to(dtype), [r.to(dtype) for r in rows]
    for s, c in enumerate(ctx):
        for first in range(0, c, page_size):
            m = min(page_size, c - first)
            pool[int(tables[s, first // page_size]), :m] = rows[s][first : first + m].to("cuda")
    out = torch.empty(n, heads * v_dim, dtype=dtype, device="cuda")
    ops.latent_attention(dev(q.reshape(n, heads * key_dim)), out, heads, key_dim, v_dim, positions, token_seq, dev(tables),
                         pool, page_size, window, scale)
    want = torch.zeros(n, heads, v_dim, dtype=torch.float64)
    for t in range(n):
        s, p = int(token_seq[t]), int(pos[t])
        lo = max(0, p - window + 1)
        kr = rows[s][lo : p + 1].double()
        for h in range(heads):
            w = torch.softmax((kr @ q[t, h].double()) * scale, dim=0)
            want[t, h] = w @ kr[:, :v_dim]
    assert torch.isfinite(out).all(), "a row outside the sequence's pages or its window was read"
    close(out.view(n, heads, v_dim), want, dtype)
    if dtype == torch.bfloat16 and ops.latent_attention_supports_mfma(heads, key_dim, v_dim):
        # the same on the matrix units, each token's rows taken by one workgroup and shared among three
        # ... and with up to four neighbouring tokens a workgroup (the first workgroups hold single tokens
        # of different sequences, one holds a portion's first tokens beside one of them)
        for nsplit, group in ((1, 1), (3, 1), (1, 4), (2, 2)):
            again = torch.full((n, heads * v_dim), float("nan"), dtype=dtype, device="cuda")
            partial = torch.full((n * heads * nsplit * (v_dim + 2),), float("nan"), device="cuda")
            ops.latent_attention_mfma(dev(q.reshape(n, heads * key_dim)), again, heads, key_dim, v_dim, positions, token_seq,
                                      dev(tables), pool, page_size, window, scale, partial=partial, nsplit=nsplit,
                                      tokens_per_group=group)
            assert torch.isfinite(again).all(), f"{nsplit} shares: a row outside the window or the pages was read"
            close(again.view(n, heads, v_dim), want, dtype, f"matrix units, {nsplit} shares, {group} tokens a workgroup")
    assert window >= 300 or (any(inside for _, inside in marks) and any(not inside for _, inside in marks))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n, batch, m, k", [(1, 6, 96, 40), (70, 3, 10, 24), (5, 2, 65, 130), (32, 4, 7, 300), (33, 2, 64, 64),
                                            (17, 28, 448, 128), (200, 3, 130, 72), (8, 5, 16, 8)])
def test_batched_product(ops, dtype, n, batch, m, k):
    """Slices of a that are 16-byte aligned (what bfloat16 then runs on the matrix units) and slices
    that are not (the general kernels)."""
    torch.manual_seed(7)
    for a_pad in (3, 8):
        a_step, out_step = k + a_pad, m + 5
        a = torch.randn(n, batch * a_step).to(dtype)
        w = (torch.randn(batch, m, k) / k**0.5).to(dtype)
        out = torch.zeros(n, batch * out_step, dtype=dtype, device="cuda")
        ops.gemm_batched(dev(a), dev(w), out, batch, a_step, out_step)
        for b in range(batch):
            want = a[:, b * a_step : b * a_step + k].double() @ w[b].double().T
            close(out[:, b * out_step : b * out_step + m], want, dtype, f"product {b}, slices {a_step} apart")
            assert float(out[:, b * out_step + m : (b + 1) * out_step].abs().max()) == 0.0


# ------------------------------------------------------------------ matrix memory

def selection_weights(prefix, heads, dim, vdim, ld, off):
    """Weights for the plain mixer that pick the scan's inputs out of a row of projections."""
    eye = torch.eye(ld, dtype=torch.float64)
    hv = heads * vdim
    return {prefix + ".q": eye[off["q"] : off["q"] + heads * dim], prefix + ".k": eye[off["k"] : off["k"] + heads * dim],
            prefix + ".v": eye[off["v"] : off["v"] + hv], prefix + ".g": eye[off["g"] : off["g"] + hv],
            prefix + ".i": eye[off["i"] : off["i"] + heads], prefix + ".f": eye[off["f"] : off["f"] + heads],
            prefix + ".o": torch.eye(hv, dtype=torch.float64)}


@pytest.mark.parametrize("heads, dim, vdim, cap", [(2, 24, 36, 14.0), (1, 8, 5, 3.0), (3, 33, 16, 30.0), (2, 100, 40, 8.0),
                                                   (1, 200, 17, 12.0)])
def test_matrix_memory_in_pieces_against_the_whole_and_the_plain_recurrence(ops, heads, dim, vdim, cap):
    """Three sequences in slots 2, 0 and the spare slot's neighbour, cut differently: whole,
    in portions of many sizes, token by token; all three equal bit for bit, and equal the plain
    recurrence; then the slots are used again by other sequences without being cleared."""
    torch.manual_seed(8)
    eps = 1e-6
    qk, hv = heads * dim, heads * vdim
    off = {"q": 0, "k": qk, "v": 2 * qk, "g": 2 * qk + hv, "i": 2 * qk + 2 * hv, "f": 2 * qk + 2 * hv + heads}
    ld = 2 * qk + 2 * hv + 2 * heads
    T = 150
    floats = ops.mlstm_state_floats(heads, dim, vdim)
    state = torch.full((4, floats), float("nan"), device="cuda")  # slots 0..2 and the spare; never cleared
    i_bias, f_bias = torch.randn(heads), torch.randn(heads) + 2.0
    norm_w = 1 + 0.1 * torch.randn(hv)

    def run(proj, cuts, slot):
        outs, p = [], 0
        for n in cuts:
            n = min(n, T - p)
            if n <= 0:
                break
            positions, _, cu = step_arrays([p], [n])
            rows = dev(proj[p : p + n])
            read = torch.empty(n, hv, device="cuda")
            ops.mlstm_scan(rows, off["q"], off["k"], off["v"], off["i"], off["f"], dev(i_bias), dev(f_bias), cap,
                           dim**-0.5, 1, heads, dim, vdim, positions, cu, i32([slot]), state, read)
            gated = torch.empty(n, hv, device="cuda")
            ops.headnorm_gate(read, rows[:, off["g"] :], dev(norm_w), eps, gated, heads, vdim)
            outs.append(gated.cpu())
            p += n
        assert p == T
        return torch.cat(outs)

    for round_ in range(2):  # the second round finds the slots full of the first round's state
        proj = torch.randn(T, ld)
        proj[:, off["i"] : off["i"] + heads] *= 6.0  # gates that swing between closed and wide open
        proj[:, off["f"] :] *= 6.0
        whole = run(proj, [T], 2)
        pieces = run(proj, [3, 2, 9, 1, 1, 8, 17, 2, 40, 64, 5, 1000], 0)
        singles = run(proj, [1] * T, 1)
        assert torch.equal(whole, pieces) and torch.equal(whole, singles), "the result depends on how the tokens were cut"
        w = selection_weights("m", heads, dim, vdim, ld, off)
        w.update({"m.i.b": i_bias.double(), "m.f.b": f_bias.double(), "m.norm": norm_w.double()})
        want, _ = plain.mlstm_mixer(proj.double(), w, "m", {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, eps)
        # gates that swing by tens in the exponent, and readouts that the unit norm rescales:
        # float32 keeps four digits of such a row
        err = float((whole.double() - want).abs().max() / want.abs().max())
        assert err <= 2e-4, f"round {round_}: rel err {err:.3e}"


def test_matrix_memory_of_several_sequences_in_one_step(ops):
    """A step with a single token, a portion and another single token: each sequence's
    state is its own, whatever else is in the batch."""
    torch.manual_seed(9)
    heads, dim, vdim, cap = 2, 16, 20, 6.0
    qk, hv = heads * dim, heads * vdim
    off = {"q": 0, "k": qk, "v": 2 * qk, "g": 2 * qk + hv, "i": 2 * qk + 2 * hv, "f": 2 * qk + 2 * hv + heads}
    ld = 2 * qk + 2 * hv + 2 * heads
    floats = ops.mlstm_state_floats(heads, dim, vdim)
    bias = dev(torch.zeros(heads))
    lens_total = [30, 41, 12]
    projs = [torch.randn(t, ld) for t in lens_total]

    def scan(entries, state):
        """entries: (sequence, slot, first, count)."""
        rows = dev(torch.cat([projs[s][a : a + c] for s, _, a, c in entries]))
        positions, _, cu = step_arrays([a for _, _, a, _ in entries], [c for _, _, _, c in entries])
        read = torch.empty(rows.shape[0], hv, device="cuda")
        ops.mlstm_scan(rows, off["q"], off["k"], off["v"], off["i"], off["f"], bias, bias, cap, dim**-0.5,
                       len(entries), heads, dim, vdim, positions, cu, i32([slot for _, slot, _, _ in entries]), state, read)
        return read.cpu()

    alone = []
    state = torch.zeros(4, floats, device="cuda")
    for s, t in enumerate(lens_total):
        alone.append(scan([(s, 0, 0, t)], state))
    state = torch.zeros(4, floats, device="cuda")
    got = [[] for _ in lens_total]
    done = [0, 0, 0]
    plan = [[(0, 1), (1, 7)], [(0, 1), (2, 1), (1, 2)], [(2, 11), (0, 28), (1, 32)]]
    for step in plan:
        entries = [(s, 2 - s, done[s], c) for s, c in step]
        out = scan(entries, state)
        row = 0
        for s, c in step:
            got[s].append(out[row : row + c])
            row, done[s] = row + c, done[s] + c
    for s in range(3):
        assert torch.equal(torch.cat(got[s]), alone[s]), f"sequence {s} depends on its batch"


@pytest.mark.parametrize("dtype", DTYPES)
def test_xielu(ops, dtype):
    torch.manual_seed(10)
    x = torch.cat([torch.randn(1000) * 3, torch.tensor([0.0, -0.0, 1e-4, -1e-4, 30.0, -30.0])]).to(dtype)
    p, q = torch.tensor(0.3, dtype=torch.float64), torch.tensor(-0.7, dtype=torch.float64)
    a_pos, a_neg = float(torch.nn.functional.softplus(p)), 0.5 + float(torch.nn.functional.softplus(q))
    out = torch.empty_like(x, device="cuda")
    ops.xielu(dev(x), out, a_pos, a_neg)
    close(out, plain.xielu(x.double(), p, q), dtype)
