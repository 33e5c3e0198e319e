"""The kernels and kernel options that the Mofarax decoder brought, each alone against a
plain computation: the rotation of neighbouring pairs with values taken from the keys,
the block-local mask in every attention kernel (with one key made to stand out just
inside and just outside a block's first position, far back, and at page borders), the
sum of two products' outputs into the stream, the normed add fused with the next norm,
the gated gather, the scaled embedding and the per-pass additions."""

import pytest
import torch

from .plain import mofarax as plain
from .test_kernels_gpu import close, dev, fill_pools_from, get_key, paged_setup

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from shrike_amd.kernels import ops

    return ops


def test_first_key_of_a_query_on_the_host():
    """PagedSpec.first_needed: what the cache manager and the step's checks go by."""
    from shrike_amd.parts import PagedSpec, PageTensor

    t = (PageTensor("k", (1,)),)
    assert [PagedSpec(t, chunk=5).first_needed(p) for p in (0, 4, 5, 9, 10, 14)] == [0, 0, 5, 5, 10, 10]
    assert [PagedSpec(t, window=3).first_needed(p) for p in (0, 2, 3, 7)] == [0, 0, 1, 5]
    assert [PagedSpec(t, window=3, chunk=5).first_needed(p) for p in (4, 5, 6, 8)] == [2, 5, 5, 6]
    assert not PagedSpec(t).bounded and PagedSpec(t, chunk=1).bounded


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, head_dim, rot_dim, page_size, theta, splits",
                         [(6, 3, 48, 48, 8, 5e4, 0), (4, 2, 64, 32, 16, 1e6, 0), (5, 5, 24, 10, 4, 300.0, 3),
                          (2, 1, 96, 0, 16, 1.0, 0), (8, 2, 128, 128, 16, 1e4, 2)])
def test_rotation_of_neighbouring_pairs_and_values_from_keys(ops, dtype, heads, kv_heads, head_dim, rot_dim,
                                                             page_size, theta, splits):
    """Queries come back rotated in place, the cache holds rotated keys, and the values
    are the keys as they came in.  Also from the partial sums of a split product, and
    with more than 64 tokens (the path that bfloat16 rows rotated whole would take)."""
    torch.manual_seed(3)
    seq_lens, starts = [37, 1, 40], [5, 0, 3000]
    n = sum(seq_lens)
    tables, k_pool, v_pool = paged_setup([s + l for s, l in zip(starts, seq_lens)], page_size, 1024, kv_heads,
                                         head_dim, dtype)
    width = (heads + kv_heads) * head_dim
    x = torch.randn(n, width)
    if splits:
        parts = torch.randn(splits, n, width) * 0.3
        x = parts.sum(0)
    stored = x.to(dtype) if not splits else x  # what the kernel reads
    positions = torch.cat([torch.arange(s, s + l) for s, l in zip(starts, seq_lens)])
    token_seq = torch.cat([torch.full((l,), i) for i, l in enumerate(seq_lens)])
    inv_freq = (theta ** (-torch.arange(0, rot_dim, 2, dtype=torch.float64) / max(rot_dim, 1))).float()
    qkv = dev(stored.to(dtype)).contiguous() if not splits else torch.empty(n, width, device="cuda", dtype=dtype)
    split_sum = ops.SplitSum(dev(parts).contiguous()) if splits else None
    ops.rope_kv_store(qkv, heads, kv_heads, head_dim, rot_dim, dev(inv_freq) if rot_dim else None,
                      dev(positions.int()), dev(token_seq.int()), tables, k_pool, v_pool, page_size,
                      split_sum=split_sum, adjacent_pairs=True, values_from_keys=True)
    src = stored.double()
    # (angles as 32-bit products, as the design and the kernel form them: at position 3,000
    # an angle is known to 2e-4, which is what a float64 angle would differ by)
    q = plain.rotate_interleaved(src[:, : heads * head_dim].view(n, heads, head_dim), positions, theta, rot_dim,
                                 angle_dtype=torch.float32)
    k_in = src[:, heads * head_dim :].view(n, kv_heads, head_dim)
    k = plain.rotate_interleaved(k_in, positions, theta, rot_dim, angle_dtype=torch.float32)
    close(qkv[:, : heads * head_dim].view(n, heads, head_dim), q, dtype, scale=1.0)
    got_k = torch.empty(n, kv_heads, head_dim, dtype=dtype)
    got_v = torch.empty(n, kv_heads, head_dim, dtype=dtype)
    for t in range(n):
        p, s = int(positions[t]), int(token_seq[t])
        page = int(tables[s, p // page_size])
        got_k[t] = get_key(k_pool, page, p % page_size).cpu()
        got_v[t] = v_pool[page, :, :, p % page_size].cpu()
    close(got_k, k, dtype, scale=1.0)
    close(got_v, k_in, dtype, scale=1.0)  # the keys before their rotation
    if rot_dim == head_dim and rot_dim:
        assert not torch.equal(got_k, got_v)


def standing_out(ctx, heads, kv_heads, head_dim, target, seed):
    """Keys and values of a sequence and one query at its last position whose score for
    key `target` towers over all others (in every head)."""
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(ctx, kv_heads, head_dim, generator=g) * 0.1
    v = torch.randn(ctx, kv_heads, head_dim, generator=g)
    direction = torch.randn(head_dim, generator=g)
    direction /= direction.norm()
    k[target] = 4.0 * direction
    q = (6.0 * direction).expand(1, heads, head_dim).clone()
    return q, k, v


def run_attention(ops, kind, q, positions, tables, k_pool, v_pool, heads, kv_heads, head_dim, page_size, chunk, scale,
                  q_lens, starts, window=None):
    """One of the attention kernels on a step of len(q_lens) sequences (single tokens
    for "decode")."""
    n = q.shape[0]
    dtype = k_pool.dtype
    qd = dev(q.to(dtype)).view(n, -1).contiguous()
    out = torch.full((n, heads * head_dim), float("nan"), device="cuda", dtype=dtype)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    token_seq = i32([s for s, l in enumerate(q_lens) for _ in range(l)])
    if kind == "general":
        ops.attention(qd, out, heads, kv_heads, head_dim, i32(positions), token_seq, tables, k_pool, v_pool,
                      page_size, window, scale, chunk=chunk)
    elif kind == "decode":
        nsplit = 3
        partial = torch.full((n * heads * nsplit * (head_dim + 2),), float("nan"), device="cuda")
        ops.attention_decode(qd, out, n, heads, kv_heads, head_dim, i32(positions), tables, k_pool, v_pool,
                             page_size, window, scale, partial, nsplit, chunk=chunk)
    else:
        cu = [0]
        for l in q_lens:
            cu.append(cu[-1] + l)
        ctx = [s + l for s, l in zip(starts, q_lens)]
        run = 16 * (ops.attention_prefill_shared_tiles(heads, kv_heads, head_dim) if kind == "shared" else 1)
        wg_seq = [s for s, l in enumerate(q_lens) for _ in range(0, l, run)]
        wg_q0 = [q0 for l in q_lens for q0 in range(0, l, run)]
        launch = ops.attention_prefill_shared if kind == "shared" else ops.attention_prefill
        launch(qd, out, len(wg_seq), heads, kv_heads, head_dim, i32(cu), i32(ctx), i32(wg_seq), i32(wg_q0), tables,
               k_pool, v_pool, page_size, window, scale, chunk=chunk)
    return out.view(n, heads, head_dim)


KINDS = [("general", torch.float32), ("general", torch.bfloat16), ("decode", torch.bfloat16),
         ("shared", torch.bfloat16), ("tiles", torch.bfloat16)]


@pytest.mark.parametrize("kind, dtype", KINDS)
@pytest.mark.parametrize("chunk, ctx", [(48, 150), (33, 100), (16, 65), (7, 40), (1, 9), (500, 700), (120, 361),
                                        (4096, 1500)])  # the last: one block, the key 1,499 positions back
def test_a_key_just_inside_and_just_outside_the_block(ops, kind, dtype, chunk, ctx):
    """The last query's block starts at `first`.  A key that stands out at `first` is
    all the query sees; the same key one position earlier (the last of the block
    before, across a page border where the sizes fall so) is not seen at all."""
    heads, kv_heads, head_dim, page_size = 4, 2, 64, 16
    pos = ctx - 1
    first = pos // chunk * chunk
    for target, inside in ((first, True), (first - 1, False), (max(first - chunk, 0), first == 0)):
        if target < 0:
            continue
        q, k, v = standing_out(ctx, heads, kv_heads, head_dim, target, seed=ctx + target)
        tables, k_pool, v_pool = paged_setup([ctx], page_size, 128, kv_heads, head_dim, dtype, seed=1)
        fill_pools_from(tables, k_pool, v_pool, 0, k, v, page_size)
        if kind == "decode" or kind == "general":
            got = run_attention(ops, kind, q, [pos], tables, k_pool, v_pool, heads, kv_heads, head_dim, page_size,
                                chunk, 1.0, [1], [pos])
        else:  # the query is the last of a portion of 21 tokens (or of the whole sequence)
            n = min(21, ctx)
            qs = torch.cat([torch.randn(n - 1, heads, head_dim), q])
            got = run_attention(ops, kind, qs, list(range(ctx - n, ctx)), tables, k_pool, v_pool, heads, kv_heads,
                                head_dim, page_size, chunk, 1.0, [n], [ctx - n])[-1:]
        kd, vd = k.to(dtype).double(), v.to(dtype).double()
        want = plain.block_local_attention(q.to(dtype).double(), kd, vd, 1.0, chunk, first=pos)
        close(got, want, dtype, scale=1.0)
        group = heads // kv_heads
        seen = vd[target].repeat_interleave(group, dim=0)[None]
        near = float((got.double().cpu() - seen).abs().max())
        if inside and target != pos:
            assert near < 0.05, "the key that stands out at the block's first position was not found"
        elif not inside:
            assert near > 0.3, "a key before the block's first position was read"


@pytest.mark.parametrize("window", [None, 25])
@pytest.mark.parametrize("kind, dtype", KINDS)
def test_block_local_attention_on_a_mixed_batch(ops, kind, dtype, window):
    """Several sequences at once, contexts before, on and after block and page edges;
    also with a window beside the block: the later of the two first keys holds."""
    torch.manual_seed(21)
    heads, kv_heads, head_dim, page_size, chunk = 6, 3, 32, 16, 40
    if kind in ("decode", "general"):
        ctx = [1, 15, 16, 17, 40, 41, 80, 81, 119, 120, 121, 333]
        q_lens = [1] * len(ctx)
    else:
        ctx = [40, 41, 100, 260, 7]
        q_lens = [40, 2, 61, 130, 7]
    starts = [c - l for c, l in zip(ctx, q_lens)]
    tables, k_pool, v_pool = paged_setup(ctx, page_size, 128, kv_heads, head_dim, dtype, seed=4)
    keys = [torch.randn(c, kv_heads, head_dim) for c in ctx]
    values = [torch.randn(c, kv_heads, head_dim) for c in ctx]
    for s in range(len(ctx)):
        fill_pools_from(tables, k_pool, v_pool, s, keys[s], values[s], page_size)
    q = torch.randn(sum(q_lens), heads, head_dim)
    positions = [p for s, l in zip(starts, q_lens) for p in range(s, s + l)]
    scale = 0.9 * head_dim**-0.5
    got = run_attention(ops, kind, q, positions, tables, k_pool, v_pool, heads, kv_heads, head_dim, page_size, chunk,
                        scale, q_lens, starts, window=window)
    assert not torch.isnan(got.float()).any(), "a slot outside the context was read"
    off = 0
    for s, l in enumerate(q_lens):
        want = plain.block_local_attention(q[off : off + l].to(dtype).double(), keys[s].to(dtype).double(),
                                           values[s].to(dtype).double(), scale, chunk, first=starts[s], window=window)
        close(got[off : off + l], want, dtype, scale=1.0)
        off += l


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden, n", [(64, 5), (100, 3), (4096, 70), (2047, 2), (8192, 2)])
@pytest.mark.parametrize("form", ["tensors", "splits", "one"])
def test_two_outputs_join_the_stream(ops, dtype, hidden, n, form):
    torch.manual_seed(5)
    resid = torch.randn(n, hidden)
    if form == "splits":
        a, b = torch.randn(3, n, hidden), torch.randn(2, n, hidden)
        d1, d2 = ops.SplitSum(dev(a)), ops.SplitSum(dev(b))
        want = resid.double() + (a.double().sum(0).float().double() + b.double().sum(0).float().double())
    else:
        a, b = torch.randn(n, hidden).to(dtype), torch.randn(n, hidden).to(dtype)
        d1, d2 = dev(a), (dev(b) if form == "tensors" else None)
        want = resid.double() + a.double() + (b.double() if form == "tensors" else 0)
    r = dev(resid)
    cast = torch.empty(n, hidden, device="cuda", dtype=dtype)
    ops.add_deltas(r, d1, d2, cast=cast)
    assert float((r.double().cpu() - want).abs().max()) <= 3e-6 * float(want.abs().max())
    close(cast, want, dtype)
    r2 = dev(resid)
    ops.add_deltas(r2, d1, d2, dtype=dtype)  # without the copy in the compute dtype
    assert torch.equal(r, r2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden, n", [(64, 5), (100, 3), (4096, 33), (2046, 2)])
@pytest.mark.parametrize("splits", [0, 3])
def test_normed_add_fused_with_the_next_norm(ops, dtype, hidden, n, splits):
    """resid += y / rms(y) * w_y, and the norm of the sum in the same pass; with rows
    chosen (the final norm) and without writing the stream back; alone, with no norm
    behind it."""
    torch.manual_seed(6)
    resid = torch.randn(n, hidden) * 3
    w_y, w = torch.randn(hidden), 1 + 0.1 * torch.randn(hidden)
    eps_y, eps = 1e-3, 1e-5
    if splits:
        parts = torch.randn(splits, n, hidden)
        y, delta = parts.double().sum(0), ops.SplitSum(dev(parts))
    else:
        y = torch.randn(n, hidden).to(dtype)
        delta, y = dev(y), y.double()
    x = resid.double() + plain.plain_weight_norm(y, w_y.double(), eps_y)
    want = plain.plain_weight_norm(x, w.double(), eps)
    r = dev(resid)
    out = torch.empty(n, hidden, device="cuda", dtype=dtype)
    ops.add_normed_rmsnorm(r, delta, dev(w_y), eps_y, dev(w), eps, out)
    assert float((r.double().cpu() - x).abs().max()) <= 3e-6 * float(x.abs().max())
    close(out, want, dtype)
    rows = torch.tensor([n - 1, 0], dtype=torch.int32, device="cuda")
    r2, out2 = dev(resid), torch.empty(2, hidden, device="cuda", dtype=dtype)
    ops.add_normed_rmsnorm(r2, delta, dev(w_y), eps_y, dev(w), eps, out2, rows=rows, write_resid=False)
    assert torch.equal(r2.cpu(), resid) and torch.equal(out2.cpu(), out[[n - 1, 0]].cpu())
    r3 = dev(resid)
    ops.add_normed_rmsnorm(r3, delta, dev(w_y), eps_y, dtype=dtype)
    assert torch.equal(r3, r)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width, slices, index, vocab, n", [(16, 6, 4, 97, 9), (5, 3, 0, 31, 70), (256, 2, 1, 50, 3)])
def test_gate_times_a_slice_of_the_tokens_row(ops, dtype, width, slices, index, vocab, n):
    torch.manual_seed(7)
    a = (torch.randn(n, width) * 2).to(dtype)
    table = torch.randn(vocab, slices * width).to(dtype)
    ids = torch.randint(0, vocab, (n,))
    out = torch.empty(n, width, device="cuda", dtype=dtype)
    ops.act_mul_rows(dev(a), dev(table), dev(ids.int()), index * width, out, "gelu_tanh")
    want = plain.gelu_tanh(a.double()) * table.double()[ids][:, index * width : (index + 1) * width]
    close(out, want, dtype, scale=1.0)
    # the gate as partial sums of a product split along k
    parts = torch.randn(11, n, width) * 0.6
    ops.act_mul_rows(ops.SplitSum(dev(parts)), dev(table), dev(ids.int()), index * width, out, "gelu_tanh")
    want = plain.gelu_tanh(parts.sum(0).double()) * table.double()[ids][:, index * width : (index + 1) * width]
    close(out, want, dtype, scale=1.0)


def test_scaled_embedding_and_additions_per_pass(ops):
    torch.manual_seed(8)
    table = torch.randn(50, 72).to(torch.bfloat16)
    ids = torch.randint(0, 50, (11,))
    out = torch.empty(11, 72, device="cuda")
    ops.embed(dev(table), dev(ids.int()), out, 3.5)
    want = plain.embed(ids, table.float(), 3.5)
    assert torch.equal(out.cpu(), want)
    other, vec = torch.randn(11, 72), torch.randn(72)
    ops.add_rows(out, dev(other), dev(vec))
    assert torch.allclose(out.cpu(), want + other + vec, atol=1e-6)
    before = out.clone()
    ops.add_rows(out, None, dev(vec))
    assert torch.allclose(out.cpu(), before.cpu() + vec, atol=1e-6)
