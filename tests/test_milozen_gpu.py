"""Milozen on the GPU against the plain implementation (tests/plain_milozen.py, float64 on the CPU):
each mechanism alone, then whole models of small made-up sizes in every way of cutting a request into steps,
with pages and slots that are freed and used again, and greedy generation through the entry point.

Which experts a token uses is a discrete choice: the 32-bit engine makes the plain implementation's choices (their
scores differ by 1e-6 of the gaps), so every position is compared there.  The bfloat16 engine's hidden states differ
from the exact ones by a percent after a few layers, which turns the choice of a token in a few hundred; whole models
in bfloat16 are therefore held to a bound that three positions in four meet (every position that attends to such a
token follows it), and a tighter one on the median."""

import math

import pytest
import torch

import plain_milozen as pm
import traces
from milozen_configs import SMALL, SMALL_B, SMALL_C, SMALL_D, config_of, moe

pytestmark = pytest.mark.gpu

DEV = torch.device("cuda:0")
DTYPES = [torch.float32, torch.bfloat16]
F64 = torch.float64


def rnd(*shape, seed=0, scale=1.0):
    return scale * torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64)


def close(got, ref, dtype, what="", loose=1.0):
    got, ref = got.double().cpu(), ref.double()
    assert got.shape == ref.shape, f"{what}: {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{what}: not finite"
    scale = max(1e-6, float(ref.abs().max()))
    worst = float((got - ref).abs().max()) / scale
    assert worst <= loose * (2.0 ** -6 if dtype == torch.bfloat16 else 2e-5), f"{what}: off by {worst:.2e} of the largest value"


def dev(x, dtype=torch.float32):
    return x.to(dtype).to(DEV).contiguous()


def ints(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


# ------------------------------------------------------------------------------ streams and the layer norm
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("streams,hidden", [(1, 100), (2, 98), (3, 2048), (8, 40)])
def test_streams_are_written_read_and_normed_in_one_pass(dtype, streams, hidden):
    from llmserve.ops import library as ops

    n, eps = 7, 1e-5
    source, y = rnd(n, hidden, seed=1, scale=3.0) + 0.7, rnd(n, hidden, seed=2)
    mix, write, read = rnd(streams, streams, seed=3) + torch.eye(streams, dtype=F64), rnd(streams, seed=4) + 1, rnd(streams, seed=5) + 0.5
    w = rnd(hidden, seed=6) + 1
    # the first read: every copy is the source
    x = torch.full((n, streams, hidden), float("nan"), dtype=torch.float32, device=DEV)
    out = torch.empty((n, hidden), dtype=dtype, device=DEV)
    ops.streams_norm(out, x, dev(w), eps, source=dev(source), read=dev(read))
    xs = source[None].repeat(streams, 1, 1)
    close(x.permute(1, 0, 2), xs, torch.float32, "copies")
    close(out, pm.layer_norm(pm.streams_read(xs, read), w, eps), dtype, "first read")
    # a write and the next read
    ops.streams_norm(out, x, dev(w), eps, y=dev(y), mix=dev(mix), write=dev(write), read=dev(read))
    xs = pm.streams_write(xs, y, mix, write)
    close(x.permute(1, 0, 2), xs, torch.float32, "written streams")
    close(out, pm.layer_norm(pm.streams_read(xs, read), w, eps), dtype, "second read")
    # picked rows for the last norm: the plain sum of the streams after one more write; nothing is stored
    before = x.clone()
    rows = [5, 0, 3]
    picked = torch.empty((3, hidden), dtype=dtype, device=DEV)
    ops.streams_norm(picked, x, dev(w), eps, y=dev(y), mix=dev(mix), write=dev(write), rows=ints(rows))
    assert torch.equal(x, before)
    close(picked, pm.layer_norm(pm.streams_write(xs, y, mix, write).sum(0), w, eps)[rows], dtype, "picked rows")
    # without coefficients a write is the plain residual sum
    if streams == 1:
        ops.streams_norm(out, x, dev(w), eps, y=dev(y))
        close(x[:, 0], xs[0] + y, torch.float32, "plain sum")
        close(out, pm.layer_norm(xs[0] + y, w, eps), dtype, "norm of the plain sum")


def test_the_variance_is_taken_about_the_mean():
    """Rows far from zero: a norm by the root mean square, or a variance from E[x^2] - E[x]^2 in 32-bit, shows."""
    from llmserve.ops import library as ops

    x = rnd(4, 1, 64, seed=9) + 300.0
    w = torch.ones(64, dtype=F64)
    out = torch.empty((4, 64), dtype=torch.float32, device=DEV)
    ops.streams_norm(out, dev(x), dev(w), 1e-5)
    close(out, pm.layer_norm(x[:, 0], w, 1e-5), torch.float32, "offset rows", loose=20)


# ------------------------------------------------------------------------------ latents, rotation, queries
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("q_rank,r,dr,dims,base", [(40, 32, 8, 8, 10000.0), (24, 48, 16, 4, 100.0), (16, 20, 2, 2, 3.0),
                                                   (300, 260, 64, 64, 10000.0)])
def test_latents_are_normed_rotated_and_stored(dtype, q_rank, r, dr, dims, base):
    from llmserve.ops import library as ops

    n, bs, eps = 9, 4, 1e-5
    positions = [0, 1, 2, 700, 701, 5, 6, 7, 8]
    z = rnd(n, 5 + q_rank + r + dr + 3, seed=11, scale=2.0)
    wq, wc = rnd(q_rank, seed=12) + 1, rnd(r, seed=13) + 1
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    pool = torch.full((6, 1, bs, r + dr), float("nan"), dtype=dtype, device=DEV)
    slots = [20, 21, 22, 3, -1, 8, 9, 10, 11]  # (a padding row stores nothing)
    cq = torch.empty((n, q_rank), dtype=dtype, device=DEV)
    ops.latent_prepare(dev(z), col_q=5, q_rank=q_rank, col_c=5 + q_rank, r=r, dr=dr, wq=dev(wq), wc=dev(wc),
                       freq=dev(freq), positions=ints(positions), eps=eps, cq=cq, pool=pool, slots=ints(slots))
    close(cq, pm.rms_unit(z[:, 5: 5 + q_rank], eps) * wq, dtype, "query latent")
    zc = z[:, 5 + q_rank:]
    want_c = pm.rms_unit(zc[:, :r], eps) * wc
    want_r = pm.rotate_interleaved(zc[:, r: r + dr], torch.tensor(positions), base, dims)
    rows = pool.reshape(-1, r + dr)
    keep = [i for i, s in enumerate(slots) if s >= 0]
    close(rows[[slots[i] for i in keep], :r], want_c[keep], dtype, "latent")
    close(rows[[slots[i] for i in keep], r:], want_r[keep], dtype, "rotated key part")
    untouched = [s for s in range(6 * bs) if s not in slots]
    assert torch.isnan(rows[untouched].float()).all()
    # a layer without a latent of its own stores nothing
    ops.latent_prepare(dev(z), col_q=5, q_rank=q_rank, col_c=None, r=r, dr=dr, wq=dev(wq), wc=None, freq=dev(freq),
                       positions=ints(positions), eps=eps, cq=cq)
    # queries: plain parts side by side, rotated parts turned into the folded rows
    heads, dn = 3, 12
    q = rnd(n, heads, dn + dr, seed=14)
    plain = torch.empty((n, heads * dn), dtype=dtype, device=DEV)
    folded = torch.full((n, heads * (r + dr)), float("nan"), dtype=dtype, device=DEV)
    ops.latent_query(plain, folded, dev(q.reshape(n, -1)), heads=heads, dn=dn, dr=dr, r=r, freq=dev(freq),
                     positions=ints(positions))
    close(plain.view(n, heads, dn), q[..., :dn], dtype, "plain parts")
    close(folded.view(n, heads, r + dr)[..., r:], pm.rotate_interleaved(q[..., dn:], torch.tensor(positions), base, dims),
          dtype, "rotated parts")
    assert torch.isnan(folded.view(n, heads, r + dr)[..., :r].float()).all()


# ------------------------------------------------------------------------------ the attention kernel alone
def paged_rows(rows, bs, dtype, seed=0, spare=3):
    """rows [t, D] -> pool [pages, 1, bs, D] in shuffled pages (unused slots NaN) and the request's block table."""
    t = rows.shape[0]
    need = -(-t // bs)
    order = torch.randperm(need + spare, generator=torch.Generator().manual_seed(seed)).tolist()
    pool = torch.full((need + spare, 1, bs, rows.shape[1]), float("nan"), dtype=dtype)
    table = torch.zeros((1, need), dtype=torch.int32)
    for i in range(need):
        table[0, i] = order[i]
        n = min(bs, t - i * bs)
        pool[order[i], 0, :n] = rows[i * bs: i * bs + n].to(dtype)
    return pool.to(DEV), table.to(DEV)


def attend(q, rows, r, dtype, bs, window, scale, at=None):
    """The kernel on a whole sequence: q [t, H, r + dr], rows [t, r + dr] -> [len(at), H, r]."""
    from llmserve.ops import library as ops

    t, heads, dk = q.shape
    at = list(range(t)) if at is None else at
    pool, table = paged_rows(rows, bs, dtype)
    out = torch.empty((len(at), heads * r), dtype=dtype, device=DEV)
    ops.attend_latent(out, dev(q[at].reshape(len(at), -1), dtype), pool, table, ints([0] * len(at)), ints(at), ints([t]),
                      heads=heads, r=r, dr=dk - r, block_size=bs, window=window or 0, scale=scale)
    return out.view(len(at), heads, r)


def attend_plain(q, rows, r, window, scale):
    t, heads, _ = q.shape
    visible = pm.window_visible(t, window)
    out = torch.zeros(t, heads, r, dtype=F64)
    for a in range(heads):
        p = torch.softmax(((q[:, a] @ rows.T) * scale).masked_fill(~visible, float("-inf")), dim=-1)
        out[:, a] = p @ rows[:, :r]
    return out


LATENT_CASES = [  # heads, r, dr, window, block size
    (3, 32, 8, 11, 8), (1, 20, 12, 1, 4), (5, 16, 8, None, 16), (2, 48, 16, 19, 8), (6, 72, 4, 40, 16), (2, 130, 62, 33, 8),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,r,dr,window,bs", LATENT_CASES)
def test_attention_over_latent_rows(dtype, heads, r, dr, window, bs):
    t = 77
    q, rows = rnd(t, heads, r + dr, seed=21), rnd(t, r + dr, seed=22)
    rows_seen, q_seen = rows.to(dtype).double(), q.to(dtype).double()
    got = attend(q, rows, r, dtype, bs, window, 0.3)
    close(got, attend_plain(q_seen, rows_seen, r, window, 0.3), dtype, "attention over the latent")


def test_a_key_that_stands_out_shows_the_windows_edge():
    """One key is made to take nearly all the weight of the queries that see it: whether query i sees key j is then
    read off the result.  Far back, at a page's border, just inside and just outside the window, the first tokens."""
    t, heads, r, dr, bs = 300, 2, 24, 8, 16
    for window in (1, 2, 16, 17, 150, None):
        for j in (0, 1, 15, 16, 17, 140, 255, 256):
            q, rows = rnd(t, heads, r + dr, seed=31, scale=0.1), rnd(t, r + dr, seed=32, scale=0.1)
            rows[j, r:] = 4.0  # (in the part that is no value, so the marker does not change what is summed)
            q[:, :, r:] = 4.0
            marker = torch.zeros(r, dtype=F64)
            marker[3] = 50.0
            rows[j, :r] += marker
            last_seen = t - 1 if window is None else min(t - 1, j + window - 1)
            at = sorted({i for i in (j - 1, j, j + 1, last_seen - 1, last_seen, last_seen + 1, t - 1) if 0 <= i < t})
            got = attend(q, rows, r, torch.float32, bs, window, 1.0, at=at).cpu()
            for k, i in enumerate(at):
                sees = j <= i and (window is None or i - j < window)
                assert (float(got[k, 0, 3]) > 25.0) == sees, f"window {window}: query {i} and key {j}"
            close(got, attend_plain(q, rows, r, window, 1.0)[at], torch.float32, f"window {window} key {j}", loose=5)


MFMA_CASES = [  # heads, r, dr, window, block size
    (3, 32, 8, 11, 8), (6, 112, 24, 130, 16), (1, 16, 8, 1, 4), (5, 48, 40, None, 16), (16, 64, 32, 33, 8), (40, 32, 32, 70, 16),
    (4, 256, 32, 50, 16), (2, 512, 64, 100, 16), (7, 144, 24, 64, 8),
]


@pytest.mark.parametrize("heads,r,dr,window,bs", MFMA_CASES)
@pytest.mark.parametrize("splits", [1, 3])
def test_matrix_core_attention_over_latent_rows(heads, r, dr, window, bs, splits):
    """Several requests in one launch: portions of different lengths behind different prefixes, single tokens, a
    request without keys; against the plain attention and, closely, against the kernel that takes any size."""
    from llmserve.ops import library as ops

    assert ops.attend_latent_mfma_supported(torch.bfloat16, r, dr)
    dt = torch.bfloat16
    lengths = [(150, 1), (97, 97), (200, 37), (64, 2), (33, 1), (300, 130)]  # (context after the step, tokens of the step)
    scale = 0.5 / math.sqrt(r + dr)
    pools, tables, qs, refs = [], [], [], []
    for b, (ctx, count) in enumerate(lengths):
        q, rows = rnd(ctx, heads, r + dr, seed=80 + b), rnd(ctx, r + dr, seed=90 + b)
        refs.append(attend_plain(q.to(dt).double(), rows.to(dt).double(), r, window, scale)[ctx - count:])
        qs.append(q[ctx - count:].reshape(count, -1))
        pool, table = paged_rows(rows, bs, dt, seed=b)
        pools.append(pool)
        tables.append(table[0].tolist())
    base, width = [0], max(len(t) for t in tables)
    for pool in pools:
        base.append(base[-1] + pool.shape[0])
    pool = torch.cat(pools)
    table = torch.zeros((len(lengths) + 2, width), dtype=torch.int32)
    order = [3, 0, 5, 1, 7, 2]  # (a request's row of the block tables is its state slot, not its place in the step)
    for b, t in enumerate(tables):
        table[order[b], : len(t)] = torch.tensor(t) + base[b]
    counts = [c for _, c in lengths] + [4]  # the last request has no keys (padding rows of a captured step)
    cu = [0]
    for c in counts:
        cu.append(cu[-1] + c)
    q_all = torch.cat(qs + [rnd(4, heads * (r + dr), seed=99)])
    n = q_all.shape[0]
    out = torch.full((n, heads * r), float("nan"), dtype=dt, device=DEV)
    args = dict(heads=heads, r=r, dr=dr, block_size=bs, window=window or 0, scale=scale, table_rows=ints(order + [4]))
    ops.attend_latent_mfma(out, dev(q_all, dt), pool, table.to(DEV), ints(cu), ints([c for c, _ in lengths] + [0]),
                           n_seqs=len(counts), max_count=max(counts), splits=splits, **args)
    assert (out[cu[-2]:] == 0).all()
    token_seq = [b for b, c in enumerate(counts) for _ in range(c)]
    positions = [ctx - count + i for ctx, count in lengths for i in range(count)] + [0] * 4
    other = torch.empty_like(out)
    ops.attend_latent(other, dev(q_all, dt), pool, table.to(DEV), ints(token_seq), ints(positions),
                      ints([c for c, _ in lengths] + [0]), **args)
    for b in range(len(lengths)):
        got = out[cu[b]: cu[b + 1]].view(-1, heads, r)
        close(got, refs[b], dt, f"request {b}")
        close(got, other[cu[b]: cu[b + 1]].view(-1, heads, r).double().cpu(), dt, f"request {b} against the plain kernel")


# ------------------------------------------------------------------------------ products with a weight per group
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,g,n,k,pad", [(70, 3, 32, 16, 5), (1, 5, 20, 24, 8), (130, 2, 66, 70, 3), (300, 3, 144, 64, 16),
                                         (17, 2, 24, 152, 0)])
def test_a_product_per_head_on_strided_views(dtype, m, g, n, k, pad):
    """(strides of x in multiples of 8 and bfloat16: the matrix-core kernel; all else the multiply-add kernel)"""
    from llmserve.ops import library as ops

    x, w, z = rnd(m, g, k + pad, seed=41), rnd(g, n, k, seed=42, scale=0.3), rnd(m, 7 + g * n, seed=43)
    xd, wd = dev(x, dtype), dev(w, dtype)
    out = torch.full((m, g, n + 3), float("nan"), dtype=dtype, device=DEV)
    ops.grouped_product(out[:, :, :n], xd[:, :, :k], wd)
    ref = torch.einsum("mgk,gnk->mgn", xd[:, :, :k].double().cpu(), wd.double().cpu())
    close(out[:, :, :n], ref, dtype, "per head")
    assert torch.isnan(out[:, :, n:].float()).all()
    ops.grouped_product(out[:, :, :n], xd[:, :, :k], wd, epilogue="gated", gate=dev(z), gate_column=7)
    close(out[:, :, :n], ref * torch.sigmoid(z[:, 7:]).reshape(m, g, n), dtype, "gated")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k,units", [(40, 24), (36, 70), (64, 32)])
@pytest.mark.parametrize("counts", [[5, 0, 70, 1], [0, 0, 3], [64, 64], [129], [200, 1, 130]])
def test_a_product_per_segment_of_rows(dtype, counts, k, units):
    from llmserve.ops import library as ops

    g, limit = len(counts), 0.9
    m = sum(counts)
    seg, tiles = [0], [[0], [0]]
    for c in counts:
        seg.append(seg[-1] + c)
        tiles[0].append(tiles[0][-1] + -(-c // ops.GROUPED_TILE))
        tiles[1].append(tiles[1][-1] + -(-c // ops.GROUPED_TILE_MFMA))
    segments = (ints(seg), ints(tiles[0] + tiles[1]))
    x, wa, wb = rnd(m, k, seed=51), rnd(g, units, k, seed=52, scale=0.3), rnd(g, units, k, seed=53, scale=0.3)
    xd = dev(x, dtype)
    wd = ops.stack_paired(dev(wa, dtype), dev(wb, dtype))
    assert wd.shape == (g, 64 * -(-units // 32), k)
    out = torch.empty((m, wd.shape[1]), dtype=torch.float32, device=DEV)
    ops.grouped_product(out, xd, wd, segments=segments)
    xs = xd.double().cpu()
    ref_a = torch.cat([xs[seg[e]: seg[e + 1]] @ wa[e].to(dtype).double().T for e in range(g)])
    ref_b = torch.cat([xs[seg[e]: seg[e + 1]] @ wb[e].to(dtype).double().T for e in range(g)])
    first = min(32, units)
    close(out[:, :first], ref_a[:, :first], dtype, "segments, first block of the first projection")
    close(out[:, 32: 32 + first], ref_b[:, :first], dtype, "segments, first block of the second projection")
    assert (out[:, first: 32] == 0).all()  # (rows of units that do not exist are zero)
    act = torch.full((m, units), float("nan"), dtype=dtype, device=DEV)
    ops.grouped_product(act, xd, wd, epilogue="paired", segments=segments, limit=limit, units=units)
    a = ref_a.to(dtype).double().clamp(max=limit)
    b = ref_b.to(dtype).double().clamp(min=-limit, max=limit)
    close(act, a * torch.sigmoid(1.702 * a) * (b + 1), dtype, "gated unit", loose=2)


@pytest.mark.parametrize("k,parts", [(64, 2), (200, 3), (1024, 4)])
def test_shares_of_k_add_up_to_the_product(k, parts):
    from llmserve.ops import library as ops

    counts, n = [3, 0, 17, 1], 72
    g, m = len(counts), sum(counts)
    seg, tiles = [0], [[0], [0]]
    for c in counts:
        seg.append(seg[-1] + c)
        tiles[0].append(tiles[0][-1] + -(-c // ops.GROUPED_TILE))
        tiles[1].append(tiles[1][-1] + -(-c // ops.GROUPED_TILE_MFMA))
    segments = (ints(seg), ints(tiles[0] + tiles[1]))
    x, w = dev(rnd(m, k, seed=55), torch.bfloat16), dev(rnd(g, n, k, seed=56, scale=0.2), torch.bfloat16)
    whole = ops.grouped_product(torch.empty((m, n), dtype=torch.float32, device=DEV), x, w, segments=segments)
    shares = ops.grouped_product(torch.full((parts, m, n), float("nan"), dtype=torch.float32, device=DEV), x, w,
                                 segments=segments, k_parts=parts)
    close(shares.sum(0), whole.double().cpu(), torch.float32, "shares of K", loose=5)
    place = ints(range(m))
    y = ops.moe_combine(torch.empty((m, n), dtype=torch.float32, device=DEV), shares, place)
    close(y, whole.double().cpu(), torch.float32, "added up by the sum over choices", loose=5)
    assert ops.grouped_k_parts(x, w) == min(4, 256 // 4, k // 512) or k < 512


# ------------------------------------------------------------------------------ experts
def test_the_largest_scores_are_chosen_and_a_tie_goes_to_the_lower_expert():
    from llmserve.ops import library as ops

    hidden, experts = 16, 9
    w = torch.zeros(experts, hidden, dtype=F64)
    w[:, 0] = torch.tensor([0.1, 0.9, 0.9, -0.5, 0.3, 0.9, -2.0, 0.0, 0.2])
    h = torch.zeros(3, hidden, dtype=F64)
    h[0, 0], h[1, 0], h[2, 0] = 1.0, -1.0, 0.0  # (all scores one half in the last row)
    for top in (1, 2, 4):
        chosen = torch.empty((3, top), dtype=torch.int32, device=DEV)
        weight = torch.empty((3, top), dtype=torch.float32, device=DEV)
        ops.moe_router(chosen, weight, dev(h), dev(w))
        assert chosen.cpu().tolist() == [[1, 2, 5, 4][:top], [6, 3, 7, 0][:top], [0, 1, 2, 3][:top]]
        scores = torch.sigmoid(h @ w.T)
        close(weight, torch.gather(scores, 1, chosen.cpu().long()), torch.float32, "weights are the scores, not renormalised")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("experts,top,ff,limit,rows", [(5, 2, 24, 1.25, 150), (3, 1, 40, 0.3, 1), (8, 8, 4, 5.0, 37),
                                                        (2, 1, 8, 1.0, 200)])
def test_experts_against_the_plain_sum(dtype, experts, top, ff, limit, rows):
    from llmserve.parts.experts import Experts
    from llmserve.parts.registry import BuildContext
    from llmserve.parts.spec import PartSpec

    hidden = 48
    part = Experts(PartSpec("experts", {"hidden": hidden, "intermediate": ff, "experts": experts, "top": top, "limit": limit}),
                   BuildContext(dtype, DEV))
    w = {name: rnd(*info.shape, seed=60 + i, scale=0.4).to(dtype) for i, (name, info) in enumerate(part.param_infos().items())}
    w["router"] = (torch.arange(experts, dtype=F64)[:, None] - experts / 2 + 0.37) * rnd(1, hidden, seed=59, scale=0.5)
    w["router"] = w["router"].to(dtype)  # (scores that lie far apart: a rounding does not change a choice)
    part.load({k: v.to(DEV) for k, v in w.items()})
    h = rnd(rows, hidden, seed=58).to(dtype)
    got = part.forward(h.to(DEV))
    assert got.dtype == torch.float32
    mlp = {"router": {"top": top, "experts": experts}, "expert": {"limit": limit, "ff": ff}}
    close(got, pm.moe_ff(h.double(), mlp, {k: v.double() for k, v in w.items()}), dtype, "experts", loose=4)


# ------------------------------------------------------------------------------ whole models
def write_model(folder, config, seed):
    from safetensors.torch import load_file

    from llmserve.weights import write_random_model

    # stored in bfloat16, so that both engines and the plain implementation hold the same numbers
    write_random_model(folder, config, seed=seed, dtype=torch.bfloat16, std=0.08, norm_std=0.05)
    return {k: v.double() for k, v in load_file(str(folder / "model.safetensors")).items()}


def logits_close(got, ref, dtype, what):
    """Per position: the difference of the logits (mean taken off, root mean square over the vocabulary) against the
    root mean square of the logits themselves.  32-bit: every position.  bfloat16: the median, and three positions
    in four (a token whose choice of experts was a close call, and all that attend to it, are off by more).
    `got` and `ref` may be lists of requests, which are then judged together."""
    if isinstance(got, (list, tuple)):
        scale = torch.cat([r.double().flatten() for r in ref]).pow(2).mean().sqrt()
        got, ref = torch.cat(list(got)), torch.cat(list(ref))
    else:
        scale = ref.double().pow(2).mean().sqrt()
    got, ref = got.double(), ref.double()
    assert got.shape == ref.shape and torch.isfinite(got).all(), what
    d = got - ref
    d = d - d.mean(dim=-1, keepdim=True)
    err = d.pow(2).mean(dim=-1).sqrt() / scale
    worst = int(err.argmax())
    if dtype == torch.float32:
        assert float(err.max()) <= 5e-5, f"{what}: position {worst} is off by {float(err.max()):.2e}"
    else:
        assert float(err.median()) <= 0.02, f"{what}: the median position is off by {float(err.median()):.2e}"
        over = int((err > 0.04).sum())
        assert over <= max(1, len(err) // 4), f"{what}: {over} of {len(err)} positions are off by more than 0.04 (worst {worst})"


MODELS = {"small": (SMALL, 8), "small_b": (SMALL_B, 16), "small_c": (SMALL_C, 4), "small_d": (SMALL_D, 8)}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for i, (name, (config, bs)) in enumerate(MODELS.items()):
        folder = tmp_path_factory.mktemp(f"milozen_{name}")
        out[name] = (folder, config, write_model(folder, config, seed=70 + i), bs)
    return out


def run_trace(runner, steps):
    from llmserve.engine.replay import Replayer

    rep, outputs = Replayer(runner), {}
    for rec in steps:
        out = rep.run(rec)
        runner.manager.check_invariants()
        if out.shape[0]:
            outputs[rec["step"]] = out.float().cpu()
    return traces.collect(steps, outputs)


def test_the_streams_after_every_layer(models):
    """Layer by layer against the plain implementation, in 32-bit: the sum of the streams after each layer."""
    from llmserve.config import EngineConfig
    from llmserve.engine.batch import build_batch
    from llmserve.engine.runner import ModelRunner

    folder, config, w, bs = models["small"]
    ids = traces.random_ids(config["vocab"], 45, 5)
    want = []
    pm.forward(config, w, ids, layers_out=want)
    runner = ModelRunner.from_folder(folder, EngineConfig(dtype="float32", block_size=bs, num_blocks=16, max_num_seqs=2,
                                                          use_graphs=False))
    runner.add_sequence("a")
    layout = runner.manager.append(["a"], [len(ids)])
    batch = build_batch(layout, [ids], [0], runner._uploader, runner.storage)
    model = runner.model
    x, delta = model.embedding.forward(batch.token_ids), None
    sources = model.cache_sources()
    for pos, index in enumerate(model.spec.schedule):
        x, delta = model.blocks[index].forward(x, delta, batch, runner.storage.layer_cache(pos, sources[pos]))
        c = delta.connection
        after = pm.streams_write(x.double().cpu().permute(1, 0, 2), delta.y.double().cpu(), c.mix.double().cpu(),
                                 c.write.double().cpu()).sum(0)
        close(after, want[pos], torch.float32, f"after layer {pos}")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(MODELS))
@pytest.mark.parametrize("graphs", [True, False])
def test_every_way_of_cutting_gives_the_plain_logits(models, name, dtype_name, graphs):
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner

    folder, config, w, bs = models[name]
    dtype = getattr(torch, dtype_name)
    seqs = {f"r{i}": traces.random_ids(config["vocab"], n, 300 + i) for i, n in enumerate([67, 1, 30, 41, 2, 75])}
    ref = {rid: pm.forward(config, w, ids) for rid, ids in seqs.items()}
    modes = {"whole": traces.whole(seqs), "decode": traces.prefill_then_decode(seqs, tail=40),
             "portions": traces.portions(seqs), "mixed": traces.mixed(seqs, seed=3, live_max=3)}
    for mode, steps in modes.items():
        pages = -(-traces.tokens_needed(steps, round_to=bs) // bs)
        runner = ModelRunner.from_folder(folder, EngineConfig(dtype=dtype_name, block_size=bs, num_blocks=pages,
                                                              max_num_seqs=3, use_graphs=graphs))
        assert runner._use_graphs == graphs  # every part of the model can be captured
        runner.storage.poison()
        got = run_trace(runner, steps)
        logits_close([got[rid] for rid in seqs], [ref[rid] for rid in seqs], dtype, f"{name} {mode} {dtype_name}")
        assert runner.manager.num_free_slots == 3
        assert all(a.num_free == pages for a in runner.manager.allocators.values())
        if graphs and mode == "decode":
            assert runner._graphs, "steps of single tokens were not replayed from a graph"


def test_a_batch_gives_each_request_what_it_gets_alone(models):
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner

    folder, config, _w, bs = models["small"]
    seqs = {f"b{i}": traces.random_ids(config["vocab"], n, 500 + i) for i, n in enumerate([50, 13, 29])}
    runner = ModelRunner.from_folder(folder, EngineConfig(dtype="float32", block_size=bs, num_blocks=64, max_num_seqs=3))
    alone = run_trace(runner, traces.portions(seqs))
    together = run_trace(runner, traces.mixed(seqs, seed=9, live_max=3))
    for rid in seqs:
        assert (alone[rid] - together[rid]).abs().max() <= 2e-5 * float(alone[rid].abs().max())


def test_long_decoding_on_a_pool_that_only_passed_pages_keep_alive(models):
    """280 tokens, most of them decoded one by one, on pools of 12 pages of 8: the request fits only because the
    pages behind the widest window among a cache's readers come back while it runs."""
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner

    folder, config, w, bs = models["small"]
    ids = traces.random_ids(config["vocab"], 280, 77)
    ref = pm.forward(config, w, ids)
    for graphs in (True, False):
        runner = ModelRunner.from_folder(folder, EngineConfig(dtype="float32", block_size=bs, num_blocks=12,
                                                              max_num_seqs=2, use_graphs=graphs))
        runner.storage.poison()
        got = run_trace(runner, traces.prefill_then_decode({"long": ids}, tail=250))
        logits_close(got["long"], ref, torch.float32, "long decoding")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(models, dtype_name):
    from llmserve import LLM, EngineConfig, SamplingParams

    folder, config, w, bs = models["small_d"]
    prompts = [traces.random_ids(config["vocab"], n, 600 + i) for i, n in enumerate([19, 3, 33, 8, 1])]
    llm = LLM(folder, dtype=dtype_name, engine=EngineConfig(block_size=bs, num_blocks=40, max_num_seqs=3,
                                                            max_num_batched_tokens=16))
    assert llm.runner.takes_device_tokens  # decode steps are replayed graphs, fed from the sampler's ids
    results = llm.generate(prompts, SamplingParams(max_new_tokens=24))
    for prompt, result in zip(prompts, results):
        assert len(result.tokens) == 24
        if dtype_name == "float32":
            assert result.tokens == pm.greedy(config, w, prompt, 24)
        else:  # a tie may fall either way in bfloat16: nearly every token must be near the top of the plain logits
            ref = pm.forward(config, w, prompt + result.tokens)
            far = 0
            for i, tok in enumerate(result.tokens):
                row = ref[len(prompt) - 1 + i]
                far += float(row.max() - row[tok]) > 0.08 * float(ref.pow(2).mean().sqrt()) + 1e-3
            assert far <= 2
    assert llm.runner.manager.num_free_slots == 3


def test_named_sizes_run_from_the_command_line_entry(capsys):
    from llmserve.cli import main

    assert main(["--model", "milozen-tiny", "--random-weights", "--max-new-tokens", "5", "--dtype", "float32"]) == 0
    assert "decode=" in capsys.readouterr().out


def drawn_config(seed: int) -> tuple[dict, int]:
    """A configuration drawn at random from what config.json allows: 1 to 4 streams or none, dense layers, layers of
    experts and layers without feed-forward in any order, layers that read an earlier layer's cache rows with a
    window of their own, 1 to 7 heads, sizes from 2 up, a rotation over all or part of the rotated dimensions,
    windows from one key up or none; and a page size."""
    import random

    rng = random.Random(seed)
    layers = []
    owners = []
    for i in range(rng.randint(2, 6)):
        mask = {} if rng.random() < 0.15 else {"size": rng.choice([1, 2, 7, 16, 33, 64, 150])}
        if owners and rng.random() < 0.35:
            mixer = {"kv_from": rng.choice(owners), "heads": rng.randint(1, 7), "dim": rng.choice([4, 8, 12, 16, 32]),
                     "vdim": rng.choice([4, 8, 24, 32]), "q_rank": rng.choice([8, 24, 48]), "mask": mask,
                     "scale": rng.choice([0.1, 0.2, 0.35])}
        else:
            rot_dim = rng.choice([2, 4, 8, 16, 32])
            mixer = {"heads": rng.randint(1, 7), "dim": rng.choice([4, 8, 12, 16, 32]), "rot_dim": rot_dim,
                     "vdim": rng.choice([4, 8, 24, 32]), "q_rank": rng.choice([8, 24, 48]),
                     "kv_rank": rng.choice([8, 20, 32, 64, 100]), "scale": rng.choice([0.1, 0.2, 0.35]), "mask": mask,
                     "rot": {"base": rng.choice([10.0, 10000.0, 500000.0]), "dims": rng.choice([rot_dim, max(2, rot_dim // 2)])}}
            owners.append(i)
        kind = rng.random()
        if kind < 0.2:
            mlp = None
        elif kind < 0.45:
            mlp = {"kind": "dense", "ff": rng.choice([24, 64, 120])}
        else:
            experts = rng.randint(2, 9)
            mlp = moe(experts=experts, top=rng.randint(1, min(experts, 4)), ff=rng.choice([8, 24, 40]),
                      limit=rng.choice([0.5, 1.25, 7.0]))
        layers.append({"mixer": mixer, "mlp": mlp})
    return config_of(width=rng.choice([40, 64, 72, 100]), vocab=rng.choice([61, 128, 257]), scale=rng.choice([0.5, 1.0, 12.0]),
                     eps=rng.choice([1e-6, 1e-5]), streams=rng.choice([None, 1, 2, 3, 4]), layers=layers), rng.choice([4, 8, 16])


@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_at_random(tmp_path, seed):
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner

    config, bs = drawn_config(seed)
    w = write_model(tmp_path, config, seed=900 + seed)
    seqs = {f"q{i}": traces.random_ids(config["vocab"], n, 40 * seed + i) for i, n in enumerate([90, 3, 47, 160, 18])}
    ref = {rid: pm.forward(config, w, ids) for rid, ids in seqs.items()}
    for dtype_name in ("float32", "bfloat16"):
        steps = traces.mixed(seqs, seed=seed, live_max=3, tail=30)
        pages = -(-traces.tokens_needed(steps, round_to=bs) // bs)
        runner = ModelRunner.from_folder(tmp_path, EngineConfig(dtype=dtype_name, block_size=bs, num_blocks=pages,
                                                                max_num_seqs=3))
        runner.storage.poison()
        got = run_trace(runner, steps)
        logits_close([got[rid] for rid in seqs], [ref[rid] for rid in seqs], getattr(torch, dtype_name),
                     f"seed {seed} {dtype_name}: {config['layers']}")
        assert runner.manager.num_free_slots == 3
        assert all(a.num_free == pages for a in runner.manager.allocators.values())
