"""Dibepel on the GPU against the plain implementation (tests/plain_dibepel.py, float64 on the CPU):
each mechanism alone, then whole models of small made-up sizes in every way of cutting a request into steps,
with pages and state slots that are freed and used again, and greedy generation through the entry point."""

import math

import pytest
import torch

import plain_dibepel as pd
import traces
from dibepel_configs import SMALL, SMALL_B, SMALL_C, config_of

pytestmark = pytest.mark.gpu

DEV = torch.device("cuda:0")
DTYPES = [torch.float32, torch.bfloat16]
F64 = torch.float64


def rnd(*shape, seed=0, scale=1.0):
    return scale * torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64)


def close(got, ref, dtype, what=""):
    """32-bit: the order of sums differs; bfloat16: single roundings of operands and results."""
    got, ref = got.double().cpu(), ref.double()
    assert got.shape == ref.shape, f"{what}: {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{what}: not finite"
    scale = max(1e-6, float(ref.abs().max()))
    worst = float((got - ref).abs().max()) / scale
    assert worst <= (2.0 ** -5 if dtype == torch.bfloat16 else 2e-5), f"{what}: off by {worst:.2e} of the largest value"


# ------------------------------------------------------------------------------ the 32-bit stream's kernels
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [100, 98, 2048])  # rows of a multiple of 4 go to the kernels that read 16 bytes a thread
def test_scaled_embedding_norm_and_gated_sum(dtype, hidden):
    from llmserve.ops import library as ops

    table = rnd(50, 72, seed=1).to(dtype)
    ids = torch.tensor([0, 49, 7, 7], dtype=torch.int32)
    x = ops.embed_scale(torch.empty(4, 72, device=DEV), table.to(DEV), ids.to(DEV), 1.7)
    close(x, table.double()[ids.long()] * 1.7, torch.float32, "embedding")

    stream = rnd(6, hidden, seed=2).float()
    w = rnd(hidden, seed=3, scale=0.2).float()
    out = ops.rmsnorm32(torch.empty(6, hidden, dtype=dtype, device=DEV), stream.to(DEV), w.to(DEV), 1e-5, 1.0)
    close(out, pd.norm_zero_centred(stream.double(), w.double(), 1e-5), dtype, "norm")
    rows = torch.tensor([4, 0], dtype=torch.int32, device=DEV)
    out = ops.rmsnorm32(torch.empty(2, hidden, dtype=dtype, device=DEV), stream.to(DEV), w.to(DEV), 1e-5, 1.0, rows=rows)
    close(out, pd.norm_zero_centred(stream.double(), w.double(), 1e-5)[[4, 0]], dtype, "norm of rows")

    z, a, f = rnd(6, 2 * hidden, seed=4).float(), rnd(6, hidden, seed=5).float(), rnd(6, hidden, seed=6).float()
    b1, b2 = rnd(hidden, seed=7).float(), rnd(hidden, seed=8).float()
    ref = stream.double() + torch.sigmoid(z[:, :hidden].double() + b1.double()) * a.double() \
        + torch.sigmoid(z[:, hidden:].double() + b2.double()) * f.double()
    got = ops.gated_add(stream.clone().to(DEV), [(a.to(DEV), 0, b1.to(DEV)), (f.to(DEV), hidden, b2.to(DEV))], z.to(DEV))
    close(got, ref, torch.float32, "two gated branches")
    got = ops.gated_add(stream.clone().to(DEV), [(a.to(DEV), None, None)])
    close(got, stream.double() + a.double(), torch.float32, "one branch without a gate")
    ref = stream.double() + a.double() + torch.sigmoid(z[:, hidden:].double() + b2.double()) * f.double()
    got = ops.gated_add(stream.clone().to(DEV), [(a.to(DEV), None, None), (f.to(DEV), hidden, b2.to(DEV))], z.to(DEV))
    close(got, ref, torch.float32, "a plain branch beside a gated one")
    # the sum and the norm of the summed rows in one kernel (rows that are no multiple of 4: one after the other)
    summed = stream.clone().to(DEV)
    out = ops.gated_add_norm(torch.empty(6, hidden, dtype=dtype, device=DEV), summed,
                             [(a.to(DEV), None, None), (f.to(DEV), hidden, b2.to(DEV))], z.to(DEV), w.to(DEV), 1e-5, 1.0)
    close(summed, ref, torch.float32, "the summed rows")
    close(out, pd.norm_zero_centred(ref, w.double(), 1e-5), dtype, "their norm")
    many = ops.GATED_ADD_NORM_ROWS + 3  # beyond this many rows: two kernels
    big, ya = rnd(many, hidden, seed=9).float(), rnd(many, hidden, seed=10).float()
    summed = big.clone().to(DEV)
    out = ops.gated_add_norm(torch.empty(many, hidden, dtype=dtype, device=DEV), summed, [(ya.to(DEV), None, None)], None,
                             w.to(DEV), 1e-5, 1.0)
    close(out, pd.norm_zero_centred(big.double() + ya.double(), w.double(), 1e-5), dtype, "many rows")


# ------------------------------------------------------------------------------ convolution, state and cache store
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [1, 2, 4])
def test_short_convolution_in_portions_with_state_and_store(dtype, taps):
    """Two requests whose portions alternate, down to single tokens: queries, and keys and values read back from
    their pages, must be the convolution of the whole sequences."""
    from llmserve.ops import library as ops

    kh, dk, vh, dv, cq, bs = 2, 8, 1, 12, 24, 4
    channels = cq + kh * dk + vh * dv
    lens = [23, 9]
    u = [rnd(n, channels, seed=10 + i).float() for i, n in enumerate(lens)]
    w = rnd(channels, taps, seed=12).float()
    ref = [pd.short_conv(x.double(), w.double()) for x in u]
    state = torch.full((3, max(taps - 1, 1), channels), float("nan"), device=DEV)[:, : taps - 1].contiguous()
    state[[2, 0]] = 0  # request 0 owns slot 2, request 1 slot 0; slot 1 stays poisoned
    k_pool = torch.full((12, kh, bs, dk), float("nan"), dtype=dtype, device=DEV)
    v_pool = torch.full((12, vh, dv, bs), float("nan"), dtype=dtype, device=DEV)
    pages = [[7, 2, 9, 0, 4, 11], [5, 1, 8]]
    slot_of = [2, 0]
    done = [0, 0]
    got_q = [[], []]
    steps = [{0: 5}, {0: 1, 1: 2}, {1: 1}, {0: 2, 1: 1}, {0: 1}, {0: 14, 1: 5}]
    for step in steps:
        ids = sorted(step)
        rows = torch.cat([u[b][done[b]: done[b] + step[b]] for b in ids]).to(DEV)
        pos, seq, cu, slots = [], [], [0], []
        for i, b in enumerate(ids):
            for p in range(done[b], done[b] + step[b]):
                pos.append(p)
                seq.append(i)
                slots.append(pages[b][p // bs] * bs + p % bs)
            cu.append(cu[-1] + step[b])
        as_i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)  # noqa: E731
        state_slots = as_i32([slot_of[b] for b in ids])
        q = torch.empty((rows.shape[0], cq), dtype=dtype, device=DEV)
        ops.conv_store(q, rows, cq=cq, k_heads=kh, dk=dk, v_heads=vh, dv=dv, taps_w=w.to(DEV),
                       state=state if taps > 1 else None, state_slots=state_slots if taps > 1 else None,
                       token_seq=as_i32(seq), positions=as_i32(pos), cu_seqlens=as_i32(cu), slots=as_i32(slots),
                       k_pool=k_pool, v_pool=v_pool, block_size=bs)
        if taps > 1:
            ops.conv_state(state, rows, state_slots, as_i32(cu), as_i32([done[b] + step[b] for b in ids]))
        row = 0
        for b in ids:
            got_q[b].append(q[row: row + step[b]].cpu())
            row += step[b]
            done[b] += step[b]
    for b, n in enumerate(lens):
        close(torch.cat(got_q[b]), ref[b][:, :cq], dtype, f"queries of request {b}")
        k = torch.stack([k_pool[pages[b][p // bs], :, p % bs] for p in range(n)]).reshape(n, -1)
        v = torch.stack([v_pool[pages[b][p // bs], :, :, p % bs] for p in range(n)]).reshape(n, -1)
        close(k, ref[b][:, cq: cq + kh * dk], dtype, f"keys of request {b}")
        close(v, ref[b][:, cq + kh * dk:], dtype, f"values of request {b}")
    if taps > 1:
        assert torch.isnan(state[1]).all()  # nobody's slot was touched


# ------------------------------------------------------------------------------ the attention kernel alone
def paged(k, v, bs, dtype, seed=0):
    """k [t, Hk, dk], v [t, Hv, dv] -> pools in shuffled pages (unused slots NaN) and the request's block table."""
    t = k.shape[0]
    need = -(-t // bs)
    order = torch.randperm(need + 3, generator=torch.Generator().manual_seed(seed)).tolist()
    k_pool = torch.full((need + 3, k.shape[1], bs, k.shape[2]), float("nan"), dtype=dtype)
    v_pool = torch.full((need + 3, v.shape[1], v.shape[2], bs), float("nan"), dtype=dtype)
    table = torch.zeros((1, need), dtype=torch.int32)
    for i in range(need):
        page = order[i]
        table[0, i] = page
        n = min(bs, t - i * bs)
        k_pool[page, :, :n] = k[i * bs: i * bs + n].transpose(0, 1).to(dtype)
        v_pool[page, :, :, :n] = v[i * bs: i * bs + n].permute(1, 2, 0).to(dtype)
    return k_pool.to(DEV), v_pool.to(DEV), table.to(DEV)


def attend(q, k, v, dtype, bs, rows=None, **kw):
    """The kernel on a whole sequence (every position a query, or `rows`): q [t, S, dk] -> [rows, H * dv]."""
    from llmserve.ops import library as ops

    t = q.shape[0]
    rows = list(range(t)) if rows is None else rows
    k_pool, v_pool, table = paged(k, v, bs, dtype)
    qd = q[rows].reshape(len(rows), -1).to(dtype).to(DEV)
    heads, dv = kw["heads"], v.shape[2]
    out = torch.empty((len(rows), heads * dv), dtype=dtype, device=DEV)
    ops.attend_composed(out, qd, k_pool, v_pool, table, torch.zeros(len(rows), dtype=torch.int32, device=DEV),
                        torch.tensor(rows, dtype=torch.int32, device=DEV), dk=q.shape[2], dv=dv, block_size=bs, **kw)
    return out


def rounded(x, dtype):
    return x.to(dtype).double()


DIFF_CASES = [  # heads, kv_heads, dk, dv, window, keep_first, block size
    (2, 1, 24, 16, 9, 4, 8),
    (4, 4, 8, 8, 5, 0, 4),
    (3, 1, 8, 24, 6, 11, 16),
    (2, 2, 10, 6, None, 0, 8),  # sizes that are no multiple of 8: rows are read element by element
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv,dk,dv,window,keep,bs", DIFF_CASES)
def test_two_score_maps_window_and_kept_tokens(dtype, heads, kv, dk, dv, window, keep, bs):
    t = 45
    q, k, v = rnd(t, heads, 2, dk, seed=20), rnd(t, kv, 2, dk, seed=21), rnd(t, kv, dv, seed=22)
    q, k, v = (rounded(x, dtype) for x in (q, k, v))
    lam, diff, eps, scale = 0.83, 0.3, 1e-5, 0.37
    ref = pd.differential_heads(q, k, v, pd.visible_window(t, window, keep), scale, lam, diff, eps)
    got = attend(q.reshape(t, heads * 2, dk), k.reshape(t, kv * 2, dk), v, dtype, bs, heads=heads, kv_heads=kv, maps=2,
                 window=window or 0, keep_first=keep, scale=scale, lam=lam, head_norm=True, eps=eps, out_scale=1 - diff)
    close(got, ref.reshape(t, -1), dtype, "differential attention")


TALK_CASES = [  # heads, kv_heads, dk, dv, chunk, block size
    (4, 2, 16, 24, 12, 8),
    (3, 3, 8, 8, 7, 4),
    (2, 1, 16, 8, 16, 16),
    (5, 5, 12, 20, 3, 8),
    (6, 2, 8, 8, None, 8),  # no chunks: every earlier key, more than one tile of them
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv,dk,dv,chunk,bs", TALK_CASES)
def test_chunks_distance_slopes_and_mixed_heads(dtype, heads, kv, dk, dv, chunk, bs):
    t = 90
    q, k, v = (rounded(x, dtype) for x in (rnd(t, heads, dk, seed=30), rnd(t, kv, dk, seed=31), rnd(t, kv, dv, seed=32)))
    talk = torch.eye(heads, dtype=F64) + rnd(heads, heads, seed=33, scale=0.3)
    slopes = pd.distance_slopes(heads)
    ref = pd.talking_heads(q, k, v, pd.visible_chunk(t, chunk), 0.3, slopes, talk)
    got = attend(q, k, v, dtype, bs, heads=heads, kv_heads=kv, chunk=chunk or 0, scale=0.3,
                 slopes=slopes.float().to(DEV), talk=talk.float().to(DEV))
    close(got, ref.reshape(t, -1), dtype, "mixed heads")
    # each ingredient alone
    ref = pd.talking_heads(q, k, v, pd.visible_chunk(t, chunk), 0.3, None, None)
    close(attend(q, k, v, dtype, bs, heads=heads, kv_heads=kv, chunk=chunk or 0, scale=0.3), ref.reshape(t, -1), dtype,
          "chunks alone")
    ref = pd.talking_heads(q, k, v, pd.visible_chunk(t, None), 0.3, slopes, None)
    close(attend(q, k, v, dtype, bs, heads=heads, kv_heads=kv, scale=0.3, slopes=slopes.float().to(DEV)),
          ref.reshape(t, -1), dtype, "slopes alone")


def test_a_key_that_stands_out_shows_every_edge():
    """One key is made to carry nearly all the weight of one query; its value is a marker.  Just inside a window, a
    chunk or the kept first tokens the marker must come out, just outside it must be gone; also far back, and where
    the key lies on a page's border."""
    t, dk, dv, bs = 300, 16, 16, 16
    g = torch.Generator().manual_seed(5)
    q = torch.randn(t, 1, dk, generator=g, dtype=F64)
    k = torch.randn(t, 1, dk, generator=g, dtype=F64)
    v = 0.01 * torch.randn(t, 1, dv, generator=g, dtype=F64)

    def marked(i, j):
        kk, vv = k.clone(), v.clone()
        kk[j, 0] = 40.0 * q[i, 0] / q[i, 0].norm() ** 2 * dk ** 0.5  # score 40 at scale 1/sqrt(dk)
        vv[j, 0] = 7.0
        return kk, vv

    def marker_seen(i, j, **kw):
        """By the kernel for any size (32-bit, the query alone) and by the matrix-core kernel (bfloat16), there both as
        a request's only new token and as the last token of a whole prompt: all three must agree."""
        kk, vv = marked(i, j)
        out = attend(q, kk, vv, torch.float32, bs, rows=[i], heads=1, kv_heads=1, scale=dk ** -0.5, **kw)
        seen = float(out[0, 0]) > 3.5
        cut = (q[: i + 1], kk[: i + 1], vv[: i + 1])
        decoded = attend_mfma([(*cut, i, 1)], bs, heads=1, kv_heads=1, scale=dk ** -0.5, **kw)[0]
        prompt = attend_mfma([(*cut, 0, i + 1)], bs, heads=1, kv_heads=1, scale=dk ** -0.5, **kw)[0]
        assert (float(decoded[0, 0]) > 3.5) == seen and (float(prompt[-1, 0]) > 3.5) == seen, (i, j, kw)
        return seen

    window, keep, chunk = 40, 20, 64
    for i in (40, 63, 64, 200, 299):
        assert marker_seen(i, i - window + 1, window=window, keep_first=keep)  # the window's last key
        if i - window >= keep:
            assert not marker_seen(i, i - window, window=window, keep_first=keep)  # one further back
        assert marker_seen(i, keep - 1, window=window, keep_first=keep)  # the last kept token
        assert marker_seen(i, 0, window=window, keep_first=keep)
        if i - window >= keep:
            assert not marker_seen(i, keep, window=window, keep_first=keep)  # the first one not kept
    assert marker_seen(30, 25, window=window, keep_first=keep)  # before the window has passed anything
    for i in (63, 64, 65, 127, 128, 255, 299):
        start = i // chunk * chunk
        assert marker_seen(i, start, chunk=chunk)  # the chunk's first key
        if start:
            assert not marker_seen(i, start - 1, chunk=chunk)  # the chunk before
            assert not marker_seen(i, 0, chunk=chunk)
        assert marker_seen(i, i, chunk=chunk)  # a chunk's first query sees itself
    assert marker_seen(299, 3)  # no mask: a key far back among hundreds
    assert marker_seen(299, 15) and marker_seen(299, 16)  # a page's last and first slot
    # with slopes the far key pays for its distance: slope 1/4 over 200 positions outweighs a score of 40
    slope = torch.tensor([0.25], device=DEV)
    assert not marker_seen(299, 99, slopes=slope) and marker_seen(299, 290, slopes=slope)


# ------------------------------------------------------------------------------ the matrix-core kernel
def attend_mfma(seqs, bs, shares=1, **kw):
    """`seqs`: per request (q [t, S, dk], k, v, first new row, number of new rows); requests that bring one row
    first.  All share one pool.  Returns the kernel's rows per request."""
    from llmserve.ops import library as ops

    dt = torch.bfloat16
    pools = [paged(k, v, bs, dt, seed=i) for i, (_q, k, v, _a, _n) in enumerate(seqs)]
    k_pool = torch.cat([p[0] for p in pools])
    v_pool = torch.cat([p[1] for p in pools])
    width = max(p[2].shape[1] for p in pools)
    table = torch.zeros((len(seqs) + 2, width), dtype=torch.int32, device=DEV)
    rows_of = [len(seqs) + 1 - i for i in range(len(seqs))]  # (a request's row of the table is not its index)
    base = 0
    for i, p in enumerate(pools):
        table[rows_of[i], : p[2].shape[1]] = p[2][0] + base
        base += p[0].shape[0]
    qs = torch.cat([q[a: a + n].reshape(n, -1) for q, _k, _v, a, n in seqs]).to(dt).to(DEV)
    cu = [0]
    for *_x, n in seqs:
        cu.append(cu[-1] + n)
    as_i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)  # noqa: E731
    heads, dv = kw["heads"], seqs[0][2].shape[2]
    out = torch.full((qs.shape[0], heads * dv), float("nan"), dtype=dt, device=DEV)
    n_dec = sum(1 for *_x, n in seqs if n == 1)
    args = (out, qs, k_pool, v_pool, table, as_i32(cu), as_i32([a + n for *_x, a, n in seqs]))
    common = dict(dk=seqs[0][0].shape[2], dv=dv, block_size=bs, table_rows=as_i32(rows_of), **kw)
    if n_dec:
        ops.attend_composed_mfma(*args, 0, n_dec, 1, shares=shares, **common)
    if n_dec < len(seqs):
        ops.attend_composed_mfma(*args, n_dec, len(seqs) - n_dec, max(n for *_x, n in seqs), shares=shares, **common)
    return [out[cu[i]: cu[i + 1]] for i in range(len(seqs))]


MFMA_DIFF = [  # heads, kv_heads, dk, dv, window, keep_first, block size
    (2, 1, 32, 16, 11, 6, 8),
    (4, 4, 16, 48, 40, 20, 16),
    (16, 2, 64, 128, 33, 0, 16),
    (3, 1, 16, 16, None, 0, 4),  # three heads in a unit of 16 columns: five tokens and a padded column
    (16, 1, 16, 32, 21, 3, 8),  # sixteen heads on one key/value head: a unit is one token
    (2, 1, 128, 128, 50, 9, 16),  # the widest keys and values the kernel takes
    (4, 4, 128, 64, 1000, 0, 16),
    (8, 2, 96, 112, 37, 20, 8),
]


@pytest.mark.parametrize("heads,kv,dk,dv,window,keep,bs", MFMA_DIFF)
def test_matrix_core_kernel_two_maps(heads, kv, dk, dv, window, keep, bs):
    dt = torch.bfloat16
    lam, diff, eps, scale = 0.83, 0.3, 1e-5, 0.3
    seqs, refs = [], []
    for i, (t, first, n) in enumerate([(71, 70, 1), (150, 149, 1), (90, 0, 90), (58, 33, 25), (40, 38, 2)]):
        q, k, v = (rounded(x, dt) for x in (rnd(t, heads, 2, dk, seed=60 + i), rnd(t, kv, 2, dk, seed=70 + i),
                                            rnd(t, kv, dv, seed=80 + i)))
        ref = pd.differential_heads(q, k, v, pd.visible_window(t, window, keep), scale, lam, diff, eps)
        refs.append(ref.reshape(t, -1)[first: first + n])
        seqs.append((q.reshape(t, heads * 2, dk), k.reshape(t, kv * 2, dk), v, first, n))
    got = attend_mfma(seqs, bs, heads=heads, kv_heads=kv, maps=2, window=window or 0, keep_first=keep, scale=scale,
                      lam=lam, head_norm=True, eps=eps, out_scale=1 - diff)
    for i, (g, r) in enumerate(zip(got, refs)):
        close(g, r, dt, f"request {i}")


MFMA_TALK = [  # heads, kv_heads, dk, dv, chunk, block size
    (4, 2, 16, 32, 20, 8),
    (8, 1, 16, 16, 64, 16),
    (3, 3, 16, 16, 9, 8),
    (32, 4, 64, 64, 128, 16),
    (32, 32, 32, 128, None, 16),  # two units a wave
    (6, 2, 16, 16, 50, 4),
    (16, 1, 32, 16, 40, 8),  # a unit is one token
    (24, 24, 16, 16, 30, 16),  # 24 units in 12 waves
    (4, 2, 128, 128, 70, 16),  # the widest keys and values the kernel takes
    (20, 20, 128, 128, 64, 16),  # ... with two units a wave
    (8, 4, 80, 96, 33, 8),
]


@pytest.mark.parametrize("heads,kv,dk,dv,chunk,bs", MFMA_TALK)
def test_matrix_core_kernel_mixed_heads(heads, kv, dk, dv, chunk, bs):
    dt = torch.bfloat16
    talk = torch.eye(heads, dtype=F64) + rnd(heads, heads, seed=33, scale=0.3 / heads ** 0.5)
    slopes = pd.distance_slopes(heads)
    seqs, refs = [], []
    for i, (t, first, n) in enumerate([(71, 70, 1), (130, 129, 1), (90, 0, 90), (58, 33, 25), (40, 38, 2)]):
        q, k, v = (rounded(x, dt) for x in (rnd(t, heads, dk, seed=60 + i), rnd(t, kv, dk, seed=70 + i),
                                            rnd(t, kv, dv, seed=80 + i)))
        ref = pd.talking_heads(q, k, v, pd.visible_chunk(t, chunk), 0.3, slopes, talk)
        refs.append(ref.reshape(t, -1)[first: first + n])
        seqs.append((q, k, v, first, n))
    got = attend_mfma(seqs, bs, heads=heads, kv_heads=kv, chunk=chunk or 0, scale=0.3, slopes=slopes.float().to(DEV),
                      talk=talk.float().to(DEV))
    for i, (g, r) in enumerate(zip(got, refs)):
        close(g, r, dt, f"request {i}")
    # every request's keys shared out to several workgroups: single tokens and portions of prompts alike
    for shares in (2, 5):
        got = attend_mfma(seqs, bs, shares=shares, heads=heads, kv_heads=kv, chunk=chunk or 0, scale=0.3,
                          slopes=slopes.float().to(DEV), talk=talk.float().to(DEV))
        for i, (g, r) in enumerate(zip(got, refs)):
            close(g, r, dt, f"request {i} in {shares} shares")
    got = attend_mfma(seqs[2:3], bs, heads=heads, kv_heads=kv, chunk=chunk or 0, scale=0.3)  # neither slopes nor mixing
    ref = pd.talking_heads(seqs[2][0].double(), seqs[2][1].double(), seqs[2][2].double(), pd.visible_chunk(90, chunk), 0.3,
                           None, None)
    close(got[0], ref.reshape(90, -1), dt, "plain")


# ------------------------------------------------------------------------------ whole models
def write_model(folder, config, seed):
    from safetensors.torch import load_file

    from llmserve.weights import write_random_model

    # weights large enough for attention to have favourites and for gates to leave one half; stored in bfloat16, so
    # that both engines and the plain implementation hold the same numbers and only the arithmetic differs
    write_random_model(folder, config, seed=seed, dtype=torch.bfloat16, std=0.08, norm_std=0.02)
    return {k: v.double() for k, v in load_file(str(folder / "model.safetensors")).items()}


def logits_close(got, ref, dtype, what):
    """Per position: the difference of the logits (mean taken off, root mean square over the vocabulary) against the
    root mean square of the logits themselves."""
    got, ref = got.double(), ref.double()
    assert got.shape == ref.shape and torch.isfinite(got).all(), what
    d = got - ref
    d = d - d.mean(dim=-1, keepdim=True)
    err = d.pow(2).mean(dim=-1).sqrt() / ref.pow(2).mean().sqrt()
    limit = 0.03 if dtype == torch.bfloat16 else 5e-5
    worst = int(err.argmax())
    assert float(err.max()) <= limit, f"{what}: position {worst} is off by {float(err.max()):.2e} (limit {limit})"


MODELS = {"small": (SMALL, 8), "small_b": (SMALL_B, 16), "small_c": (SMALL_C, 8)}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for i, (name, (config, bs)) in enumerate(MODELS.items()):
        folder = tmp_path_factory.mktemp(f"dibepel_{name}")
        out[name] = (folder, config, write_model(folder, config, seed=40 + i), bs)
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


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(MODELS))
@pytest.mark.parametrize("graphs", [True, False])
def test_every_way_of_cutting_gives_the_plain_logits(models, name, dtype_name, graphs):
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner

    folder, config, w, bs = models[name]
    dtype = getattr(torch, dtype_name)
    vocab = config["vocab"]
    seqs = {f"r{i}": traces.random_ids(vocab, n, 300 + i) for i, n in enumerate([67, 1, 30, 41, 2, 75])}
    ref = {rid: pd.forward(config, w, ids) for rid, ids in seqs.items()}
    modes = {"whole": traces.whole(seqs), "decode": traces.prefill_then_decode(seqs, tail=40),
             "portions": traces.portions(seqs), "mixed": traces.mixed(seqs, seed=3, live_max=3)}
    for mode, steps in modes.items():
        pages = -(-traces.tokens_needed(steps, round_to=bs) // bs)
        runner = ModelRunner.from_folder(folder, EngineConfig(dtype=dtype_name, block_size=bs, num_blocks=pages,
                                                              max_num_seqs=3, use_graphs=graphs))
        assert runner._use_graphs == graphs  # every part of the model can be captured
        runner.storage.poison()
        got = run_trace(runner, steps)
        for rid in seqs:
            logits_close(got[rid], ref[rid], dtype, f"{name} {mode} {rid} {dtype_name}")
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
    pages behind the window and of passed chunks come back while it runs, and the kept first tokens stay."""
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner

    folder, config, w, bs = models["small"]
    ids = traces.random_ids(config["vocab"], 280, 77)
    ref = pd.forward(config, w, ids)
    for graphs in (True, False):
        runner = ModelRunner.from_folder(folder, EngineConfig(dtype="float32", block_size=bs, num_blocks=12,
                                                              max_num_seqs=2, use_graphs=graphs))
        runner.storage.poison()
        steps = traces.prefill_then_decode({"long": ids}, tail=250)
        got = run_trace(runner, steps)
        logits_close(got["long"], ref, torch.float32, "long decoding")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(models, dtype_name):
    from llmserve import LLM, EngineConfig, SamplingParams

    folder, config, w, bs = models["small_b"]
    prompts = [traces.random_ids(config["vocab"], n, 600 + i) for i, n in enumerate([19, 3, 33, 8, 1])]
    llm = LLM(folder, dtype=dtype_name, engine=EngineConfig(block_size=bs, num_blocks=24, max_num_seqs=3,
                                                            max_num_batched_tokens=16))
    assert llm.runner.takes_device_tokens  # decode steps are replayed graphs, fed from the sampler's ids
    results = llm.generate(prompts, SamplingParams(max_new_tokens=24))
    for prompt, result in zip(prompts, results):
        assert len(result.tokens) == 24
        if dtype_name == "float32":
            assert result.tokens == pd.greedy(config, w, prompt, 24)
        else:  # a tie may fall either way in bfloat16: every token must be near the top of the plain logits
            ref = pd.forward(config, w, prompt + result.tokens)
            for i, tok in enumerate(result.tokens):
                row = ref[len(prompt) - 1 + i]
                assert float(row.max() - row[tok]) <= 0.05 * float(ref.pow(2).mean().sqrt()) + 1e-3
    assert llm.runner.manager.num_free_slots == 3


def test_named_sizes_run_from_the_command_line_entry(capsys):
    from llmserve.cli import main

    assert main(["--model", "dibepel-tiny", "--random-weights", "--max-new-tokens", "5", "--dtype", "float32"]) == 0
    assert "decode=" in capsys.readouterr().out


def drawn_config(seed: int) -> tuple[dict, int]:
    """A configuration drawn at random from what config.json allows: layer kinds in any order, some layers on
    another's tensors, some without feed-forward, 1 to 16 query heads per key/value head, key and value sizes that
    the matrix-core kernel takes (multiples of 16) and that it does not, windows, kept tokens and chunks from 1 key
    up, 1 to 5 taps; and a page size."""
    import random

    rng = random.Random(seed)
    sizes = [8, 16, 16, 24, 32, 40, 48, 64]
    layers = []
    for i in range(rng.randint(2, 5)):
        kind = rng.choice(["attention", "attention_2"])
        kv = rng.choice([1, 1, 2, 3, 4])
        heads = kv * rng.choice([1, 1, 2, 4, 8, 16] if kv == 1 else [1, 2, 3])
        mixer = {"heads": heads, "kv_heads": kv, "dim": rng.choice(sizes), "vdim": rng.choice(sizes),
                 "scale": rng.choice([0.1, 0.2, 0.35])}
        if kind == "attention":
            mixer["diff"] = rng.choice([0.0, 0.2, 0.5, 0.8])
            mixer["mask"] = {} if rng.random() < 0.15 else {"size": rng.choice([1, 2, 7, 16, 33, 64]),
                                                            "keep_first": rng.choice([0, 1, 5, 16, 40])}
        else:
            mixer["conv"] = rng.randint(1, 5)
            mixer["mask"] = {} if rng.random() < 0.15 else {"size": rng.choice([1, 3, 16, 31, 64, 100])}
        changes = {"mixer": mixer}
        if rng.random() < 0.25:
            changes["mlp"] = None
        layers.append((kind, changes))
    for _ in range(rng.randint(0, 3)):  # further runs of earlier layers, appended (so no index moves)
        src = rng.randrange(len(layers))
        layers.append((layers[src][0], {"weights_of": src}))  # (a layer that itself runs on another's tensors makes a chain)
    width = rng.choice([40, 64, 72, 100])
    return config_of(width=width, vocab=rng.choice([61, 128, 257]), scale=rng.choice([0.5, 1.0, 2.5]),
                     eps=rng.choice([1e-6, 1e-5]), ff=rng.choice([24, 64, 120]), layers=layers), rng.choice([4, 8, 16])


@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_at_random(tmp_path, seed):
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner

    config, bs = drawn_config(seed)
    w = write_model(tmp_path, config, seed=900 + seed)
    seqs = {f"q{i}": traces.random_ids(config["vocab"], n, 40 * seed + i) for i, n in enumerate([90, 3, 47, 130, 18])}
    ref = {rid: pd.forward(config, w, ids) for rid, ids in seqs.items()}
    for dtype_name in ("float32", "bfloat16"):
        steps = traces.mixed(seqs, seed=seed, live_max=3, tail=30)
        pages = -(-traces.tokens_needed(steps, round_to=bs) // bs)
        runner = ModelRunner.from_folder(tmp_path, EngineConfig(dtype=dtype_name, block_size=bs, num_blocks=pages,
                                                                max_num_seqs=3))
        runner.storage.poison()
        got = run_trace(runner, steps)
        for rid in seqs:
            logits_close(got[rid], ref[rid], getattr(torch, dtype_name), f"seed {seed} {rid} {dtype_name}: {config['layers']}")
        assert runner.manager.num_free_slots == 3
        assert all(a.num_free == pages for a in runner.manager.allocators.values())
