"""Debusun on the GPU against the plain implementation (tests/plain_debusun.py): each mechanism's kernel
alone, then whole models under every way of cutting the work, in float32 and bfloat16."""
import json
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

import harness
import plain_debusun as plain
from debusun_models import MODELS, make_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]
TD = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 2e-5, "bfloat16": 2e-2}


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("debusun")
    made = {}

    def get(name):
        if name not in made:
            made[name] = make_model(str(root / name), name)
        return made[name]
    return get


def _i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def _i64(x):
    return torch.tensor(x, dtype=torch.int64, device=DEV)


def _steps(cuts):
    """cuts: for each request the sizes of its portions, one a step.  Yields for every step the rows
    (request, first token, tokens) of the requests that still bring something."""
    at = [0] * len(cuts)
    for step in range(max(len(c) for c in cuts)):
        rows = []
        for b, c in enumerate(cuts):
            if step < len(c):
                rows.append((b, at[b], c[step]))
                at[b] += c[step]
        yield rows


def _step_index(rows):
    cu, tok_seq, positions = [0], [], []
    for i, (_, a, n) in enumerate(rows):
        cu.append(cu[-1] + n)
        tok_seq += [i] * n
        positions += list(range(a, a + n))
    return cu, tok_seq, positions


# ---- the embedding of pairs ------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("vocab,buckets,mul_prev,mul_cur,width", [(311, 97, 31, 7, 96), (70000, 5, 1000003, 99991, 50), (9, 1, 0, 0, 8)])
def test_pair_embedding_keeps_the_token_before(vocab, buckets, mul_prev, mul_cur, width, dtype):
    """Three requests in slots that are not in order and were used before, cut into portions down to one token:
    a portion's first token pairs with the last token of the portion before; a sequence's first token takes the
    table's last row whatever its slot held."""
    from xinfer_amd import kernels
    dt = TD[dtype]
    g = torch.Generator().manual_seed(vocab)
    table = torch.randn(vocab, width, generator=g).to(dt)
    pairs = torch.randn(buckets + 1, width, generator=g).to(dt)
    rng = random.Random(vocab)
    toks = [harness.random_prompt(rng, n, vocab) for n in (23, 1, 40)]
    toks[2][:3] = [vocab - 1, vocab - 1, vocab - 2]                     # the largest products
    cuts = [[2, 20, 1], [1], [1, 1, 2, 33, 3]]
    slots = [3, 0, 2]
    last = torch.full((5,), 7, dtype=torch.int32, device=DEV)          # what other requests left
    got = [[] for _ in toks]
    for rows in _steps(cuts):
        cu, tok_seq, positions = _step_index(rows)
        ids = _i32([t for b, a, n in rows for t in toks[b][a:a + n]])
        st = _i64([slots[b] for b, _, _ in rows])
        out = kernels.embed_pair(table.to(DEV), pairs.to(DEV), ids, _i32(positions), _i32(tok_seq), _i32(cu), st, last, 2.5,
                                 buckets, mul_prev, mul_cur)
        kernels.keep_last_token(ids, _i32(cu), st, last)
        assert out.dtype == torch.float32
        for i, (b, _, _) in enumerate(rows):
            got[b].append(out[cu[i]:cu[i + 1]].cpu())
    assert int(last[1]) == 7 and int(last[4]) == 7
    for b, t in enumerate(toks):
        want = plain.embed(t, table.double(), 2.5, pairs.double(), dict(buckets=buckets, mul_prev=mul_prev, mul_cur=mul_cur))
        assert int(last[slots[b]]) == t[-1]
        assert (torch.cat(got[b]).double() - want).abs().max() < 1e-5 * want.abs().max()


# ---- heads: rotation, then the unit norm, then the cache ---------------------------------------------------------
def _pools(L, G, d, dv, page, dtype, grouped, seed=0):
    """Empty K and V pools with more pages than L tokens need, and a block table of shuffled pages."""
    n_pages = -(-L // page)
    order = list(range(n_pages + 3))
    random.Random(seed).shuffle(order)
    table = torch.tensor([order[:n_pages]], dtype=torch.int32)
    k_pool = torch.zeros(n_pages + 3, G, page, d, dtype=dtype)
    v_pool = torch.zeros((n_pages + 3, G, page // 8, dv, 8) if grouped else (n_pages + 3, G, page, dv), dtype=dtype)
    slots = torch.tensor([order[p // page] * page + p % page for p in range(L)], dtype=torch.int64)
    return k_pool, v_pool, table, slots


def _read_pools(k_pool, v_pool, table, L, grouped):
    page = k_pool.shape[2]
    k = torch.stack([k_pool[table[0, p // page], :, p % page] for p in range(L)])
    if grouped:
        v = torch.stack([v_pool[table[0, p // page], :, (p % page) // 8, :, p % 8] for p in range(L)])
    else:
        v = torch.stack([v_pool[table[0, p // page], :, p % page] for p in range(L)])
    return k, v


def _tables(rot, n):
    """cos and sin [n, dims / 2] as float32, from the plain frequencies."""
    f, m = plain.rotary_frequencies(rot)
    ang = torch.arange(n, dtype=torch.float64)[:, None] * f[None, :]
    return (ang.cos() * m).float().to(DEV), (ang.sin() * m).float().to(DEV)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d,dv,rot", [(6, 2, 16, 24, 8), (3, 3, 32, 8, 32), (4, 1, 48, 48, 2), (2, 2, 12, 20, 0)])
def test_heads_turned_then_divided_by_their_root_mean_square(H, G, d, dv, rot, dtype):
    from xinfer_amd import kernels
    dt = TD[dtype]
    grouped = dt == torch.bfloat16
    g = torch.Generator().manual_seed(H * d)
    L, page = 37, 8
    qkv = (torch.randn(L, H * d + G * d + G * dv, generator=g) * 3).to(dt)
    positions = [100 + 3 * p for p in range(L)]                        # not the rows' own numbers
    r = {"dims": rot, "base": 50.0} if rot else None
    cos, sin = _tables(r, 100 + 3 * L) if rot else (None, None)
    k_pool, v_pool, table, slots = _pools(L, G, d, dv, page, dt, grouped)
    slots[5] = -1                                                       # stores nothing
    k_d, v_d = k_pool.to(DEV), v_pool.to(DEV)
    q = kernels.head_rows(qkv.to(DEV), slots.to(DEV), k_d, v_d, H, G, d, dv, v_grouped=grouped, cos=cos, sin=sin, rotary_dim=rot,
                          interleaved=True, positions=_i32(positions), unit_norm=True, eps=1e-3)
    x = qkv.double()
    want_q, want_k = x[:, :H * d].view(L, H, d), x[:, H * d:H * d + G * d].view(L, G, d)
    if rot:
        want_q, want_k = plain.rotate(want_q, r, torch.tensor(positions)), plain.rotate(want_k, r, torch.tensor(positions))
    want_q, want_k = plain.rms_norm(want_q, 1e-3), plain.rms_norm(want_k, 1e-3)
    want_v = x[:, H * d + G * d:].view(L, G, dv)
    tol = 1e-5 if dt == torch.float32 else 1e-2
    assert (q.cpu().double() - want_q).abs().max() < tol * want_q.abs().max()
    k, v = _read_pools(k_d.cpu(), v_d.cpu(), table, L, grouped)
    keep = [p for p in range(L) if p != 5]
    assert (k.double()[keep] - want_k[keep]).abs().max() < tol * want_k.abs().max()
    assert torch.equal(v[keep], qkv[:, H * d + G * d:].view(L, G, dv)[keep])
    assert float(k[5].abs().max()) == 0 and float(v[5].abs().max()) == 0
    assert want_v.shape == v.shape


# ---- attention over planted keys -----------------------------------------------------------------------------------
def _planted(L, H, G, d, window, scale, seed, big_score=30.0):
    """q [L, H, d] and k [L, G, d] of one sequence in which chosen (query, key) pairs have a score that stands far
    out: keys just inside and just outside the window, at page borders, the first token, far back."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(L, H, d, generator=g) * 0.3
    k = torch.randn(L, G, d, generator=g) * 0.3
    big = big_score / scale
    pairs = []
    w = window or L
    for i in list(range(L - 12, L)) + [w - 1, w, w + 1, 17, 31, 32, 63, 64, 65]:
        if not (0 <= i < L):
            continue
        for j in (i - w + 1, i - w, i - 15, i - 16, i - 17, i - 63, i - 64, 0, 1, i - L // 2):
            if 0 <= j <= i:
                pairs.append((i, j))
    rng = random.Random(seed)
    for n, (i, j) in enumerate(pairs):
        h = rng.randrange(H)
        u = torch.zeros(d)
        u[n % d] = 1.0
        q[i, h] = u * (big ** 0.5)
        k[j, h // (H // G)] = u * (big ** 0.5)
    return q, k


def _windowed(q, k, v, scale, window, sinks=None):
    """The plain attention of a whole sequence: q [L, H, d], k [L, G, d], v [L, G, dv] -> [L, H dv]."""
    L, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(L, H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        p = plain.window_softmax((q[:, h] @ k[:, h // (H // G)].T) * scale, window or (1 << 30), None if sinks is None else sinks[h])
        out[:, h] = p @ v[:, h // (H // G)]
    return out.reshape(L, -1)


LATENT_CASES = [  # H, rank, r, window, scale, L, page
    (4, 40, 8, 21, 0.3, 90, 16),
    (8, 96, 32, 70, 0.1, 210, 64),
    (2, 24, 4, 9, 0.25, 40, 8),
    (3, 18, 6, None, 0.3, 150, 8),
    (8, 128, 32, 150, 0.1, 400, 64),
    (5, 64, 64, 64, 0.12, 200, 32),
]


def _latent_case(case, dtype, matrix_cores, tail=9, head_rows=False):
    """One pool holds [latent | turned key part] for every token, and a key's first `rank` dims are its value.  A
    sink as large as the planted scores shows in every row it belongs to; a sink of -40 must not show at all."""
    from xinfer_amd import kernels
    H, rank, r, window, scale, L, page = case
    dt = TD[dtype]
    q, k = _planted(L, H, 1, rank + r, window, scale, seed=L)
    q, k = q.to(dt), k.to(dt)
    sinks = torch.tensor([(30.0, -40.0, 0.0, 28.0)[h % 4] for h in range(H)])
    want = _windowed(q.double(), k.double(), k.double()[:, :, :rank], scale, window, sinks.double())
    plain_softmax = _windowed(q.double(), k.double(), k.double()[:, :, :rank], scale, window)
    assert (want - plain_softmax).abs().max() > 0.1 * want.abs().max()         # the sinks matter here
    pool, vt, table, slots = _pools(L, 1, rank + r, rank, page, dt, True, seed=L)
    for p in range(L):
        pg, off = int(slots[p]) // page, int(slots[p]) % page
        pool[pg, 0, off] = k[p, 0]
        vt[pg, 0, off // 8, :, off % 8] = k[p, 0, :rank]
    pool, vt, table, sinks = pool.to(DEV), vt.to(DEV), table.to(DEV), sinks.to(DEV)

    def run(positions):
        qs = q[positions[0]:positions[-1] + 1].to(DEV)
        pos = _i32(positions)
        if not matrix_cores:
            return kernels.attention_generic(qs, pool, None, table, torch.zeros_like(pos), pos, scale, window or 0, sinks=sinks,
                                             value_dim=rank)
        n, ctx = len(positions), positions[-1] + 1
        if head_rows and n == 1:                    # the token's heads as the rows of blocks of one head
            shape = 1 if kernels.attention_biased_block(rank + r, rank, 1, 1) >= H else 0
            per = kernels.attention_biased_block(rank + r, rank, 1, shape)
            tiles = _i32([[0, i * per] for i in range(-(-H // per))])
            span = min(ctx, window + 63) if window else ctx
            out = kernels.attention_biased_bf16(qs.view(H, 1, rank + r), pool, vt, table, tiles, _i32([0, H]), _i32([ctx]), scale,
                                                window or 0, small=shape, split_keys=64 if positions[0] % 2 else 0, span=span,
                                                sinks=sinks, rows_heads=H)
            return out.view(1, H * rank)
        rows, shape = kernels.prefill_tiles([n], [ctx], rank + r, H, 1, block_of=lambda s_: kernels.attention_biased_block(rank + r, rank, H, s_))
        tiles = torch.tensor(rows, dtype=torch.int32, device=DEV).reshape(-1, 2)
        split, span = 0, 0
        if n == 1 and positions[0] % 2:             # single tokens: every other one in slices of 64 keys put together afterwards
            span = min(ctx, window + 63) if window else ctx
            split = 64
        return kernels.attention_biased_bf16(qs, pool, vt, table, tiles, _i32([0, n]), _i32([ctx]), scale, window or 0, small=shape,
                                             split_keys=split, span=span, sinks=sinks)
    head = L - tail
    outs = [run(list(range(head)))] + [run([p]) for p in range(head, L)]
    got = torch.cat([o.cpu() for o in outs]).double()
    err = (got - want).abs().max(dim=1).values
    bad = (err > TOL[dtype] * want.abs().max()).nonzero()
    assert bad.numel() == 0, f"first wrong position {int(bad[0])} of {L} (window {window}): {float(err[int(bad[0])]):.3e}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", LATENT_CASES)
def test_attention_over_a_latent_with_sinks_and_planted_keys(case, dtype):
    _latent_case(case, dtype, matrix_cores=False)


@pytest.mark.parametrize("case", [c for c in LATENT_CASES if c[1] % 8 == 0 and c[2] % 8 == 0])
def test_attention_over_a_latent_on_the_matrix_cores(case):
    _latent_case(case, "bfloat16", matrix_cores=True)
    _latent_case(case, "bfloat16", matrix_cores=True, tail=70)


@pytest.mark.parametrize("case", [c for c in LATENT_CASES if c[1] % 8 == 0 and c[2] % 8 == 0] + [(144, 136, 8, 40, 0.1, 120, 16)])
def test_single_tokens_whose_heads_are_the_rows_of_a_block(case):
    """Steps of single tokens over one kv head: all heads of a token in one block (or several, for many heads), whole
    and in slices of 64 keys, each head with its own sink."""
    _latent_case(case, "bfloat16", matrix_cores=True, tail=70, head_rows=True)


def test_a_sink_of_the_matrix_core_kernel_with_several_kv_heads():
    """Sinks belong to query heads: with groups of query heads on kv heads, each head's own sink joins its sum."""
    from xinfer_amd import kernels
    H, G, d, dv, L, page, scale, window = 6, 2, 32, 16, 100, 16, 0.2, 33
    q, k = _planted(L, H, G, d, window, scale, seed=3)
    g = torch.Generator().manual_seed(1)
    v = torch.randn(L, G, dv, generator=g)
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    sinks = torch.tensor([30.0, -40.0, 1.0, 29.0, 2.0, 31.0])
    want = _windowed(q.double(), k.double(), v.double(), scale, window, sinks.double())
    k_pool, v_pool, table, slots = _pools(L, G, d, dv, page, torch.bfloat16, True)
    for p in range(L):
        pg, off = int(slots[p]) // page, int(slots[p]) % page
        k_pool[pg, :, off] = k[p]
        v_pool[pg, :, off // 8, :, off % 8] = v[p]
    rows, shape = kernels.prefill_tiles([L], [L], d, H, G, block_of=lambda s_: kernels.attention_biased_block(d, dv, H // G, s_))
    got = kernels.attention_biased_bf16(q.to(DEV), k_pool.to(DEV), v_pool.to(DEV), table.to(DEV),
                                        torch.tensor(rows, dtype=torch.int32, device=DEV).reshape(-1, 2), _i32([0, L]), _i32([L]),
                                        scale, window, small=shape, sinks=sinks.to(DEV))
    assert (got.cpu().double() - want).abs().max() < 2e-2 * want.abs().max()
    pos = torch.arange(L, dtype=torch.int32, device=DEV)
    ref = kernels.attention_generic(q.to(DEV), k_pool.to(DEV), v_pool.to(DEV), table.to(DEV), torch.zeros_like(pos), pos, scale,
                                    window, v_grouped=True, sinks=sinks.to(DEV))
    assert (ref.cpu().double() - want).abs().max() < 2e-2 * want.abs().max()


ATTN_CASES = [  # H, G, d, dv, window, scale, L
    (6, 2, 16, 24, 12, 0.4, 70),
    (5, 5, 20, 12, 5, 0.35, 60),
    (3, 1, 12, 20, 1, 0.5, 40),
    (8, 2, 64, 128, 100, 0.125, 330),
    (4, 4, 128, 128, 300, 0.09, 420),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", ATTN_CASES)
def test_window_attention_with_heads_of_two_sizes(case, dtype):
    """Keys just inside and just outside the window, at page borders and far back, in a portion and token by token,
    through the kernel the engine chooses for the sizes and the precision."""
    from xinfer_amd import kernels
    from xinfer_amd.parts import StepContext
    H, G, d, dv, window, scale, L = case
    dt = TD[dtype]
    page = 16
    grouped = dt == torch.bfloat16
    q, k = _planted(L, H, G, d, window, scale, seed=L)
    v = torch.randn(L, G, dv, generator=torch.Generator().manual_seed(L))
    q, k, v = q.to(dt), k.to(dt), v.to(dt)
    want = _windowed(q.double(), k.double(), v.double(), scale, window)
    k_pool, v_pool, table, slots = _pools(L, G, d, dv, page, dt, grouped, seed=L)
    for p in range(L):
        pg, off = int(slots[p]) // page, int(slots[p]) % page
        k_pool[pg, :, off] = k[p]
        if grouped:
            v_pool[pg, :, off // 8, :, off % 8] = v[p]
        else:
            v_pool[pg, :, off] = v[p]
    k_pool, v_pool, table = k_pool.to(DEV), v_pool.to(DEV), table.to(DEV)
    outs = []
    head = L - 9
    for positions in [list(range(head))] + [[p] for p in range(head, L)]:
        n, ctx_len = len(positions), positions[-1] + 1
        ctx = StepContext(num_tokens=n, num_seqs=1, dtype=dt, device=torch.device(DEV), positions=_i32(positions),
                          tok_seq=_i32([0] * n), cu_q=_i32([0, n]), ctx_lens=_i32([ctx_len]), state_slots=_i64([0]),
                          slots=[_i64([-1] * n)], block_tables=[table], cu_q_host=[0, n], ctx_lens_host=[ctx_len],
                          max_q_len=n, max_ctx_len=ctx_len)
        outs.append(kernels.attention(q[positions[0]:positions[-1] + 1].to(DEV), k_pool, v_pool, ctx, 0, scale, window,
                                      v_grouped=grouped).cpu())
    got = torch.cat(outs).double()
    err = (got - want).abs().max(dim=1).values
    bad = (err > TOL[dtype] * want.abs().max()).nonzero()
    assert bad.numel() == 0, f"first wrong position {int(bad[0])} of {L} (window {window}): {float(err[int(bad[0])]):.3e}"


# ---- the latent's rows and the heads' products ----------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,d,r,dv,rank,page", [(4, 16, 8, 24, 40, 16), (2, 24, 4, 16, 24, 8), (3, 12, 6, 10, 18, 8), (8, 64, 32, 64, 128, 64)])
def test_latent_rows_and_the_heads_products(H, d, r, dv, rank, page, dtype):
    """The packed projection [q | down | gate]: the normed latent and the turned key part go into the pool (and the
    latent once more in groups of eight tokens), the queries' turned parts into q'; the plain parts go through U_k;
    U_v and the gate come behind."""
    from xinfer_amd import kernels
    dt = TD[dtype]
    g = torch.Generator().manual_seed(rank)
    L = 45
    rot = {"dims": r, "base": 100.0, "scaling": dict(factor=4.0, original=16, fast=8.0, slow=1.0)}
    m = dict(heads=H, dim=d, rot_dim=r, vdim=dv, kv_rank=rank, scale=0.3, rot=rot)
    width = H * (d + r) + rank + r + H * dv
    proj = (torch.randn(L, width, generator=g) * 2).to(dt)
    w = 1 + 0.3 * torch.randn(rank, generator=g)
    uk = (torch.randn(H * d, rank, generator=g) * 0.3).to(dt)
    uv = (torch.randn(H * dv, rank, generator=g) * 0.3).to(dt)
    positions = [7 + 2 * p for p in range(L)]
    cos, sin = _tables(rot, 7 + 2 * L)
    pool, vt, table, slots = _pools(L, 1, rank + r, rank, page, dt, True)
    slots[11] = -1
    pool_d, vt_d = pool.to(DEV), vt.to(DEV)
    proj_d = proj.to(DEV)
    q_full = torch.zeros(L, H, rank + r, dtype=dt, device=DEV)
    kernels.latent_rows(proj_d, 0, H * (d + r), w.to(DEV), 1e-4, slots.to(DEV), pool_d, q_full, H, d, r, rank, cos, sin, True,
                        _i32(positions), values=vt_d)
    q_plain = proj_d[:, :H * (d + r)].view(L, H, d + r)[:, :, :d]
    kernels.head_linear(q_plain, uk.to(DEV).view(H, d, rank).transpose(1, 2), q_full[:, :, :rank])
    turned = torch.empty(L, H, rank, dtype=dt, device=DEV)          # U_k turned over in memory: the same product
    kernels.head_linear(q_plain, uk.to(DEV).view(H, d, rank).transpose(1, 2).contiguous(), turned)
    assert (turned.float() - q_full[:, :, :rank].float()).abs().max() <= (0 if dt == torch.float32 else 1e-2) * q_full.float().abs().max()
    x = proj.double()
    pos = torch.tensor(positions)
    qs = x[:, :H * (d + r)].view(L, H, d + r)
    down = x[:, H * (d + r):H * (d + r) + rank + r]
    c = plain.rms_norm(down[:, :rank], 1e-4, w.double())
    k_turned = plain.rotate(down[:, None, rank:], rot, pos)[:, 0]
    want_q = torch.cat([torch.einsum("thi,hij->thj", qs[..., :d], uk.double().view(H, d, rank)),
                        plain.rotate(qs[..., d:], rot, pos)], dim=-1)
    tol = 1e-5 if dt == torch.float32 else 1.5e-2
    assert (q_full.cpu().double() - want_q).abs().max() < tol * want_q.abs().max()
    k, v = _read_pools(pool_d.cpu(), vt_d.cpu(), table, L, True)
    keep = [p for p in range(L) if p != 11]
    want_k = torch.cat([c, k_turned], dim=-1)
    assert (k.double()[keep, 0] - want_k[keep]).abs().max() < tol * want_k.abs().max()
    assert torch.equal(v[keep, 0], k[keep, 0, :rank])                  # the same latent in both layouts
    assert float(k[11].abs().max()) == 0 and float(v[11].abs().max()) == 0
    # behind the attention: every head's sum of the latent through U_v, times sigmoid(gate)
    a = (torch.randn(L, H, rank, generator=g)).to(dt)
    heads = torch.empty(L, H, dv, dtype=dt, device=DEV)
    gate = proj_d[:, H * (d + r) + rank + r:].view(L, H, dv)
    kernels.head_linear(a.to(DEV), uv.to(DEV).view(H, dv, rank), heads, gate=gate)
    want = torch.einsum("thj,hnj->thn", a.double(), uv.double().view(H, dv, rank)) * torch.sigmoid(x[:, H * (d + r) + rank + r:].view(L, H, dv))
    assert (heads.cpu().double() - want).abs().max() < tol * want.abs().max()
    assert m["heads"] == H


# ---- the state space ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,taps,pad,long", [(40, 3, 2, False), (7, 2, 2, False), (130, 5, 2, False), (64, 4, 2, False), (9, 1, 2, False),
                                             (40, 3, 8, False), (64, 4, 8, True), (128, 5, 16, True), (16, 2, 8, True), (8, 1, 8, False),
                                             (24, 6, 8, False)])
def test_causal_convolution_over_portions(C, taps, pad, long, dtype):
    """Three requests in slots used before, in portions down to one token (shorter than the taps): a portion's first
    outputs read the inputs the portion before left, a sequence's first outputs read zeros.  Channels that start at a
    whole 16-byte chunk of rows made of such chunks take eight channels a thread, and long steps runs of tokens, with
    sequences that start inside a run."""
    from xinfer_amd import kernels
    dt = TD[dtype]
    g = torch.Generator().manual_seed(C)
    lens = [300, 2, 1100] if long else [23, 2, 40]
    cuts = [[2, 297, 1], [2], [1, 1, 2, 1093, 3]] if long else [[2, 20, 1], [2], [1, 1, 2, 33, 3]]
    slots = [3, 0, 2]
    u = [(torch.randn(n, C + 2 * pad, generator=g)).to(dt) for n in lens]         # columns of wider rows
    wt, bias = torch.randn(C, taps, generator=g) * 0.5, torch.randn(C, generator=g) * 0.1
    tails = torch.full((5, taps - 1, C), 9.0, device=DEV)
    tails[slots] = 0                                                          # what the runner does when a request starts
    got = [[] for _ in lens]
    for rows in _steps(cuts):
        cu, tok_seq, _ = _step_index(rows)
        x = torch.cat([u[b][a:a + n] for b, a, n in rows]).to(DEV)[:, pad:pad + C]
        st = _i64([slots[b] for b, _, _ in rows])
        out = kernels.causal_conv(x, wt.to(DEV), bias.to(DEV), tails, st, _i32(tok_seq), _i32(cu))
        if taps > 1:
            kernels.conv_tail(x, tails, st, _i32(cu))
        for i, (b, _, _) in enumerate(rows):
            got[b].append(out[cu[i]:cu[i + 1]].cpu())
    if taps > 1:
        assert torch.all(tails[1] == 9.0) and torch.all(tails[4] == 9.0)
    for b, n in enumerate(lens):
        want = plain.silu(plain.causal_conv(u[b][:, pad:pad + C].double(), wt.double(), bias.double()))
        err = (torch.cat(got[b]).double() - want).abs().max(dim=1).values
        bad = (err > (1e-5 if dt == torch.float32 else 1e-2) * want.abs().max()).nonzero()
        assert bad.numel() == 0, f"request {b}: first wrong token {int(bad[0])} of {n}"
        if taps > 1 and n >= taps - 1:
            assert torch.equal(tails[slots[b]].cpu(), u[b][n - (taps - 1):, pad:pad + C].float())


def _ssm_inputs(T, H, G, N, dv, dt, seed):
    g = torch.Generator().manual_seed(seed)
    packed = (torch.randn(T, H * dv + 2 * G * N + H + 3, generator=g) * 0.7).to(dt)       # x | B | C | dt | something else
    x, B, C = packed[:, :H * dv], packed[:, H * dv:H * dv + G * N], packed[:, H * dv + G * N:H * dv + 2 * G * N]
    step = packed[:, H * dv + 2 * G * N:H * dv + 2 * G * N + H]
    return packed, x, B, C, step


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk", [0, 16])
@pytest.mark.parametrize("H,G,N,dv", [(4, 2, 16, 24), (3, 3, 8, 20), (2, 1, 12, 20), (8, 1, 64, 64), (6, 3, 16, 12), (1, 1, 128, 8),
                                      (2, 1, 40, 80), (4, 2, 256, 136)])
def test_state_space_walk_of_unequal_requests_in_portions(H, G, N, dv, chunk, dtype, monkeypatch):
    from xinfer_amd import kernels
    monkeypatch.setattr(kernels, "SCAN_CHUNK", chunk)
    dt = TD[dtype]
    lens = [37, 5, 70]
    cuts = [[2, 33, 1, 1], [5], [1, 1, 2, 64, 2]]
    slots = [3, 0, 2]
    g = torch.Generator().manual_seed(H)
    step_bias, decay_log = torch.randn(H, generator=g) * 0.5 - 1.0, torch.randn(H, generator=g) * 0.5 - 1.0
    data = [_ssm_inputs(n, H, G, N, dv, dt, 10 * i + H) for i, n in enumerate(lens)]
    want = []
    for n, (_, x, B, C, step) in zip(lens, data):
        y, S = plain.state_space(x.double().view(n, H, dv), B.double().view(n, G, N), C.double().view(n, G, N),
                                 plain.softplus(step.double() + step_bias.double()), decay_log.double(), torch.zeros(H, dtype=torch.float64))
        want.append((y, S))
    state = torch.full((5, H, N, dv), 7.0, device=DEV)
    state[slots] = 0
    got = [[] for _ in lens]
    for k, rows in enumerate(_steps(cuts)):
        cu, _, _ = _step_index(rows)
        packed = torch.cat([data[b][0][a:a + n] for b, a, n in rows]).to(DEV)
        x, B, C = packed[:, :H * dv], packed[:, H * dv:H * dv + G * N], packed[:, H * dv + G * N:H * dv + 2 * G * N]
        step = packed[:, H * dv + 2 * G * N:H * dv + 2 * G * N + H]
        o = kernels.linear_scan(C, B, x, state, _i64([slots[b] for b, _, _ in rows]), _i32(cu), H, N, dv, step=step,
                                step_bias=step_bias.to(DEV), decay_log=decay_log.to(DEV), groups=G,
                                q_lens=[n for _, _, n in rows] if chunk else None, plan_cache={} if k % 2 else None)
        for i, (b, _, _) in enumerate(rows):
            got[b].append(o[cu[i]:cu[i + 1]].cpu())
    assert torch.all(state[1] == 7.0) and torch.all(state[4] == 7.0)
    for b, n in enumerate(lens):
        y, S = want[b]
        o = torch.cat(got[b]).double()
        assert (o - y).abs().max() < 2e-5 * y.abs().max(), (b, float((o - y).abs().max()))
        assert (state[slots[b]].cpu().double() - S).abs().max() < 2e-5 * S.abs().max()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rate,far", [(-30.0, 599), (-6.0, 300), (-2.0, 40)])
def test_state_space_keeps_a_far_token(rate, far, dtype):
    """One token far back is made to stand out (its B and the last C along one direction of their own): the last
    token's result is that token's value times its step and the decays since, which a lost or reset state would not
    give; the prompt is cut at a place of its own and decoded one by one at the end."""
    from xinfer_amd import kernels
    dt = TD[dtype]
    T, H, G, N, dv = 600, 2, 1, 32, 40
    g = torch.Generator().manual_seed(far)
    B = (torch.randn(T, G * N, generator=g) * 0.1).to(dt)
    C = (torch.randn(T, G * N, generator=g) * 0.1).to(dt)
    x = torch.randn(T, H * dv, generator=g).to(dt)
    step = torch.zeros(T, H).to(dt)                                          # every step softplus(0) = ln 2
    at = T - 1 - far
    B[:, 3] = 0
    B[at] = 0
    B[at, 3] = 30.0
    C[T - 1, 3] = 30.0
    decay_log = torch.full((H,), rate)
    want, _ = plain.state_space(x.double().view(T, H, dv), B.double().view(T, G, N), C.double().view(T, G, N),
                                plain.softplus(step.double()), decay_log.double(), torch.zeros(H, dtype=torch.float64))
    d = float(np.log(2.0))
    share = 900.0 * d * float(np.exp(-np.exp(rate) * d * far)) * x.double().view(T, H, dv)[at]
    assert (want[T - 1] - share).abs().max() < 0.1 * share.abs().max()        # the planted token dominates
    state = torch.zeros(1, H, N, dv, device=DEV)
    slot = _i64([0])
    outs = []
    for a, b in [(0, 257), (257, T - 5)] + [(t, t + 1) for t in range(T - 5, T)]:
        outs.append(kernels.linear_scan(C[a:b].to(DEV), B[a:b].to(DEV), x[a:b].to(DEV), state, slot, _i32([0, b - a]), H, N, dv,
                                        step=step[a:b].to(DEV), step_bias=torch.zeros(H, device=DEV), decay_log=decay_log.to(DEV),
                                        groups=G, q_lens=[b - a]).cpu())
    got = torch.cat(outs).double()
    assert (got[T - 1] - want[T - 1]).abs().max() < 1e-4 * want[T - 1].abs().max()
    assert (got - want).abs().max() < 1e-4 * want.abs().max()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("pad", [5, 8])
@pytest.mark.parametrize("H,dv,parts", [(4, 24, 2), (3, 20, 3), (2, 20, 1), (8, 64, 1), (6, 12, 6), (5, 7, 1), (160, 64, 1), (6, 16, 3)])
def test_gate_before_the_norm_in_equal_parts(H, dv, parts, pad, dtype):
    from xinfer_amd import kernels
    dt = TD[dtype]
    g = torch.Generator().manual_seed(H * dv)
    T = 19
    y = torch.randn(T, H, dv, generator=g)
    packed = torch.randn(T, 2 * H * dv + pad, generator=g).to(dt)        # z | something else | x
    z, x = packed[:, :H * dv], packed[:, H * dv + pad:]
    skip, w = torch.randn(H, generator=g), 1 + 0.2 * torch.randn(H * dv, generator=g)
    pd = packed.to(DEV)
    got = kernels.gated_group_norm(y.to(DEV), pd[:, H * dv + pad:], skip.to(DEV), pd[:, :H * dv], w.to(DEV), 1e-3, parts, dt)
    full = y.double() + skip.double()[None, :, None] * x.double().view(T, H, dv)
    want = plain.gated_group_norm(full.reshape(T, H * dv), z.double(), w.double(), 1e-3, parts)
    assert got.dtype == dt
    assert (got.cpu().double() - want).abs().max() < (1e-5 if dt == torch.float32 else 1e-2) * want.abs().max()


# ---- the start of a pass ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("width", [96, 100, 50])
def test_the_start_of_a_pass(width):
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(width)
    T = 11
    resid, first, vec = torch.randn(T, width, generator=g), torch.randn(T, width, generator=g), torch.randn(width, generator=g)
    for pending in (torch.randn(T, width, generator=g), torch.randn(T, width, generator=g).bfloat16(), torch.randn(3, T, width, generator=g), None):
        for use_first in (True, False):
            r = resid.clone().to(DEV)
            kernels.stream_start(r, None if pending is None else pending.to(DEV), 0.5, first.to(DEV) if use_first else None, vec.to(DEV))
            want = resid.double() + vec.double()
            if pending is not None:
                want = want + 0.5 * (pending.double() if pending.dim() == 2 else pending.double().sum(0))
            if use_first:
                want = want + first.double()
            assert (r.cpu().double() - want).abs().max() < 1e-5


# ---- whole models ----------------------------------------------------------------------------------------------------
LENGTHS = {"A": [1, 2, 12, 13, 33, 77, 130], "B": [3, 9, 10, 18, 64, 101], "C": [1, 7, 8, 40, 75, 210], "D": [2, 1, 30, 140],
           "R": [5, 101, 330, 64, 301], "S": [3, 70, 71, 260, 129]}


def _requests(name):
    rng = random.Random(900 + ord(name))
    vocab = MODELS[name]["config"]["vocab"]
    return {f"r{i}": harness.random_prompt(rng, n, vocab) for i, n in enumerate(LENGTHS[name])}


_plain_cache = {}
_model_cache = {}


def _plain_logits(name, model_dir):
    if name not in _plain_cache:
        pm = plain.PlainDebusun(model_dir, torch.float64)
        _plain_cache[name] = {rid: pm.logits(toks).float() for rid, toks in _requests(name).items()}
    return _plain_cache[name]


def _model(name, dtype, model_dir):
    from xinfer_amd.engine import load_model
    if (name, dtype) not in _model_cache:
        _model_cache[(name, dtype)] = load_model(model_dir, dtype, DEV)
    return _model_cache[(name, dtype)]


def _run(name, dtype, dirs, steps, what, **kw):
    from xinfer_amd.engine import ModelRunner
    page = MODELS[name]["page_size"]
    need = harness.tokens_needed(steps, page)
    model = _model(name, dtype, dirs(name))
    runner = ModelRunner(model, page_size=page, num_pages=max(1, need // page), max_requests=4, **kw)     # exactly enough pages
    got = harness.replay(runner, steps)
    for g in range(len(runner.cache.groups)):
        assert runner.cache.free_pages(g) == max(1, need // page)
    rel = harness.compare(got, _plain_logits(name, dirs(name)), harness.TOL[dtype], f"{name}/{dtype}/{what}")
    print(f"{name}/{dtype}/{what}: worst error {rel:.2e} of the largest logit")
    return got, runner


@pytest.mark.parametrize("name", list(MODELS))
def test_the_models_are_what_they_are_meant_to_be(name, dirs):
    cfg = MODELS[name]["config"]
    model = _model(name, "float32", dirs(name))
    loop = cfg.get("loop")
    runs = len(cfg["layers"]) + ((loop["stop"] - loop["start"]) * (loop["times"] - 1) if loop else 0)
    assert len(model.spec.schedule) == runs
    assert len(model.blocks) == len(cfg["layers"])
    assert model.graph_safe
    if name == "R":        # the latent of this one runs on the matrix cores in bfloat16
        m16 = _model(name, "bfloat16", dirs(name))
        assert m16.blocks[0].mixer.values_pool and not model.blocks[0].mixer.values_pool


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_whole(name, dtype, dirs):
    got, _ = _run(name, dtype, dirs, harness.trace_whole(_requests(name)), "whole")
    assert len(got) == sum(LENGTHS[name])


@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_the_stream_after_every_layer(name, dirs):
    """float32, one request: the residual stream after every run of a layer against the plain one."""
    from xinfer_amd.engine import ModelRunner, StepEntry
    model = _model(name, "float32", dirs(name))
    toks = _requests(name)["r2"]
    want = plain.PlainDebusun(dirs(name), torch.float64).stream(toks)[1:]
    seen = []
    kept = [(b, b.forward) for b in model.blocks]
    try:
        for blk, orig in kept:
            def fwd(stream, ctx, c, _o=orig, **kw):
                s = _o(stream, ctx, c, **kw)
                p = s.pending.float() if s.pending.dim() == 2 else s.pending.float().sum(0)
                seen.append((s.resid + s.pending_scale * p).cpu().double())
                return s
            blk.forward = fwd
        runner = ModelRunner(model, page_size=MODELS[name]["page_size"], num_pages=8, max_requests=1, use_graphs=False)
        runner.add_request(0)
        runner.step([StepEntry(0, toks, [])])
    finally:
        for blk, orig in kept:
            blk.forward = orig
    assert len(seen) == len(want)
    for i, (a, b) in enumerate(zip(seen, want)):
        assert (a - b).abs().max() < 1e-5 * b.abs().max(), f"the stream after layer run {i} differs"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_prefill_against_decoding_one_by_one(name, dtype, dirs):
    _run(name, dtype, dirs, harness.trace_tail_one_by_one(_requests(name), tail=40), "tail")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_portions(name, dtype, dirs):
    _run(name, dtype, dirs, harness.trace_portions(_requests(name)), "portions")
    _run(name, dtype, dirs, harness.trace_portions(_requests(name), sizes=(2, 2, 3, 40, 2, 5)), "small portions")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype, dirs):
    """More requests than state slots, one after the other in the same slots and pages: a request that starts
    finds no state, no last token and no convolution inputs of the one before."""
    for seed in (1, 2):
        _run(name, dtype, dirs, harness.trace_mixed(_requests(name), seed, max_live=3), f"mixed {seed}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "R"])
def test_short_chunks_of_the_states_walk(name, dtype, dirs, monkeypatch):
    """Portions from 32 tokens on are walked in chunks of 16: whole prompts, portions and mixed batches again."""
    from xinfer_amd import kernels
    monkeypatch.setattr(kernels, "SCAN_CHUNK", 16)
    _run(name, dtype, dirs, harness.trace_whole(_requests(name)), "whole, chunks of 16")
    _run(name, dtype, dirs, harness.trace_portions(_requests(name), sizes=(33, 2, 47, 32, 5)), "portions, chunks of 16")
    _run(name, dtype, dirs, harness.trace_mixed(_requests(name), 3, max_live=3, sizes=(40, 2, 35, 64)), "mixed, chunks of 16")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "R", "S"])
def test_unequal_requests_decoding_together(name, dtype, dirs):
    reqs = {k: v for k, v in _requests(name).items() if len(v) > 8}
    reqs = dict(list(reqs.items())[:4])
    _run(name, dtype, dirs, harness.trace_batch_decode(reqs, tail=7), "batch decode", use_graphs=False)
    got, runner = _run(name, dtype, dirs, harness.trace_batch_decode(reqs, tail=7), "batch decode, graphs", graph_after=1)
    assert runner.graph_replays > 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "R"])
def test_long_decoding_passes_every_window(name, dtype, dirs):
    """Three tokens of prompt, then the rest one by one: every window passes over decoded tokens, pages behind the
    windows come back, the states grow token by token."""
    n = 253 if name == "A" else 340
    toks = harness.random_prompt(random.Random(9), n, MODELS[name]["config"]["vocab"])
    from xinfer_amd.engine import ModelRunner
    ref = {"a": plain.PlainDebusun(dirs(name), torch.float64).logits(toks).float()}
    steps = harness.trace_tail_one_by_one({"a": toks}, tail=n - 3)
    page = MODELS[name]["page_size"]
    runner = ModelRunner(_model(name, dtype, dirs(name)), page_size=page, num_pages=-(-n // page) + 1, max_requests=2, graph_after=2)
    got = harness.replay(runner, steps)
    assert runner.graph_replays > 200
    harness.compare(got, ref, harness.TOL[dtype], f"long decoding {name} {dtype}")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_greedy_generation_through_the_engine(dtype, dirs):
    """The framework's own entry point and scheduler: five prompts, three at a time, prompts cut into
    portions of 16 tokens, greedy tokens against the plain implementation."""
    from xinfer_amd import Engine, EngineConfig, SamplingParams
    name = "A"
    rng = random.Random(3)
    vocab = MODELS[name]["config"]["vocab"]
    prompts = [harness.random_prompt(rng, n, vocab) for n in (5, 40, 17, 33, 2)]
    eng = Engine(EngineConfig(weight_path=dirs(name), page_size=16, num_pages=24, max_num_seqs=3, prefill_chunk_size=16,
                              max_model_len=128, seed=1), dtype)
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True))
    pm = plain.PlainDebusun(dirs(name), torch.float64)
    for p, o in zip(prompts, outs):
        assert o.prompt_length == len(p) and o.decoded_length == 24
        if dtype == "f32":
            assert o.token_ids == pm.greedy(p, 24)
        else:
            ids = list(p)
            for t in o.token_ids:
                lg = pm.logits(ids)[-1]
                assert float(lg.max() - lg[t]) <= 2 * harness.TOL["bfloat16"] * float(lg.abs().max())
                ids.append(t)
    assert eng.runner.cache.live_requests() == 0


def test_command_line_runs_the_model(dirs, capsys):
    from xinfer_amd import cli
    rc = cli.main(["--w", dirs("A"), "--prompt-ids", "1,2,3,4,5,6,7,8,9", "--max-tokens", "4", "--max-model-len", "256",
                   "--temperature", "0", "--ignore-eos", "--page-size", "16", "--max-num-seqs", "4", "--dtype", "bf16"])
    assert rc == 0 and "Decoded tokens: 4 in" in capsys.readouterr().out
    rc = cli.main(["--w", dirs("B"), "--prompt-ids", "1,2,3|4,5,6,7", "--max-tokens", "5", "--max-model-len", "64",
                   "--temperature", "0", "--ignore-eos", "--page-size", "8", "--num-pages", "16", "--dtype", "f32"])
    assert rc == 0 and "Decoded tokens: 10 in" in capsys.readouterr().out


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_run_program(dtype, dirs, tmp_path):
    name = "R"
    vocab = MODELS[name]["config"]["vocab"]
    reqs = {f"r{i}": harness.random_prompt(random.Random(60 + i), n, vocab) for i, n in enumerate([33, 170, 5, 64, 200, 9])}
    steps = harness.trace_mixed(reqs, 4)
    need = harness.tokens_needed(steps, 64)
    out = tmp_path / "out"
    proc = subprocess.Popen(
        [sys.executable, os.path.join(REPO, "bin", "trace_run"), "--model", dirs(name), "--dtype", dtype,
         "--out", str(out), "--max-tokens", str(need)],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for st in steps:
        proc.stdin.write(json.dumps(st) + "\n")
        proc.stdin.flush()
        assert proc.stdout.readline().strip() == f"done {st['step']}"
    proc.stdin.close()
    assert proc.wait(timeout=120) == 0
    pm = plain.PlainDebusun(dirs(name), torch.float64)
    ref = {rid: pm.logits(t).float() for rid, t in reqs.items()}
    got, fed = {}, {rid: 0 for rid in reqs}
    for st in steps:
        wanted = sum(len(e["want"]) for e in st["entries"])
        arr = np.fromfile(out / f"{st['step']}.f32", dtype="<f4").reshape(wanted, vocab)
        row = 0
        for e in st["entries"]:
            for w in e["want"]:
                got[(e["id"], fed[e["id"]] + w)] = torch.from_numpy(arr[row].copy())
                row += 1
            fed[e["id"]] += len(e["tokens"])
    assert len(got) == sum(len(t) for t in reqs.values())
    harness.compare(got, ref, harness.TOL[dtype], f"trace_run {dtype}")


def test_decode_graph_replays_equal_launches(dirs):
    """float32: steps replayed from a recorded graph give the bits of the same steps launched one by one (the
    states, the convolution's inputs and the tokens before are advanced once a step, in the step that records too)."""
    from xinfer_amd.engine import ModelRunner, StepEntry
    name = "A"
    model = _model(name, "float32", dirs(name))
    vocab, page = MODELS[name]["config"]["vocab"], MODELS[name]["page_size"]
    rng = random.Random(21)
    prompts = {i: harness.random_prompt(rng, rng.randrange(3, 50), vocab) for i in range(4)}
    feed = {i: harness.random_prompt(rng, 30, vocab) for i in prompts}

    def run(use_graphs):
        runner = ModelRunner(model, page, 24, 4, use_graphs=use_graphs, graph_after=1)
        out = []
        for i in prompts:
            runner.add_request(i)
            runner.step([StepEntry(i, prompts[i], [])])
        for step in range(30):
            out.append(runner.step([StepEntry(i, [feed[i][step]], [0]) for i in prompts]).cpu())
        return out, runner
    want, _ = run(False)
    got, r1 = run(True)
    assert r1.graph_replays >= 25
    for k, (a, b) in enumerate(zip(want, got)):
        assert torch.equal(a, b), f"step {k} differs between graph and launches"
