"""Vuzazen on the GPU against the plain implementation (tests/plain_vuzazen.py): each mechanism's kernel
alone, then whole models under every way of cutting the work, in float32 and bfloat16."""
import json
import math
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

import harness
import plain_vuzazen as plain
from vuzazen_models import MODELS, make_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]
TD = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 2e-5, "bfloat16": 2e-2}


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("vuzazen")
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


# ---- small kernels -----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,pad", [(80, 13), (7, 0), (24, 8), (300, 1)])
def test_rows_normed_out_of_a_packed_projection(n, pad, dtype):
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(n)
    packed = (torch.randn(9, n + pad, generator=g) * 3).to(TD[dtype])
    w = torch.randn(n, generator=g)
    got = kernels.rows_rmsnorm(packed.to(DEV)[:, :n], w.to(DEV), 1e-5, TD[dtype]).cpu().double()
    want = plain.rms_norm(packed[:, :n].double(), 1e-5, w.double())
    assert (got - want).abs().max() < (1e-6 if dtype == "float32" else 1e-2) * want.abs().max()
    one = kernels.rows_rmsnorm(packed.to(DEV)[:1, :n], None, 1e-5, torch.float32).cpu().double()
    assert (one - plain.rms_norm(packed[:1, :n].double(), 1e-5)).abs().max() < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
def test_one_gate_a_head(dtype):
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(4)
    T, H, dv = 11, 5, 12
    x = torch.randn(T, H * dv, generator=g).to(TD[dtype])
    packed = torch.randn(T, 7 + H, generator=g).to(TD[dtype])
    want = (x.double().view(T, H, dv) * torch.sigmoid(packed[:, 7:].double())[:, :, None]).reshape(T, H * dv)
    got = kernels.head_gate_(x.to(DEV).clone(), packed.to(DEV)[:, 7:], H).cpu().double()
    assert (got - want).abs().max() < (1e-6 if dtype == "float32" else 1e-2) * want.abs().max()
    # the same gate where the heads' products are stored
    K, N = 16, 24
    a = torch.randn(T, H, K, generator=g).to(TD[dtype])
    w = torch.randn(H, N, K, generator=g).to(TD[dtype])
    out = torch.empty(T, H, N, dtype=TD[dtype], device=DEV)
    kernels.head_linear(a.to(DEV), w.to(DEV), out, gate=packed.to(DEV)[:, 7:])
    want = torch.einsum("thk,hnk->thn", a.double(), w.double()) * torch.sigmoid(packed[:, 7:].double())[:, :, None]
    assert (out.cpu().double() - want).abs().max() < (1e-5 if dtype == "float32" else 1e-2) * want.abs().max()


# ---- the matrix memory --------------------------------------------------------------------------------------------
def _memory_inputs(T, H, dk, dv, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    packed = (torch.randn(T, 2 * H * dk + 2 * H * dv, generator=g) * 0.7).to(dtype)
    a = H * dk
    packed[:, a:2 * a] = (packed[:, :a].float() + 0.5 * packed[:, a:2 * a].float()).to(dtype)     # keys lean towards queries
    z = torch.randn(T, 2 * H, generator=g) * 5
    bias = torch.randn(2 * H, generator=g)
    bias[H:] += 2.0
    w = 1 + 0.2 * torch.randn(H * dv, generator=g)
    return packed, z, bias, w


def _plain_memory(packed, z, bias, w, H, dk, dv, cap, eps):
    T = packed.shape[0]
    p = packed.double()
    a, b = H * dk, H * dv
    q = p[:, :a].view(T, H, dk) * dk ** -0.5
    k, v, g = p[:, a:2 * a].view(T, H, dk), p[:, 2 * a:2 * a + b].view(T, H, dv), p[:, 2 * a + b:]
    zz = z.double() + bias.double()
    o, state = plain.matrix_memory(q, k, v, plain.capped(zz[:, :H], cap), plain.log_sigmoid(plain.capped(zz[:, H:], cap)))
    return plain.rms_norm(o, eps).reshape(T, b) * w.double() * torch.sigmoid(g), state


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk", [0, 16])
@pytest.mark.parametrize("H,dk,dv,cap", [(3, 16, 24, 8.0), (1, 20, 20, 15.0), (2, 24, 64, 4.0), (5, 6, 10, 30.0), (2, 128, 65, 12.5)])
def test_matrix_memory_of_unequal_requests_in_portions(H, dk, dv, cap, chunk, dtype, monkeypatch):
    """Three requests in slots that are not in order and were used before (the runner's part, clearing a slot, is done
    here by hand), cut into portions down to one token; long portions in chunks side by side."""
    from xinfer_amd import kernels
    monkeypatch.setattr(kernels, "SCAN_CHUNK", chunk)
    dt, eps = TD[dtype], 1e-5
    lens = [70, 1, 45]
    cuts = [[2, 64, 1, 3], [1], [40, 1, 1, 3]]
    slots = [3, 0, 2]
    ins = [_memory_inputs(n, H, dk, dv, 10 * H + i, dt) for i, n in enumerate(lens)]
    bias, w = ins[0][2], ins[0][3]
    state = torch.full((5, H, dk, dv + 1), 7.0, device=DEV)
    m_state = torch.full((5, H), 3.0, device=DEV)
    for s in slots:
        state[s] = 0
        m_state[s] = 0
    got = [[] for _ in lens]
    a, b = H * dk, H * dv
    for rows in _steps(cuts):
        cu, _, _ = _step_index(rows)
        p = torch.cat([ins[r][0][s:s + n] for r, s, n in rows]).to(DEV)
        z = torch.cat([ins[r][1][s:s + n] for r, s, n in rows]).to(DEV)
        st = _i64([slots[r] for r, _, _ in rows])
        gates, floor = kernels.mlstm_gates(z, bias.to(DEV), cap, m_state, st, _i32(cu), H)
        o = kernels.linear_scan(p[:, :a], p[:, a:2 * a], p[:, 2 * a:2 * a + b], state, st, _i32(cu), H, dk, dv + 1, gates=gates,
                                value_cols=dv, q_scale=dk ** -0.5, q_lens=[n for _, _, n in rows], plan_cache={})
        out = kernels.mlstm_finish(o, floor, w.to(DEV), eps, p[:, 2 * a + b:], dt)
        for i, (r, _, _) in enumerate(rows):
            got[r].append(out[cu[i]:cu[i + 1]].cpu())
    assert float(state[1].min()) == 7.0 and float(m_state[4].min()) == 3.0
    for r, n in enumerate(lens):
        want, (S, nn, m) = _plain_memory(ins[r][0], ins[r][1], bias, w, H, dk, dv, cap, eps)
        err = (torch.cat(got[r]).double() - want).abs().max(dim=1).values
        bad = (err > (1e-4 if dtype == "float32" else 3e-2) * want.abs().max()).nonzero()
        assert bad.numel() == 0, f"request {r}: first wrong token {int(bad[0])}: {float(err[int(bad[0])]):.3e}"
        assert (m_state[slots[r]].cpu().double() - m).abs().max() < 1e-5
        assert (state[slots[r], :, :, :dv].cpu().double() - S).abs().max() < 1e-4 * max(1.0, float(S.abs().max()))
        assert (state[slots[r], :, :, dv].cpu().double() - nn).abs().max() < 1e-4 * max(1.0, float(nn.abs().max()))


@pytest.mark.parametrize("far", [599, 300, 40])
def test_matrix_memory_keeps_a_far_token(far):
    """One token's input gate is wide open and every forget gate nearly 1: the token planted `far` back is what a
    query that matches its key reads, through single tokens and through chunks."""
    from xinfer_amd import kernels
    H, dk, dv, cap, eps = 2, 16, 8, 20.0, 1e-6
    T = far + 5
    g = torch.Generator().manual_seed(far)
    packed = torch.randn(T, 2 * H * dk + 2 * H * dv, generator=g) * 0.1
    a, b = H * dk, H * dv
    u = torch.zeros(dk)
    u[3] = 4.0
    packed[2, a:a + dk] = u                               # head 0's key of token 2
    packed[2, 2 * a:2 * a + dv] = torch.arange(dv) - 3.0     # and its value
    packed[T - 1, :dk] = u * 4                             # the last token's query
    packed[:, 2 * a + b:] = 0                              # every output gate half open
    z = torch.zeros(T, 2 * H)
    z[:, :H] = -18.0                                       # input gates shut
    z[2, 0] = 18.0                                         # but this one
    z[:, H:] = 19.0                                        # forget gates as open as the cap lets them be
    bias = torch.zeros(2 * H)
    w = torch.ones(H * dv)
    want, _ = _plain_memory(packed, z, bias, w, H, dk, dv, cap, eps)
    v2 = packed[2, 2 * a:2 * a + dv].double()
    assert (want[T - 1, :dv] / want[T - 1, 0] - v2 / v2[0]).abs().max() < 1e-3        # the planted value, up to the norm
    for cut in ([T], [T - 3, 1, 1, 1], [7] + [1] * (T - 7)):
        state = torch.zeros(1, H, dk, dv + 1, device=DEV)
        m_state = torch.zeros(1, H, device=DEV)
        outs, at = [], 0
        for n in cut:
            p, zz = packed[at:at + n].to(DEV), z[at:at + n].to(DEV)
            gates, floor = kernels.mlstm_gates(zz, bias.to(DEV), cap, m_state, _i64([0]), _i32([0, n]), H)
            o = kernels.linear_scan(p[:, :a], p[:, a:2 * a], p[:, 2 * a:2 * a + b], state, _i64([0]), _i32([0, n]), H, dk, dv + 1,
                                    gates=gates, value_cols=dv, q_scale=dk ** -0.5, q_lens=[n], plan_cache={})
            outs.append(kernels.mlstm_finish(o, floor, w.to(DEV), eps, p[:, 2 * a + b:], torch.float32).cpu())
            at += n
        got = torch.cat(outs).double()
        assert (got - want).abs().max() < 1e-4 * want.abs().max(), f"cut {cut[:4]}"


# ---- rows of the attention with a convolution and mixed heads ------------------------------------------------------
def _pools(L, G, d, dv, page, dtype, grouped, one_key_head, seed=0):
    """Empty K and V pools with more pages than L tokens need, and a block table of shuffled pages."""
    n_pages = -(-L // page)
    order = list(range(n_pages + 3))
    random.Random(seed).shuffle(order)
    table = torch.tensor([order[:n_pages]], dtype=torch.int32)
    k_pool = torch.zeros((n_pages + 3, 1, page, G * d) if one_key_head else (n_pages + 3, G, page, d), dtype=dtype)
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
    return k.reshape(L, -1), v


def _folded_queries(q, talk, G):
    """q [T, H, d] -> q' [T, H, G d]: part c of q'_h is sum over the heads g of kv head c of talk[h, g] q_g."""
    T, H, d = q.shape
    per = H // G
    out = torch.zeros(T, H, G, d, dtype=q.dtype)
    for h in range(H):
        for g_ in range(H):
            out[:, h, g_ // per] += talk[h, g_] * q[:, g_]
    return out.reshape(T, H, G * d)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d,dv,taps,page,norms,talks", [
    (6, 2, 16, 24, 3, 16, True, True), (5, 5, 20, 20, 2, 8, True, True), (3, 1, 12, 20, 5, 8, True, True),
    (4, 2, 8, 16, 1, 16, True, True), (4, 2, 8, 24, 0, 16, True, True), (4, 2, 128, 64, 3, 64, True, True), (6, 3, 8, 16, 4, 8, False, False), (2, 2, 16, 8, 3, 8, True, False)])
def test_rows_after_the_convolution_the_norms_and_the_heads_mix(H, G, d, dv, taps, page, norms, talks, dtype):
    """A request in portions (some shorter than the taps), beside another request whose tail must not be touched: q (or
    q' with mixed heads) and what the cache holds against the plain convolution, norms and unit values."""
    from xinfer_amd import kernels
    dt, eps = TD[dtype], 1e-5
    grouped = dtype == "bfloat16"
    L = 61
    C = H * d + G * d + G * dv
    g = torch.Generator().manual_seed(H * 100 + taps)
    packed = torch.randn(L, C + H, generator=g).to(dt)                      # the heads' gates ride behind
    cw = torch.randn(C, max(taps, 1), generator=g) * 0.6
    qw, kw = (1 + 0.3 * torch.randn(H * d, generator=g), 1 + 0.3 * torch.randn(G * d, generator=g)) if norms else (None, None)
    talk = (torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)).to(torch.bfloat16).float() if talks else None
    u = packed[:, :C].double()
    y = plain.short_conv(u, cw.double()) if taps >= 1 else u          # one tap: a factor a channel; none: no convolution
    q, k, v = y[:, :H * d], y[:, H * d:H * d + G * d], y[:, H * d + G * d:].view(L, G, dv)
    if norms:
        q, k = plain.rms_norm(q, eps, qw.double()), plain.rms_norm(k, eps, kw.double())
    v = plain.rms_norm(v, eps)
    want_q = _folded_queries(q.view(L, H, d), talk.double(), G) if talks else q.view(L, H, d)
    k_pool, v_pool, table, slots = _pools(L, G, d, dv, page, dt, grouped, talks, seed=taps)
    k_pool, v_pool = k_pool.to(DEV), v_pool.to(DEV)
    tails = torch.full((3, max(taps - 1, 1), C), 5.0, device=DEV)[:, :taps - 1] if taps > 1 else None
    if taps > 1:
        tails = tails.contiguous()
        tails[1] = 0
    cuts = [1, 1, 3, 2, 20, 1, 33] if taps > 1 else [L]
    outs, at = [], 0
    for n in cuts:
        rows = packed[at:at + n].to(DEV)
        sl = slots[at:at + n].clone()
        if at <= 5 < at + n:
            sl[5 - at] = -1                                                   # a token that stores nothing
        qo = kernels.conv_qkv_rows(rows, cw.to(DEV) if taps >= 1 else None, tails, _i64([1]), _i32([0] * n), _i32([0, n]),
                                   None if qw is None else qw.to(DEV), None if kw is None else kw.to(DEV), eps, sl.to(DEV), k_pool, v_pool,
                                   H, G, d, dv, v_grouped=grouped, value_unit_norm=True, talk=None if talk is None else talk.to(DEV))
        if taps > 1:
            kernels.conv_tail(rows[:, :C], tails, _i64([1]), _i32([0, n]))
        outs.append(qo.cpu())
        at += n
    tol = 1e-5 if dtype == "float32" else 1.5e-2
    got_q = torch.cat(outs).double()
    assert got_q.shape == want_q.shape and (got_q - want_q).abs().max() < tol * want_q.abs().max()
    got_k, got_v = _read_pools(k_pool.cpu(), v_pool.cpu(), table, L, grouped)
    keep = [p for p in range(L) if p != 5]
    assert (got_k.double()[keep] - k[keep]).abs().max() < tol * k.abs().max()
    assert (got_v.double()[keep] - v[keep]).abs().max() < tol * v.abs().max()
    assert float(got_k[5].abs().max()) == 0 and float(got_v[5].abs().max()) == 0
    if taps > 1:
        assert torch.equal(tails[1].cpu(), packed[L - taps + 1:, :C].float()) and float(tails[0].min()) == 5.0 and float(tails[2].max()) == 5.0


# ---- mixed heads' attention over planted keys -------------------------------------------------------------------------
def _planted(L, H, G, d, scale, seed, big_score=30.0):
    """q [L, H, d] and k [L, G, d] of one sequence in which chosen (query, key) pairs have a score that stands far
    out: keys at page borders, the first tokens, far back among hundreds."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(L, H, d, generator=g) * 0.3
    k = torch.randn(L, G, d, generator=g) * 0.3
    big = big_score / scale
    pairs = []
    for i in list(range(L - 12, L)) + [1, 2, 17, 31, 32, 63, 64, 65, 128]:
        if not (0 <= i < L):
            continue
        for j in (i, i - 1, i - 15, i - 16, i - 17, i - 63, i - 64, i - 65, 0, 1, i - L // 2, i - L + 3):
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


MIXED_CASES = [  # H, G, d, dv, scale, L, page
    (6, 2, 16, 24, 0.4, 90, 16),
    (8, 2, 64, 64, 0.11, 300, 64),
    (5, 5, 24, 24, 0.3, 70, 8),
    (3, 1, 12, 20, 0.5, 150, 8),
    (4, 2, 128, 64, 0.09, 400, 64),
    (6, 3, 32, 128, 0.18, 200, 32),
    (24, 2, 64, 128, 0.12, 130, 16),          # twelve heads a group: a group's rows in one block, or in two
    (40, 2, 32, 64, 0.2, 100, 16),            # twenty heads a group
    (4, 4, 64, 64, 0.12, 200, 64),
    (12, 12, 64, 32, 0.12, 100, 16),          # a key head of 768 dims: the generic kernel alone
]


def _mixed_case(case, dtype, matrix_cores, tail=9):
    from xinfer_amd import kernels
    H, G, d, dv, scale, L, page = case
    dt = TD[dtype]
    grouped = dtype == "bfloat16"
    q, k = _planted(L, H, G, d, scale, seed=L)
    g = torch.Generator().manual_seed(L)
    v = torch.randn(L, G, dv, generator=g)
    talk = (torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)).to(torch.bfloat16).float()
    q, k, v = q.to(dt), k.to(dt), v.to(dt)
    scores = plain.mixed_head_scores(q.double(), k.double(), scale, talk.double())
    own = plain.mixed_head_scores(q.double(), k.double(), scale, torch.eye(H, dtype=torch.float64))
    want = torch.stack([plain.causal_softmax(scores[h]) @ v.double()[:, h // (H // G)] for h in range(H)], dim=1).reshape(L, H * dv)
    unmixed = torch.stack([plain.causal_softmax(own[h]) @ v.double()[:, h // (H // G)] for h in range(H)], dim=1).reshape(L, H * dv)
    assert (want - unmixed).abs().max() > 0.1 * want.abs().max()              # the mix matters here
    k_pool, v_pool, table, slots = _pools(L, G, d, dv, page, dt, grouped, True, seed=L)
    packed = torch.cat([q.reshape(L, -1), k.reshape(L, -1), v.reshape(L, -1)], dim=1).to(DEV)
    k_pool, v_pool, table = k_pool.to(DEV), v_pool.to(DEV), table.to(DEV)
    qf = kernels.conv_qkv_rows(packed, None, None, _i64([0]), _i32([0] * L), _i32([0, L]), None, None, 1e-5, slots.to(DEV), k_pool,
                               v_pool, H, G, d, dv, v_grouped=grouped, value_unit_norm=False, talk=talk.to(DEV))
    if dtype == "bfloat16":
        # what the attention kernels are held to: the scores of the mixed queries as they were rounded (the mix itself
        # is held to the plain one where the rows are tested; planted scores of 30 make its rounding show in the weights)
        mixed = torch.einsum("ihx,jx->hij", qf.cpu().double(), k.double().reshape(L, G * d)) * scale
        assert (mixed - scores).abs().max() < 0.02 * scores.abs().max()
        want = torch.stack([plain.causal_softmax(mixed[h]) @ v.double()[:, h // (H // G)] for h in range(H)], dim=1).reshape(L, H * dv)

    def run(positions):
        qs = qf[positions[0]:positions[-1] + 1]
        pos = _i32(positions)
        if not matrix_cores:
            return kernels.attention_generic(qs, k_pool, v_pool, table, torch.zeros_like(pos), pos, scale, 0, v_grouped=grouped)
        n, ctx = len(positions), positions[-1] + 1
        per = H // G
        if n == 1 and per >= 4:                     # a group's heads as the rows of blocks that read the one key head
            shape = 1 if kernels.attention_biased_block(G * d, dv, 1, 1) >= per else 0
            rows_ = kernels.attention_biased_block(G * d, dv, 1, shape)
            tiles = _i32([[0, c * per + b * rows_] for c in range(G) for b in range(-(-per // rows_))])
            out = kernels.attention_biased_bf16(qs.reshape(H, 1, G * d), k_pool, v_pool, table, tiles, _i32([0, H]), _i32([ctx]), scale, 0,
                                                small=shape, split_keys=64 if positions[0] % 2 else 0, span=ctx, rows_heads=H)
            return out.view(1, H * dv)
        rows, shape = kernels.prefill_tiles([n], [ctx], G * d, H, G, block_of=lambda s_: kernels.attention_biased_block(G * d, dv, H // G, s_))
        tiles = torch.tensor(rows, dtype=torch.int32, device=DEV).reshape(-1, 2)
        split, span = (64, ctx) if n == 1 and positions[0] % 2 else (0, 0)     # every other single token in slices of 64 keys
        return kernels.attention_biased_bf16(qs, k_pool, v_pool, table, tiles, _i32([0, n]), _i32([ctx]), scale, 0, small=shape,
                                             split_keys=split, span=span)
    head = L - tail
    outs = [run(list(range(head)))] + [run([p]) for p in range(head, L)]
    got = torch.cat([o.cpu() for o in outs]).double()
    err = (got - want).abs().max(dim=1).values
    bad = (err > TOL[dtype] * want.abs().max()).nonzero()
    assert bad.numel() == 0, f"first wrong position {int(bad[0])} of {L}: {float(err[int(bad[0])]):.3e}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", MIXED_CASES)
def test_mixed_heads_attention_with_planted_keys(case, dtype):
    _mixed_case(case, dtype, matrix_cores=False)


@pytest.mark.parametrize("case", [c for c in MIXED_CASES if c[1] * c[2] <= 256 and (c[1] * c[2]) % 8 == 0 and c[3] % 8 == 0])
def test_mixed_heads_attention_on_the_matrix_cores(case):
    _mixed_case(case, "bfloat16", matrix_cores=True)


# ---- experts that see the token times its score -------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,width,ff,experts,top", [(37, 96, 40, 4, 2), (9, 100, 24, 2, 1), (50, 50, 18, 6, 4), (300, 64, 32, 8, 3), (1, 72, 24, 3, 3)])
def test_experts_weighted_on_their_input(T, width, ff, experts, top, dtype):
    from xinfer_amd import kernels
    dt = TD[dtype]
    g = torch.Generator().manual_seed(T)
    x = torch.randn(T, width, generator=g).to(dt)
    router = torch.zeros(experts, width)
    router[:, :3] = torch.randn(experts, 3, generator=g) * 2
    x[:, :3] = (torch.randint(0, 2, (T, 3), generator=g).float() * 2 - 1).to(dt)          # the choice is clear
    w = {"router": router.to(torch.bfloat16).double()}
    gu, dn = [], []
    for e in range(experts):
        ws = [(torch.randn(ff, width, generator=g) * 0.2).to(dt), (torch.randn(ff, width, generator=g) * 0.2).to(dt),
              (torch.randn(width, ff, generator=g) * 0.2).to(dt)]
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = (t.double() for t in ws)
        gu.append(torch.cat(ws[:2]))
        dn.append(ws[2])
    want = plain.routed_experts(x.double(), w, {"router": {"experts": experts, "top": top}})
    z = x.double() @ w["router"].T
    srt = z.sort(dim=-1, descending=True).values
    if top < experts:
        assert float((srt[:, top - 1] - srt[:, top]).min()) > 0.05
    gate_up, down = torch.stack(gu).to(DEV), torch.stack(dn).to(DEV)
    idx, wt = kernels.moe_route(x.to(DEV), w["router"].float().to(DEV), None, top, sigmoid=True)
    assert (wt.cpu().double().sort(dim=-1, descending=True).values - torch.sigmoid(srt[:, :top])).abs().max() < 1e-5
    tol = 1e-5 if dtype == "float32" else 2e-2
    got = kernels.moe_experts(x.to(DEV), gate_up, down, idx, wt, "silu", grouped=False, weigh_input=True).cpu().double()
    assert (got - want).abs().max() < tol * want.abs().max()
    plain_weights = kernels.moe_experts(x.to(DEV), gate_up, down, idx, wt, "silu", grouped=False).cpu().double()
    assert (plain_weights - want).abs().max() > 0.02 * want.abs().max()        # where the weight stands matters
    if dtype == "bfloat16" and width % 8 == 0 and ff % 8 == 0:
        for rows in (32, 64, 128):
            grouped = kernels.moe_experts(x.to(DEV), gate_up, down, idx, wt, "silu", grouped=True, tile_rows=rows,
                                          weigh_input=True).cpu().double()
            assert (grouped - want).abs().max() < tol * want.abs().max(), f"tiles of {rows} rows"
        lib = kernels.moe_experts_library(x.to(DEV), gate_up, down, idx, wt, "silu", weigh_input=True).cpu().double()
        assert (lib - want).abs().max() < tol * want.abs().max()


# ---- whole models ----------------------------------------------------------------------------------------------------
LENGTHS = {"A": [1, 2, 12, 13, 33, 77, 130], "B": [3, 9, 10, 18, 64, 101], "C": [1, 7, 8, 40, 75, 210], "M": [2, 1, 30, 140],
           "R": [5, 101, 330, 64, 301], "S": [3, 70, 71, 260, 129]}


def _requests(name):
    rng = random.Random(700 + ord(name))
    vocab = MODELS[name]["config"]["vocab"]
    return {f"r{i}": harness.random_prompt(rng, n, vocab) for i, n in enumerate(LENGTHS[name])}


_plain_cache = {}
_model_cache = {}


def _plain_logits(name, model_dir):
    if name not in _plain_cache:
        pm = plain.PlainVuzazen(model_dir, torch.float64)
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
    assert len(model.spec.schedule) == len(cfg["layers"]) == len(model.blocks)
    assert model.graph_safe and model.head.tied
    toks = _requests(name)[f"r{len(LENGTHS[name]) - 1}"]
    pm = plain.PlainVuzazen(dirs(name), torch.float64)
    x = pm.stream(toks)
    for i, l in enumerate(cfg["layers"]):           # the routers' choices are clear, and not always the same
        ml = l.get("mlp")
        if ml and ml["kind"] == "moe" and ml["router"]["top"] < ml["router"]["experts"]:
            # (the stream between the layer's two sublayers is not kept: the marker columns are the same in both)
            h = plain.rms_norm(x[i + 1], cfg["norm"]["eps"], plain.layer_norm_weight(pm.w[f"l{i}.norm2"]))
            z = (h @ pm.w[f"l{i}.mlp.router"].T).sort(dim=-1, descending=True)
            top = ml["router"]["top"]
            assert float((z.values[:, top - 1] - z.values[:, top]).min()) > 0.02
            assert len(set(z.indices[:, 0].tolist())) > 1


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_whole(name, dtype, dirs):
    got, _ = _run(name, dtype, dirs, harness.trace_whole(_requests(name)), "whole")
    assert len(got) == sum(LENGTHS[name])


@pytest.mark.parametrize("name", ["A", "B", "C", "M"])
def test_the_stream_after_every_layer(name, dirs):
    """float32, one request: the residual stream after every layer against the plain one."""
    from xinfer_amd.engine import ModelRunner, StepEntry
    model = _model(name, "float32", dirs(name))
    toks = _requests(name)["r2"]
    want = plain.PlainVuzazen(dirs(name), torch.float64).stream(toks)[1:]
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
        assert (a - b).abs().max() < 2e-5 * b.abs().max(), f"the stream after layer {i} differs"


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
    finds no memory, no running maximum, no last token and no convolution inputs of the one before."""
    for seed in (1, 2):
        _run(name, dtype, dirs, harness.trace_mixed(_requests(name), seed, max_live=3), f"mixed {seed}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "R", "M"])
def test_short_chunks_of_the_memorys_walk(name, dtype, dirs, monkeypatch):
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
def test_long_decoding(name, dtype, dirs):
    """Three tokens of prompt, then the rest one by one: the memories, the convolutions' inputs and the caches grow
    token by token, over several pages."""
    n = 253 if name == "A" else 340
    toks = harness.random_prompt(random.Random(9), n, MODELS[name]["config"]["vocab"])
    from xinfer_amd.engine import ModelRunner
    ref = {"a": plain.PlainVuzazen(dirs(name), torch.float64).logits(toks).float()}
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
    pm = plain.PlainVuzazen(dirs(name), torch.float64)
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
    rc = cli.main(["--w", dirs("M"), "--prompt-ids", "1,2,3|4,5,6,7", "--max-tokens", "5", "--max-model-len", "64",
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
    pm = plain.PlainVuzazen(dirs(name), torch.float64)
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
    memories, their maxima, the convolution's inputs and the tokens before are advanced once a step, in the step that
    records too)."""
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
