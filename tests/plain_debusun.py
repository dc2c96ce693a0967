"""A plain, slow Debusun written from the design's equations: one function a mechanism, every token of a
sequence at once, no cache, no batching, no kernels.  It reads a model folder by itself (config.json,
model.safetensors through the safetensors library) and shares no code with the engine.

Notation: x the residual stream [T, width], h a sublayer's input, p a token's position (from 0).
"""
import json
import math
import os

import torch
from safetensors import safe_open


# ---- small functions ---------------------------------------------------------------------------------
def rms_norm(x, eps, w=None):
    """x / sqrt(mean(x^2) + eps) over the last axis, times w if given."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


# ---- embedding ---------------------------------------------------------------------------------------
def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """The row of the pair table for every token: (prev * mul_prev + cur * mul_cur) mod buckets, and row
    number `buckets` for a sequence's first token."""
    rows = [buckets]
    for a, b in zip(tokens[:-1], tokens[1:]):
        rows.append((a * mul_prev + b * mul_cur) % buckets)
    return rows


def embed(tokens, table, scale, pair_table, bigram):
    x = table[torch.tensor(tokens)] * scale
    return x + pair_table[torch.tensor(bigram_rows(tokens, bigram["buckets"], bigram["mul_prev"], bigram["mul_cur"]))]


# ---- rotary positions --------------------------------------------------------------------------------
def rotary_frequencies(rot):
    """(f_i, factor on cos and sin): f_i = base^(-2i / dims); with `scaling` (factor, original, fast, slow)
    frequency i becomes f_i / factor * r_i + f_i (1 - r_i), r_i a ramp from 0 to 1 between the dims at which
    `fast` and `slow` turns fit into `original` positions, and cos and sin grow by 0.1 ln(factor) + 1."""
    d, base = rot["dims"], rot["base"]
    f = [base ** (-2.0 * i / d) for i in range(d // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=torch.float64), 1.0

    def dim_of(turns):
        return d * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(dim_of(sc["fast"])), 0)
    hi = min(math.ceil(dim_of(sc["slow"])), d - 1)
    out = []
    for i, fi in enumerate(f):
        r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / sc["factor"] * r + fi * (1 - r))
    return torch.tensor(out, dtype=torch.float64), 0.1 * math.log(sc["factor"]) + 1.0


def rotate(x, rot, positions):
    """x [T, heads, n]: dims 2i and 2i + 1, i < rot.dims / 2, of every head turn by the angle p f_i:
    (u, v) -> (u cos - v sin, v cos + u sin); dims from rot.dims on pass unchanged."""
    d = rot["dims"]
    f, m = rotary_frequencies(rot)
    ang = positions.to(torch.float64)[:, None] * f[None, :]
    c, s = (ang.cos() * m)[:, None, :].to(x.dtype), (ang.sin() * m)[:, None, :].to(x.dtype)
    u, v = x[..., 0:d:2], x[..., 1:d:2]
    turned = torch.stack([u * c - v * s, v * c + u * s], dim=-1).reshape(*x.shape[:-1], d)
    return torch.cat([turned, x[..., d:]], dim=-1)


# ---- softmax over a window, with or without a sink ------------------------------------------------------
def window_softmax(scores, window, sink=None):
    """scores [T, T] (query i, key j): j is seen if 0 <= i - j < window; the weights' denominator also holds
    exp(sink) if a sink is given: one more weight that no value goes with."""
    T = scores.shape[0]
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    seen = (j <= i) & (i - j < window)
    s = scores.masked_fill(~seen, float("-inf"))
    m = s.max(dim=-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, torch.full_like(m, float(sink)))
    e = torch.exp(s - m)
    den = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink - m)
    return e / den


def _window(m):
    return m["mask"]["size"] if m.get("mask") else 1 << 30


# ---- the three mixers ------------------------------------------------------------------------------------
def attention_heads(q, k, v, m, eps, positions):
    """q [T, H, d], k [T, G, d], v [T, G, dv] as projected: rotation, then each q and k head divided by its root mean
    square, scores times scale over the window, softmax; query head i reads kv head i // (H / G).  Returns [T, H dv]."""
    T, H, _ = q.shape
    G, dv = k.shape[1], v.shape[2]
    if m.get("rot"):
        q, k = rotate(q, m["rot"], positions), rotate(k, m["rot"], positions)
    q, k = rms_norm(q, eps), rms_norm(k, eps)
    out = torch.zeros(T, H, dv, dtype=q.dtype)
    for hd in range(H):
        g = hd // (H // G)
        p = window_softmax((q[:, hd] @ k[:, g].T) * m["scale"], _window(m))
        out[:, hd] = p @ v[:, g]
    return out.reshape(T, H * dv)


def attention(h, w, m, eps, positions):
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    heads = attention_heads((h @ w["q"].T).view(T, H, d), (h @ w["k"].T).view(T, G, d), (h @ w["v"].T).view(T, G, dv), m, eps,
                            positions)
    return heads @ w["o"].T


def latent_heads(q, down, w, m, eps, positions):
    """q [T, H, d + r] and down [T, rank + r] as projected; w holds dkv.norm, uk, uv, sink.  Returns the heads
    [T, H dv] before the gate."""
    H, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = q.shape[0]
    q_plain, q_turned = q[..., :d], rotate(q[..., d:], m["rot"], positions)
    c = rms_norm(down[:, :rank], eps, w["dkv.norm"])
    k_turned = rotate(down[:, None, rank:], m["rot"], positions)[:, 0]          # one part for all heads
    k_plain = (c @ w["uk"].T).view(T, H, d)
    v = (c @ w["uv"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=q.dtype)
    for hd in range(H):
        s = (q_plain[:, hd] @ k_plain[:, hd].T + q_turned[:, hd] @ k_turned.T) * m["scale"]
        out[:, hd] = window_softmax(s, _window(m), sink=w["sink"][hd]) @ v[:, hd]
    return out.reshape(T, H * dv)


def latent_attention(h, w, m, eps, positions):
    T = h.shape[0]
    heads = latent_heads((h @ w["q"].T).view(T, m["heads"], m["dim"] + m["rot_dim"]), h @ w["dkv"].T, w, m, eps, positions)
    return (heads * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


def causal_conv(u, taps_w, bias):
    """u [T, C]; taps_w [C, taps]: column taps - 1 - k weighs the input k tokens back; nothing comes before a sequence."""
    T, C = u.shape
    taps = taps_w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u], dim=0)
    out = bias[None, :].expand(T, C).clone()
    for j in range(taps):
        out = out + padded[j:j + T] * taps_w[:, j][None, :]
    return out


def state_space(x, B, C, dt, decay_log, skip, state=None):
    """x [T, H, dv], B and C [T, G, N], dt [T, H] (step sizes, after the softplus): per head i (group i // (H / G))
    S <- exp(-exp(decay_log_i) dt) S + dt B x^T, y = S^T C + skip_i x.  Returns (y [T, H, dv], the last S [H, N, dv])."""
    T, H, dv = x.shape
    G, N = B.shape[1], B.shape[2]
    decay = torch.exp(-torch.exp(decay_log)[None, :] * dt)                     # [T, H]
    y = torch.zeros(T, H, dv, dtype=x.dtype)
    S = torch.zeros(H, N, dv, dtype=x.dtype) if state is None else state.clone()
    for hd in range(H):
        g = hd // (H // G)
        for t in range(T):
            S[hd] = decay[t, hd] * S[hd] + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S[hd].T @ C[t, g] + skip[hd] * x[t, hd]
    return y, S


def gated_group_norm(y, z, weight, eps, parts):
    """y, z [T, inner]: y * silu(z), each of `parts` equal parts of a row divided by its root mean square, times weight."""
    T, inner = y.shape
    y = y * silu(z)
    return rms_norm(y.view(T, parts, inner // parts), eps).reshape(T, inner) * weight


def mamba2(h, w, m, eps):
    H, dv, N, G, parts = m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]
    inner = H * dv
    T = h.shape[0]
    p = h @ w["in"].T
    z, xbc, dt = p[:, :inner], p[:, inner:2 * inner + 2 * G * N], p[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w["conv"], w["conv.b"]))
    x = xbc[:, :inner].view(T, H, dv)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    y, _ = state_space(x, B, C, softplus(dt + w["dt_bias"]), w["A_log"], w["D"])
    return gated_group_norm(y.reshape(T, inner), z, w["norm"], eps, parts) @ w["o"].T


def dense_mlp(h, w):
    return (torch.relu(h @ w["up"].T) ** 2) @ w["down"].T


# ---- the model ---------------------------------------------------------------------------------------------
class PlainDebusun:
    def __init__(self, model_dir, dtype=torch.float64):
        with open(os.path.join(model_dir, "config.json")) as f:
            self.cfg = json.load(f)
        self.dtype = dtype
        self.w = {}
        with safe_open(os.path.join(model_dir, "model.safetensors"), "pt") as f:
            for name in f.keys():
                t = f.get_tensor(name)
                self.w[name] = t.to(dtype) if t.is_floating_point() else t

    def _sub(self, prefix):
        return {k[len(prefix):]: v for k, v in self.w.items() if k.startswith(prefix)}

    def run_order(self):
        """(layer, number of the pass or None) for every run of a layer; a pass's first run is marked."""
        n = len(self.cfg["layers"])
        loop = self.cfg.get("loop")
        if not loop:
            return [(i, None, False) for i in range(n)]
        a, b, times = loop["start"], loop["stop"], loop["times"]
        order = [(i, None, False) for i in range(a)]
        for t in range(times):
            order += [(i, t, i == a) for i in range(a, b)]
        return order + [(i, None, False) for i in range(b, n)]

    def stream(self, tokens):
        """The residual stream after the embedding and after every run of a layer."""
        cfg, eps = self.cfg, self.cfg["norm"]["eps"]
        T = len(tokens)
        positions = torch.arange(T)
        e = cfg["embedding"]
        x = embed(tokens, self.w["embed"], e["scale"], self.w["bigram"], e["bigram"])
        first = x.clone()
        out = [x.clone()]
        for i, t, starts in self.run_order():
            if starts:
                if t > 0:
                    x = x + first
                x = x + self.w["loop.step"][t]
            l = cfg["layers"][i]
            h = rms_norm(x, eps, self.w[f"l{i}.norm1"])
            w = self._sub(f"l{i}.mix.")
            if l["type"] == "attention":
                x = x + attention(h, w, l["mixer"], eps, positions)
            elif l["type"] == "latent_attention":
                x = x + latent_attention(h, w, l["mixer"], eps, positions)
            elif l["type"] == "mamba2":
                x = x + mamba2(h, w, l["mixer"], eps)
            else:
                raise ValueError(l["type"])
            if l.get("mlp") is not None:
                x = x + dense_mlp(rms_norm(x, eps, self.w[f"l{i}.norm2"]), self._sub(f"l{i}.mlp."))
            out.append(x.clone())
        return out

    def logits(self, tokens):
        x = self.stream(tokens)[-1]
        return rms_norm(x, self.cfg["norm"]["eps"], self.w["final.norm"]) @ self.w["head"].T

    def greedy(self, prompt, n):
        ids = list(prompt)
        for _ in range(n):
            ids.append(int(self.logits(ids)[-1].argmax()))
        return ids[len(prompt):]
