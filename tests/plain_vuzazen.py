"""A plain, slow Vuzazen written from the design's equations: one function a mechanism, every token of a
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


def layer_norm_weight(w):
    """A norm's tensor holds its factor's distance from one: the factor is 1 + w."""
    return 1.0 + w


def silu(z):
    return z * torch.sigmoid(z)


def log_sigmoid(z):
    return -torch.where(z < -30, -z, torch.log1p(torch.exp(-torch.clamp(z, min=-30))))


def causal_softmax(scores):
    """scores [T, T] (query i, key j): j is seen if j <= i."""
    T = scores.shape[0]
    seen = torch.arange(T)[None, :] <= torch.arange(T)[:, None]
    return torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1)


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


# ---- rotary positions, pairs (i, i + dims / 2) ----------------------------------------------------------
def rotate_half(x, rot, positions):
    """x [T, heads, n]: dims i and i + dims / 2, i < dims / 2, of every head turn by the angle p f_i, f_i =
    base^(-2i / dims): (u, v) -> (u cos - v sin, v cos + u sin); dims from rot.dims on pass unchanged."""
    d, half = rot["dims"], rot["dims"] // 2
    f = torch.tensor([rot["base"] ** (-2.0 * i / d) for i in range(half)], dtype=torch.float64)
    ang = positions.to(torch.float64)[:, None] * f[None, :]
    c, s = ang.cos()[:, None, :].to(x.dtype), ang.sin()[:, None, :].to(x.dtype)
    u, v = x[..., :half], x[..., half:d]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., d:]], dim=-1)


# ---- the matrix memory ------------------------------------------------------------------------------------
def capped(z, cap):
    return cap * torch.tanh(z / cap)


def matrix_memory(q, k, v, log_in, log_keep, state=None):
    """q, k [T, H, dk], v [T, H, dv], log_in and log_keep [T, H] (the logarithms of the input gate and of the
    forget gate).  Per head, with the running maximum m (0 at the start, like S and n):
        m' = max(log_keep + m, log_in);  S' = exp(log_keep + m - m') S + exp(log_in - m') k v^T;  n' likewise with k
        o = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)
    Returns (o [T, H, dv], (S, n, m))."""
    T, H, dk = q.shape
    dv = v.shape[2]
    if state is None:
        S, n, m = torch.zeros(H, dk, dv, dtype=q.dtype), torch.zeros(H, dk, dtype=q.dtype), torch.zeros(H, dtype=q.dtype)
    else:
        S, n, m = (s.clone() for s in state)
    o = torch.zeros(T, H, dv, dtype=q.dtype)
    for t in range(T):
        m_new = torch.maximum(log_keep[t] + m, log_in[t])
        keep = torch.exp(log_keep[t] + m - m_new)
        take = torch.exp(log_in[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        m = m_new
        num = torch.einsum("hkv,hk->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        o[t] = num / den[:, None]
    return o, (S, n, m)


def mlstm(h, w, m, eps):
    H, dk, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    T = h.shape[0]
    q = (h @ w["q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ w["k"].T).view(T, H, dk)
    v = (h @ w["v"].T).view(T, H, dv)
    log_in = capped(h @ w["i"].T + w["i.b"], cap)
    log_keep = log_sigmoid(capped(h @ w["f"].T + w["f.b"], cap))
    o, _ = matrix_memory(q, k, v, log_in, log_keep)
    o = rms_norm(o, eps).reshape(T, H * dv) * w["norm"]
    return (o * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


# ---- attention over a latent -----------------------------------------------------------------------------
def latent_heads(q, down, w, m, eps, positions):
    """q [T, H, d + r] (plain dims first, then the turned ones) and down [T, rank + r] as projected; w holds dkv.norm,
    uk, uv.  Returns the heads [T, H, dv] before the gate."""
    H, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = q.shape[0]
    q_plain, q_turned = q[..., :d], rotate_half(q[..., d:], m["rot"], positions)
    c = rms_norm(down[:, :rank], eps, w["dkv.norm"])
    k_turned = rotate_half(down[:, None, rank:], m["rot"], positions)[:, 0]          # one part for all heads
    k_plain = (c @ w["uk"].T).view(T, H, d)
    v = (c @ w["uv"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=q.dtype)
    for hd in range(H):
        s = (q_plain[:, hd] @ k_plain[:, hd].T + q_turned[:, hd] @ k_turned.T) * m["scale"]
        out[:, hd] = causal_softmax(s) @ v[:, hd]
    return out


def latent_attention(h, w, m, eps, positions):
    T = h.shape[0]
    H, d, r = m["heads"], m["dim"], m["rot_dim"]
    cq = rms_norm(h @ w["dq"].T, eps, w["dq.norm"])
    q = (cq @ w["uq"].T).view(T, H, d + r)
    heads = latent_heads(q, h @ w["dkv"].T, w, m, eps, positions)
    gate = torch.sigmoid(h @ w["g"].T)                                    # [T, H]: one number a head
    return (heads * gate[:, :, None]).reshape(T, -1) @ w["o"].T


# ---- attention with a short convolution, whole-row norms and mixed heads -------------------------------------
def short_conv(u, taps_w):
    """u [T, C]; taps_w [C, taps]: y_t = sum_j taps_w[:, j] u_(t - taps + 1 + j), nothing before a sequence."""
    T, C = u.shape
    taps = taps_w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u], dim=0)
    out = torch.zeros(T, C, dtype=u.dtype)
    for j in range(taps):
        out = out + padded[j:j + T] * taps_w[:, j][None, :]
    return out


def mixed_head_scores(q, k, scale, talk):
    """q [T, H, d], k [T, G, d] -> scores [H, T, T]: head h's own scores (q_h . k of its kv head) * scale, then
    head h gets sum_g talk[h, g] * (head g's)."""
    H, G = q.shape[1], k.shape[1]
    own = torch.stack([(q[:, g] @ k[:, g // (H // G)].T) * scale for g in range(H)])
    return torch.einsum("hg,gij->hij", talk, own)


def conv_attention(h, w, m, eps):
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q, k, v = h @ w["q"].T, h @ w["k"].T, h @ w["v"].T
    if m.get("conv"):
        q, k, v = short_conv(q, w["q.conv"]), short_conv(k, w["k.conv"]), short_conv(v, w["v.conv"])
    q = rms_norm(q, eps, w["q.norm"]).view(T, H, d)                        # one mean over the whole projection
    k = rms_norm(k, eps, w["k.norm"]).view(T, G, d)
    v = rms_norm(v.view(T, G, dv), eps)                                    # head by head, no weight
    scores = mixed_head_scores(q, k, m["scale"], w["talk"])
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hd in range(H):
        out[:, hd] = causal_softmax(scores[hd]) @ v[:, hd // (H // G)]
    gate = torch.sigmoid(h @ w["g"].T)                                     # [T, H]
    return (out * gate[:, :, None]).reshape(T, H * dv) @ w["o"].T


# ---- feed-forwards -------------------------------------------------------------------------------------------
def dense_mlp(h, w):
    return (silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def routed_experts(h, w, mlp):
    """Scores sigmoid(router h); each token's `top` largest; an expert sees the token times its score."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    s = torch.sigmoid(h.to(torch.float64) @ w["router"].to(torch.float64).T)
    chosen = torch.topk(s, top, dim=-1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for r in range(top):
            e = int(chosen.indices[t, r])
            xin = h[t] * chosen.values[t, r].to(h.dtype)
            out[t] += (silu(w[f"e{e}.gate"] @ xin) * (w[f"e{e}.up"] @ xin)) @ w[f"e{e}.down"].T
    return out


# ---- the model ---------------------------------------------------------------------------------------------
class PlainVuzazen:
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

    def mixer(self, i, h, positions):
        l, eps = self.cfg["layers"][i], self.cfg["norm"]["eps"]
        w = self._sub(f"l{i}.mix.")
        if l["type"] == "mlstm":
            return mlstm(h, w, l["mixer"], eps)
        if l["type"] == "latent_attention":
            return latent_attention(h, w, l["mixer"], eps, positions)
        if l["type"] == "attention":
            return conv_attention(h, w, l["mixer"], eps)
        raise ValueError(l["type"])

    def stream(self, tokens):
        """The residual stream after the embedding and after every layer."""
        cfg, eps = self.cfg, self.cfg["norm"]["eps"]
        positions = torch.arange(len(tokens))
        e = cfg["embedding"]
        x = embed(tokens, self.w["embed"], e["scale"], self.w["bigram"], e["bigram"])
        out = [x.clone()]
        for i, l in enumerate(cfg["layers"]):
            x = x + self.mixer(i, rms_norm(x, eps, layer_norm_weight(self.w[f"l{i}.norm1"])), positions)
            if l.get("mlp") is not None:
                h = rms_norm(x, eps, layer_norm_weight(self.w[f"l{i}.norm2"]))
                w = self._sub(f"l{i}.mlp.")
                x = x + (dense_mlp(h, w) if l["mlp"].get("kind", "dense") == "dense" else routed_experts(h, w, l["mlp"]))
            out.append(x.clone())
        return out

    def logits(self, tokens):
        x = self.stream(tokens)[-1]
        return rms_norm(x, self.cfg["norm"]["eps"], layer_norm_weight(self.w["final.norm"])) @ self.w["embed"].T

    def greedy(self, prompt, n):
        ids = list(prompt)
        for _ in range(n):
            ids.append(int(self.logits(ids)[-1].argmax()))
        return ids[len(prompt):]
