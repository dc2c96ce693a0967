"""Attention over a cached latent, as a mixer: "latent_attention".

    q = W_q h                          heads of [dim plain | rot_dim turned] dims
    down = W_dkv h                     rank + rot_dim rows: c = RMSNorm(down[:rank]) * w, and down[rank:], turned by the
                                       token's position, is one key part shared by all heads
    head i: k = [U_k,i c | turned part], v = U_v,i c
    score = (q_plain . U_k,i c + q_turned . k_turned) * scale over the last `window` tokens (0: all)
    softmax, with exp(sink_i) in its denominator if the spec says `sinks`
    o = W_o (heads * sigmoid(W_g h))   (the gate only if the spec says `gate`; `gate="head"`: W_g has one row a head
                                       and a head is multiplied by one number)

With `q_rank` the queries come through a latent of their own: q = W_uq (RMSNorm(W_dq h) * w_dq), the down projection
packed with the others, its norm in float32.

What a token keeps in the cache is c and the turned key part: one pool "latent" [pages, 1, page, rank + rot_dim].  The
heads' matrices move to the query's side: q' = [U_k,i^T q_plain | q_turned] is scored against the cached rows directly,
the weighted sum of the cached c is taken once a head, and U_v,i is applied to that sum; a token's keys and values are
never made.  The gate is applied where U_v's product is stored.  Rotation tables, the latent's norm, scores, softmax and
sinks are float32 in both precisions.  In bfloat16, where the matrix-core attention kernel takes the sizes (rank + rot_dim
up to 256, both multiples of 8), a second pool "latent_t" [pages, 1, page / 8, rank, 8] holds c once more, in the groups
of eight tokens that kernel reads values in: portions and single tokens then run on the matrix cores, with one kv head
of rank + rot_dim dims and values of rank dims; other sizes, and float32, read keys and values from the one pool
with the generic kernel.  Tensor names under the part's prefix: q (or dq, dq.norm, uq), dkv, dkv.norm, uk, uv, sink,
g, o (the spec's `names` replaces any).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import KVNeed, LayerCache, Mixer, PAGE, PAGE_BY_8, PoolNeed, StepContext, position_encoding_class, register_mixer
from .linear import Linear


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    graph_safe = True
    NAMES: Dict[str, str] = {"q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "sink": "sink",
                             "g": "g", "o": "o", "dq": "dq", "dq_norm": "dq.norm", "uq": "uq"}

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.d = int(spec["head_dim"])              # plain dims of a head's q and k
        self.r = int(spec["rot_dim"])               # turned dims
        self.dv = int(spec["value_dim"])
        self.rank = int(spec["kv_rank"])
        self.scale = float(spec["scale"])
        self.window = int(spec.get("window") or 0)
        self.eps = float(spec["norm_eps"])
        self.has_sinks = bool(spec.get("sinks", False))
        self.has_gate = bool(spec.get("gate", False))
        self.head_gate = spec.get("gate") == "head"          # one number a head
        self.q_rank = int(spec.get("q_rank") or 0)           # 0: q straight from h
        if min(self.hidden, self.heads, self.d, self.dv, self.rank) <= 0 or self.r <= 0 or self.r % 2:
            raise ValueError(f"{self.heads} heads of {self.d} + {self.r} dims with values of {self.dv} over a latent of "
                             f"{self.rank} cannot be run")
        pos = spec.get("position")
        if pos is None or int(pos.get("rotary_dim", pos["head_dim"])) != self.r:
            raise ValueError("latent attention turns the whole of its rot_dim dims: it needs a position encoding of that size")
        self.position = position_encoding_class(pos.kind)(pos, dtype)
        # values in groups of eight tokens beside the keys: what the matrix-core kernel reads (any page it is given
        # is a power of two of at least 8 where the engine runs bfloat16 attention on the matrix cores)
        self.values_pool = (dtype == torch.bfloat16 and spec.get("matrix_cores", True)
                            and kernels.attention_biased_supported(self.heads, 1, self.rank + self.r, self.rank, 64))
        self.proj: Optional[Linear] = None          # [q (or the queries' down projection) | dkv | g] rows
        self.uq: Optional[Linear] = None
        self.q_norm_w = None
        self.o: Optional[Linear] = None
        self.uk = self.uv = None                    # [heads, rank, dim] (turned over) and [heads, vdim, rank] (as stored)
        self.norm_w = self.sinks = None

    @classmethod
    def _names(cls, spec: PartSpec, prefix: str) -> Dict[str, str]:
        given = spec.get("names") or {}
        return {k: f"{prefix}.{given.get(k, v)}" for k, v in cls.NAMES.items()}

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        h, H, d, r, dv, rank = (int(spec[k]) for k in ("hidden_size", "num_heads", "head_dim", "rot_dim", "value_dim", "kv_rank"))
        n = cls._names(spec, prefix)
        out = [TensorDecl(n["dkv"], (rank + r, h)), TensorDecl(n["dkv_norm"], (rank,), "norm"),
               TensorDecl(n["uk"], (H * d, rank)), TensorDecl(n["uv"], (H * dv, rank)), TensorDecl(n["o"], (h, H * dv))]
        qr = int(spec.get("q_rank") or 0)
        if qr:
            out += [TensorDecl(n["dq"], (qr, h)), TensorDecl(n["dq_norm"], (qr,), "norm"), TensorDecl(n["uq"], (H * (d + r), qr))]
        else:
            out.append(TensorDecl(n["q"], (H * (d + r), h)))
        if spec.get("sinks", False):
            out.append(TensorDecl(n["sink"], (H,), "normal(0,1)"))
        if spec.get("gate", False):
            out.append(TensorDecl(n["g"], (H if spec.get("gate") == "head" else H * dv, h)))
        return out

    def _lin(self, store: WeightStore, name: str, device) -> torch.Tensor:
        t = store.get(name, None, device)
        return t.to(self.dtype) if (self.dtype == torch.float32 or t.dtype != torch.float32) else t

    def load(self, store: WeightStore, prefix: str, device) -> None:
        n = self._names(self.spec, prefix)
        first = "dq" if self.q_rank else "q"
        parts = [self._lin(store, n[k], device) for k in ((first, "dkv", "g") if self.has_gate else (first, "dkv"))]
        if self.q_rank:
            self.uq = Linear(self._lin(store, n["uq"], device).to(self.dtype))
            self.q_norm_w = store.get(n["dq_norm"], torch.float32, device).contiguous()
        self.proj = Linear(torch.cat([p.to(self.dtype) for p in parts], dim=0))
        self.o = Linear(self._lin(store, n["o"], device).to(self.dtype))
        # U_k with a head's inputs (its plain query dims) side by side, as the queries' product reads it
        self.uk = self._lin(store, n["uk"], device).to(self.dtype).view(self.heads, self.d, self.rank).transpose(1, 2).contiguous()
        self.uv = self._lin(store, n["uv"], device).to(self.dtype).contiguous().view(self.heads, self.dv, self.rank)
        self.norm_w = store.get(n["dkv_norm"], torch.float32, device).contiguous()
        if self.has_sinks:
            self.sinks = store.get(n["sink"], torch.float32, device).contiguous()
        self.position.load(store, prefix, device)

    def cache_need(self) -> KVNeed:
        pools = [PoolNeed("latent", (1, PAGE, self.rank + self.r))]
        if self.values_pool:
            pools.append(PoolNeed("latent_t", (1, PAGE_BY_8, self.rank, 8)))
        return KVNeed(self.window, tuple(pools))

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        H, d, r, dv, rank = self.heads, self.d, self.r, self.dv, self.rank
        T = x.shape[0]
        p = self.proj(x, out_dtype=self.dtype)
        q_cols = H * (d + r)
        if self.q_rank:            # the queries through their latent: the heads' q parts are rows of their own
            qp = self.uq(kernels.rows_rmsnorm(p[:, :self.q_rank], self.q_norm_w, self.eps, self.dtype), out_dtype=self.dtype)
            q_rows, q_at, down_at = qp, 0, self.q_rank
        else:
            q_rows, q_at, down_at = p, 0, q_cols
        pool = cache.pools["latent"]
        values = cache.pools.get("latent_t")
        if values is not None and not kernels.attention_biased_supported(H, 1, rank + r, rank, pool.shape[2]):
            values = None                                           # a page the matrix-core kernel does not take
        slots = ctx.slots[cache.group] if cache.write else ctx.no_slots
        pos = self.position
        q_full = torch.empty((T, H, rank + r), dtype=self.dtype, device=x.device)
        kernels.latent_rows(p, q_at, down_at, self.norm_w, self.eps, slots, pool, q_full, H, d, r, rank, pos.cos, pos.sin,
                            pos.interleaved, ctx.positions, values=values, q_rows=None if q_rows is p else q_rows)
        # the plain part of every head's query through its U_k: out[t, h, j] = sum_i q[t, h, i] U_k[h, i, j]
        q_plain = q_rows[:, :q_cols].view(T, H, d + r)[:, :, :d]
        kernels.head_linear(q_plain, self.uk, q_full[:, :, :rank])
        a = kernels.attention(q_full, pool, values, ctx, cache.group, self.scale, self.window, v_grouped=values is not None,
                              sinks=self.sinks, value_dim=rank)
        # the heads' weighted sums of the latent through their U_v, times the gate
        heads = torch.empty((T, H, dv), dtype=self.dtype, device=x.device)
        gate = None
        if self.head_gate:
            gate = p[:, down_at + rank + r:]                       # [T, H]
        elif self.has_gate:
            gate = p[:, down_at + rank + r:].view(T, H, dv)
        kernels.head_linear(a.view(T, H, rank), self.uv, heads, gate=gate)
        return self.o(heads.view(T, H * dv), out_dtype=self.dtype, allow_split=True)
