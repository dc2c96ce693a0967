"""Token embedding and the language-model head, as kinds of their own registries.

"embedding": x = E[ids] (times `scale` if the spec gives one; Qwen3 gives none) into the
float32 residual stream; with `sinusoid_base` b a sinusoidal position vector is added, entry 2i =
sin(p b^(-2i / dim)), entry 2i + 1 = cos of the same angle, for the token's position p (float32) (reference: /root/reference/src/models/qwen3.rs:211-220,302-309).
With `pairs` (name, buckets, mul_prev, mul_cur) a row of a second table [buckets + 1, dim] is added, chosen by the
token and the one before it: row (prev * mul_prev + token * mul_cur) mod buckets, and the last row for a sequence's
first token.  The token before is state of the request: the embedding keeps one int32 a live request
(`state_need`), written after every step, so a prompt may be cut anywhere.
"lm_head": logits = h @ W^T in float32; W is the embedding table when the spec says `tied`
(qwen3.rs:267-287,367-373); `scale` s, if the spec gives one, multiplies them; `softcap` c, if the spec
gives one, then makes them c * tanh(logits / c).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import Head, LayerCache, StateNeed, StepContext, TokenEmbedding, register_embedding, register_head
from .linear import Linear


@register_embedding("embedding")
class Embedding(TokenEmbedding):
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.vocab = int(spec["vocab_size"])
        self.dim = int(spec["dim"])
        self.scale = float(spec.get("scale") or 1.0)
        self.sinusoid_base = float(spec.get("sinusoid_base") or 0.0)
        self.freq: Optional[torch.Tensor] = None      # float32 [(dim + 1) / 2]: base^(-2i / dim)
        self.rows: Optional[torch.Tensor] = None      # the last step's result rounded to the activation dtype
        self.table: Optional[torch.Tensor] = None
        pairs = spec.get("pairs")
        self.pairs = None if not pairs else dict(name=str(pairs["name"]), buckets=int(pairs["buckets"]),
                                                 mul_prev=int(pairs["mul_prev"]), mul_cur=int(pairs["mul_cur"]))
        if self.pairs is not None and (self.pairs["buckets"] <= 0 or min(self.pairs["mul_prev"], self.pairs["mul_cur"]) < 0):
            raise ValueError("an embedding of pairs needs buckets and multipliers that are not negative")
        if self.pairs is not None and self.sinusoid_base > 0:
            raise NotImplementedError("an embedding with sinusoidal positions and a table of pairs")
        self.pair_table: Optional[torch.Tensor] = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str = "") -> List[TensorDecl]:
        out = [TensorDecl(spec["name"], (int(spec["vocab_size"]), int(spec["dim"])))]
        if spec.get("pairs"):
            out.append(TensorDecl(spec["pairs"]["name"], (int(spec["pairs"]["buckets"]) + 1, int(spec["dim"]))))
        return out

    def state_need(self) -> Optional[StateNeed]:
        return StateNeed((), torch.int32, "last_token") if self.pairs is not None else None

    def load(self, store: WeightStore, prefix: str, device) -> None:
        t = store.get(self.spec["name"], None, device)
        if self.dtype == torch.float32 or t.dtype != torch.float32:
            t = t.to(self.dtype)
        self.table = t.contiguous()
        if self.pairs is not None:
            self.pair_table = store.get(self.pairs["name"], None, device).to(self.table.dtype).contiguous()
        if self.sinusoid_base > 0:
            i = torch.arange((self.dim + 1) // 2, dtype=torch.float32)
            self.freq = (torch.tensor(self.sinusoid_base, dtype=torch.float32) ** (-2.0 * i / self.dim)).to(device).contiguous()

    def forward(self, ids: torch.Tensor, ctx: Optional[StepContext] = None, cache: Optional[LayerCache] = None) -> torch.Tensor:
        if self.pairs is not None:
            if ctx is None or cache is None or cache.state is None:
                raise ValueError("an embedding of pairs needs the step and its slots of the tokens before")
            p = self.pairs
            out = kernels.embed_pair(self.table, self.pair_table, ids, ctx.positions, ctx.tok_seq, ctx.cu_q, ctx.state_slots,
                                     cache.state, self.scale, p["buckets"], p["mul_prev"], p["mul_cur"])
            kernels.keep_last_token(ids, ctx.cu_q, ctx.state_slots, cache.state)
            return out
        if self.freq is None:
            return kernels.embed(self.table, ids, scale=self.scale)
        if ctx is None:
            raise ValueError("an embedding with sinusoidal positions needs the step's positions")
        out, self.rows = kernels.embed_sinusoid(self.table, ids, ctx.positions, self.freq, self.scale,
                                                None if self.dtype == torch.float32 else self.dtype)
        return out


@register_head("lm_head")
class LMHead(Head):
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.tied = bool(spec.get("tied", False))
        self.softcap = float(spec.get("softcap") or 0.0)
        self.scale = float(spec.get("scale") or 1.0)
        self.proj: Optional[Linear] = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str = "") -> List[TensorDecl]:
        return [TensorDecl(spec["name"], (int(spec["vocab_size"]), int(spec["dim"])))]

    def load(self, store: WeightStore, prefix: str, device, shared: Optional[torch.Tensor] = None) -> None:
        if self.tied and shared is not None:
            self.proj = Linear(shared)
            return
        t = store.get(self.spec["name"], None, device)
        if self.dtype == torch.float32 or t.dtype != torch.float32:
            t = t.to(self.dtype)
        self.proj = Linear(t)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        # float32 logits straight from the float32 sums.  In float32 a row's logits do not depend on
        # how many rows were asked for (one fixed-order kernel); in bfloat16 the kernel is chosen by
        # the number of rows (thin or streaming up to 3, tiled up to 128, the library beyond), each
        # with its own order of sums, so they agree to rounding only
        logits = self.proj(h, out_dtype=torch.float32, skinny_rows=kernels.SKINNY_MAX_ROWS)
        if self.scale != 1.0:
            logits = kernels.scale_(logits, self.scale)
        return kernels.softcap_(logits, self.softcap) if self.softcap > 0 else logits
