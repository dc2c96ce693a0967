"""A matrix memory with exponential gating (the mLSTM of xLSTM), as a mixer: "mlstm".

Per request and head a float32 matrix S [key_dim, value_dim], a vector n [key_dim] and a running maximum m, all zero
when the request starts.  For every token, with q = W_q h * q_scale (key_dim^-1/2 unless given), k = W_k h, v = W_v h
and per head the logits zi = w_i . h + b_i, zf = w_f . h + b_f:

    log_in = cap tanh(zi / cap)                  log_keep = logsigmoid(cap tanh(zf / cap))
    m' = max(log_keep + m, log_in)
    S' = exp(log_keep + m - m') S + exp(log_in - m') k v^T          n' likewise with k alone
    o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)

then each head's o is divided by its root mean square over value_dim (eps inside the root), the heads side by side are
multiplied by a weight [heads * value_dim] and by sigmoid(W_g h), and projected (`o`).

The state is walked by the kernel of the other decaying-state mixers (`kernels.linear_scan` with ready-made gates, long
portions in chunks side by side): n rides along as one more value column whose value is always 1, so a slot of "state"
is [heads, key_dim, value_dim + 1]; m is a second state of the request, "max" [heads], walked by the kernel that makes
the gates.  Logits, gates, their exponentials, the state, its results and the norm are float32 in both precisions (the
logits leave their product as float32); q, k, v and g are one packed product in the activation dtype.  Tensor names
under the part's prefix: q, k, v, g, o, norm, i, i.b, f, f.b (the spec's `names` replaces any).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import LayerCache, Mixer, StateNeed, StepContext, register_mixer
from .linear import Linear


@register_mixer("mlstm")
class MatrixMemory(Mixer):
    graph_safe = True
    NAMES: Dict[str, str] = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "i": "i", "i_bias": "i.b",
                             "f": "f", "f_bias": "f.b"}

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.dk = int(spec["key_dim"])
        self.dv = int(spec["value_dim"])
        self.cap = float(spec["gate_cap"])
        self.eps = float(spec["norm_eps"])
        self.q_scale = float(spec.get("q_scale") or self.dk ** -0.5)
        if min(self.hidden, self.heads, self.dk, self.dv) <= 0 or not self.cap > 0:
            raise ValueError(f"{self.heads} heads of {self.dk} by {self.dv} with a gate cap of {self.cap} cannot be run")
        self.proj: Optional[Linear] = None           # [q | k | v | g] rows
        self.gates: Optional[Linear] = None          # [i | f] rows: the gates' logits
        self.o: Optional[Linear] = None
        self.gate_bias = self.norm_w = None

    @classmethod
    def _names(cls, spec: PartSpec, prefix: str) -> Dict[str, str]:
        given = spec.get("names") or {}
        return {k: f"{prefix}.{given.get(k, v)}" for k, v in cls.NAMES.items()}

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        h, H, dk, dv = (int(spec[k]) for k in ("hidden_size", "num_heads", "key_dim", "value_dim"))
        n = cls._names(spec, prefix)
        return [TensorDecl(n["q"], (H * dk, h)), TensorDecl(n["k"], (H * dk, h)), TensorDecl(n["v"], (H * dv, h)),
                TensorDecl(n["g"], (H * dv, h)), TensorDecl(n["o"], (h, H * dv)), TensorDecl(n["norm"], (H * dv,), "norm"),
                TensorDecl(n["i"], (H, h)), TensorDecl(n["i_bias"], (H,), "normal(0,1)"),
                TensorDecl(n["f"], (H, h)), TensorDecl(n["f_bias"], (H,), "normal(2,1)")]

    def _lin(self, store: WeightStore, name: str, device) -> torch.Tensor:
        t = store.get(name, None, device)
        return t.to(self.dtype) if (self.dtype == torch.float32 or t.dtype != torch.float32) else t

    def load(self, store: WeightStore, prefix: str, device) -> None:
        n = self._names(self.spec, prefix)
        self.proj = Linear(torch.cat([self._lin(store, n[k], device).to(self.dtype) for k in ("q", "k", "v", "g")], dim=0))
        self.gates = Linear(torch.cat([self._lin(store, n[k], device).to(self.dtype) for k in ("i", "f")], dim=0))
        self.o = Linear(self._lin(store, n["o"], device).to(self.dtype))
        self.gate_bias = torch.cat([store.get(n[k], torch.float32, device).reshape(-1) for k in ("i_bias", "f_bias")]).contiguous()
        self.norm_w = store.get(n["norm"], torch.float32, device).contiguous()

    def state_need(self) -> Tuple[StateNeed, ...]:
        return (StateNeed((self.heads, self.dk, self.dv + 1), torch.float32, "state"),
                StateNeed((self.heads,), torch.float32, "max"))

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        if cache.state is None or "max" not in cache.states:
            raise RuntimeError("a matrix memory was given no state slots")
        H, dk, dv = self.heads, self.dk, self.dv
        p = self.proj(x, out_dtype=self.dtype)
        a, b = H * dk, H * dv
        q, k, v, g = p[:, :a], p[:, a:2 * a], p[:, 2 * a:2 * a + b], p[:, 2 * a + b:]
        z = self.gates(x, out_dtype=torch.float32)                  # the gates' logits leave their product in float32
        gates, floor = kernels.mlstm_gates(z, self.gate_bias, self.cap, cache.states["max"], ctx.state_slots, ctx.cu_q, H)
        cut = {}
        if ctx.max_q_len > 1 and ctx.cu_q_host:
            cu = ctx.cu_q_host
            cut = dict(q_lens=[cu[i + 1] - cu[i] for i in range(ctx.num_seqs)], plan_cache=ctx.scratch)
        o = kernels.linear_scan(q, k, v, cache.state, ctx.state_slots, ctx.cu_q, H, dk, dv + 1, gates=gates, value_cols=dv,
                                q_scale=self.q_scale, **cut)
        return self.o(kernels.mlstm_finish(o, floor, self.norm_w, self.eps, g, self.dtype), out_dtype=self.dtype, allow_split=True)
