"""A selective state-space mixer (state-space duality form), as a mixer: "mamba2".

    [z | x | B | C | dt] = W_in h          inner = heads * value_dim; B, C: groups * state_dim each; dt: heads
    x, B, C <- silu(conv(x, B, C))         a causal convolution per channel over the last `conv` tokens, with a bias
    d = softplus(dt + dt_bias)             no clamp
    head i (group i // (heads / groups)):  S <- exp(-exp(A_log_i) d) S + d B x^T      (S: state_dim x value_dim)
                                           y = S^T C + D_i x
    y <- y * silu(z), RMS-normed in `norm_groups` equal parts (eps inside the root), times a weight, then W_o

What a request keeps from token to token, one slot each: the float32 matrices S of every head ("state") and the last
conv - 1 inputs of the convolution ("conv_tail", float32, oldest first).  Both start at zero (the runner clears a slot
when its request starts), and a step leaves them as they are after its last token, so a prompt may be cut anywhere.
Step sizes, decays and their exponentials, d x, the state, y, the gate and the norm are float32 in both precisions; the
projections and the convolution's result are in the activation dtype.  The state is walked by the kernel of the other
decaying-state mixers (`kernels.linear_scan` with a decay per token and head; long portions in chunks side by side).
Tensor names under the part's prefix: in, conv, conv.b, dt_bias, A_log, D, norm, o (the spec's `names` replaces any).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import LayerCache, Mixer, StateNeed, StepContext, register_mixer
from .linear import Linear


@register_mixer("mamba2")
class Mamba2(Mixer):
    graph_safe = True
    NAMES: Dict[str, str] = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "A_log": "A_log",
                             "D": "D", "norm": "norm", "o": "o"}

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.dv = int(spec["value_dim"])
        self.n = int(spec["state_dim"])
        self.groups = int(spec["groups"])
        self.taps = int(spec["conv"])
        self.norm_groups = int(spec.get("norm_groups") or 1)
        self.eps = float(spec["norm_eps"])
        self.inner = self.heads * self.dv
        self.channels = self.inner + 2 * self.groups * self.n
        if (min(self.hidden, self.heads, self.dv, self.n, self.groups, self.taps, self.norm_groups) <= 0
                or self.heads % self.groups or self.inner % self.norm_groups):
            raise ValueError(f"{self.heads} heads of {self.dv} in {self.groups} groups with states of {self.n}, {self.taps} taps "
                             f"and {self.norm_groups} norm groups cannot be run")
        self.proj: Optional[Linear] = None
        self.o: Optional[Linear] = None
        self.conv_w = self.conv_b = self.dt_bias = self.a_log = self.skip = self.norm_w = None

    @classmethod
    def _names(cls, spec: PartSpec, prefix: str) -> Dict[str, str]:
        given = spec.get("names") or {}
        return {k: f"{prefix}.{given.get(k, v)}" for k, v in cls.NAMES.items()}

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        h, H, dv, N, G, taps = (int(spec[k]) for k in ("hidden_size", "num_heads", "value_dim", "state_dim", "groups", "conv"))
        inner, C = H * dv, H * dv + 2 * G * N
        n = cls._names(spec, prefix)
        return [TensorDecl(n["in"], (2 * inner + 2 * G * N + H, h)), TensorDecl(n["conv"], (C, taps), "normal(0,0.3)"),
                TensorDecl(n["conv_bias"], (C,), "normal(0,0.1)"), TensorDecl(n["dt_bias"], (H,), "normal(-1.5,0.5)"),
                TensorDecl(n["A_log"], (H,), "normal(-1,0.5)"), TensorDecl(n["D"], (H,), "norm"),
                TensorDecl(n["norm"], (inner,), "norm"), TensorDecl(n["o"], (h, inner))]

    def load(self, store: WeightStore, prefix: str, device) -> None:
        n = self._names(self.spec, prefix)
        self.proj = Linear(store.get(n["in"], None, device).to(self.dtype))
        self.o = Linear(store.get(n["o"], None, device).to(self.dtype))
        f32 = lambda k: store.get(n[k], torch.float32, device).contiguous()
        self.conv_w, self.conv_b, self.dt_bias = f32("conv"), f32("conv_bias"), f32("dt_bias")
        self.a_log, self.skip, self.norm_w = f32("A_log"), f32("D"), f32("norm")

    def state_need(self) -> Tuple[StateNeed, ...]:
        needs = [StateNeed((self.heads, self.n, self.dv), torch.float32, "state")]
        if self.taps > 1:
            needs.append(StateNeed((self.taps - 1, self.channels), torch.float32, "conv_tail"))
        return tuple(needs)

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        if cache.state is None or (self.taps > 1 and "conv_tail" not in cache.states):
            raise RuntimeError("a state-space mixer was given no state slots")
        H, dv, N, G, inner, C = self.heads, self.dv, self.n, self.groups, self.inner, self.channels
        p = self.proj(x, out_dtype=self.dtype)
        z, u, dt = p[:, :inner], p[:, inner:inner + C], p[:, inner + C:]
        if self.taps > 1:
            tails = cache.states["conv_tail"]
        else:
            tails = torch.empty((cache.state.shape[0], 0, C), dtype=torch.float32, device=x.device)
        xbc = kernels.causal_conv(u, self.conv_w, self.conv_b, tails, ctx.state_slots, ctx.tok_seq, ctx.cu_q)
        if self.taps > 1:
            kernels.conv_tail(u, tails, ctx.state_slots, ctx.cu_q)
        xs, b, c = xbc[:, :inner], xbc[:, inner:inner + G * N], xbc[:, inner + G * N:]
        cut = {}
        if ctx.max_q_len > 1 and ctx.cu_q_host:
            cu = ctx.cu_q_host
            cut = dict(q_lens=[cu[i + 1] - cu[i] for i in range(ctx.num_seqs)], plan_cache=ctx.scratch)
        y = kernels.linear_scan(c, b, xs, cache.state, ctx.state_slots, ctx.cu_q, H, N, dv, step=dt, step_bias=self.dt_bias,
                                decay_log=self.a_log, groups=G, **cut)
        out = kernels.gated_group_norm(y, xs, self.skip, z, self.norm_w, self.eps, self.norm_groups, self.dtype)
        return self.o(out, out_dtype=self.dtype, allow_split=True)
