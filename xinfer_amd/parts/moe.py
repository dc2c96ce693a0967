"""Routed experts (mixture of experts) as a feed-forward.

z = W_router x (+ b) in float32; each token takes the `top` experts with the largest z, weighted by
the softmax over the chosen logits only; an expert is a gated feed-forward without biases,
down(act(gate x) * (up x)); the result is the weighted sum of the chosen experts' outputs, in
float32.  The experts' weights are stacked at load: gate and up [E, 2F, H] (gate rows first), down
[E, H, F].  In steps of single tokens nothing is read on the host: the router's choice stays on the
device and the experts' kernels find their rows from it, so decode steps can be recorded.

Options, each a parameter of the spec: `gated: False` makes an expert down(act(up x)) with the up rows
alone ([E, F, H]) and takes the activations without a gate as well ("relu2": the square of relu);
`scores: "all"` weighs the chosen experts by their softmax scores over ALL experts, divided by the
chosen ones' sum + 1e-20 (in place of the softmax over the chosen logits), `scores: "sigmoid"` by sigmoid(z) of each
chosen expert as it is (nothing is divided; the largest logits are the largest scores); `weigh: "input"` lets the
weight multiply what the expert SEES, sum of expert_e(weight_e * x), instead of what it returns (the experts' first
products are linear, so the kernels put the weight on their float32 sums, before the activation); `shared` = {intermediate_size,
activation, gated, gate}: one more expert of the same form that every token takes, added to the result,
times sigmoid(w_g . x) with a vector w_g of its own if `gate` says so (that product rides with the
router's, in float32).

Tensor names under the part's prefix (`names` of the spec replaces any of them): `router`,
`router_bias`, and per expert i `expert{i}.gate`, `expert{i}.up`, `expert{i}.down`, in which "{i}" is
the expert's number; `shared_gate`, `shared_up`, `shared_down` and `shared_open` (the vector w_g, [1, H]).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import FeedForward, StepContext, register_feed_forward
from .linear import Linear


@register_feed_forward("routed_experts")
class RoutedExperts(FeedForward):
    graph_safe = True
    LIBRARY = True       # False: the hand-written kernels for every step
    NAMES = {"router": "router.weight", "router_bias": "router.bias", "gate": "experts.{i}.gate_proj.weight",
             "up": "experts.{i}.up_proj.weight", "down": "experts.{i}.down_proj.weight",
             "shared_gate": "shared_expert.gate_proj.weight", "shared_up": "shared_expert.up_proj.weight",
             "shared_down": "shared_expert.down_proj.weight", "shared_open": "shared_expert_gate.weight"}

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])          # of one expert
        self.experts = int(spec["num_experts"])
        self.top = int(spec["top"])
        self.router_bias = bool(spec.get("router_bias", False))
        self.activation = str(spec.get("activation", "silu"))
        self.gated = bool(spec.get("gated", True))
        self._check_act(self.activation, self.gated)
        self.all_scores = self._scores(spec) == "all"
        self.sigmoid_scores = self._scores(spec) == "sigmoid"
        self.weigh_input = str(spec.get("weigh", "output")) == "input"
        if str(spec.get("weigh", "output")) not in ("input", "output"):
            raise ValueError(f"weigh {spec.get('weigh')!r}: 'output' (the expert's result) or 'input'")
        if self.weigh_input and not self.gated:
            raise NotImplementedError("a weight on the experts' input is built for gated experts")
        if not (0 < self.top <= self.experts):
            raise ValueError(f"{self.top} of {self.experts} experts cannot be chosen")
        sh = spec.get("shared")
        self.shared = None if not sh else dict(inter=int(sh["intermediate_size"]), act=str(sh.get("activation", self.activation)),
                                               gated=bool(sh.get("gated", self.gated)), open=bool(sh.get("gate", False)))
        if self.shared:
            self._check_act(self.shared["act"], self.shared["gated"])
        self.shared_up: Optional[Linear] = None          # [gate; up] rows if the shared expert is gated
        self.shared_down: Optional[Linear] = None
        self.router_w: Optional[torch.Tensor] = None     # float32 [E, H]
        self.router_b: Optional[torch.Tensor] = None     # float32 [E]
        self.gate_up: Optional[torch.Tensor] = None      # [E, 2F, H]
        self.down: Optional[torch.Tensor] = None         # [E, H, F]

    @staticmethod
    def _check_act(act: str, gated: bool) -> None:
        known = kernels.ACTIVATIONS if gated else kernels.UNGATED_ACTIVATIONS
        if act not in known:
            raise NotImplementedError(f"activation {act!r} is not built for experts {'with' if gated else 'without'} "
                                      f"a gate ({', '.join(known)})")

    @staticmethod
    def _scores(spec: PartSpec) -> str:
        scores = str(spec.get("scores", "chosen"))
        if scores not in ("chosen", "all", "sigmoid"):
            raise ValueError(f"router scores {scores!r}: 'chosen' (softmax over the chosen logits), 'all' or 'sigmoid'")
        return scores

    @classmethod
    def _names(cls, spec: PartSpec, prefix: str):
        given = spec.get("names") or {}
        return {k: f"{prefix}.{given.get(k, v)}" for k, v in cls.NAMES.items()}

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        h, f, e = int(spec["hidden_size"]), int(spec["intermediate_size"]), int(spec["num_experts"])
        n = cls._names(spec, prefix)
        out = [TensorDecl(n["router"], (e, h))]
        if spec.get("router_bias", False):
            out.append(TensorDecl(n["router_bias"], (e,)))
        gated = bool(spec.get("gated", True))
        for i in range(e):
            if gated:
                out.append(TensorDecl(n["gate"].replace("{i}", str(i)), (f, h)))
            out += [TensorDecl(n["up"].replace("{i}", str(i)), (f, h)), TensorDecl(n["down"].replace("{i}", str(i)), (h, f))]
        sh = spec.get("shared")
        if sh:
            fs = int(sh["intermediate_size"])
            if bool(sh.get("gated", gated)):
                out.append(TensorDecl(n["shared_gate"], (fs, h)))
            out += [TensorDecl(n["shared_up"], (fs, h)), TensorDecl(n["shared_down"], (h, fs))]
            if sh.get("gate", False):
                out.append(TensorDecl(n["shared_open"], (1, h)))
        return out

    def load(self, store: WeightStore, prefix: str, device) -> None:
        n = self._names(self.spec, prefix)
        self.router_w = store.get(n["router"], torch.float32, device).contiguous()
        if self.router_bias:
            self.router_b = store.get(n["router_bias"], torch.float32, device).contiguous()
        gu, dn = [], []
        for i in range(self.experts):
            u, d = (store.get(n[k].replace("{i}", str(i)), self.dtype, device) for k in ("up", "down"))
            if self.gated:
                u = torch.cat([store.get(n["gate"].replace("{i}", str(i)), self.dtype, device), u], dim=0)
            gu.append(u)
            dn.append(d)
        self.gate_up = torch.stack(gu).contiguous()
        self.down = torch.stack(dn).contiguous()
        if self.shared:
            u = store.get(n["shared_up"], self.dtype, device)
            if self.shared["gated"]:
                u = torch.cat([store.get(n["shared_gate"], self.dtype, device), u], dim=0)
            self.shared_up = Linear(u)
            self.shared_down = Linear(store.get(n["shared_down"], self.dtype, device))
            if self.shared["open"]:        # the vector that opens the shared branch: one more row of the router's product
                row = store.get(n["shared_open"], torch.float32, device).reshape(1, self.hidden)
                self.router_w = torch.cat([self.router_w, row], dim=0).contiguous()

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        opens = bool(self.shared and self.shared["open"])
        routed = kernels.moe_route(x, self.router_w, self.router_b, self.top, all_scores=self.all_scores,
                                   extra_rows=1 if opens else 0, sigmoid=self.sigmoid_scores)
        idx, wt = routed[0], routed[1]
        # a step that brings portions is never recorded: with many rows an expert it may read the experts' row
        # counts on the host and hand each expert's rows to the vendor library, as the dense products of many rows go
        if (ctx.max_q_len > 1 and x.dtype == torch.bfloat16 and self.LIBRARY
                and x.shape[0] * self.top >= kernels.MOE_LIBRARY_ROWS * self.experts):
            out = kernels.moe_experts_library(x, self.gate_up, self.down, idx, wt, self.activation, gated=self.gated,
                                              weigh_input=self.weigh_input)
        else:
            out = kernels.moe_experts(x, self.gate_up, self.down, idx, wt, self.activation, gated=self.gated,
                                      weigh_input=self.weigh_input)
        if self.shared:
            out = self._add_shared(out, x, routed[2][:, 0] if opens else None)
        return out

    def _add_shared(self, out: torch.Tensor, x: torch.Tensor, opening: Optional[torch.Tensor]) -> torch.Tensor:
        """out (float32) += [sigmoid(opening) *] the shared expert's result for every row."""
        sh = self.shared
        if sh["gated"]:
            m = self.shared_up(x, out_dtype=self.dtype, gated=True, act=sh["act"])
            if m is None:
                m = kernels.act_mul(self.shared_up(x, out_dtype=self.dtype), sh["act"])
        else:
            m = kernels.act_(self.shared_up(x, out_dtype=self.dtype), sh["act"])
        y = self.shared_down(m, out_dtype=self.dtype)
        if opening is None:
            return kernels.scaled_sum(out, y, 1.0)
        return kernels.gated_add_(out, y, opening)
