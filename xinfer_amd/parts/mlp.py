"""Gated feed-forward: down(act(gate(x)) * up(x)), act = silu (SwiGLU) or the tanh form of gelu.

gate and up are concatenated at load into one [2I, H] weight, the product lands in a
packed [T, 2I] buffer and one kernel applies silu(g) * u (reference: MLP::forward,
/root/reference/src/models/layers/mlp.rs:613-633; merge at load mlp.rs:447-466).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import FeedForward, StepContext, register_feed_forward
from .linear import Linear


@register_feed_forward("gated_mlp")
class GatedMLP(FeedForward):
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.activation = str(spec.get("activation", "silu"))
        if self.activation not in kernels.ACTIVATIONS:
            raise NotImplementedError(f"activation {self.activation!r} is not built ({', '.join(kernels.ACTIVATIONS)})")
        self.gate_up: Optional[Linear] = None
        self.down: Optional[Linear] = None

    NAMES = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}

    @classmethod
    def _names(cls, spec: PartSpec, prefix: str):
        """The three tensors' names: the spec's `names` (what follows the prefix) over the defaults."""
        given = spec.get("names") or {}
        return {k: f"{prefix}.{given.get(k, v)}" for k, v in cls.NAMES.items()}

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        h, i = int(spec["hidden_size"]), int(spec["intermediate_size"])
        n = cls._names(spec, prefix)
        return [TensorDecl(n["gate"], (i, h)), TensorDecl(n["up"], (i, h)), TensorDecl(n["down"], (h, i))]

    def load(self, store: WeightStore, prefix: str, device) -> None:
        def lin(name):
            t = store.get(name, None, device)
            return t.to(self.dtype) if (self.dtype == torch.float32 or t.dtype != torch.float32) else t
        n = self._names(self.spec, prefix)
        g, u = lin(n["gate"]), lin(n["up"])
        common = torch.float32 if torch.float32 in (g.dtype, u.dtype) else g.dtype
        self.gate_up = Linear(torch.cat([g.to(common), u.to(common)], dim=0))
        self.down = Linear(lin(n["down"]))

    takes_sink = True
    takes_folded = True

    def forward(self, x, ctx: StepContext, sink=None):
        """`x`: rows or a `Folded`; `sink`: see `Part.takes_sink`."""
        m = self.gate_up(x, out_dtype=self.dtype, gated=True, act=self.activation)    # gate, up and act*mul in one pass
        if m is None and self.activation != "silu":
            m = kernels.act_mul(self.gate_up(x, out_dtype=self.dtype), self.activation)
        elif m is None:
            m = kernels.silu_mul(self.gate_up(x, out_dtype=self.dtype))
        return self.down(m, out_dtype=self.dtype, allow_split=True, sink=sink)   # the next norm adds the parts


@register_feed_forward("mlp")
class DenseMLP(FeedForward):
    """Feed-forward without a gate: down(act(up(x))), act one of `kernels.UNGATED_ACTIVATIONS` (silu, the tanh form
    of gelu, or relu2: the square of relu).  Tensor names as data (`names`: up, down)."""
    graph_safe = True
    NAMES = {"up": "up_proj.weight", "down": "down_proj.weight"}

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.activation = str(spec.get("activation", "relu2"))
        if self.activation not in kernels.UNGATED_ACTIVATIONS:
            raise NotImplementedError(f"activation {self.activation!r} is not built ({', '.join(kernels.UNGATED_ACTIVATIONS)})")
        self.up: Optional[Linear] = None
        self.down: Optional[Linear] = None

    @classmethod
    def _names(cls, spec: PartSpec, prefix: str):
        given = spec.get("names") or {}
        return {k: f"{prefix}.{given.get(k, v)}" for k, v in cls.NAMES.items()}

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        h, i = int(spec["hidden_size"]), int(spec["intermediate_size"])
        n = cls._names(spec, prefix)
        return [TensorDecl(n["up"], (i, h)), TensorDecl(n["down"], (h, i))]

    def load(self, store: WeightStore, prefix: str, device) -> None:
        def lin(name):
            t = store.get(name, None, device)
            return t.to(self.dtype) if (self.dtype == torch.float32 or t.dtype != torch.float32) else t
        n = self._names(self.spec, prefix)
        self.up = Linear(lin(n["up"]))
        self.down = Linear(lin(n["down"]))

    def forward(self, x, ctx: StepContext):
        m = kernels.act_(self.up(x, out_dtype=self.dtype), self.activation)
        return self.down(m, out_dtype=self.dtype, allow_split=True)      # the next norm adds the parts
