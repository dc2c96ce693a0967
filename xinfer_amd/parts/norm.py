"""RMSNorm on the float32 residual stream, fused with the residual add.

out = s * rsqrt(mean(s^2) + eps) * w with s = resid (+ add), everything in float32 and
one rounding to the output type (reference: NormX::forward and forward_add,
/root/reference/src/models/layers/others.rs:22-62; weight kept in float32,
/root/reference/src/models/qwen3.rs:83).  With `weight_offset` c the stored tensor lies around -c + 1
and the factor is c + w (c = 1: the tensor is the factor's distance from one); the sum is made once, in float32, when the
tensor is loaded.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import Norm, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True
    foldable = True      # the products around it can carry it (parts.base.Folded)

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.dim = int(spec["dim"])
        self.eps = float(spec["eps"])
        self.weight_offset = float(spec.get("weight_offset") or 0.0)
        self.weight: Optional[torch.Tensor] = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        # random weights lie around 1 - offset, so that the factor lies around 1 either way
        init = "norm" if not spec.get("weight_offset") else f"normal({1.0 - float(spec['weight_offset'])},0.1)"
        return [TensorDecl(f"{prefix}.weight" if "name" not in spec.params else spec["name"],
                           (int(spec["dim"]),), init)]

    def load(self, store: WeightStore, prefix: str, device) -> None:
        name = self.spec.get("name") or f"{prefix}.weight"
        w = store.get(name, torch.float32, device)
        self.weight = (w + self.weight_offset if self.weight_offset else w).contiguous()

    def forward(self, resid, add, out_dtype, rows=None, out=None, add_scale: float = 1.0):
        return kernels.add_rmsnorm(resid, add, self.weight, self.eps, out_dtype, rows=rows, out=out, y_scale=add_scale)

    def forward_branch(self, resid, y, rows_dtype):
        return kernels.rmsnorm_add(resid, y, self.weight, self.eps, rows_dtype)
