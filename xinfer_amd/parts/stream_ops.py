"""What may run on the residual stream between two runs of layers (`ScheduleEntry.before`).

"pass_start": what a pass over a span of layers adds to the stream when it starts,

    x <- x (+ the branch that is still to be added) (+ the embedding's output, `add_first`) + table[row]

with `table` a tensor [rows, dim] named by the spec and `row` the number of the pass.  One float32 kernel; the
stream goes on with nothing pending.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import StepContext, Stream, StreamOp, register_stream_op


@register_stream_op("pass_start")
class PassStart(StreamOp):
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.dim = int(spec["dim"])
        self.rows = int(spec.get("rows") or 0)          # 0: no table
        self.row = int(spec.get("row") or 0)
        self.needs_first = bool(spec.get("add_first", False))
        if self.rows and not (0 <= self.row < self.rows):
            raise ValueError(f"row {self.row} of a table of {self.rows}")
        self.vec: Optional[torch.Tensor] = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str = "") -> List[TensorDecl]:
        if not int(spec.get("rows") or 0):
            return []
        return [TensorDecl(spec["name"], (int(spec["rows"]), int(spec["dim"])))]

    def load(self, store: WeightStore, prefix: str, device) -> None:
        if self.rows:
            self.vec = store.get(self.spec["name"], torch.float32, device)[self.row].contiguous()

    def forward(self, stream: Stream, first: Optional[torch.Tensor], ctx: StepContext) -> Stream:
        if stream.folded is not None:
            raise RuntimeError("the stream carries a half-done norm of the block before")
        if self.needs_first and first is None:
            raise RuntimeError("the embedding's output was not kept for the start of a pass")
        kernels.stream_start(stream.resid, stream.pending, stream.pending_scale, first if self.needs_first else None, self.vec)
        return Stream(stream.resid, None)
