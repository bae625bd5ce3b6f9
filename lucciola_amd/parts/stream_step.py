"""Things done to the residual stream between two layers, as parts of their own family
(``stream_step``): ``forward(stream)`` changes the stream in place.  A run order names one right
before the site it belongs to (``RunEntry.before``)."""
from __future__ import annotations

from typing import Dict

from ..config.registry import STREAM_STEPS
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part, ResidualStream


@STREAM_STEPS.register("row_offset")
class RowOffset(Part):
    """Adds row ``row`` of a learned table [rows, size] to every token's stream: the mark of a
    pass where a stack of layers runs several times.  The branch output that still waits is
    added by the same kernel."""

    graph_safe = True

    def __init__(self, size: int, rows: int, row: int):
        super().__init__(size=size, rows=rows, row=row)
        self.size, self.rows, self.row = int(size), int(rows), int(row)
        if not 0 <= self.row < self.rows:
            raise ValueError(f"row_offset: row {row} of a table of {rows}")
        self.vector = None

    def declare(self) -> Dict[str, ParamDecl]:
        return {"table": ParamDecl((self.rows, self.size), role="vector", init="normal")}

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.vector = tensors["table"][self.row].contiguous()

    def forward(self, stream: ResidualStream) -> None:
        ops.stream_add(stream.h, ops.value(stream.pending), self.vector)
        stream.pending = None
