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
    added by the same kernel.  ``add_origin``: the stream as the embedding left it is added as
    well (a pass that starts again from the tokens themselves)."""

    graph_safe = True

    def __init__(self, size: int, rows: int, row: int, add_origin: bool = False):
        super().__init__(size=size, rows=rows, row=row, add_origin=add_origin)
        self.size, self.rows, self.row = int(size), int(rows), int(row)
        self.needs_origin = bool(add_origin)
        if not 0 <= self.row < self.rows:
            raise ValueError(f"row_offset: row {row} of a table of {rows}")
        self.vector = None

    def declare(self) -> Dict[str, ParamDecl]:
        return {"table": ParamDecl((self.rows, self.size), role="vector", init="normal")}

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.vector = tensors["table"][self.row].contiguous()

    def forward(self, stream: ResidualStream) -> None:
        if self.needs_origin and stream.origin is None:
            raise ValueError("row_offset: the stream's origin was not kept")
        ops.stream_add(stream.h, ops.value(stream.pending), self.vector,
                       more=stream.origin if self.needs_origin else None)
        stream.pending = None
