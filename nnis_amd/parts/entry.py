"""What happens to the residual stream where a pass through repeated layers
begins.  A model whose schedule runs a stretch of layers several times with
the same weights may mark each pass: the embedding's output is added again
(from the second pass on), and a learned vector of the pass's own, one row of
a table [passes, width], is added before the pass's first layer.
"""

from __future__ import annotations

from ..errors import InvalidInput
from .base import PassEntry, TensorSpec, register_part
from .lazy import PostNormed, PreparedRows


class PassRestart(PassEntry):
    """x <- x (+ pending) (+ the embedding's output) (+ table[row]).  One
    kernel, which also runs the first norm of the layer behind it where that
    norm is one the kernel takes (``following``), and the norm that a
    ``PostNormed`` pending part still owes."""

    graph_safe = True

    def __init__(self, width, table=None, rows=0, row=0, add_embedding=False):
        self.width, self.table_name, self.rows, self.row = int(width), table, int(rows), int(row)
        self.needs_embedding = bool(add_embedding)
        if table is not None and not 0 <= self.row < self.rows:
            raise InvalidInput(f"a pass's entry names row {row} of a table of {rows}")
        self.vector = None

    def tensors(self):
        return [TensorSpec(self.table_name, (self.rows, self.width))] if self.table_name else []

    def bind(self, weights, rt):
        if self.table_name:
            self.vector = weights[self.table_name][self.row].contiguous()

    def weight_bytes(self):
        return 0 if self.vector is None else self.vector.numel() * self.vector.element_size()

    def forward(self, stream, embedded, rt, following=None):
        if isinstance(stream, PreparedRows):
            raise InvalidInput("a pass's entry takes the stream itself, not a norm of it that has already run")
        x, pending = stream
        y = post = None
        if isinstance(pending, PostNormed):
            if hasattr(pending.norm, "triple"):
                y, post = pending.y, pending.norm.triple()
            else:
                y = pending.materialize(rt)
        elif pending is not None:
            y = pending
        # the embedding's output is kept as it is: a stream that still is that tensor goes on in a new one
        x_out = rt.empty(*x.shape, dtype=x.dtype) if x is embedded else x
        takes = following is not None and hasattr(following, "triple")
        h = rt.empty(x.shape[0], self.width) if takes else None
        rt.ops.tanh_norm_step(x, x_out=x_out, y=y, post=post, rows_add=embedded if self.needs_embedding else None,
                              vec_add=self.vector, following=following.triple() if takes else None, h=h)
        return PreparedRows(following, x_out, h) if takes else (x_out, None)


register_part("pass_entry", "restart", PassRestart)
