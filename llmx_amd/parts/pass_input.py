"""What a repeated run of layers adds to the residual at the start of a pass.

"pass_vector": x <- (x + embedding rows) + table[index], the embedding rows only where the part says so (every pass but a
loop's first), table a tensor [passes, hidden] with one learned vector a pass.  All float32.
"""

from __future__ import annotations

from .. import ops
from .base import ResidualInput, register
from .spec import TensorSpec


class PassVector(ResidualInput):
    """params: hidden, passes (rows of the table), index (the pass), add_embedding (bool).  Tensor: the prefix itself,
    (passes, hidden); every pass's part lists it, and all read the one device tensor."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.hidden = int(params["hidden"])
        self.passes = int(params["passes"])
        self.index = int(params["index"])
        if not 0 <= self.index < self.passes:
            raise ValueError(f"pass vector: pass {self.index} outside the table's {self.passes}")
        self.wants_embedding = bool(params.get("add_embedding", False))
        self.vector = None

    def tensor_specs(self, available):
        if self.index:          # the table is listed once, by the first pass's part
            return []
        return [TensorSpec(self.prefix, (self.passes, self.hidden), "bias", init=("normal", 0.0, 0.02))]

    def load(self, tensors):
        self.vector = tensors[self.prefix][self.index]

    def forward(self, step, x, embedding_rows):
        ops.add_rows_vector(x, embedding_rows if self.wants_embedding else None, self.vector)


register("residual_input", "pass_vector", PassVector)
