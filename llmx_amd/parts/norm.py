"""Norms of float32 rows.  RMSNorm: y = x * (r * w), r = 1/sqrt(mean(x^2) + eps); LayerNorm (a weight, no bias):
y = (x - mean) / sqrt(var + eps) * w, var the mean of the squared deviations.  All in float32.

Order of operations as the reference computes it (/root/reference/src/backends/cpu/cpu_backend.hpp:1437-1459): the
reciprocal root times the weight is formed first, then multiplied into x.
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import ops
from .base import Norm, register
from .spec import TensorSpec


class RMSNorm(Norm):
    """params: width, eps; gain ("vector", the default: one weight a coordinate; "scalar": the file holds one number for
    all coordinates); tensor (the name's last part, "weight" by default; "" when the prefix is the whole name); optional
    (True: a norm that nothing runs, listed only so that a file which holds its tensor all the same is not refused);
    offset (0 by default; 1 for a weight that is stored around zero: the gain is offset + the stored weight, formed once
    at load in float32).  Tensor: <prefix><tensor>, (width,) or ().  `add_into` is the form an arrangement uses that norms
    a sublayer's result on its way into the residual."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.width = int(params["width"])
        self.eps = float(params["eps"])
        self.gain = str(params.get("gain", "vector"))
        if self.gain not in ("vector", "scalar"):
            raise ValueError(f"norm gain {self.gain!r} is not one of ['scalar', 'vector']")
        self.tensor = str(params.get("tensor", "weight"))
        self.optional = bool(params.get("optional", False))
        self.offset = float(params.get("offset", 0.0))
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self, available):
        if self.optional and self.name(self.tensor) not in available:
            return []
        # random weights: the gain lies around 1 either way, so a stored weight with an offset lies around 1 - offset
        init = ("normal", 1.0 - self.offset, 0.05) if self.offset else None
        return [TensorSpec(self.name(self.tensor), (self.width,) if self.gain == "vector" else (), "norm", init=init)]

    def load(self, tensors):
        if self.optional and self.name(self.tensor) not in tensors:
            return
        w = tensors[self.name(self.tensor)]
        if self.offset:
            w = w + self.offset
        # one number for all coordinates is kept as a row of that number, which every norm kernel takes as it is
        self.weight = w if self.gain == "vector" else w.reshape(1).expand(self.width).contiguous()

    def forward(self, step, x, out, out32=None, pick=None):
        ops.rmsnorm(x, self.weight, self.eps, out, out32, pick)

    def deferred(self, x):
        return ops.NormedRows(x, self.weight, self.eps)

    def add_into(self, step, x, y, copy=None):
        """x += norm(y); `copy` (optional) receives the new rows in its own type."""
        ops.rmsnorm_add(x, y, self.weight, self.eps)
        if copy is not None:
            ops.cast_rows(x, copy)

    def add_into_then_norm(self, step, x, y, then: "RMSNorm", out, out32=None):
        """x += norm(y); out / out32 = then(x): the join and the next sublayer's norm in one launch."""
        ops.rmsnorm_add_norm(x, y, self.weight, self.eps, then.weight, then.eps, out, out32)


class LayerNorm(Norm):
    """params: width, eps; tensor (the name's last part, "weight" by default; "" when the prefix is the whole name).
    Tensor: <prefix><tensor>, (width,).  `add_into` is the form an arrangement uses that norms a sublayer's result on its
    way into the residual."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.width = int(params["width"])
        self.eps = float(params["eps"])
        self.tensor = str(params.get("tensor", "weight"))
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self, available):
        return [TensorSpec(self.name(self.tensor), (self.width,), "norm")]

    def load(self, tensors):
        self.weight = tensors[self.name(self.tensor)]

    def forward(self, step, x, out, out32=None, pick=None):
        ops.layernorm(x, self.weight, self.eps, out, out32, pick)

    def add_into(self, step, x, y, copy=None):
        """x += norm(y); `copy` (optional) receives the new rows in its own type."""
        ops.layernorm_add(x, y, self.weight, self.eps, copy)


register("norm", "rmsnorm", RMSNorm)
register("norm", "layernorm", LayerNorm)
