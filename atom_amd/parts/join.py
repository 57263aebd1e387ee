"""What a model does to its stream where a pass over a run of repeated layers begins.

``concat_projection``: ``x <- W [x ; x0]`` with x the residual stream, x0 the embedding's output and W
[width, 2 width] (x's columns first).  The stream's pending summand is added on the way in; the product's float32
result starts the stream anew.
"""

from __future__ import annotations

import torch

from .base import JOINS, Join, ParamSpec


class ConcatProjection(Join):
    def __init__(self, hidden_size: int, prefix: str = "", weight_name: str = "weight"):
        super().__init__(prefix)
        self.hidden_size = hidden_size
        self.weight_name = weight_name

    def param_specs(self):
        return {"weight": ParamSpec.single(self.weight_name, (self.hidden_size, 2 * self.hidden_size))}

    def forward(self, ctx, hidden, residual, first):
        ops = ctx.ops
        hidden = ops.materialize(hidden)
        both = torch.empty((hidden.shape[0], 2 * self.hidden_size), dtype=ctx.dtype, device=hidden.device)
        ops.sum_concat(hidden, residual, first, both)
        return ops.linear(both, self.params["weight"], None, out_dtype=torch.float32), None


JOINS.register("concat_projection", ConcatProjection)
