"""A per-layer input that depends on the token itself: with ``e`` the layer's ``dim`` columns of a table that has a
row per token id (shared by all layers: columns ``[layer * dim, (layer + 1) * dim)``),

    g = gelu_tanh(W_gate x) * e[token];   y = W_proj g;   x += y / rms(y) * w

The norm is an RMS norm with a plain weight.  The table is one of the model's shared token tables
(``ctx.tables[table_name]``); the token ids are the step's (``ctx.token_ids``).  The part adds to the stream
itself (``forward_stream``), since what it adds is normed in float32 like every other summand of the stream.
"""

from __future__ import annotations

import torch

from .base import FEED_FORWARDS, FeedForward, ParamSpec


class TokenSide(FeedForward):
    def __init__(self, hidden_size: int, vocab_size: int, dim: int, layer: int, num_layers: int, norm_eps: float,
                 table_name: str, prefix: str = "", names: dict[str, str] | None = None):
        super().__init__(prefix)
        if not 0 <= layer < num_layers:
            raise ValueError(f"layer {layer} of {num_layers}")
        self.hidden_size, self.vocab_size, self.dim = hidden_size, vocab_size, dim
        self.layer, self.num_layers = layer, num_layers
        self.norm_eps = float(norm_eps)
        self.table_name = table_name
        self.names = {"gate": "gate", "proj": "proj", "norm": "norm", **(names or {})}

    def param_specs(self):
        n = self.names
        return {"gate.weight": ParamSpec.single(n["gate"], (self.dim, self.hidden_size)),
                "proj.weight": ParamSpec.single(n["proj"], (self.hidden_size, self.dim)),
                "norm.weight": ParamSpec.single(n["norm"], (self.hidden_size,), kind="vector", init="one_plus_normal")}

    def forward(self, ctx, x):
        raise NotImplementedError("this part adds to the stream itself: forward_stream")

    def forward_stream(self, ctx, reads, stream):
        """``reads``: the stream's rows in the step's type; ``stream``: float32, added to in place.  Returns the
        stream's new rows in the step's type."""
        ops = ctx.ops
        table = ctx.tables[self.table_name].params["weight"]
        if table.shape[1] != self.num_layers * self.dim:
            raise ValueError(f"the token table has {table.shape[1]} columns, {self.num_layers} layers of {self.dim} "
                             "need others")
        raw = ops.linear(reads, self.params["gate.weight"], None, out_dtype=torch.float32)
        gated = torch.empty((raw.shape[0], self.dim), dtype=ctx.dtype, device=raw.device)
        ops.token_gate(raw, table, self.layer * self.dim, ctx.token_ids, gated)
        y = ops.linear(gated, self.params["proj.weight"], None, out_dtype=torch.float32)
        out = None
        if ctx.dtype != torch.float32:
            out = torch.empty(tuple(stream.shape), dtype=ctx.dtype, device=stream.device)
        ops.rmsnorm_post(y, self.params["norm.weight"], self.norm_eps, stream, out)
        return stream if out is None else out


FEED_FORWARDS.register("token_side", TokenSide)
