"""Grouped-query attention whose values are its keys, over the paged cache.

``q = W_q x + b_q`` and ``k = W_k x + b_k``; the values are k as projected.  Then q and k are RMS-normed over the
whole projection (all heads at once, one weight per entry), rotated (interleaved pairs of the first ``dims``
entries of each head), and

    score = cap * tanh((q . k) * scale / cap)        (no cap: the scaled product itself)

over the keys a query may see: those at or before it, within the last ``window`` positions where a window is set,
and within its own chunk of ``chunk`` positions (counted from position 0 of the request) where chunks are set.
Ordinary softmax.  The heads' outputs are multiplied by ``sigmoid(W_g x)`` before the output projection.

Key pages hold the normed, rotated keys; value pages hold the keys as projected.  One packed product gives q, k
and the gate's input as float32; one kernel norms, rotates and writes both page kinds.
"""

from __future__ import annotations

import torch

from .attention import GroupedQueryAttention
from .base import MIXERS, POSITION_ENCODINGS, KVCacheNeed, ParamSpec, PartChoice, Source


class KeyValueAttention(GroupedQueryAttention):
    graph_safe = True
    accepts_deferred = False

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, scale: float,
                 softcap: float | None = None, chunk: int | None = None, window: int | None = None,
                 bias: bool = True, wide_norm: bool = True, gate: bool = True, norm_eps: float = 1e-6,
                 position_encoding: PartChoice | None = None, prefix: str = "", names: dict[str, str] | None = None):
        super().__init__(hidden_size, num_heads, num_kv_heads, head_dim, norm_eps=norm_eps, scale=scale, window=window,
                         position_encoding=None, prefix=prefix)
        self.softcap = float(softcap) if softcap else None
        self.chunk = int(chunk) if chunk else None
        self.bias, self.wide_norm, self.gate = bool(bias), bool(wide_norm), bool(gate)
        self.names = {"q": "q", "k": "k", "gate": "g", "o": "o", "norm": "norm", "bias": "b", **(names or {})}
        self.rope = position_encoding.build(POSITION_ENCODINGS, head_dim=head_dim) if position_encoding else None

    def cache_need(self):
        return KVCacheNeed(self.num_kv_heads, self.head_dim, self.window, self.chunk)

    def param_specs(self):
        n = self.names
        q_rows, k_rows = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        rows = [(n["q"], q_rows), (n["k"], k_rows)] + ([(n["gate"], q_rows)] if self.gate else [])
        specs = {"proj.weight": ParamSpec.stacked(rows, (self.hidden_size,)),
                 "o.weight": ParamSpec.single(n["o"], (self.hidden_size, q_rows))}
        if self.bias:
            # the gate's rows have no bias: theirs stays zero
            specs["proj.bias"] = ParamSpec((sum(r for _, r in rows),), "vector",
                                           (Source(f"{n['q']}.{n['bias']}", 0, q_rows),
                                            Source(f"{n['k']}.{n['bias']}", q_rows, k_rows)))
        if self.wide_norm:
            specs["q_norm.weight"] = ParamSpec.single(f"{n['q']}.{n['norm']}", (q_rows,), kind="vector",
                                                      init="one_plus_normal")
            specs["k_norm.weight"] = ParamSpec.single(f"{n['k']}.{n['norm']}", (k_rows,), kind="vector",
                                                      init="one_plus_normal")
        return specs

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        tokens = x.shape[0]
        H, G, D = self.num_heads, self.num_kv_heads, self.head_dim
        proj = ops.linear(x, self.params["proj.weight"], self.p("proj.bias"), out_dtype=torch.float32)
        meta = self._meta(ctx, cache.group)
        rope = self.rope
        q = torch.empty((tokens, H, D), dtype=x.dtype, device=x.device)
        ops.keys_as_values_write(proj, q, cache.k_cache, cache.v_cache, self.p("q_norm.weight"), self.p("k_norm.weight"),
                                 rope.freq if rope else None, rope.dims if rope else 0, ctx.positions,
                                 ctx.slot_mappings[cache.group], H, G, D, meta.page_size, self.norm_eps,
                                 write_kv=cache.writes)
        out = torch.empty((tokens, H, D), dtype=x.dtype, device=x.device)
        ops.paged_attention(q, cache.k_cache, cache.v_cache, out, meta, self.scale, self.window, softcap=self.softcap,
                            chunk=self.chunk)
        heads = out.view(tokens, H * D)
        if self.gate:
            gated = torch.empty((tokens, H * D), dtype=x.dtype, device=x.device)
            heads = ops.sigmoid_gate(heads, proj, (H + G) * D, gated)
        return ops.linear(heads, self.params["o.weight"], None, defer=True)


MIXERS.register("key_value_attention", KeyValueAttention)
