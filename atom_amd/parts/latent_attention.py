"""Attention whose keys and values are expanded from one cached latent per token.

Per token the mixer caches ``c`` (an RMS-normed down-projection of ``kv_rank`` entries) and one rotated key part
of ``rot_dim`` entries that all heads share.  Head h's key is ``[W_uk,h c ; k_rot]``, its value ``W_uv,h c``, its
query ``[q_h ; q_rot,h]`` with rotation on the ``rot`` parts only.  Since ``q_h . (W_uk,h c) = (W_uk,h^T q_h) . c``
the queries are brought into the latent space instead of the keys out of it: attention then runs over the cached
rows themselves, which all heads share, and the weighted sum of latents is expanded by ``W_uv,h`` afterwards.
Options: a learned sink per head in the softmax's denominator, a sigmoid gate per head on the output.

Order of kernels: one product for q | down-projection | gate (float32 out); norm, rotation and cache write; the
queries' absorption (a product per head); attention; the expansion by ``W_uv`` with the gate folded in; the output
product.
"""

from __future__ import annotations

import torch

from ..kernels.hip import AttentionMeta
from .base import MIXERS, POSITION_ENCODINGS, LatentCacheNeed, Mixer, ParamSpec, PartChoice


class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, kv_rank: int,
                 scale: float, norm_eps: float, position_encoding: PartChoice | None = None, sink: bool = False,
                 gate: bool = False, window: int | None = None, prefix: str = "", names: dict[str, str] | None = None):
        super().__init__(prefix)
        self.hidden_size, self.num_heads = hidden_size, num_heads
        self.head_dim, self.rot_dim, self.value_dim, self.kv_rank = head_dim, rot_dim, value_dim, kv_rank
        self.scale = float(scale)
        self.norm_eps = float(norm_eps)
        self.has_sink, self.has_gate = bool(sink), bool(gate)
        self.window = window
        self.names = {"q": "q", "down": "dkv", "down_norm": "dkv.norm", "up_k": "uk", "up_v": "uv", "sink": "sink",
                      "gate": "g", "o": "o", **(names or {})}
        self.rope = position_encoding.build(POSITION_ENCODINGS) if position_encoding is not None else None
        if self.rope is not None and self.rope.dims > rot_dim:
            raise ValueError(f"{self.rope.dims} rotated dimensions do not fit a rotated part of {rot_dim}")
        self.up_k = self.up_v = None

    def children(self):
        return [self.rope] if self.rope is not None else []

    def cache_need(self):
        return LatentCacheNeed(self.kv_rank + self.rot_dim, self.window)

    @property
    def q_width(self) -> int:
        return self.num_heads * (self.head_dim + self.rot_dim)

    def param_specs(self):
        n, h = self.names, self.hidden_size
        rows = [(n["q"], self.q_width), (n["down"], self.kv_rank + self.rot_dim)]
        if self.has_gate:
            rows.append((n["gate"], self.num_heads))
        specs = {
            "proj.weight": ParamSpec.stacked(rows, (h,)),
            "down_norm.weight": ParamSpec.single(n["down_norm"], (self.kv_rank,), kind="vector", init="one_plus_normal"),
            "up_k.weight": ParamSpec.single(n["up_k"], (self.num_heads * self.head_dim, self.kv_rank)),
            "up_v.weight": ParamSpec.single(n["up_v"], (self.num_heads * self.value_dim, self.kv_rank)),
            "o.weight": ParamSpec.single(n["o"], (h, self.num_heads * self.value_dim)),
        }
        if self.has_sink:
            specs["sink"] = ParamSpec.single(n["sink"], (self.num_heads,), kind="vector")
        return specs

    def finalize(self, device, dtype):
        # per head: the key up-projection transposed, [heads, rank, dim], so that absorbing a query is x W^T like
        # every other product; the value up-projection is [heads, vdim, rank] as stored
        H, d, dv, rank = self.num_heads, self.head_dim, self.value_dim, self.kv_rank
        self.up_k = self.params["up_k.weight"].view(H, d, rank).transpose(1, 2).contiguous()
        self.up_v = self.params["up_v.weight"].view(H, dv, rank)

    def _meta(self, ctx, group: int) -> AttentionMeta:
        key = ("latent attention meta", group)
        meta = ctx.memo.get(key)
        if meta is None:
            meta = AttentionMeta(
                token_seq=ctx.token_seq, positions=ctx.positions, block_tables=ctx.block_tables[group],
                cu_seqlens_q=ctx.cu_seqlens_q, context_lens=ctx.context_lens, num_seqs=ctx.num_seqs,
                num_tokens=ctx.num_tokens, max_q_len=ctx.max_q_len, max_context_len=ctx.max_context_len,
                page_size=ctx.page_sizes[group], num_prefill=ctx.num_prefill)
            ctx.memo[key] = meta
        return meta

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        T = x.shape[0]
        H, d, r, dv, rank = self.num_heads, self.head_dim, self.rot_dim, self.value_dim, self.kv_rank
        width = rank + r
        proj = ops.linear(x, self.params["proj.weight"], None, out_dtype=torch.float32)
        ld = proj.shape[1]
        q_abs = torch.empty((T, H, width), dtype=x.dtype, device=x.device)
        rope = self.rope
        ops.latent_prepare(proj, 0, self.q_width, H, d, r, rank, rope.dims if rope else 0,
                           self.params["down_norm.weight"], self.norm_eps, rope.freq if rope else None,
                           rope.mult if rope else 1.0, ctx.positions,
                           ctx.slot_mappings[cache.group] if cache.writes else None, cache.pages, q_abs, self.scale)
        ops.heads_gemm(proj, 0, ld, d + r, self.up_k, q_abs, 0, H * width, width, H, T, rank, d, alpha=self.scale)
        latent = torch.empty((T, H, rank), dtype=x.dtype, device=x.device)
        ops.latent_attention(q_abs, cache.pages, latent, self._meta(ctx, cache.group), rank,
                             self.p("sink") if self.has_sink else None, self.window)
        out = torch.empty((T, H * dv), dtype=x.dtype, device=x.device)
        ops.heads_gemm(latent, 0, H * rank, rank, self.up_v, out, 0, H * dv, dv, H, T, dv, rank,
                       gate=proj if self.has_gate else None, gate_offset=self.q_width + width, ldg=ld)
        return ops.linear(out, self.params["o.weight"], None, defer=True)


MIXERS.register("latent_attention", LatentAttention)
