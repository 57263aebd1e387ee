"""The gated delta rule: a recurrent mixer with a matrix state per head.

Per head, with unit-length q and k (q also times ``dim^-1/2``), ``beta = sigmoid(W_b x)`` and the decay
``g = exp(-exp(A_log) softplus(W_a x + dt_bias))``:

    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

(Yang et al., "Gated Delta Networks: Improving Mamba2 with Delta Rule").  q, k and v first pass a short causal
convolution over time per channel and SiLU; the read-out is RMS-normed per head, weighted, and gated by
``silu(W_g x)``.  ``kv_heads`` q/k heads serve ``heads`` value heads in groups.

A request keeps one float32 row in its state slot: the convolution's last ``taps - 1`` inputs, then S of every
head.  All of the batch is read through the step's device arrays, so single tokens, prompt portions cut anywhere
and padded rows of a replayed graph run the same kernels.
"""

from __future__ import annotations

import torch

from .base import MIXERS, Mixer, ParamSpec, StateNeed


class GatedDeltaRule(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                 conv_taps: int, norm_eps: float, prefix: str = "", names: dict[str, str] | None = None):
        super().__init__(prefix)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} q/k heads")
        if conv_taps < 1:
            raise ValueError("the short convolution needs at least one tap")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.value_dim, self.conv_taps = head_dim, value_dim, conv_taps
        self.norm_eps = float(norm_eps)
        self.names = {"q": "q", "k": "k", "v": "v", "gate": "g", "beta": "b", "decay": "a", "conv": "conv",
                      "A_log": "A_log", "dt_bias": "dt_bias", "norm": "norm", "o": "o", **(names or {})}

    @property
    def channels(self) -> int:
        """Columns that pass the convolution: q | k | v."""
        return 2 * self.num_kv_heads * self.head_dim + self.num_heads * self.value_dim

    @property
    def conv_floats(self) -> int:
        return (self.conv_taps - 1) * self.channels

    def cache_need(self):
        return StateNeed((self.conv_floats + self.num_heads * self.head_dim * self.value_dim,), torch.float32)

    def param_specs(self):
        n, h = self.names, self.hidden_size
        qk, v = self.num_kv_heads * self.head_dim, self.num_heads * self.value_dim
        conv = lambda name: f"{n[name]}.{n['conv']}"  # noqa: E731
        return {
            "proj.weight": ParamSpec.stacked([(n["q"], qk), (n["k"], qk), (n["v"], v), (n["gate"], v),
                                              (n["beta"], self.num_heads), (n["decay"], self.num_heads)], (h,)),
            "conv.weight": ParamSpec.stacked([(conv("q"), qk), (conv("k"), qk), (conv("v"), v)], (self.conv_taps,)),
            "A_log": ParamSpec.single(n["A_log"], (self.num_heads,), kind="vector"),
            "dt_bias": ParamSpec.single(n["dt_bias"], (self.num_heads,), kind="vector"),
            "norm.weight": ParamSpec.single(n["norm"], (self.value_dim,), kind="vector", init="one_plus_normal"),
            "o.weight": ParamSpec.single(n["o"], (h, v)),
        }

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        T = x.shape[0]
        H, dv, C = self.num_heads, self.value_dim, self.channels
        proj = ops.linear(x, self.params["proj.weight"], None, out_dtype=torch.float32)
        qkv = torch.empty((T, C), dtype=torch.float32, device=x.device)
        ops.conv_silu_state(proj, C, self.params["conv.weight"], cache.state, ctx.cu_seqlens_q, ctx.slot_of_seq, qkv,
                            max_q_len=ctx.max_q_len)
        read = torch.empty((T, H, dv), dtype=torch.float32, device=x.device)
        gate_off = C
        beta_off = C + H * dv
        ops.delta_rule(qkv, proj, beta_off + H, beta_off, self.params["A_log"], self.params["dt_bias"], cache.state,
                       self.conv_floats, ctx.cu_seqlens_q, ctx.slot_of_seq, read, H, self.num_kv_heads, self.head_dim,
                       dv)
        out = torch.empty((T, H * dv), dtype=x.dtype, device=x.device)
        ops.delta_out(read, proj, gate_off, self.params["norm.weight"], self.norm_eps, out)
        return ops.linear(out, self.params["o.weight"], None, defer=True)


MIXERS.register("gated_delta", GatedDeltaRule)
