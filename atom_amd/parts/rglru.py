"""A real-gated linear recurrence between two branches (the recurrent block of De et al., "Griffin: Mixing Gated
Linear Recurrences with Local Attention for Efficient Language Models").

With ``C = width`` channels in ``blocks`` equal parts:

    y = gelu_tanh(W_y x + b_y)                    u = conv(W_x x + b_x)        (short causal convolution per channel,
    r = sigmoid(R_b u_b + c_b)                    i = sigmoid(I_b u_b + d_b)    bias, no activation; gates per part b)
    a = exp(-8 r softplus(lam))                   S <- a S + sqrt(1 - a^2) (i u)
    out = W_o (S y)

S starts at zero, also for a request's first token.  A request keeps one float32 row in its state slot: the
convolution's last ``taps - 1`` inputs, then S.  Gates, decay and state are float32; the gates' small products
take the convolution's float32 output as it is.
"""

from __future__ import annotations

import torch

from .base import MIXERS, Mixer, ParamSpec, StateNeed


class RealGatedRecurrence(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, width: int, blocks: int, conv_taps: int, decay_scale: float = 8.0,
                 prefix: str = "", names: dict[str, str] | None = None):
        super().__init__(prefix)
        if width % blocks:
            raise ValueError(f"{width} channels do not split into {blocks} equal parts")
        if conv_taps < 1:
            raise ValueError("the short convolution needs at least one tap")
        self.hidden_size, self.width, self.blocks, self.conv_taps = hidden_size, width, blocks, conv_taps
        self.decay_scale = float(decay_scale)
        self.names = {"x": "x", "y": "y", "conv": "conv", "recurrence_gate": "ra", "input_gate": "ri", "lam": "lam",
                      "o": "o", "bias": "b", **(names or {})}

    @property
    def conv_floats(self) -> int:
        return (self.conv_taps - 1) * self.width

    def cache_need(self):
        return StateNeed((self.conv_floats + self.width,), torch.float32)

    def param_specs(self):
        n, c, h = self.names, self.width, self.hidden_size
        part = c // self.blocks
        b = lambda name: f"{n[name]}.{n['bias']}"  # noqa: E731
        return {
            "in.weight": ParamSpec.stacked([(n["x"], c), (n["y"], c)], (h,)),
            "in.bias": ParamSpec.stacked([(b("x"), c), (b("y"), c)], (), kind="vector"),
            "conv.weight": ParamSpec.single(n["conv"], (c, self.conv_taps)),
            "conv.bias": ParamSpec.single(b("conv"), (c,), kind="vector"),
            "ra.weight": ParamSpec.single(n["recurrence_gate"], (self.blocks, part, part)),
            "ra.bias": ParamSpec.single(b("recurrence_gate"), (self.blocks, part), kind="vector"),
            "ri.weight": ParamSpec.single(n["input_gate"], (self.blocks, part, part)),
            "ri.bias": ParamSpec.single(b("input_gate"), (self.blocks, part), kind="vector"),
            "lam": ParamSpec.single(n["lam"], (c,), kind="vector"),
            "o.weight": ParamSpec.single(n["o"], (h, c)),
        }

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        T, c = x.shape[0], self.width
        part = c // self.blocks
        proj = ops.linear(x, self.params["in.weight"], self.params["in.bias"], out_dtype=torch.float32)   # x | y
        u = torch.empty((T, c), dtype=torch.float32, device=x.device)
        ops.conv_silu_state(proj, c, self.params["conv.weight"], cache.state, ctx.cu_seqlens_q, ctx.slot_of_seq, u,
                            max_q_len=ctx.max_q_len, bias=self.params["conv.bias"], activation="none")
        gates = torch.empty((2, T, c), dtype=torch.float32, device=x.device)
        for which, name in enumerate(("ra.weight", "ri.weight")):
            ops.heads_gemm(u, 0, c, part, self.params[name], gates, which * T * c, c, part, self.blocks, T, part, part,
                           exact=True)
        out = torch.empty((T, c), dtype=x.dtype, device=x.device)
        ops.rglru_scan(u, gates, self.params["ra.bias"], self.params["ri.bias"], self.params["lam"], proj, c,
                       cache.state, self.conv_floats, ctx.cu_seqlens_q, ctx.slot_of_seq, out, self.decay_scale,
                       max_q_len=ctx.max_q_len)
        return ops.linear(out, self.params["o.weight"], None, defer=True)


MIXERS.register("rglru", RealGatedRecurrence)
