"""A feed-forward of routed experts: every token runs ``top`` of ``experts`` small gated feed-forwards and takes
the weighted sum of their outputs.

The router's logits are a float32 product; the scores are their sigmoids.  A per-expert ``correction`` is added to
the scores for the choice only (a load-balancing bias that leaves the weights alone); the weights are the chosen
experts' scores, renormalised to sum to one only when asked.  Experts have no biases; their matrices are stacked
[experts, 2 ff, width] (gate rows, then up rows) and [experts, width, ff].
"""

from __future__ import annotations

from .base import FEED_FORWARDS, FeedForward, ParamSpec


class RoutedExperts(FeedForward):
    def __init__(self, hidden_size: int, expert_size: int, num_experts: int, top: int, activation: str = "silu",
                 correction: bool = True, renormalize: bool = False, prefix: str = "",
                 names: dict[str, str] | None = None):
        super().__init__(prefix)
        if not 0 < top <= num_experts:
            raise ValueError(f"a token cannot use {top} of {num_experts} experts")
        self.hidden_size, self.expert_size, self.num_experts, self.top = hidden_size, expert_size, num_experts, top
        self.activation = activation
        self.has_correction, self.renormalize = bool(correction), bool(renormalize)
        self.names = {"router": "router", "correction": "correction", "expert": "e{}", "gate": "gate", "up": "up",
                      "down": "down", **(names or {})}
        self.gate_up = self.down = None

    def param_specs(self):
        n, h, f = self.names, self.hidden_size, self.expert_size
        gate_up, down = [], []
        for e in range(self.num_experts):
            ex = n["expert"].format(e)
            gate_up += [(f"{ex}.{n['gate']}", f), (f"{ex}.{n['up']}", f)]
            down.append((f"{ex}.{n['down']}", h))
        specs = {
            "router.weight": ParamSpec.single(n["router"], (self.num_experts, h)),
            "gate_up.weight": ParamSpec.stacked(gate_up, (h,)),
            "down.weight": ParamSpec.stacked(down, (f,)),
        }
        if self.has_correction:
            specs["correction"] = ParamSpec.single(n["correction"], (self.num_experts,), kind="vector")
        return specs

    def finalize(self, device, dtype):
        self.gate_up = self.params["gate_up.weight"].view(self.num_experts, 2 * self.expert_size, self.hidden_size)
        self.down = self.params["down.weight"].view(self.num_experts, self.hidden_size, self.expert_size)

    def forward(self, ctx, x):
        ops = ctx.ops
        logits = ops.linear_f32(x, self.params["router.weight"])
        ids, weights = ops.router_choose(logits, self.p("correction"), self.top, self.renormalize)
        return ops.experts_forward(x, self.gate_up, self.down, ids, weights, self.activation)


FEED_FORWARDS.register("routed_experts", RoutedExperts)
