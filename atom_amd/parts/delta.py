"""The gated delta rule: a recurrent mixer with a matrix state per head.

Per head, with unit-length q and k (q also times ``dim^-1/2``), ``beta = sigmoid(W_b x)`` and the decay
``g = exp(-exp(A_log) softplus(W_a x + dt_bias))``:

    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

(Yang et al., "Gated Delta Networks: Improving Mamba2 with Delta Rule").  q, k and v first pass a short causal
convolution over time per channel and SiLU; the read-out is RMS-normed per head, weighted, and gated by
``silu(W_g x)``.  ``kv_heads`` q/k heads serve ``heads`` value heads in groups.

Options: ``decay`` "head" (one decay per head) or "channel" (one per head and key channel, acting on the rows of
S: ``A_log`` stays per head, ``dt_bias`` and the decay's projection have heads x dim entries); ``decay_low_rank`` /
``gate_low_rank``: the projection is a product of two, ``W_2 (W_1 x)`` (checkpoint names with 1 and 2 appended),
whose inner size is ``decay_rank`` / ``gate_rank`` or, where that is None, the checkpoint tensor's own;
``gate_activation`` "silu" or "sigmoid".

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
                 conv_taps: int, norm_eps: float, decay: str = "head", decay_low_rank: bool = False,
                 gate_low_rank: bool = False, gate_activation: str = "silu", decay_rank: int | None = None,
                 gate_rank: int | None = None, prefix: str = "", names: dict[str, str] | None = None):
        super().__init__(prefix)
        if decay not in ("head", "channel"):
            raise ValueError(f"decay is per 'head' or per 'channel', got {decay!r}")
        if gate_activation not in ("silu", "sigmoid"):
            raise ValueError(f"the read-out's gate is 'silu' or 'sigmoid', got {gate_activation!r}")
        self.decay, self.decay_low_rank, self.gate_low_rank = decay, bool(decay_low_rank), bool(gate_low_rank)
        self.gate_activation = gate_activation
        self.decay_rank, self.gate_rank = decay_rank, gate_rank
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

    @property
    def decay_width(self) -> int:
        return self.num_heads * (self.head_dim if self.decay == "channel" else 1)

    def adopt_shapes(self, shape_of):
        n = self.names
        for low, rank, name in ((self.decay_low_rank, "decay_rank", n["decay"]), (self.gate_low_rank, "gate_rank", n["gate"])):
            if low and getattr(self, rank) is None:
                shape = shape_of(f"{name}1")
                if shape is not None and len(shape) == 2:
                    setattr(self, rank, int(shape[0]))

    def _rank(self, which: str) -> int:
        rank = getattr(self, which)
        if rank is None:
            raise ValueError(f"{which} is not known: name it, or load the model from a checkpoint whose tensors say it")
        return rank

    def _layout(self):
        """Rows of the stacked projection, in order, as (checkpoint name, rows), and where each piece begins."""
        n = self.names
        qk, v = self.num_kv_heads * self.head_dim, self.num_heads * self.value_dim
        rows = [(n["q"], qk), (n["k"], qk), (n["v"], v),
                (f"{n['gate']}1", self._rank("gate_rank")) if self.gate_low_rank else (n["gate"], v),
                (n["beta"], self.num_heads),
                (f"{n['decay']}1", self._rank("decay_rank")) if self.decay_low_rank else (n["decay"], self.decay_width)]
        at, offsets = 0, []
        for _, r in rows:
            offsets.append(at)
            at += r
        return rows, {"gate": offsets[3], "beta": offsets[4], "decay": offsets[5], "total": at}

    def param_specs(self):
        n, h = self.names, self.hidden_size
        qk, v = self.num_kv_heads * self.head_dim, self.num_heads * self.value_dim
        conv = lambda name: f"{n[name]}.{n['conv']}"  # noqa: E731
        specs = {
            "proj.weight": ParamSpec.stacked(self._layout()[0], (h,)),
            "conv.weight": ParamSpec.stacked([(conv("q"), qk), (conv("k"), qk), (conv("v"), v)], (self.conv_taps,)),
            "A_log": ParamSpec.single(n["A_log"], (self.num_heads,), kind="vector"),
            "dt_bias": ParamSpec.single(n["dt_bias"], (self.decay_width,), kind="vector"),
            "norm.weight": ParamSpec.single(n["norm"], (self.value_dim,), kind="vector", init="one_plus_normal"),
            "o.weight": ParamSpec.single(n["o"], (h, v)),
        }
        if self.decay_low_rank:
            specs["decay2.weight"] = ParamSpec.single(f"{n['decay']}2", (self.decay_width, self._rank("decay_rank")))
        if self.gate_low_rank:
            specs["gate2.weight"] = ParamSpec.single(f"{n['gate']}2", (v, self._rank("gate_rank")))
        return specs

    def _second(self, ops, proj, offset: int, weight):
        """``W_2`` applied to the columns of the float32 projection that hold ``W_1 x``, as float32 sums."""
        T, ld = proj.shape
        n, k = weight.shape
        out = torch.empty((T, n), dtype=torch.float32, device=proj.device)
        return ops.heads_gemm(proj, offset, ld, 0, weight.view(1, n, k), out, 0, n, 0, 1, T, n, k, exact=True)

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        T = x.shape[0]
        H, dv, C = self.num_heads, self.value_dim, self.channels
        proj = ops.linear(x, self.params["proj.weight"], None, out_dtype=torch.float32)
        qkv = torch.empty((T, C), dtype=torch.float32, device=x.device)
        ops.conv_silu_state(proj, C, self.params["conv.weight"], cache.state, ctx.cu_seqlens_q, ctx.slot_of_seq, qkv,
                            max_q_len=ctx.max_q_len)
        read = torch.empty((T, H, dv), dtype=torch.float32, device=x.device)
        at = self._layout()[1]
        decay, decay_off = proj, at["decay"]
        if self.decay_low_rank:
            decay, decay_off = self._second(ops, proj, at["decay"], self.params["decay2.weight"]), 0
        gate, gate_off = proj, at["gate"]
        if self.gate_low_rank:
            gate, gate_off = self._second(ops, proj, at["gate"], self.params["gate2.weight"]), 0
        ops.delta_rule(qkv, proj, decay_off, at["beta"], self.params["A_log"], self.params["dt_bias"], cache.state,
                       self.conv_floats, ctx.cu_seqlens_q, ctx.slot_of_seq, read, H, self.num_kv_heads, self.head_dim,
                       dv, decay=decay, per_channel=self.decay == "channel")
        out = torch.empty((T, H * dv), dtype=x.dtype, device=x.device)
        ops.delta_out(read, gate, gate_off, self.params["norm.weight"], self.norm_eps, out,
                      activation=self.gate_activation)
        return ops.linear(out, self.params["o.weight"], None, defer=True)


MIXERS.register("gated_delta", GatedDeltaRule)
