"""Token embedding and the language-model head (atom/model_ops/embed_head.py:138-178,
225-263).  The head may share the embedding's table (atom/models/qwen3.py:339-340);
it is applied only to the rows whose logits are asked for (embed_head.py:249-252)."""

from __future__ import annotations

import torch

from .base import EMBEDDINGS, HEADS, Embedding, Head, ParamSpec


class TokenEmbedding(Embedding):
    def __init__(self, vocab_size: int, hidden_size: int, prefix: str = "", weight_name: str = "weight"):
        super().__init__(prefix)
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.weight_name = weight_name   # the table's checkpoint name under the prefix (empty: the prefix itself)

    def param_specs(self):
        return {"weight": ParamSpec.single(self.weight_name, (self.vocab_size, self.hidden_size))}

    def forward(self, ctx, ids: torch.Tensor) -> torch.Tensor:
        out = torch.empty((ids.numel(), self.hidden_size), dtype=ctx.dtype, device=ids.device)
        return ctx.ops.embedding(self.params["weight"], ids, out)


class ScaledEmbedding(TokenEmbedding):
    """``table[ids] * scale`` as float32 rows: the start of a float32 residual stream, not rounded to the
    serving type on the way."""

    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0, prefix: str = "",
                 weight_name: str = "weight"):
        super().__init__(vocab_size, hidden_size, prefix, weight_name)
        self.scale = float(scale)

    def forward(self, ctx, ids: torch.Tensor) -> torch.Tensor:
        out = torch.empty((ids.numel(), self.hidden_size), dtype=torch.float32, device=ids.device)
        return ctx.ops.embedding_scaled(self.params["weight"], ids, out, self.scale)


class LMHead(Head):
    """``logits = x @ W.T`` in float32 out.  ``tied_to`` names the embedding whose table it shares."""

    def __init__(self, vocab_size: int, hidden_size: int, tied_to: TokenEmbedding | None = None, prefix: str = "",
                 weight_name: str = "weight"):
        super().__init__(prefix)
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.tied_to = tied_to
        self.weight_name = weight_name

    def param_specs(self):
        if self.tied_to is not None:
            return {}
        return {"weight": ParamSpec.single(self.weight_name, (self.vocab_size, self.hidden_size))}

    @property
    def weight(self) -> torch.Tensor:
        return self.tied_to.params["weight"] if self.tied_to is not None else self.params["weight"]

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        return ctx.ops.linear(x, self.weight, None, out_dtype=torch.float32)


EMBEDDINGS.register("token_embedding", TokenEmbedding)
EMBEDDINGS.register("scaled_f32_embedding", ScaledEmbedding)
HEADS.register("lm_head", LMHead)
