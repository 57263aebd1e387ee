"""Ralitar as a ``ModelSpec``.

The stream starts as the token's embedding row plus a row of a second table chosen by a hash of the previous
and the current token (a row of its own for a request's first token); it is float32 throughout.  Every layer is
a block whose sublayers read the stream itself and whose outputs are RMS-normed on the way in:
``x += norm1(mixer(x))``, then ``x += norm2(ff(x))`` where the layer has a feed-forward, then a small input that
depends on the token: ``x += rmsnorm(W_proj (gelu(W_gate x) * e_layer[token]))``.  The mixer is a real-gated
linear recurrence (two branches, short convolution, block-diagonal gates), the gated delta rule with one decay
per key channel and low-rank decay and gate projections, or grouped-query attention within chunks of positions
whose values are its unnormed, unrotated keys, with a tanh cap on the scores and a sigmoid output gate.  The
feed-forward is dense and gated by tanh-GELU.  A final RMS norm and an untied head.

Checkpoint names: ``embed``, ``bigram``, ``side.embed``, ``l<i>.norm1`` / ``.norm2`` (weights), ``l<i>.mix.*``,
``l<i>.mlp.*``, ``l<i>.side.{gate,proj,norm}``, ``final.norm``, ``head``; matrices carry no ``.weight`` suffix,
biases end in ``.b``.
"""

from __future__ import annotations

from ..config.model_config import RalitarConfig
from ..parts.base import PartChoice
from .model import ModelSpec


def _mixer(cfg: RalitarConfig, layer: dict) -> PartChoice:
    m = layer["mixer"]
    if layer["type"] == "rglru":
        return PartChoice("rglru", {"hidden_size": cfg.hidden_size, "width": m["width"], "blocks": m["blocks"],
                                    "conv_taps": m["conv"]})
    if layer["type"] == "channel_delta":
        return PartChoice("gated_delta", {
            "hidden_size": cfg.hidden_size, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"],
            "head_dim": m["dim"], "value_dim": m["vdim"], "conv_taps": m["conv"], "norm_eps": cfg.norm_eps,
            "decay": "channel", "decay_low_rank": True, "gate_low_rank": True, "gate_activation": "sigmoid",
            # the inner sizes of the two low-rank projections are the checkpoint tensors' own; a configuration may
            # name them for weights that are drawn, not loaded
            "decay_rank": m.get("decay_rank"), "gate_rank": m.get("gate_rank")})
    rope = None
    rot = m.get("rot")
    if rot is not None and rot["dims"] > 0:
        scaling = rot.get("scaling") or {}
        rope = PartChoice("banded_rotary", {"dims": rot["dims"], "base": rot["base"], "factor": scaling.get("factor"),
                                            "low": scaling.get("low"), "high": scaling.get("high"),
                                            "original": scaling.get("original")})
    return PartChoice("key_value_attention", {
        "hidden_size": cfg.hidden_size, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
        "scale": m["scale"], "softcap": m.get("softcap"), "chunk": (m.get("mask") or {}).get("size"),
        "norm_eps": cfg.norm_eps, "position_encoding": rope})


def _feed_forward(cfg: RalitarConfig, layer: dict) -> PartChoice | None:
    mlp = layer.get("mlp")
    if mlp is None:
        return None
    return PartChoice("gated_mlp", {"hidden_size": cfg.hidden_size, "intermediate_size": mlp["ff"],
                                    "activation": "gelu_tanh", "weight_suffix": "",
                                    "names": {"gate": "gate", "up": "up", "down": "down"}})


def ralitar_spec(cfg: RalitarConfig) -> ModelSpec:
    norm = PartChoice("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.norm_eps, "weight_name": ""})
    blocks = []
    for i, layer in enumerate(cfg.layers):
        side = None
        if cfg.side_dim:
            side = PartChoice("token_side", {"hidden_size": cfg.hidden_size, "vocab_size": cfg.vocab_size,
                                             "dim": cfg.side_dim, "layer": i, "num_layers": len(cfg.layers),
                                             "norm_eps": cfg.norm_eps, "table_name": "side.embed"})
        blocks.append(PartChoice("postnorm", {"mixer": _mixer(cfg, layer), "feed_forward": _feed_forward(cfg, layer),
                                              "norm": norm, "side": side}))
    if cfg.bigram is not None:
        buckets, mul_prev, mul_cur = cfg.bigram
        embedding = PartChoice("bigram_embedding", {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur,
                                                    "weight_name": "embed", "bigram_name": "bigram"})
        embedding_prefix = ""
    else:
        embedding = PartChoice("scaled_f32_embedding", {"scale": 1.0, "weight_name": ""})
        embedding_prefix = "embed"
    tables = {}
    if cfg.side_dim:
        tables["side.embed"] = PartChoice("token_embedding", {
            "vocab_size": cfg.vocab_size, "hidden_size": len(cfg.layers) * cfg.side_dim, "weight_name": ""})
    return ModelSpec(
        vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, blocks=blocks, final_norm=norm, tables=tables,
        tie_word_embeddings=False, embedding=embedding, head=PartChoice("lm_head", {"weight_name": ""}),
        max_positions=0, embedding_prefix=embedding_prefix, layer_prefix="l{}", final_norm_prefix="final.norm",
        head_prefix="head")
