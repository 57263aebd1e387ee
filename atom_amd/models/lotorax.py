"""Lotorax as a ``ModelSpec``.

The embedding's rows are multiplied by a constant and start a float32 residual stream.  Every layer is a block
with layer norms before and after each sublayer: ``x += norm1b(mixer(norm1(x)))``, then
``x += norm2b(ff(norm2(x)))`` where the layer has a feed-forward.  The mixer is attention over cached latents
(rotated part stretched for long contexts, a sink in the softmax, a gate per head) or the gated delta rule; the
feed-forward is ReLU-gated and dense, or SiLU-gated routed experts with sigmoid scores.  Layers ``start .. stop - 1``
of ``loop`` run ``times`` times in a row with the same weights, each pass with memory of its own, and every pass
begins with ``x <- W_in [x ; x0]``, x0 being the embedding's output.  A final layer norm and an untied head.

Checkpoint names: ``embed``, ``loop.in``, ``l<i>.norm1`` (weight) and ``l<i>.norm1.b`` (bias) and so on,
``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``; matrices carry no ``.weight`` suffix.
"""

from __future__ import annotations

from ..config.model_config import LotoraxConfig
from ..parts.base import PartChoice
from .model import LayerRun, ModelSpec


def _mixer(cfg: LotoraxConfig, layer: dict) -> PartChoice:
    m = layer["mixer"]
    if layer["type"] == "latent_attention":
        rot = m["rot"]
        scaling = rot.get("scaling") or {}
        rope = PartChoice("scaled_rotary", {"dims": rot["dims"], "base": rot["base"], "factor": scaling.get("factor"),
                                            "original": scaling.get("original"), "fast": scaling.get("fast"),
                                            "slow": scaling.get("slow")})
        return PartChoice("latent_attention", {
            "hidden_size": cfg.hidden_size, "num_heads": m["heads"], "head_dim": m["dim"], "rot_dim": m["rot_dim"],
            "value_dim": m["vdim"], "kv_rank": m["kv_rank"], "scale": m["scale"], "norm_eps": cfg.norm_eps,
            "position_encoding": rope, "sink": True, "gate": True})
    return PartChoice("gated_delta", {
        "hidden_size": cfg.hidden_size, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
        "value_dim": m["vdim"], "conv_taps": m["conv"], "norm_eps": cfg.norm_eps})


def _feed_forward(cfg: LotoraxConfig, layer: dict) -> PartChoice | None:
    mlp = layer.get("mlp")
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return PartChoice("gated_mlp", {"hidden_size": cfg.hidden_size, "intermediate_size": mlp["ff"],
                                        "activation": "relu", "weight_suffix": "",
                                        "names": {"gate": "gate", "up": "up", "down": "down"}})
    return PartChoice("routed_experts", {"hidden_size": cfg.hidden_size, "expert_size": mlp["expert"]["ff"],
                                         "num_experts": mlp["router"]["experts"], "top": mlp["router"]["top"],
                                         "activation": "silu", "correction": True, "renormalize": False})


def lotorax_order(num_layers: int, loop: tuple | None) -> list[LayerRun]:
    if loop is None:
        return [LayerRun(i) for i in range(num_layers)]
    start, stop, times = loop
    runs = [LayerRun(i) for i in range(start)]
    for _ in range(times):
        runs += [LayerRun(i, enters=(i == start)) for i in range(start, stop)]
    return runs + [LayerRun(i) for i in range(stop, num_layers)]


def lotorax_spec(cfg: LotoraxConfig) -> ModelSpec:
    norm = PartChoice("layernorm", {"size": cfg.hidden_size, "eps": cfg.norm_eps, "weight_name": "", "bias_name": "b"})
    blocks = [PartChoice("sandwich", {"mixer": _mixer(cfg, layer), "feed_forward": _feed_forward(cfg, layer),
                                      "norm": norm}) for layer in cfg.layers]
    return ModelSpec(
        vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, blocks=blocks, final_norm=norm,
        tie_word_embeddings=False,
        embedding=PartChoice("scaled_f32_embedding", {"scale": cfg.embedding_scale, "weight_name": ""}),
        head=PartChoice("lm_head", {"weight_name": ""}),
        order=lotorax_order(len(cfg.layers), cfg.loop),
        join=PartChoice("concat_projection", {"weight_name": ""}) if cfg.loop is not None else None,
        join_prefix="loop.in", max_positions=0,
        embedding_prefix="embed", layer_prefix="l{}", final_norm_prefix="final.norm", head_prefix="head")
