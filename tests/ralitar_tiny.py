"""Tiny Ralitar configurations for the tests, as raw config.json dictionaries, and model folders with weights drawn
so that every mechanism shows in the logits: pair-table rows, token-side columns, decays per channel, convolution
taps, gate biases and norm weights of a size that moves the result when they are dropped or misplaced.

The configurations differ from each other in every size.  Query heads outnumber key heads (or not), key and value
sizes of the delta rule differ, the inner sizes of its two low-rank projections differ from each other and from the
token-side size, chunks are smaller than, equal to and larger than a cache page and never a multiple of 64, the
recurrence has one, three or four parts, the layers come in different orders, one layer has no feed-forward, and one
model has neither the pair table nor the token side.
"""

from __future__ import annotations

import functools
import json
import os
import tempfile
import zlib

import torch

# inner sizes of the delta rule's low-rank projections: a tensor's shape says them, the configuration does not
RANKS = {"U": {"a1": 6, "g1": 10}, "V": {"a1": 9, "g1": 4}, "W": {"a1": 16, "g1": 24}, "X": {"a1": 40, "g1": 24}}


def _rglru(width, blocks, conv):
    return {"width": width, "blocks": blocks, "conv": conv}


def _delta(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def _attn(heads, kv_heads, dim, chunk, scale, softcap=None, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if chunk:
        m["mask"] = {"size": chunk}
    if softcap:
        m["softcap"] = softcap
    if rot:
        m["rot"] = rot
    return m


def _dense(ff):
    return {"kind": "dense", "ff": ff}


BANDS = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}

# U: delta, attention (chunks of 7, smaller than a page), recurrence; pair table and token side
RALI_U = {
    "architecture": "Ralitar", "vocab": 97, "width": 40, "norm": {"eps": 2e-5},
    "embedding": {"bigram": {"buckets": 53, "mul_prev": 31, "mul_cur": 5}}, "token_side": {"dim": 5},
    "layers": [
        {"type": "channel_delta", "mixer": _delta(4, 2, 8, 12, 3), "mlp": _dense(56)},
        {"type": "attention", "mixer": _attn(6, 2, 10, 7, 0.6, softcap=3.0, rot={"base": 300.0, "dims": 6, "scaling": BANDS}),
         "mlp": None},
        {"type": "rglru", "mixer": _rglru(24, 3, 2), "mlp": _dense(48)},
    ],
}

# V: recurrence first (one part), attention with as many key heads as query heads, chunks of a page, no cap, plain
# frequencies over the whole head; a delta layer whose q/k heads are its value heads; five taps
RALI_V = {
    "architecture": "Ralitar", "vocab": 131, "width": 48, "norm": {"eps": 1e-6},
    "embedding": {"bigram": {"buckets": 17, "mul_prev": 3, "mul_cur": 101}}, "token_side": {"dim": 3},
    "layers": [
        {"type": "rglru", "mixer": _rglru(20, 1, 5), "mlp": None},
        {"type": "attention", "mixer": _attn(3, 3, 8, 16, 0.35, rot={"base": 10000.0, "dims": 8}), "mlp": _dense(40)},
        {"type": "channel_delta", "mixer": _delta(3, 3, 12, 4, 5), "mlp": _dense(32)},
        {"type": "attention", "mixer": _attn(4, 1, 6, 40, 0.5, softcap=8.0), "mlp": _dense(24)},
    ],
}

# W: sizes the matrix-core kernels take (heads of 64 and 128, multiples of 16), chunks of 48 and 160, neither the
# pair table nor the token side
RALI_W = {
    "architecture": "Ralitar", "vocab": 160, "width": 64, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "attention", "mixer": _attn(4, 2, 64, 48, 0.11, softcap=20.0, rot={"base": 50000.0, "dims": 32, "scaling": BANDS}),
         "mlp": _dense(96)},
        {"type": "rglru", "mixer": _rglru(64, 4, 4), "mlp": _dense(64)},
        {"type": "channel_delta", "mixer": _delta(4, 2, 16, 32, 4), "mlp": None},
        {"type": "attention", "mixer": _attn(2, 1, 128, 160, 0.08, rot={"base": 1000.0, "dims": 64}), "mlp": _dense(80)},
    ],
}

# X: wide enough that prompts of 5, 40, 130 and 300 tokens reach every kernel the engine has for matrix products
# (few rows, up to 64, up to 256, the library's), with widths that are not powers of two
RALI_X = {
    "architecture": "Ralitar", "vocab": 1000, "width": 384, "norm": {"eps": 1e-6},
    "embedding": {"bigram": {"buckets": 509, "mul_prev": 65537, "mul_cur": 257}}, "token_side": {"dim": 24},
    "layers": [
        {"type": "attention", "mixer": _attn(6, 3, 64, 96, 0.125, softcap=30.0, rot={"base": 10000.0, "dims": 16, "scaling": BANDS}),
         "mlp": _dense(1056)},
        {"type": "channel_delta", "mixer": _delta(6, 3, 64, 32, 4), "mlp": _dense(1056)},
        {"type": "rglru", "mixer": _rglru(448, 7, 4), "mlp": _dense(1056)},
    ],
}

CONFIGS = {"U": RALI_U, "V": RALI_V, "W": RALI_W, "X": RALI_X}
SEEDS = {"U": 5, "V": 13, "W": 31, "X": 43}


def _draw(name: str, shape, seed: int) -> torch.Tensor:
    g = torch.Generator().manual_seed((seed * 1000003 + zlib.crc32(name.encode())) % (2 ** 63))
    last = name.rsplit(".", 1)[-1]
    z = torch.randn(shape, generator=g)
    if name.endswith(".conv"):
        return 0.5 * z
    if last == "dt_bias":
        return 0.5 + z
    if last == "A_log":
        return 0.7 * z
    if last == "lam":
        return z - 1.0
    if last == "b":
        return 0.3 * z if len(shape) <= 2 and ".mix.r" in name or len(shape) == 1 else z / shape[-1] ** 0.5
    if len(shape) == 1:                       # norm weights
        return 1.0 + 0.2 * z
    if last in ("embed", "bigram"):
        return z
    if ".mix.r" in name:                      # the recurrence's gates: wide enough for the gates to move
        return 2.0 * z / shape[-1] ** 0.5
    return z / shape[-1] ** 0.5               # matrices: outputs of unit size


def shapes(which: str) -> dict:
    """Every tensor a checkpoint of configuration ``which`` holds, by name, written out here from the design
    (not taken from the engine's own list): the tests compare the two."""
    cfg = CONFIGS[which]
    w, v = cfg["width"], cfg["vocab"]
    out = {"embed": (v, w), "final.norm": (w,), "head": (v, w)}
    if "embedding" in cfg:
        out["bigram"] = (cfg["embedding"]["bigram"]["buckets"] + 1, w)
    side = (cfg.get("token_side") or {}).get("dim", 0)
    if side:
        out["side.embed"] = (v, side * len(cfg["layers"]))
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (w,)
        if layer["type"] == "rglru":
            c, b = m["width"], m["blocks"]
            out.update({p + "mix.y": (c, w), p + "mix.y.b": (c,), p + "mix.x": (c, w), p + "mix.x.b": (c,),
                        p + "mix.conv": (c, m["conv"]), p + "mix.conv.b": (c,), p + "mix.ra": (b, c // b, c // b),
                        p + "mix.ra.b": (b, c // b), p + "mix.ri": (b, c // b, c // b), p + "mix.ri.b": (b, c // b),
                        p + "mix.lam": (c,), p + "mix.o": (w, c)})
        elif layer["type"] == "channel_delta":
            H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            ra, rg = RANKS[which]["a1"], RANKS[which]["g1"]
            out.update({p + "mix.q": (G * D, w), p + "mix.k": (G * D, w), p + "mix.v": (H * V, w),
                        p + "mix.q.conv": (G * D, m["conv"]), p + "mix.k.conv": (G * D, m["conv"]),
                        p + "mix.v.conv": (H * V, m["conv"]), p + "mix.b": (H, w), p + "mix.A_log": (H,),
                        p + "mix.norm": (V,), p + "mix.a1": (ra, w), p + "mix.a2": (H * D, ra),
                        p + "mix.dt_bias": (H * D,), p + "mix.g1": (rg, w), p + "mix.g2": (H * V, rg),
                        p + "mix.o": (w, H * V)})
        else:
            H, G, D = m["heads"], m["kv_heads"], m["dim"]
            out.update({p + "mix.q": (H * D, w), p + "mix.q.b": (H * D,), p + "mix.k": (G * D, w), p + "mix.k.b": (G * D,),
                        p + "mix.q.norm": (H * D,), p + "mix.k.norm": (G * D,), p + "mix.g": (H * D, w),
                        p + "mix.o": (w, H * D)})
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            out.update({p + "norm2": (w,), p + "mlp.gate": (ff, w), p + "mlp.up": (ff, w), p + "mlp.down": (w, ff)})
        if side:
            out.update({p + "side.gate": (side, w), p + "side.proj": (w, side), p + "side.norm": (w,)})
    return out


@functools.lru_cache(maxsize=None)
def folder(which: str, stored: str = "bfloat16") -> str:
    """A model folder (config.json + model.safetensors) of configuration ``which``."""
    from safetensors.torch import save_file

    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[stored]
    path = os.path.join(_TMP.name, f"rali_{which}_{stored}")
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(CONFIGS[which], f)
    tensors = {name: _draw(name, shape, SEEDS[which]).to(dtype).contiguous() for name, shape in shapes(which).items()}
    save_file(tensors, os.path.join(path, "model.safetensors"))
    return path


@functools.lru_cache(maxsize=None)
def tensors(which: str, stored: str = "bfloat16") -> dict:
    from safetensors.torch import load_file

    return load_file(os.path.join(folder(which, stored), "model.safetensors"))


def ids(which: str, n: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, CONFIGS[which]["vocab"], (n,), generator=g).tolist()


_ORACLE: dict = {}


def oracle(which: str, tokens: list[int], stored: str = "bfloat16") -> torch.Tensor:
    import plain_ralitar as pr

    key = (which, stored, tuple(tokens))
    if key not in _ORACLE:
        _ORACLE[key] = pr.forward(CONFIGS[which], tensors(which, stored), tokens)[0]
    return _ORACLE[key]


def float32_error(which: str, tokens: list[int], stored: str = "bfloat16") -> torch.Tensor:
    """Per position, how far the plain implementation run in float32 is from itself in float64 (largest difference
    of a logit): what rounding alone does at that token with these weights.  A sublayer's output is normed on its
    way into the stream, so a token whose output is small carries its rounding along enlarged."""
    import plain_ralitar as pr

    key = (which, stored, tuple(tokens), "float32")
    if key not in _ORACLE:
        wide = pr.WIDE
        pr.WIDE = torch.float32
        try:
            narrow = pr.forward(CONFIGS[which], tensors(which, stored), tokens)[0]
        finally:
            pr.WIDE = wide
        _ORACLE[key] = (narrow.double() - oracle(which, tokens, stored)).abs().amax(dim=1)
    return _ORACLE[key]


def core(which: str, dtype: str, ops, device: str, num_pages: int = 64, max_num_seqs: int = 4, page_size: int = 16,
         graph_sizes=None, stored: str = "bfloat16"):
    from atom_amd.engine.core import TORCH_DTYPES, build_core, load_model

    model, _ = load_model(folder(which, stored), dtype=TORCH_DTYPES[dtype], device=device)
    return build_core(model, ops, dtype=TORCH_DTYPES[dtype], device=device, page_size=page_size, num_pages=num_pages,
                      max_num_seqs=max_num_seqs, max_model_len=num_pages * page_size, graph_sizes=graph_sizes)


_TMP = tempfile.TemporaryDirectory(prefix="atom_amd_ralitar_")
