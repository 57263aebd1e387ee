"""Tiny Lotorax configurations for the tests, as raw config.json dictionaries, and model folders with weights
drawn so that every mechanism shows in the logits: sinks, router corrections, decays, convolution taps and norm
biases of a size that moves the result when they are dropped or misplaced.

The configurations differ from each other in every size: the unrotated, rotated and value sizes of a head are
never equal, q/k heads are fewer than value heads, the router takes one, two or three experts, layers are looped
once, three times or not at all, from the first layer or from a later one, and one layer has no feed-forward.
"""

from __future__ import annotations

import functools
import json
import os
import tempfile
import zlib

import torch


def _latent(heads, dim, rot_dim, vdim, rank, base=10000.0, scaling=None, scale=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = scaling
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "rot": rot,
            "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}


def _delta(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


YARN = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}

# P: attention, delta, attention with experts; the last two looped three times
LOTO_P = {
    "architecture": "Lotorax", "vocab": 131, "width": 48, "embedding": {"scale": 3.5}, "norm": {"eps": 2e-5},
    "layers": [
        {"type": "latent_attention", "mixer": _latent(3, 8, 4, 12, 24, base=5000.0, scaling=YARN), "mlp": _dense(72)},
        {"type": "delta", "mixer": _delta(4, 2, 8, 12, 3), "mlp": _moe(40, 5, 2)},
        {"type": "latent_attention", "mixer": _latent(2, 16, 8, 20, 40, base=300.0), "mlp": _moe(24, 4, 1)},
    ],
    "loop": {"start": 1, "stop": 3, "times": 3},
}

# Q: no loop; a layer without feed-forward; three experts a token; a delta layer first
LOTO_Q = {
    "architecture": "Lotorax", "vocab": 97, "width": 40, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "delta", "mixer": _delta(2, 1, 12, 20, 2), "mlp": None},
        {"type": "latent_attention", "mixer": _latent(5, 4, 6, 8, 16, base=100000.0, scaling=YARN, scale=0.4),
         "mlp": _moe(16, 6, 3)},
        {"type": "delta", "mixer": _delta(3, 3, 16, 8, 5), "mlp": _dense(56)},
    ],
}

# R: everything looped from the first layer, once; sizes the matrix-core kernels like (multiples of 16 and 32)
LOTO_R = {
    "architecture": "Lotorax", "vocab": 160, "width": 64, "embedding": {"scale": 8.0}, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "latent_attention", "mixer": _latent(4, 32, 16, 48, 64, base=10000.0, scaling=YARN), "mlp": _moe(32, 8, 2)},
        {"type": "delta", "mixer": _delta(4, 2, 16, 80, 3), "mlp": _dense(104)},
    ],
    "loop": {"start": 0, "stop": 2, "times": 1},
}

CONFIGS = {"P": LOTO_P, "Q": LOTO_Q, "R": LOTO_R}
SEEDS = {"P": 3, "Q": 11, "R": 29}


def _draw(name: str, shape, seed: int) -> torch.Tensor:
    g = torch.Generator().manual_seed((seed * 1000003 + zlib.crc32(name.encode())) % (2 ** 63))
    last = name.rsplit(".", 1)[-1]
    z = torch.randn(shape, generator=g)
    if name.endswith(".conv"):
        return 0.5 * z
    if last in ("sink", "dt_bias"):
        return 0.5 + z
    if last == "correction":
        return 0.4 * z
    if last == "A_log":
        return 0.7 * z
    if last == "b":
        return 0.2 * z if len(shape) == 1 else z / shape[-1] ** 0.5
    if len(shape) == 1:                       # norm weights
        return 1.0 + 0.2 * z
    if last in ("embed",):
        return z
    return z / shape[-1] ** 0.5               # matrices: outputs of unit size


@functools.lru_cache(maxsize=None)
def folder(which: str, stored: str = "bfloat16") -> str:
    """A model folder (config.json + model.safetensors) of configuration ``which``."""
    from safetensors.torch import save_file

    from atom_amd.config import build_model, model_config_from_dict
    from atom_amd.weights.loader import expected_tensors

    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[stored]
    path = os.path.join(_TMP.name, f"loto_{which}_{stored}")
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(CONFIGS[which], f)
    model = build_model(model_config_from_dict(CONFIGS[which]))
    tensors = {name: _draw(name, shape, SEEDS[which]).to(dtype).contiguous()
               for name, (shape, _) in expected_tensors(model).items()}
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
    import plain_lotorax as pl

    return _oracle(which, tokens, stored)[0]


def _oracle(which, tokens, stored):
    import plain_lotorax as pl

    key = (which, stored, tuple(tokens))
    if key not in _ORACLE:
        margins = []
        logits = pl.forward(CONFIGS[which], tensors(which, stored), tokens, margins=margins)[0]
        _ORACLE[key] = (logits, torch.stack(margins).min(dim=0).values if margins else None)
    return _ORACLE[key]


def router_margin(which: str, tokens: list[int], stored: str = "bfloat16"):
    """Per token, the least distance over the model's routers between the last expert taken and the first left
    out (None for a model without routers): where it is small, rounding may choose differently."""
    return _oracle(which, tokens, stored)[1]


def core(which: str, dtype: str, ops, device: str, num_pages: int = 64, max_num_seqs: int = 4, page_size: int = 16,
         graph_sizes=None, stored: str = "bfloat16"):
    from atom_amd.engine.core import TORCH_DTYPES, build_core, load_model

    model, _ = load_model(folder(which, stored), dtype=TORCH_DTYPES[dtype], device=device)
    return build_core(model, ops, dtype=TORCH_DTYPES[dtype], device=device, page_size=page_size, num_pages=num_pages,
                      max_num_seqs=max_num_seqs, max_model_len=num_pages * page_size, graph_sizes=graph_sizes)


_TMP = tempfile.TemporaryDirectory(prefix="atom_amd_lotorax_")
