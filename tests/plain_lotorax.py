"""A plain, slow implementation of the Lotorax design, one function per mechanism, in float64.
It shares no code with the engine: the GPU and CPU tests compare the engine with it.

Notation: T tokens, W the model's width, H heads.  Linear weights are [out, in].
"""

from __future__ import annotations

import math

import torch

F = torch.float64


# ----------------------------------------------------------------------------- small pieces


def layer_norm(x, w, b, eps):
    mean = x.mean(dim=-1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * w + b


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


# ----------------------------------------------------------------------------- rotation


def yarn_frequencies(dims: int, base: float, scaling: dict | None):
    """(frequency of each pair, multiplier of cos and sin)."""
    i = torch.arange(dims // 2, dtype=F)
    f = base ** (-2 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def where(turns):
        return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(where(float(scaling["fast"]))), 0)
    hi = min(math.ceil(where(float(scaling["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1


def rotate_pairs(x, positions, dims: int, base: float, scaling: dict | None):
    """x [T, ..., n]: the first ``dims`` entries of the last axis rotated pair by pair, (2i, 2i+1)."""
    f, mult = yarn_frequencies(dims, base, scaling)
    a = positions.to(F)[:, None] * f[None, :]                       # [T, dims/2]
    cos, sin = torch.cos(a) * mult, torch.sin(a) * mult
    while cos.dim() < x.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


# ----------------------------------------------------------------------------- mixers


def latent_attention(h, positions, w, m, eps, history=None):
    """h [T, W] at ``positions``; w: the mixer's tensors by short name; m: its sizes.  ``history`` may hold
    (latents, rotated keys) of earlier tokens; returns (output [T, W], (latents, rotated keys) of all tokens)."""
    T = h.shape[0]
    H, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m["rot"]
    q = (h @ w["q"].T).view(T, H, d + r)
    q_plain, q_rot = q[..., :d], q[..., d:]
    down = h @ w["dkv"].T
    c = rms_unit(down[:, :rank], eps) * w["dkv.norm"]
    k_rot = down[:, rank:]
    q_rot = rotate_pairs(q_rot, positions, rot["dims"], rot["base"], rot.get("scaling"))
    k_rot = rotate_pairs(k_rot, positions, rot["dims"], rot["base"], rot.get("scaling"))
    key_pos = positions
    if history is not None:
        c = torch.cat((history[0], c))
        k_rot = torch.cat((history[1], k_rot))
        key_pos = torch.cat((torch.arange(c.shape[0] - T), positions))
    n = c.shape[0]
    k_plain = (c @ w["uk"].T).view(n, H, d)
    v = (c @ w["uv"].T).view(n, H, dv)
    s = (torch.einsum("thd,nhd->htn", q_plain, k_plain) + torch.einsum("thr,nr->htn", q_rot, k_rot)) * m["scale"]
    seen = key_pos[None, :] <= positions[:, None]
    s = s.masked_fill(~seen[None], -math.inf)
    top = torch.maximum(s.max(dim=-1, keepdim=True).values, w["sink"].view(H, 1, 1))
    e = torch.exp(s - top)
    p = e / (e.sum(dim=-1, keepdim=True) + torch.exp(w["sink"].view(H, 1, 1) - top))
    o = torch.einsum("htn,nhv->thv", p, v)
    o = o * torch.sigmoid(h @ w["g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ w["o"].T, (c, k_rot)


def short_convolution(x, taps_w, before=None):
    """x [T, C], taps_w [C, taps] (last column: the current token); ``before`` [taps-1, C] are the inputs that
    preceded x (zeros at a sequence's start).  Returns (y [T, C], the last taps-1 inputs)."""
    taps = taps_w.shape[1]
    if before is None:
        before = torch.zeros((taps - 1, x.shape[1]), dtype=x.dtype)
    full = torch.cat((before, x))
    y = torch.zeros_like(x)
    for j in range(taps):
        y = y + full[j:j + x.shape[0]] * taps_w[:, j]
    return y, full[full.shape[0] - (taps - 1):]


def delta_rule(q, k, v, beta, g, state):
    """One head: q, k [T, d], v [T, dv], beta, g [T], state [d, dv].  Returns (o [T, dv], state)."""
    S = state.clone()
    out = []
    for t in range(q.shape[0]):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out.append(S.T @ q[t])
    return torch.stack(out), S


def delta_mixer(h, w, m, eps, carried=None):
    """h [T, W]; ``carried`` = (conv inputs of q, k, v, state [H, d, dv]) of the tokens before, or None."""
    T = h.shape[0]
    H, Hk, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    before = carried[:3] if carried is not None else (None, None, None)
    q, tail_q = short_convolution(h @ w["q"].T, w["q.conv"], before[0])
    k, tail_k = short_convolution(h @ w["k"].T, w["k.conv"], before[1])
    v, tail_v = short_convolution(h @ w["v"].T, w["v.conv"], before[2])
    q, k, v = silu(q).view(T, Hk, d), silu(k).view(T, Hk, d), silu(v).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(dim=-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(dim=-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w["b"].T)
    g = torch.exp(-torch.exp(w["A_log"]) * softplus(h @ w["a"].T + w["dt_bias"]))
    state = carried[3] if carried is not None else torch.zeros((H, d, dv), dtype=h.dtype)
    outs, states = [], []
    for head in range(H):
        kv = head // (H // Hk)
        o, S = delta_rule(q[:, kv], k[:, kv], v[:, head], beta[:, head], g[:, head], state[head])
        outs.append(o)
        states.append(S)
    o = torch.stack(outs, dim=1)                                      # [T, H, dv]
    o = rms_unit(o, eps) * w["norm"] * silu(h @ w["g"].T).view(T, H, dv)
    return o.reshape(T, H * dv) @ w["o"].T, (tail_q, tail_k, tail_v, torch.stack(states))


# ----------------------------------------------------------------------------- feed-forwards


def dense_ff(h, w):
    return (torch.relu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def routed_choice(h, w, top: int):
    """(chosen experts [T, top], their weights [T, top])."""
    s = torch.sigmoid(h @ w["router"].T)
    chosen = torch.topk(s + w["correction"], top, dim=-1).indices
    return chosen, torch.gather(s, 1, chosen)


def routed_margin(h, w, top: int):
    """Per token, how far the last chosen expert's choice score lies above the best one left out."""
    pick = torch.sigmoid(h @ w["router"].T) + w["correction"]
    if top >= pick.shape[-1]:
        return torch.full((h.shape[0],), math.inf, dtype=h.dtype)
    best = torch.topk(pick, top + 1, dim=-1).values
    return best[:, top - 1] - best[:, top]


def routed_ff(h, w, experts: int, top: int):
    chosen, weights = routed_choice(h, w, top)
    out = torch.zeros((h.shape[0], w["e0.down"].shape[0]), dtype=h.dtype)
    for e in range(experts):
        y = (silu(h @ w[f"e{e}.gate"].T) * (h @ w[f"e{e}.up"].T)) @ w[f"e{e}.down"].T
        share = (weights * (chosen == e)).sum(dim=-1, keepdim=True)
        out = out + share * y
    return out


# ----------------------------------------------------------------------------- the model


def running_order(cfg) -> list[tuple[int, bool]]:
    """(layer, whether a pass of the loop starts before it) for every run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    runs = [(i, False) for i in range(loop["start"])]
    for _ in range(loop["times"]):
        runs += [(i, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, False) for i in range(loop["stop"], n)]


def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg, tensors, ids, positions=None, carried=None, trail=None, margins=None):
    """Logits [T, vocab] of the tokens ``ids`` (one sequence).  ``carried``: what an earlier call returned
    (then ``positions`` continue); ``trail``: a list that receives the residual stream after every run;
    ``margins``: a list that receives every routed run's ``routed_margin``."""
    tensors = {k: (v.to(F) if v.is_floating_point() else v) for k, v in tensors.items()}
    T = len(ids)
    eps = cfg["norm"]["eps"]
    start = 0 if carried is None else carried["seen"]
    positions = torch.arange(start, start + T)
    x0 = tensors["embed"][torch.tensor(ids)] * cfg["embedding"]["scale"]
    x = x0
    runs = running_order(cfg)
    memory = [None] * len(runs) if carried is None else carried["runs"]
    kept = []
    for r, (i, enters) in enumerate(runs):
        layer = cfg["layers"][i]
        p = f"l{i}."
        if enters:
            x = torch.cat((x, x0), dim=-1) @ tensors["loop.in"].T
        h = layer_norm(x, tensors[p + "norm1"], tensors[p + "norm1.b"], eps)
        w = sub(tensors, p + "mix.")
        if layer["type"] == "latent_attention":
            y, keep = latent_attention(h, positions, w, layer["mixer"], eps, memory[r])
        elif layer["type"] == "delta":
            y, keep = delta_mixer(h, w, layer["mixer"], eps, memory[r])
        else:
            raise ValueError(layer["type"])
        kept.append(keep)
        x = x + layer_norm(y, tensors[p + "norm1b"], tensors[p + "norm1b.b"], eps)
        if layer.get("mlp"):
            h = layer_norm(x, tensors[p + "norm2"], tensors[p + "norm2.b"], eps)
            w = sub(tensors, p + "mlp.")
            if layer["mlp"]["kind"] == "dense":
                y = dense_ff(h, w)
            else:
                y = routed_ff(h, w, layer["mlp"]["router"]["experts"], layer["mlp"]["router"]["top"])
                if margins is not None:
                    margins.append(routed_margin(h, w, layer["mlp"]["router"]["top"]))
            x = x + layer_norm(y, tensors[p + "norm2b"], tensors[p + "norm2b.b"], eps)
        if trail is not None:
            trail.append(x)
    h = layer_norm(x, tensors["final.norm"], tensors["final.norm.b"], eps)
    return h @ tensors["head"].T, {"seen": start + T, "runs": kept}
