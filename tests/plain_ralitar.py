"""A plain, slow implementation of the Ralitar design in float64, one function per mechanism, written from the
design's equations and sharing no code with the engine.  Recurrent mixers walk the tokens one by one; attention
builds the whole score matrix.  ``forward`` takes a request's tokens (or a further portion of them together with
what the earlier portions ``carried``) and returns the logits at every position.
"""

from __future__ import annotations

import math

import torch

WIDE = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def short_convolution(x, taps_w, before=None, bias=None):
    """x [T, C]; taps_w [C, taps], the last column weighs the current token; ``before`` [taps - 1, C]: the inputs
    ahead of x (zeros at a request's start).  Returns (y [T, C], the last taps - 1 inputs)."""
    taps = taps_w.shape[1]
    if before is None:
        before = torch.zeros(taps - 1, x.shape[1], dtype=x.dtype)
    padded = torch.cat((before, x), dim=0)
    y = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for j in range(taps):
            y[t] += padded[t + j] * taps_w[:, j]
    if bias is not None:
        y = y + bias
    return y, padded[padded.shape[0] - (taps - 1):]


# ------------------------------------------------------------------ the real-gated linear recurrence


def rglru_mixer(h, w, m, carried=None, decay_scale=8.0):
    """w: the mixer's tensors by their names under '<layer>.mix.'; carried: (conv inputs, S)."""
    blocks = m["blocks"]
    y = gelu_tanh(h @ w["y"].T + w["y.b"])
    before, S = carried if carried is not None else (None, torch.zeros(m["width"], dtype=WIDE))
    u, tail = short_convolution(h @ w["x"].T + w["x.b"], w["conv"], before, w["conv.b"])
    part = m["width"] // blocks
    out = torch.zeros_like(u)
    sp = softplus(w["lam"])
    for t in range(h.shape[0]):
        r = torch.empty(m["width"], dtype=WIDE)
        i = torch.empty(m["width"], dtype=WIDE)
        for b in range(blocks):
            cols = slice(b * part, (b + 1) * part)
            r[cols] = torch.sigmoid(w["ra"][b] @ u[t, cols] + w["ra.b"][b])
            i[cols] = torch.sigmoid(w["ri"][b] @ u[t, cols] + w["ri.b"][b])
        a = torch.exp(-decay_scale * r * sp)
        S = a * S + torch.sqrt(1 - a * a) * (i * u[t])
        out[t] = S
    return (out * y) @ w["o"].T, (tail, S)


# ------------------------------------------------------------------ the gated delta rule with channel decay


def delta_step(S, q, k, v, beta, g):
    """One token of one head.  S [dim, vdim]; g [dim] weighs the rows of S.  Returns (o [vdim], S)."""
    S = g[:, None] * S
    u = beta * (v - S.T @ k)
    S = S + torch.outer(k, u)
    return S.T @ q, S


def channel_delta_mixer(h, w, m, eps, carried=None):
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    before = carried[0] if carried is not None else {"q": None, "k": None, "v": None}
    S = carried[1].clone() if carried is not None else torch.zeros(H, D, V, dtype=WIDE)
    conv, tails = {}, {}
    for name in ("q", "k", "v"):
        y, tails[name] = short_convolution(h @ w[name].T, w[f"{name}.conv"], before[name])
        conv[name] = silu(y)
    q = conv["q"].view(T, G, D)
    k = conv["k"].view(T, G, D)
    v = conv["v"].view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w["b"].T)
    step = softplus((h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]).view(T, H, D)
    g = torch.exp(-torch.exp(w["A_log"]).view(1, H, 1) * step)
    gate = torch.sigmoid((h @ w["g1"].T) @ w["g2"].T).view(T, H, V)
    o = torch.zeros(T, H, V, dtype=WIDE)
    for t in range(T):
        for head in range(H):
            kv = head // (H // G)
            o[t, head], S[head] = delta_step(S[head], q[t, kv], k[t, kv], v[t, head], beta[t, head], g[t, head])
    o = rms(o, eps) * w["norm"] * gate
    return o.reshape(T, H * V) @ w["o"].T, (tails, S)


# ------------------------------------------------------------------ chunked attention whose values are its keys


def banded_frequencies(dims: int, base: float, scaling: dict | None):
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=WIDE)
    if not scaling:
        return f
    out = f.clone()
    for i in range(dims // 2):
        length = 2 * math.pi / float(f[i])
        if length < scaling["original"] / scaling["high"]:
            continue
        if length > scaling["original"] / scaling["low"]:
            out[i] = f[i] / scaling["factor"]
        else:
            s = (scaling["original"] / length - scaling["low"]) / (scaling["high"] - scaling["low"])
            out[i] = (1 - s) * f[i] / scaling["factor"] + s * f[i]
    return out


def rotate_pairs(x, positions, freq):
    """x [T, heads, dim]: entries (2i, 2i + 1) of each head turn by positions * freq[i]; the rest stay."""
    out = x.clone()
    for i in range(freq.numel()):
        a = positions.to(WIDE) * freq[i]
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def visible(i: int, j: int, chunk: int | None) -> bool:
    return j <= i and (chunk is None or i // chunk == j // chunk)


def chunk_attention_mixer(h, positions, w, m, eps, carried=None):
    """carried: (keys [n, G, D] normed and rotated, values [n, G, D], their positions)."""
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    T = h.shape[0]
    q = h @ w["q"].T + w["q.b"]
    k = h @ w["k"].T + w["k.b"]
    v = k.view(T, G, D)
    q = (rms(q, eps) * w["q.norm"]).view(T, H, D)
    k = (rms(k, eps) * w["k.norm"]).view(T, G, D)
    rot = m.get("rot")
    if rot and rot["dims"]:
        freq = banded_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate_pairs(q, positions, freq), rotate_pairs(k, positions, freq)
    if carried is not None:
        k, v = torch.cat((carried[0], k)), torch.cat((carried[1], v))
        key_pos = torch.cat((carried[2], positions))
    else:
        key_pos = positions
    chunk = (m.get("mask") or {}).get("size")
    cap = m.get("softcap")
    out = torch.zeros(T, H, D, dtype=WIDE)
    for t in range(T):
        seen = [j for j in range(key_pos.numel()) if visible(int(positions[t]), int(key_pos[j]), chunk)]
        for head in range(H):
            kv = head // (H // G)
            s = (k[seen, kv] @ q[t, head]) * m["scale"]
            if cap:
                s = cap * torch.tanh(s / cap)
            out[t, head] = torch.softmax(s, dim=0) @ v[seen, kv]
    out = out.reshape(T, H * D) * torch.sigmoid(h @ w["g"].T)
    return out @ w["o"].T, (k, v, key_pos)


# ------------------------------------------------------------------ around the mixers


def dense_ff(h, w):
    return (gelu_tanh(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def token_side(x, e, w, eps):
    y = (gelu_tanh(x @ w["gate"].T) * e) @ w["proj"].T
    return rms(y, eps) * w["norm"]


def bigram_rows(ids, previous, bigram):
    """Row of the pair table for each token; ``previous``: the token before ids[0], None at a request's start."""
    buckets, mul_prev, mul_cur = bigram["buckets"], bigram["mul_prev"], bigram["mul_cur"]
    rows, prev = [], previous
    for t in ids:
        rows.append(buckets if prev is None else (prev * mul_prev + t * mul_cur) % buckets)
        prev = t
    return rows


def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg, tensors, ids, carried=None, trail=None):
    """Logits [len(ids), vocab] in float64 and what a continuation needs.  ``trail``: a list that receives the
    stream after every layer."""
    tensors = {k: v.to(WIDE) for k, v in tensors.items()}
    eps = cfg["norm"]["eps"]
    start = carried["n"] if carried is not None else 0
    positions = torch.arange(start, start + len(ids))
    tok = torch.tensor(ids, dtype=torch.long)
    x = tensors["embed"][tok]
    bigram = (cfg.get("embedding") or {}).get("bigram")
    if bigram:
        x = x + tensors["bigram"][torch.tensor(bigram_rows(ids, carried["last"] if carried else None, bigram))]
    side = (cfg.get("token_side") or {}).get("dim", 0)
    new = {"n": start + len(ids), "last": ids[-1], "layers": []}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        w = sub(tensors, p + "mix.")
        before = carried["layers"][i] if carried is not None else None
        if layer["type"] == "rglru":
            mixed, keep = rglru_mixer(x, w, layer["mixer"], before)
        elif layer["type"] == "channel_delta":
            mixed, keep = channel_delta_mixer(x, w, layer["mixer"], eps, before)
        else:
            mixed, keep = chunk_attention_mixer(x, positions, w, layer["mixer"], eps, before)
        new["layers"].append(keep)
        x = x + rms(mixed, eps) * tensors[p + "norm1"]
        if layer.get("mlp") is not None:
            x = x + rms(dense_ff(x, sub(tensors, p + "mlp.")), eps) * tensors[p + "norm2"]
        if side:
            e = tensors["side.embed"][tok][:, i * side:(i + 1) * side]
            x = x + token_side(x, e, sub(tensors, p + "side."), eps)
        if trail is not None:
            trail.append(x.clone())
    logits = (rms(x, eps) * tensors["final.norm"]) @ tensors["head"].T
    return logits, new
