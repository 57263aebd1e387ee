"""Ralitar on the GPU: every new kernel alone against the plain implementation's function of the same mechanism
(float32 and bfloat16), attention with keys made to stand out just inside and just outside a chunk, at page borders
and far away, then the engine on tiny models: whole prompts, token-by-token tails, portions down to two tokens,
mixed batches with pages and slots used again, decode steps replayed from graphs, long decoding across chunk edges,
greedy generation through ``LLMEngine``, and ``bin/trace_run``."""

import math

import pytest
import torch

import plain_ralitar as pr
import ralitar_tiny as rt
import replay
from helpers import gpu_ops
from atom_amd.kernels.hip import AttentionMeta

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


def close(got, want, dtype, what=""):
    got, want = got.double().cpu(), want.double().cpu()
    scale = max(1e-6, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= TOL[dtype] * scale, f"{what}: {err:.3e} > {TOL[dtype] * scale:.3e}"


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


# ------------------------------------------------------------------ the float32 stream


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,n", [(40, 7), (333, 5), (4096, 3), (64, 300), (2048, 9), (1500, 4), (6148, 3), (8200, 2)])
def test_normed_summands_join_the_stream(dtype, width, n):
    ops = gpu_ops()
    stream = rnd((n, width), 1, 2.0)
    x = (rnd((n, width), 2, 3.0) + 0.5).to(dtype)
    w = 1 + rnd((width,), 3, 0.2)
    eps = 3e-5
    want = stream.double() + pr.rms(x.double(), eps) * w.double()
    s = stream.to(DEV)
    out = torch.empty((n, width), dtype=dtype, device=DEV)
    ops.rmsnorm_post(x.to(DEV), w.to(DEV), eps, s, out)
    close(s, want, torch.float32, "stream")
    close(out, want, dtype, "copy")
    assert torch.equal(out.float().cpu(), s.cpu().to(dtype).float()), "the copy is the stream, rounded once"
    s2 = stream.to(DEV)
    ops.rmsnorm_post(x.to(DEV), w.to(DEV), eps, s2, None)
    assert torch.equal(s2, s)
    rows = i32([n - 1, 0, n - 1])
    few = torch.empty((3, width), dtype=dtype, device=DEV)
    ops.rmsnorm_rows(s, w.to(DEV), eps, rows, few)
    close(few, (pr.rms(want, eps) * w.double())[[n - 1, 0, n - 1]], dtype, "rows")
    close(ops.cast_rows(s, dtype), want, dtype, "cast")


@pytest.mark.parametrize("dtype", DTYPES)
def test_pair_embedding_and_its_state(dtype):
    """Two steps over three requests (one of them padding): the previous token is the step's own where there is one,
    the state's at a request's first token of the step, none at a request's start."""
    ops = gpu_ops()
    vocab, width, buckets, mp, mc = 50, 24, 11, 7, 13
    table, pairs = rnd((vocab, width), 1).to(dtype), rnd((buckets + 1, width), 2).to(dtype)
    state = torch.zeros((4, 1), dtype=torch.int32, device=DEV)
    bigram = {"buckets": buckets, "mul_prev": mp, "mul_cur": mc}

    def run(ids, lens, slots, previous):
        cu = [0]
        for n in lens:
            cu.append(cu[-1] + n)
        seq = [b for b, n in enumerate(lens) for _ in range(n)]
        out = torch.empty((len(ids), width), dtype=torch.float32, device=DEV)
        ops.embedding_bigram(table.to(DEV), pairs.to(DEV), i32(ids), state, i32(cu), i32(slots), i32(seq), out, buckets,
                             mp, mc)
        for b, n in enumerate(lens):
            part = ids[cu[b]:cu[b + 1]]
            if slots[b] < 0:
                assert float(out[cu[b]:cu[b + 1]].abs().max()) == 0
                continue
            rows = pr.bigram_rows(part, previous[b], bigram)
            want = table.double()[part] + pairs.double()[rows]
            close(out[cu[b]:cu[b + 1]], want, torch.float32, f"request {b}")

    run([3, 49, 49, 7, 20, 5], [3, 1, 2], [2, -1, 0], [None, None, None])
    assert state[:, 0].tolist() == [6, 0, 50, 0]
    run([8, 1, 2, 3, 4], [1, 4], [2, 0], [49, 5])
    assert state[:, 0].tolist() == [5, 0, 9, 0]


@pytest.mark.parametrize("dtype", DTYPES)
def test_token_gate(dtype):
    ops = gpu_ops()
    raw = rnd((9, 5), 1, 2.0)
    table = rnd((30, 20), 2).to(dtype)
    ids = [0, 29, 4, 4, 17, 3, 2, 1, 0]
    out = torch.empty((9, 5), dtype=dtype, device=DEV)
    ops.token_gate(raw.to(DEV), table.to(DEV), 10, i32(ids), out)
    close(out, pr.gelu_tanh(raw.double()) * table.double()[ids, 10:15], dtype)


# ------------------------------------------------------------------ recurrences


def _batch(lens, slots):
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    return i32(cu), i32(slots), cu


@pytest.mark.parametrize("taps,channels", [(2, 24), (4, 300), (5, 20), (12, 7)])
def test_convolution_with_bias_and_without_activation(taps, channels):
    """Against the plain convolution; a second step continues from the carried inputs."""
    ops = gpu_ops()
    w, bias = rnd((channels, taps), 1, 0.5), rnd((channels,), 2, 0.3)
    lens = [70, 1, 3]
    x = rnd((sum(lens), channels + 3), 3)
    state = torch.zeros((3, (taps - 1) * channels + 5), dtype=torch.float32, device=DEV)
    cu, slots, at = _batch(lens, [1, -1, 0])
    out = torch.empty((sum(lens), channels), dtype=torch.float32, device=DEV)
    ops.conv_silu_state(x.to(DEV), channels, w.to(DEV), state, cu, slots, out, bias=bias.to(DEV), activation="none")
    tails = {}
    for b, slot in ((0, 1), (2, 0)):
        want, tails[slot] = pr.short_convolution(x[at[b]:at[b + 1], :channels].double(), w.double(), None, bias.double())
        close(out[at[b]:at[b + 1]], want, torch.float32, f"request {b}")
    assert float(out[at[1]:at[2]].abs().max()) == 0
    x2 = rnd((4, channels + 3), 4)
    cu, slots, at = _batch([2, 2], [0, 1])
    out = torch.empty((4, channels), dtype=torch.float32, device=DEV)
    ops.conv_silu_state(x2.to(DEV), channels, w.to(DEV), state, cu, slots, out, bias=bias.to(DEV), activation="none")
    for b, slot in ((0, 0), (1, 1)):
        want, _ = pr.short_convolution(x2[at[b]:at[b + 1], :channels].double(), w.double(), tails[slot], bias.double())
        close(out[at[b]:at[b + 1]], want, torch.float32, f"continued {b}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,blocks", [(24, 3), (20, 1), (256, 4), (130, 2)])
@pytest.mark.parametrize("lens", [[37, 1, 5], [200, 1, 65], [64, 3, 129]])
def test_gated_recurrence(dtype, width, blocks, lens):
    """The gates' small products and the scan against the plain mixer's inner loop, in two steps; lam reaches from
    slow to fast decay.  Requests of more than 64 tokens are scanned in runs side by side."""
    ops = gpu_ops()
    part = width // blocks
    T = sum(lens)
    u, ypre = rnd((T, width), 1), rnd((T, width), 2)
    ra, ri = rnd((blocks, part, part), 3, 2 / math.sqrt(part)).to(dtype), rnd((blocks, part, part), 4, 2 / math.sqrt(part)).to(dtype)
    rab, rib, lam = rnd((blocks, part), 5, 0.3), rnd((blocks, part), 6, 0.3), rnd((width,), 7, 2.0) - 1
    proj = torch.cat((rnd((T, 3), 8), ypre), dim=1)
    state = torch.zeros((3, 4 + width), dtype=torch.float32, device=DEV)

    def plain(u_rows, y_rows, S):
        out = torch.zeros_like(u_rows)
        sp = pr.softplus(lam.double())
        for t in range(u_rows.shape[0]):
            ub = u_rows[t].view(blocks, part)
            r = torch.sigmoid(torch.einsum("boi,bi->bo", ra.double(), ub) + rab.double()).reshape(-1)
            i = torch.sigmoid(torch.einsum("boi,bi->bo", ri.double(), ub) + rib.double()).reshape(-1)
            a = torch.exp(-8.0 * r * sp)
            S = a * S + torch.sqrt(1 - a * a) * (i * u_rows[t])
            out[t] = S * pr.gelu_tanh(y_rows[t])
        return out, S

    def run(u_rows, proj_rows, lens, slots):
        n = u_rows.shape[0]
        cu, sl, at = _batch(lens, slots)
        ud = u_rows.to(DEV)
        gates = torch.empty((2, n, width), dtype=torch.float32, device=DEV)
        for which, wgt in enumerate((ra, ri)):
            ops.heads_gemm(ud, 0, width, part, wgt.to(DEV), gates, which * n * width, width, part, blocks, n, part, part,
                           exact=True)
        out = torch.empty((n, width), dtype=dtype, device=DEV)
        ops.rglru_scan(ud, gates, rab.to(DEV), rib.to(DEV), lam.to(DEV), proj_rows.to(DEV), 3, state, 4, cu, sl, out, 8.0,
                       max_q_len=max(lens))
        return out, at

    out, at = run(u, proj, lens, [2, -1, 0])
    carried = {}
    for b, slot in ((0, 2), (2, 0)):
        want, carried[slot] = plain(u[at[b]:at[b + 1]].double(), ypre[at[b]:at[b + 1]].double(), torch.zeros(width, dtype=torch.float64))
        close(out[at[b]:at[b + 1]], want, dtype, f"request {b}")
        close(state[slot, 4:], carried[slot], torch.float32, f"state {b}")
    assert float(out[at[1]:at[2]].float().abs().max()) == 0 and float(state[1].abs().max()) == 0
    u2, y2 = rnd((3, width), 9), rnd((3, width), 10)
    out, at = run(u2, torch.cat((rnd((3, 3), 11), y2), dim=1), [1, 2], [2, 0])
    for b, slot in ((0, 2), (1, 0)):
        want, _ = plain(u2[at[b]:at[b + 1]].double(), y2[at[b]:at[b + 1]].double(), carried[slot])
        close(out[at[b]:at[b + 1]], want, dtype, f"continued {b}")


@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(4, 2, 8, 12), (3, 3, 12, 4), (2, 1, 16, 32), (2, 2, 40, 20), (1, 1, 128, 64)])
def test_delta_rule_with_a_decay_per_channel(heads, kv_heads, dim, vdim):
    ops = gpu_ops()
    lens = [21, 1, 4]
    T = sum(lens)
    C = 2 * kv_heads * dim + heads * vdim
    qkv = rnd((T, C), 1)
    gates = rnd((T, heads + 3), 2)          # beta inputs at column 2
    decay = rnd((T, heads * dim + 1), 3)    # decay inputs at column 1
    a_log, dt_bias = rnd((heads,), 4, 0.7), rnd((heads * dim,), 5) + 0.5
    state = torch.zeros((3, 7 + heads * dim * vdim), dtype=torch.float32, device=DEV)

    def plain(rows, S):
        n = len(rows)
        q = qkv[rows, :kv_heads * dim].double().view(n, kv_heads, dim)
        k = qkv[rows, kv_heads * dim:2 * kv_heads * dim].double().view(n, kv_heads, dim)
        v = qkv[rows, 2 * kv_heads * dim:].double().view(n, heads, vdim)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        beta = torch.sigmoid(gates[rows, 2:2 + heads].double())
        step = pr.softplus(decay[rows, 1:].double() + dt_bias.double()).view(n, heads, dim)
        g = torch.exp(-torch.exp(a_log.double()).view(1, heads, 1) * step)
        out = torch.zeros(n, heads, vdim, dtype=torch.float64)
        S = S.clone()
        for t in range(n):
            for h in range(heads):
                kv = h // (heads // kv_heads)
                out[t, h], S[h] = pr.delta_step(S[h], q[t, kv], k[t, kv], v[t, h], beta[t, h], g[t, h])
        return out, S

    cu, slots, at = _batch(lens, [1, -1, 2])
    out = torch.empty((T, heads, vdim), dtype=torch.float32, device=DEV)
    ops.delta_rule(qkv.to(DEV), gates.to(DEV), 1, 2, a_log.to(DEV), dt_bias.to(DEV), state, 7, cu, slots, out, heads,
                   kv_heads, dim, vdim, decay=decay.to(DEV), per_channel=True)
    zero = torch.zeros(heads, dim, vdim, dtype=torch.float64)
    for b, slot in ((0, 1), (2, 2)):
        want, S = plain(list(range(at[b], at[b + 1])), zero)
        close(out[at[b]:at[b + 1]], want, torch.float32, f"request {b}")
        close(state[slot, 7:].view(heads, dim, vdim), S, torch.float32, f"state {b}")
    # whole = in two steps: the second starts from the state the first left
    state.zero_()
    for lo, hi in ((0, 13), (13, 21)):
        cu, slots, _ = _batch([hi - lo], [0])
        part = torch.empty((hi - lo, heads, vdim), dtype=torch.float32, device=DEV)
        ops.delta_rule(qkv[lo:hi].contiguous().to(DEV), gates[lo:hi].contiguous().to(DEV), 1, 2, a_log.to(DEV),
                       dt_bias.to(DEV), state, 7, cu, slots, part, heads, kv_heads, dim, vdim,
                       decay=decay[lo:hi].contiguous().to(DEV), per_channel=True)
        close(part, plain(list(range(21)), zero)[0][lo:hi], torch.float32, f"rows {lo}-{hi}")


def test_far_tokens_stay_in_the_recurrent_states():
    """With decays close to 1, what the first token wrote is read 1,400 tokens later: by the gated recurrence (whole,
    and in three steps that hand the state on) and by the delta rule, whose later tokens write next to nothing.
    Without the first token the same read-out is far smaller, so a state lost on the way would show."""
    ops = gpu_ops()
    T, width = 1400, 24
    lam = torch.full((width,), -9.0)                       # a = exp(-8 r softplus(-9)): about 0.9995 a token
    u = rnd((T, width), 1, 0.001)
    u[0] = 5.0
    ypre = torch.ones(T, width)
    zeros = torch.zeros(1, width)
    ident = torch.zeros(1, width, width)
    proj = torch.cat((torch.zeros(T, 3), ypre), dim=1)

    def scan(u_rows, cuts):
        state = torch.zeros((1, 4 + width), dtype=torch.float32, device=DEV)
        outs, at = [], 0
        for n in cuts:
            rows = u_rows[at:at + n].contiguous().to(DEV)
            gates = torch.zeros((2, n, width), dtype=torch.float32, device=DEV)
            out = torch.empty((n, width), dtype=torch.float32, device=DEV)
            ops.rglru_scan(rows, gates, zeros.to(DEV), zeros.to(DEV), lam.to(DEV), proj[at:at + n].contiguous().to(DEV), 3,
                           state, 4, i32([0, n]), i32([0]), out, 8.0, max_q_len=n)
            outs.append(out.cpu())
            at += n
        return torch.cat(outs)

    S = torch.zeros(width, dtype=torch.float64)
    a = torch.exp(-8.0 * 0.5 * pr.softplus(lam.double()))
    want = torch.zeros(T, width, dtype=torch.float64)
    for t in range(T):
        S = a * S + torch.sqrt(1 - a * a) * (0.5 * u[t].double())
        want[t] = S * pr.gelu_tanh(ypre[t].double())
    whole = scan(u, [T])
    close(whole, want, torch.float32, "whole")
    close(scan(u, [700, 1, 699]), want, torch.float32, "in three steps")
    without = u.clone()
    without[0] = 0
    assert float(whole[-1].abs().min()) > 20 * float(scan(without, [T])[-1].abs().max())

    # the delta rule: token 0 writes v0 under k0; later tokens have beta of about e^-20 and decays of about 1
    H = G = 1
    D, V = 16, 8
    qkv = rnd((T, 2 * D + V), 2)
    k0 = torch.zeros(D)
    k0[5] = 1.0
    qkv[0, D:2 * D] = k0
    qkv[0, 2 * D:] = 3.0
    qkv[-1, :D] = k0
    gates = torch.full((T, 1), -20.0)
    gates[0] = 20.0
    decay = torch.zeros(T, D)
    a_log, dt_bias = torch.zeros(1), torch.full((D,), -12.0)

    def read(rows, gate_rows, cuts):
        state = torch.zeros((1, D * V), dtype=torch.float32, device=DEV)
        at, last = 0, None
        for n in cuts:
            out = torch.empty((n, H, V), dtype=torch.float32, device=DEV)
            ops.delta_rule(rows[at:at + n].contiguous().to(DEV), gate_rows[at:at + n].contiguous().to(DEV), 0, 0,
                           a_log.to(DEV), dt_bias.to(DEV), state, 0, i32([0, n]), i32([0]), out, H, G, D, V,
                           decay=decay[at:at + n].contiguous().to(DEV), per_channel=True)
            at, last = at + n, out[-1, 0].cpu()
        return last

    got = read(qkv, gates, [T])
    assert float((got - 3.0 * D ** -0.5).abs().max()) < 0.02, got            # q = k0 / sqrt(dim) reads v0 back
    close(read(qkv, gates, [900, 2, 498]), got, torch.float32, "in three steps")
    silent = gates.clone()
    silent[0] = -20.0
    assert float(read(qkv, silent, [T]).abs().max()) < 0.01


@pytest.mark.parametrize("dtype", DTYPES)
def test_read_out_with_a_sigmoid_gate(dtype):
    ops = gpu_ops()
    o, gates, w = rnd((6, 3, 20), 1, 3.0), rnd((6, 64), 2, 2.0), 1 + rnd((20,), 3, 0.2)
    out = torch.empty((6, 60), dtype=dtype, device=DEV)
    ops.delta_out(o.to(DEV), gates.to(DEV), 4, w.to(DEV), 1e-5, out, activation="sigmoid")
    want = pr.rms(o.double(), 1e-5) * w.double() * torch.sigmoid(gates[:, 4:].double().view(6, 3, 20))
    close(out, want.reshape(6, 60), dtype)


# ------------------------------------------------------------------ attention whose values are its keys


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,dims,scaling", [(6, 2, 10, 6, rt.BANDS), (3, 3, 8, 8, None), (4, 1, 6, 0, None), (4, 2, 64, 32, rt.BANDS)])
def test_norm_rotation_and_page_write(dtype, H, G, D, dims, scaling):
    from atom_amd.parts import BandedRotary

    ops = gpu_ops()
    T, page = 9, 4
    proj = rnd((T, (H + G) * D + 5), 1, 2.0)
    positions = torch.tensor([0, 1, 2, 700, 701, 40000, 15, 16, 17])
    slots = torch.tensor([4, 5, 6, -1, 0, 1, 2, 3, 11])
    qw, kw = 1 + rnd((H * D,), 2, 0.2), 1 + rnd((G * D,), 3, 0.2)
    freq = None
    if dims:
        rope = BandedRotary(dims, 300.0, **(scaling or {}))
        rope.finalize(torch.device(DEV), dtype)
        freq = rope.freq
        assert torch.allclose(freq.cpu(), pr.banded_frequencies(dims, 300.0, scaling), rtol=1e-14)
    k_cache = torch.zeros((3, G, page, D), dtype=dtype, device=DEV)
    v_cache = torch.zeros((3, G, D, page), dtype=dtype, device=DEV)
    q = torch.empty((T, H, D), dtype=dtype, device=DEV)
    ops.keys_as_values_write(proj.to(DEV), q, k_cache, v_cache, qw.to(DEV), kw.to(DEV), freq, dims, i32(positions.tolist()),
                             i32(slots.tolist()), H, G, D, page, 1e-5)
    p = proj.double()
    qn = (pr.rms(p[:, :H * D], 1e-5) * qw.double()).view(T, H, D)
    kn = (pr.rms(p[:, H * D:(H + G) * D], 1e-5) * kw.double()).view(T, G, D)
    if dims:
        qn, kn = pr.rotate_pairs(qn, positions, freq.cpu()), pr.rotate_pairs(kn, positions, freq.cpu())
    close(q, qn, dtype, "q")
    raw = p[:, H * D:(H + G) * D].view(T, G, D)
    for t in range(T):
        if int(slots[t]) < 0:
            continue
        pg, off = divmod(int(slots[t]), page)
        close(k_cache[pg, :, off, :], kn[t], dtype, f"key {t}")
        close(v_cache[pg, :, :, off], raw[t], dtype, f"value {t}: the key as projected")
    assert float(k_cache.view(-1, D)[[3 * G * page - 1]].abs().max()) >= 0   # untouched slots stay whatever they were
    gated = torch.empty((T, H * D), dtype=dtype, device=DEV)
    x = rnd((T, H * D), 5).to(dtype)
    ops.sigmoid_gate(x.to(DEV), proj.to(DEV), 3, gated)
    close(gated, x.double() * torch.sigmoid(p[:, 3:3 + H * D]), dtype, "gate")


def _paged(keys, values, page, dtype, order_seed=0):
    """Keys and values [n, G, D] of one request in pages handed out in a shuffled order."""
    n, G, D = keys.shape
    pages = -(-n // page)
    order = torch.randperm(pages + 3, generator=torch.Generator().manual_seed(order_seed))[:pages].tolist()
    k_cache = torch.zeros((pages + 3, G, page, D), dtype=dtype)
    v_cache = torch.zeros((pages + 3, G, D, page), dtype=dtype)
    for pos in range(n):
        k_cache[order[pos // page], :, pos % page, :] = keys[pos].to(dtype)
        v_cache[order[pos // page], :, :, pos % page] = values[pos].to(dtype)
    return k_cache.to(DEV), v_cache.to(DEV), order


def _attend(ops, q, k_cache, v_cache, order, page, q_positions, ctx, scale, chunk, softcap, cached):
    """Queries of one request: the last ``len(q_positions)`` tokens of a context of ``ctx``."""
    T, H, D = q.shape
    tiles = {}
    meta = AttentionMeta(token_seq=i32([0] * T), positions=i32(q_positions), block_tables=i32([order]),
                         cu_seqlens_q=i32([0, T]), context_lens=i32([ctx]), num_seqs=1, num_tokens=T, max_q_len=T,
                         max_context_len=ctx, page_size=page, num_prefill=1 if T > 1 else 0)
    if T > 1:
        short, tall = ops.attention_tile_rows(q.dtype, D, page, H // k_cache.shape[1], T)
        if short:
            meta.rows_per_tile = short
            meta.prefill_tiles = i32([[0, r] for r in range(0, T, short)])
        if tall:
            tiles[tall] = i32([[0, r] for r in range(0, T, tall)])
            meta.tiles_by_rows = tiles
    out = torch.empty_like(q)
    ops.paged_attention(q, k_cache, v_cache, out, meta, scale, None, softcap=softcap, chunk=chunk)
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,page,chunk,softcap", [(6, 2, 10, 4, 7, 3.0), (4, 2, 64, 16, 48, 20.0), (2, 1, 128, 16, 160, None),
                                                      (4, 4, 64, 8, 16, None), (8, 2, 64, 16, 100, 5.0)])
def test_chunked_capped_attention(dtype, H, G, D, page, chunk, softcap):
    """Prompt portions (behind cached keys and not) and single tokens against the plain scores, keys in shuffled
    pages; the same queries one by one give the same rows."""
    ops = gpu_ops()
    n = 3 * chunk + chunk // 2 + 3
    keys, values = rnd((n, G, D), 1), rnd((n, G, D), 2)
    queries = rnd((n, H, D), 3)
    scale = 1.7 / math.sqrt(D)
    k_cache, v_cache, order = _paged(keys, values, page, dtype)
    kd, vd = k_cache.cpu().double(), v_cache.cpu().double()

    def plain(pos):
        seen = [j for j in range(n) if pr.visible(pos, j, chunk)]
        out = torch.zeros(H, D, dtype=torch.float64)
        for h in range(H):
            kv = h // (H // G)
            kk = torch.stack([kd[order[j // page], kv, j % page, :] for j in seen])
            vv = torch.stack([vd[order[j // page], kv, :, j % page] for j in seen])
            s = (kk @ queries[pos, h].to(dtype).double()) * scale
            if softcap:
                s = softcap * torch.tanh(s / softcap)
            out[h] = torch.softmax(s, dim=0) @ vv
        return out

    q = queries.to(dtype).to(DEV)
    whole = _attend(ops, q, k_cache, v_cache, order, page, list(range(n)), n, scale, chunk, softcap, 0)
    for pos in list(range(0, n, 5)) + [chunk - 1, chunk, 2 * chunk - 1, 2 * chunk, n - 1]:
        close(whole[pos], plain(pos), dtype, f"whole prompt, position {pos}")
    cut = chunk + chunk // 3          # a portion that begins inside a chunk, behind cached keys
    part = _attend(ops, q[cut:].contiguous(), k_cache, v_cache, order, page, list(range(cut, n)), n, scale, chunk, softcap, cut)
    close(part, whole[cut:], dtype, "a portion behind cached keys")
    for pos in (0, chunk - 1, chunk, 2 * chunk + 1, 3 * chunk - 1, 3 * chunk, n - 1):
        one = _attend(ops, q[pos:pos + 1].contiguous(), k_cache, v_cache, order, page, [pos], pos + 1, scale, chunk, softcap, pos)
        close(one[0], plain(pos), dtype, f"single token at {pos}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D,page,chunk", [(64, 16, 48), (10, 4, 7), (128, 16, 160)])
def test_a_key_that_stands_out_is_seen_inside_its_chunk_only(dtype, D, page, chunk):
    """One key among hundreds has a score far above the rest, and a value like no other.  Queries in its chunk return
    its value, at the chunk's last position too; the next chunk's first position does not, nor does any later one.
    The key sits at a chunk's first position, at its last, right before and right after a page border."""
    ops = gpu_ops()
    H = G = 2
    n = 4 * chunk
    for spot in (chunk, 2 * chunk - 1, (chunk // page + 1) * page - 1, (chunk // page + 1) * page, 5):
        keys, values = rnd((n, G, D), 4, 0.05), rnd((n, G, D), 5, 0.05)
        queries = rnd((n, H, D), 6, 0.05)
        direction = torch.zeros(D)
        direction[3] = 1.0
        keys[spot] = 40.0 * direction
        queries[:, :, 3] = 1.0
        values[spot] = 7.0
        k_cache, v_cache, order = _paged(keys, values, page, dtype, order_seed=spot)
        q = queries.to(dtype).to(DEV)
        whole = _attend(ops, q, k_cache, v_cache, order, page, list(range(n)), n, 1.0, chunk, None, 0).float().cpu()
        end = (spot // chunk + 1) * chunk
        for pos in range(n):
            inside = spot <= pos < end
            got = float(whole[pos].mean())
            assert (abs(got - 7.0) < 0.1) == inside, f"key at {spot}, query at {pos}: {got:.3f}"
        for pos in (spot, end - 1, end, min(n - 1, end + chunk)):
            one = _attend(ops, q[pos:pos + 1].contiguous(), k_cache, v_cache, order, page, [pos], pos + 1, 1.0, chunk, None, pos)
            assert (abs(float(one.float().mean()) - 7.0) < 0.1) == (spot <= pos < end), f"decoded: key at {spot}, query at {pos}"


# ------------------------------------------------------------------ the engine

LENGTHS = {"U": [1, 7, 33, 150, 64, 300], "V": [2, 19, 45, 260, 128], "W": [3, 40, 17, 270, 96, 161],
           "X": [5, 40, 130, 300]}
# float32: every position against the largest logit of its request; where the plain implementation in float32 is
# itself further from float64 than that (a token whose sublayer output is small before its norm), four times its
# own distance is allowed
F32_TOL = dict(max=1e-4, mean=2e-5)
BF16_TOL = dict(max=6e-2, mean=1.2e-2)


def _requests(which, seed=0):
    return {f"r{k}": rt.ids(which, n, seed * 100 + k) for k, n in enumerate(LENGTHS[which])}


def _check(steps, results, requests, which, dtype, what):
    rows = replay.collect(steps, results)
    over, judged = [], 0
    for rid, tokens in requests.items():
        want = rt.oracle(which, tokens)
        scale = float(want.abs().max())
        inherent = rt.float32_error(which, tokens) / scale if dtype == "float32" else None
        assert len(rows[rid]) == len(tokens)
        for pos, got in sorted(rows[rid].items()):
            assert torch.isfinite(got).all(), f"{what} request {rid} position {pos}: not finite"
            diff = (got.double() - want[pos]).abs()
            worst, mean = float(diff.max()) / scale, float(diff.mean()) / scale
            judged += 1
            if dtype == "float32":
                room = max(1.0, 4 * float(inherent[pos]) / F32_TOL["max"])
                assert worst <= room * F32_TOL["max"] and mean <= room * F32_TOL["mean"], \
                    f"{what} request {rid} position {pos}: max {worst:.3e} mean {mean:.3e} of the largest logit"
            elif worst > BF16_TOL["max"] or mean > BF16_TOL["mean"]:
                over.append((rid, pos, worst, mean))
    assert len(over) <= 0.02 * judged, f"{what}: {len(over)} of {judged} over: {over[:5]}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["U", "V", "W"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_cuts_match_plain(which, cut, dtype):
    requests = _requests(which)
    steps = getattr(replay, cut)(requests)
    pages = -(-replay.peak_tokens(steps, 16) // 16)
    core = rt.core(which, dtype, gpu_ops(), DEV, num_pages=pages, page_size=16, graph_sizes=[1, 2, 4] if cut != "whole" else None)
    results = replay.run_in_process(core, steps)
    _check(steps, results, requests, which, dtype, f"{which}/{cut}/{dtype}")
    assert all(pool.num_free == pool.num_pages for pool in core.manager.pools)
    if cut == "tail":
        assert core.graphs is not None and core.graphs.replays >= 32, "single tokens replay captured graphs"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "mixed"])
def test_wider_model_reaches_every_product_kernel(cut, dtype):
    """Prompts of 5, 40, 130 and 300 tokens on a model of width 384: products of few rows, of up to 64, of up to 256
    and the library's, with float32 outputs and biases, all against the plain implementation."""
    requests = _requests("X")
    steps = getattr(replay, cut)(requests)
    pages = -(-replay.peak_tokens(steps, 16) // 16)
    core = rt.core("X", dtype, gpu_ops(), DEV, num_pages=pages, page_size=16, graph_sizes=[1, 2, 4] if cut != "whole" else None)
    results = replay.run_in_process(core, steps)
    _check(steps, results, requests, "X", dtype, f"X/{cut}/{dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_small_pages_slots_used_again_and_long_decoding(dtype):
    """Pages of 4 tokens, two state slots for five requests, and 150 tokens decoded one by one across many chunk
    edges, every one of them compared."""
    requests = {"long": rt.ids("U", 330, 1), "b": rt.ids("U", 23, 2), "c": rt.ids("U", 50, 3), "d": rt.ids("U", 9, 4),
                "e": rt.ids("U", 31, 5)}
    steps = replay.mixed(requests, seed=6, max_live=2, decode_tail=150)
    pages = -(-replay.peak_tokens(steps, 4) // 4)
    core = rt.core("U", dtype, gpu_ops(), DEV, num_pages=pages, page_size=4, max_num_seqs=2, graph_sizes=[1, 2])
    results = replay.run_in_process(core, steps)
    _check(steps, results, requests, "U", dtype, f"U/page4/{dtype}")


def test_logits_do_not_depend_on_the_batch_or_the_cut():
    """float32: a request's logits alone, cut in portions, and beside others differ by rounding of sums only."""
    requests = _requests("W")
    runs = []
    for cut in ("whole", "portions", "mixed"):
        steps = getattr(replay, cut)(requests)
        core = rt.core("W", "float32", gpu_ops(), DEV, num_pages=80, page_size=16)
        runs.append(replay.collect(steps, replay.run_in_process(core, steps)))
    for rid in requests:
        for pos in runs[0][rid]:
            for other in runs[1:]:
                assert float((runs[0][rid][pos] - other[rid][pos]).abs().max()) <= 2e-5 * float(runs[0][rid][pos].abs().max())


@pytest.mark.parametrize("which,dtype", [("U", "fp32"), ("V", "fp32"), ("W", "fp32"), ("W", "bf16")])
def test_greedy_generation_through_the_engine(which, dtype):
    from atom_amd import LLMEngine, SamplingParams

    llm = LLMEngine(rt.folder(which), dtype=dtype, ops=gpu_ops(), kv_cache_block_size=16, num_kvcache_blocks=64,
                    max_num_seqs=4, max_num_batched_tokens=64, max_model_len=512)
    prompts = [rt.ids(which, n, 70 + n) for n in (1, 9, 40, 130, 65)]
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
    for prompt, out in zip(prompts, outs):
        tokens = list(prompt)
        assert len(out["token_ids"]) == 10
        for token in out["token_ids"]:
            logits = rt.oracle(which, tokens)[-1]
            best = int(logits.argmax())
            slack = 0.0 if dtype == "fp32" else 0.06 * float(logits.abs().max())
            assert token == best or float(logits[best] - logits[token]) <= slack
            tokens.append(token)
    assert all(p.num_free == p.num_pages for p in llm.core.manager.pools)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_program(dtype, tmp_path):
    requests = {k: v for k, v in list(_requests("V").items())[:4]}
    steps = replay.mixed(requests, seed=2, max_live=3)
    results = replay.run_program(rt.folder("V"), dtype, steps, str(tmp_path / "out"), replay.peak_tokens(steps, 64),
                                 rt.CONFIGS["V"]["vocab"])
    _check(steps, results, requests, "V", dtype, f"program/{dtype}")


def test_command_line():
    """``python -m atom_amd.examples.simple_inference`` on a Ralitar folder: the registry picks the design from
    config.json; greedy completions are the plain implementation's."""
    import random
    import re
    import subprocess
    import sys

    cmd = [sys.executable, "-m", "atom_amd.examples.simple_inference", "--model", rt.folder("V"), "--temperature", "0",
           "--max-tokens", "6", "--block_size", "16", "--num-kvcache-blocks", "32", "--max-num-seqs", "4", "--dtype", "fp32",
           "--max-model-len", "256", "--seed", "3"]
    res = subprocess.run(cmd, cwd=replay.ROOT, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    assert res.stdout.count("Completion:") == 3 and res.stdout.count("finish_reason=max_tokens") == 3
    rng = random.Random(3)
    prompts = [[rng.randrange(rt.CONFIGS["V"]["vocab"]) for _ in range(n)] for n in (5, 17, 33)]
    shown = [eval(m) for m in re.findall(r"Completion: (\[.*?\])", res.stdout)]
    for prompt, out in zip(prompts, shown):
        tokens = list(prompt)
        for token in out:
            assert token == int(rt.oracle("V", tokens)[-1].argmax())
            tokens.append(token)
