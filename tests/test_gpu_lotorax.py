"""Lotorax on the GPU: every new kernel alone against the plain implementation's function of the same
mechanism (float32 and bfloat16), then the engine on tiny models: whole prompts, token-by-token tails, portions
down to two tokens, mixed batches with pages and slots used again, decode steps replayed from graphs, long
decoding across the attention kernel's key chunks, greedy generation through ``LLMEngine``, and ``bin/trace_run``."""

import math

import pytest
import torch

import lotorax_tiny as lt
import plain_lotorax as pl
import replay
from helpers import gpu_ops
from atom_amd.engine.core import StepEntry
from atom_amd.kernels.hip import AttentionMeta

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


def close(got, want, dtype, what=""):
    got, want = got.double().cpu(), want.double()
    scale = max(1e-6, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= TOL[dtype] * scale, f"{what}: {err:.3e} > {TOL[dtype] * scale:.3e}"


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


# ------------------------------------------------------------------ norms and the stream


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,n", [(48, 7), (200, 7), (1031, 7), (200, 300), (5000, 7), (1031, 260)])
def test_layernorm_modes(dtype, width, n):
    """Few rows and wide rows (a block a row), many rows (a wave a row)."""
    ops = gpu_ops()
    x = (rnd((n, width), 1, 2.0) + 0.7).to(dtype)
    w, b, w2, b2 = 1 + rnd((width,), 2, 0.2), rnd((width,), 3, 0.3), 1 + rnd((width,), 4, 0.2), rnd((width,), 5, 0.3)
    dev = lambda t: t.to(DEV)  # noqa: E731
    eps = 3e-5
    out = torch.empty((n, width), dtype=dtype, device=DEV)
    close(ops.layernorm(dev(x), dev(w), dev(b), eps, out), pl.layer_norm(x.double(), w.double(), b.double(), eps), dtype, "plain")
    res = torch.empty((n, width), dtype=torch.float32, device=DEV)
    ops.layernorm(dev(x), dev(w), dev(b), eps, out, residual=res, mode="init")
    assert torch.equal(res.cpu(), x.float())
    y = rnd((n, width), 6).to(dtype)
    ops.layernorm(dev(y), dev(w), dev(b), eps, out, residual=res, mode="add")
    total = x.double() + y.double()
    close(res, total, torch.float32, "sum")
    close(out, pl.layer_norm(total, w.double(), b.double(), eps), dtype, "add")
    # the normed rows join the stream unrounded, and the stream is normed for what follows
    z = rnd((n, width), 7, 3.0).to(dtype)
    ops.layernorm(dev(z), dev(w), dev(b), eps, out, residual=res, mode="post", next_weight=dev(w2), next_bias=dev(b2))
    total = total + pl.layer_norm(z.double(), w.double(), b.double(), eps)
    close(res, total, torch.float32, "post sum")
    close(out, pl.layer_norm(total, w2.double(), b2.double(), eps), dtype, "post")
    rows = i32([5, 0, 5])
    few = torch.empty((3, width), dtype=dtype, device=DEV)
    before = res.clone()
    ops.layernorm(dev(y), dev(w), dev(b), eps, few, residual=res, mode="add", rows=rows)
    assert torch.equal(res, before)
    close(few, pl.layer_norm((total + y.double())[[5, 0, 5]], w.double(), b.double(), eps), dtype, "rows")
    # a float32 input (the stream's own summand) with an output of the serving type
    f32 = torch.empty((n, width), dtype=torch.float32, device=DEV)
    close(ops.layernorm(dev(x.float()), dev(w), dev(b), eps, f32), pl.layer_norm(x.double(), w.double(), b.double(), eps),
          torch.float32, "float32 out")


@pytest.mark.parametrize("dtype", DTYPES)
def test_scaled_embedding_join_input_and_activations(dtype):
    ops = gpu_ops()
    table = rnd((37, 24), 1).to(dtype)
    ids = i32([3, 36, 0, 3])
    out = torch.empty((4, 24), dtype=torch.float32, device=DEV)
    ops.embedding_scaled(table.to(DEV), ids, out, 3.7)
    close(out, table.double()[[3, 36, 0, 3]] * 3.7, torch.float32)
    hidden, res, first = rnd((4, 24), 2).to(dtype), rnd((4, 24), 3), rnd((4, 24), 4)
    both = torch.empty((4, 48), dtype=dtype, device=DEV)
    ops.sum_concat(hidden.to(DEV), res.to(DEV), first.to(DEV), both)
    close(both, torch.cat((hidden.double() + res.double(), first.double()), 1), dtype)
    ops.sum_concat(hidden.to(DEV), None, first.to(DEV), both)
    close(both, torch.cat((hidden.double(), first.double()), 1), dtype)
    x = rnd((5, 2 * 20), 5, 2.0).to(dtype)
    act = torch.empty((5, 20), dtype=dtype, device=DEV)
    for name, f in (("relu", torch.relu), ("silu", pl.silu), ("gelu_tanh", pl.gelu_tanh)):
        ops.gated_act(x.to(DEV), act, name)
        close(act, f(x.double()[:, :20]) * x.double()[:, 20:], dtype, name)


# ------------------------------------------------------------------ attention over latents


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,rot,rank,dims,scaling", [(3, 8, 4, 24, 4, lt.YARN), (2, 16, 8, 40, 8, None),
                                                             (5, 4, 6, 16, 4, lt.YARN), (1, 32, 64, 128, 64, lt.YARN)])
def test_latent_prepare(dtype, heads, dim, rot, rank, dims, scaling):
    from atom_amd.parts import ScaledRotary

    ops = gpu_ops()
    T, pre = 9, 5
    ld = pre + heads * (dim + rot) + rank + rot + 3
    proj = rnd((T, ld), 1)
    positions = torch.tensor([0, 1, 2, 700, 701, 40000, 15, 16, 17])
    rope = ScaledRotary(dims, 5000.0, **(scaling or {}))
    rope.finalize(torch.device(DEV), dtype)
    f, mult = pl.yarn_frequencies(dims, 5000.0, scaling)
    assert torch.allclose(rope.freq.cpu(), f, rtol=1e-14) and rope.mult == pytest.approx(mult)
    w = 1 + rnd((rank,), 2, 0.2)
    slots = torch.tensor([4, 5, 6, -1, 0, 1, 2, 3, 11])
    pages = torch.zeros((3, 4, rank + rot), dtype=dtype, device=DEV)
    q_abs = torch.zeros((T, heads, rank + rot), dtype=dtype, device=DEV)
    kv_off = pre + heads * (dim + rot)
    ops.latent_prepare(proj.to(DEV), pre, kv_off, heads, dim, rot, rank, dims, w.to(DEV), 1e-5, rope.freq, rope.mult,
                       positions.int().to(DEV), slots.int().to(DEV), pages, q_abs, 0.37)
    p = proj.double()
    q = p[:, pre:kv_off].view(T, heads, dim + rot)[..., dim:]
    close(q_abs[..., rank:], pl.rotate_pairs(q, positions, dims, 5000.0, scaling) * 0.37, dtype, "rotated queries")
    c = pl.rms_unit(p[:, kv_off:kv_off + rank], 1e-5) * w.double()
    k = pl.rotate_pairs(p[:, kv_off + rank:kv_off + rank + rot], positions, dims, 5000.0, scaling)
    want = torch.zeros((12, rank + rot), dtype=torch.float64)
    for t in range(T):
        if slots[t] >= 0:
            want[slots[t]] = torch.cat((c[t], k[t]))
    close(pages.view(12, -1), want, dtype, "pages")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("x_dtype", DTYPES)
@pytest.mark.parametrize("H,m,n,k", [(3, 70, 21, 16), (2, 200, 100, 40), (5, 33, 64, 128)])
def test_heads_gemm_on_the_matrix_cores(dtype, x_dtype, H, m, n, k):
    """Strides that keep 16-byte pieces aligned: bfloat16 weights with 32 rows or more take the matrix-core kernel."""
    ops = gpu_ops()
    ldx, hsx, ldy, hsy = H * (k + 8) + 16, k + 8, H * (n + 3), n + 3
    x = rnd((m, ldx), 1).to(x_dtype)
    w = rnd((H, n, k), 2, k ** -0.5).to(dtype)
    y = torch.zeros((m, ldy), dtype=dtype, device=DEV)
    gate = rnd((m, H + 2), 3)
    ops.heads_gemm(x.to(DEV), 8, ldx, hsx, w.to(DEV), y, 1, ldy, hsy, H, m, n, k, alpha=0.7, gate=gate.to(DEV),
                   gate_offset=2, ldg=H + 2)
    for h in range(H):
        want = 0.7 * x.double()[:, 8 + h * hsx:8 + h * hsx + k] @ w.double()[h].T * torch.sigmoid(gate.double()[:, 2 + h])[:, None]
        close(y[:, 1 + h * hsy:1 + h * hsy + n], want, torch.bfloat16 if torch.bfloat16 in (dtype, x_dtype) else dtype, f"head {h}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_heads_gemm_with_strides_and_gate(dtype):
    ops = gpu_ops()
    H, m, n, k = 3, 70, 21, 13
    ldx, hsx, ldy, hsy = H * 20 + 7, 20, H * 30, 30
    x = rnd((m, ldx), 1)
    w = rnd((H, n, k), 2).to(dtype)
    y = torch.zeros((m, ldy), dtype=dtype, device=DEV)
    gate = rnd((m, 9), 3)
    ops.heads_gemm(x.to(DEV), 4, ldx, hsx, w.to(DEV), y, 2, ldy, hsy, H, m, n, k, alpha=0.5, gate=gate.to(DEV),
                   gate_offset=1, ldg=9)
    for h in range(H):
        want = 0.5 * x.double()[:, 4 + h * hsx:4 + h * hsx + k] @ w.double()[h].T * torch.sigmoid(gate.double()[:, 1 + h])[:, None]
        close(y[:, 2 + h * hsy:2 + h * hsy + n], want, dtype, f"head {h}")


def _plain_latent_attention(q_abs, rows, rank, sink, positions, window=None):
    out = []
    for t, pos in enumerate(positions):
        first = max(0, pos - window + 1) if window else 0
        keys = rows[first:pos + 1]
        s = q_abs[t] @ keys.T
        top = s.max(dim=-1, keepdim=True).values
        if sink is not None:
            top = torch.maximum(top, sink[:, None])
        e = torch.exp(s - top)
        denom = e.sum(-1, keepdim=True) + (torch.exp(sink[:, None] - top) if sink is not None else 0)
        out.append((e / denom) @ keys[:, :rank])
    return torch.stack(out)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rank,rot,heads,page,window", [(24, 4, 3, 8, None), (64, 16, 4, 16, None), (40, 8, 2, 4, 37),
                                                        (128, 32, 7, 16, None), (32, 16, 5, 8, 41), (256, 64, 16, 16, None),
                                                        (512, 64, 3, 16, None), (48, 8, 70, 4, None)])
def test_latent_attention_far_keys_page_and_chunk_edges(dtype, rank, rot, heads, page, window):
    """Queries at the first positions, around page borders and around the kernel's chunks of 256 keys, and at the
    end of a long context; key 3 is made to stand out for the last queries, so that a lost far key shows; the sink
    is large for one head, so that leaving it out shows."""
    ops = gpu_ops()
    n = 700
    width = rank + rot
    rows = rnd((n, width), 1, 0.5)
    # requests that share one context's pages; each brings a few consecutive tokens that end its own context
    groups = [[0, 1, 2], [page - 1, page, page + 1], [254, 255, 256, 257], [511, 512, 513], [n - 2, n - 1]]
    positions = [pos for grp in groups for pos in grp]
    q_abs = rnd((len(positions), heads, width), 2, 0.4)
    rows[3] = 0.1 * rows[3]
    rows[3, :8] = 2.0
    q_abs[-2:, :, :8] = 1.5                      # the last queries look for key 3, 690 tokens back
    sink = rnd((heads,), 3)
    sink[0] = 6.0
    rows, q_abs = rows.to(dtype), q_abs.to(dtype)
    want = _plain_latent_attention(q_abs.double(), rows.double(), rank, sink.double(), positions, window)
    if window is None:
        lost = _plain_latent_attention(q_abs.double(), torch.cat((rows[:3], rows[3:4] * 0, rows[4:])).double(), rank,
                                       sink.double(), positions)
        assert float((lost[-1] - want[-1]).abs().max()) > 0.05, "the far key must matter in this test"
    # scatter the context over pages in a shuffled order
    num_pages = -(-n // page) + 3
    order = torch.randperm(num_pages, generator=torch.Generator().manual_seed(4))[:-(-n // page)]
    pages = torch.zeros((num_pages, page, width), dtype=dtype)
    for j in range(n):
        pages[order[j // page], j % page] = rows[j]
    starts = [0]
    for grp in groups:
        starts.append(starts[-1] + len(grp))
    meta = AttentionMeta(token_seq=i32([b for b, grp in enumerate(groups) for _ in grp]), positions=i32(positions),
                         block_tables=order.int().view(1, -1).repeat(len(groups), 1).contiguous().to(DEV),
                         cu_seqlens_q=i32(starts), context_lens=i32([grp[-1] + 1 for grp in groups]), num_seqs=len(groups),
                         num_tokens=len(positions), max_q_len=4, max_context_len=n, page_size=page, num_prefill=len(groups))
    out = torch.empty((len(positions), heads, rank), dtype=dtype, device=DEV)
    ops.latent_attention(q_abs.to(DEV), pages.to(DEV), out, meta, rank, sink.to(DEV), window)
    close(out, want, dtype, "with sink")
    ops.latent_attention(q_abs.to(DEV), pages.to(DEV), out, meta, rank, None, window)
    close(out, _plain_latent_attention(q_abs.double(), rows.double(), rank, None, positions, window), dtype, "no sink")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rank,rot,heads,page", [(64, 16, 4, 16), (128, 32, 5, 8), (40, 8, 2, 4), (512, 64, 16, 16)])
def test_latent_attention_single_tokens_with_keys_split_over_blocks(dtype, rank, rot, heads, page):
    """One token a request, contexts of 1 key to 700, a padding row, and a row's keys on one block or split over
    3 or 8 (the matrix-core kernel; the general kernel takes no split)."""
    ops = gpu_ops()
    width = rank + rot
    contexts = [1, 31, 33, 700, 256, 0, 97]
    num_pages = sum(-(-c // page) for c in contexts) + 2
    order = torch.randperm(num_pages, generator=torch.Generator().manual_seed(5)).tolist()
    pages = torch.zeros((num_pages, page, width), dtype=dtype)
    tables = torch.zeros((len(contexts), -(-700 // page)), dtype=torch.int32)
    rows, sink = [], rnd((heads,), 9)
    for b, c in enumerate(contexts):
        mine = rnd((c, width), 20 + b, 0.5).to(dtype)
        rows.append(mine)
        for j in range(c):
            if j % page == 0:
                tables[b, j // page] = order.pop()
            pages[tables[b, j // page], j % page] = mine[j]
    q_abs = rnd((len(contexts), heads, width), 3, 0.4).to(dtype)
    want = torch.zeros((len(contexts), heads, rank), dtype=torch.float64)
    for b, c in enumerate(contexts):
        if c:
            want[b] = _plain_latent_attention(q_abs[b:b + 1].double(), rows[b].double(), rank, sink.double(), [c - 1])[0]
    meta = AttentionMeta(token_seq=i32([b if c else -1 for b, c in enumerate(contexts)]), positions=i32([max(c - 1, 0) for c in contexts]),
                         block_tables=tables.to(DEV), cu_seqlens_q=i32(list(range(len(contexts) + 1))),
                         context_lens=i32(contexts), num_seqs=len(contexts), num_tokens=len(contexts), max_q_len=1,
                         max_context_len=700, page_size=page, num_prefill=0)
    for parts in (None, 1, 3, 8):
        out = torch.full((len(contexts), heads, rank), 7.0, dtype=dtype, device=DEV)
        ops.latent_attention(q_abs.to(DEV), pages.to(DEV), out, meta, rank, sink.to(DEV), None, parts=parts)
        close(out, want, dtype, f"parts {parts}")


# ------------------------------------------------------------------ the delta rule


@pytest.mark.parametrize("lens", [[5, 1, 2, 1, 9], [150, 3, 64, 2, 65]])
@pytest.mark.parametrize("taps,channels", [(2, 40), (4, 300), (5, 17), (1, 8)])
def test_conv_silu_state(taps, channels, lens):
    """Requests of one token, of fewer tokens than taps, and of several runs of 64 tokens; a padding row."""
    ops = gpu_ops()
    slots = [2, 0, 3, -1, 1]
    T = sum(lens)
    x = rnd((T, channels + 6), 1)
    w = rnd((channels, taps), 2, 0.6)
    floats = (taps - 1) * channels
    state = rnd((4, floats + 11), 3)
    want_state = state.clone().double()
    want = torch.zeros((T, channels), dtype=torch.float64)
    at = 0
    for n, slot in zip(lens, slots):
        if slot >= 0:
            tail = want_state[slot, :floats].view(taps - 1, channels)
            y, new = pl.short_convolution(x[at:at + n, :channels].double(), w.double(), tail.clone())
            want[at:at + n] = pl.silu(y)
            tail.copy_(new)
        at += n
    cu = i32([0] + list(torch.tensor(lens).cumsum(0)))
    out = torch.empty((T, channels), dtype=torch.float32, device=DEV)
    dstate = state.to(DEV)
    for wd in DTYPES:
        dstate.copy_(state)
        ops.conv_silu_state(x.to(DEV), channels, w.to(wd).to(DEV), dstate, cu, i32(slots), out)
        close(out, want if wd == torch.float32 else want, wd, "convolution")
    close(dstate, want_state, torch.bfloat16, "carried inputs")
    dstate.copy_(state)
    ops.conv_silu_state(x.to(DEV), channels, w.to(DEV), dstate, cu, i32(slots), out)
    close(dstate, want_state, torch.float32, "carried inputs")
    assert torch.equal(dstate[:, floats:].cpu(), state[:, floats:])


@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(4, 2, 8, 12), (2, 1, 12, 20), (3, 3, 48, 70), (2, 2, 128, 300)])
def test_delta_rule_and_read_out(heads, kv_heads, dim, vdim):
    ops = gpu_ops()
    lens, slots = [21, 1, 2, 1], [1, 2, -1, 0]
    T = sum(lens)
    C = 2 * kv_heads * dim + heads * vdim
    qkv = rnd((T, C), 1)
    gates = rnd((T, 3 + 2 * heads), 2, 1.5)
    a_log, dt_bias = rnd((heads,), 3, 0.7), 0.5 + rnd((heads,), 4)
    off = 5
    state = rnd((3, off + heads * dim * vdim), 5, 0.3)
    want_state = state.clone().double()
    want = torch.zeros((T, heads, vdim), dtype=torch.float64)
    at = 0
    for n, slot in zip(lens, slots):
        if slot >= 0:
            x = qkv[at:at + n].double()
            q = x[:, :kv_heads * dim].view(n, kv_heads, dim)
            k = x[:, kv_heads * dim:2 * kv_heads * dim].view(n, kv_heads, dim)
            v = x[:, 2 * kv_heads * dim:].view(n, heads, vdim)
            q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
            k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
            g = gates[at:at + n].double()
            beta = torch.sigmoid(g[:, 1:1 + heads])
            decay = torch.exp(-torch.exp(a_log.double()) * pl.softplus(g[:, 2 + heads:2 + 2 * heads] + dt_bias.double()))
            S = want_state[slot, off:].view(heads, dim, vdim)
            for h in range(heads):
                kv = h // (heads // kv_heads)
                o, new = pl.delta_rule(q[:, kv], k[:, kv], v[:, h], beta[:, h], decay[:, h], S[h].clone())
                want[at:at + n, h] = o
                S[h] = new
        at += n
    cu = i32([0] + list(torch.tensor(lens).cumsum(0)))
    out = torch.empty((T, heads, vdim), dtype=torch.float32, device=DEV)
    dstate = state.to(DEV)
    ops.delta_rule(qkv.to(DEV), gates.to(DEV), 2 + heads, 1, a_log.to(DEV), dt_bias.to(DEV), dstate, off, cu, i32(slots),
                   out, heads, kv_heads, dim, vdim)
    close(out, want, torch.float32, "read-out")
    close(dstate, want_state, torch.float32, "state")
    w = 1 + rnd((vdim,), 6, 0.2)
    gate = rnd((T, 4 + heads * vdim), 7)
    for dtype in DTYPES:
        y = torch.empty((T, heads * vdim), dtype=dtype, device=DEV)
        ops.delta_out(out, gate.to(DEV), 4, w.to(DEV), 1e-5, y)
        ref = pl.rms_unit(out.double().cpu(), 1e-5) * w.double() * pl.silu(gate.double()[:, 4:].view(T, heads, vdim))
        close(y, ref.reshape(T, -1), dtype, "gated read-out")


# ------------------------------------------------------------------ routed experts


@pytest.mark.parametrize("experts,top", [(5, 2), (4, 1), (6, 3), (64, 8)])
def test_router_choice_uses_the_correction_for_the_choice_only(experts, top):
    ops = gpu_ops()
    logits = rnd((50, experts), 1, 2.0)
    correction = rnd((experts,), 2, 0.5)
    w = {"router": torch.eye(experts, dtype=torch.float64), "correction": correction.double()}
    ids, weights = pl.routed_choice(logits.double(), w, top)
    got_ids, got_w = ops.router_choose(logits.to(DEV), correction.to(DEV), top)
    assert torch.equal(got_ids.cpu().long().sort(dim=-1).values, ids.sort(dim=-1).values)
    order = got_ids.cpu().long()
    close(got_w, torch.sigmoid(logits.double()).gather(1, order), torch.float32)
    plain_ids, _ = pl.routed_choice(logits.double(), {"router": w["router"], "correction": 0 * correction.double()}, top)
    assert not torch.equal(plain_ids.sort(dim=-1).values, ids.sort(dim=-1).values), "the correction must matter here"
    _, renorm = ops.router_choose(logits.to(DEV), correction.to(DEV), top, renormalize=True)
    close(renorm.sum(-1), torch.ones(50), torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,ff,experts,top,tokens", [(48, 40, 5, 2, 13), (40, 16, 6, 3, 1), (64, 32, 8, 1, 70),
                                                         (48, 40, 5, 2, 300), (136, 72, 33, 4, 129), (264, 88, 10, 2, 64)])
def test_experts_forward(dtype, width, ff, experts, top, tokens):
    ops = gpu_ops()
    x = rnd((tokens, width), 1).to(dtype)
    w = {"router": rnd((experts, width), 2, 0.5).to(dtype), "correction": rnd((experts,), 3, 0.3)}
    for e in range(experts):
        w[f"e{e}.gate"], w[f"e{e}.up"] = rnd((ff, width), 10 + e, width ** -0.5).to(dtype), rnd((ff, width), 30 + e, width ** -0.5).to(dtype)
        w[f"e{e}.down"] = rnd((width, ff), 50 + e, ff ** -0.5).to(dtype)
    wd = {k: v.double() for k, v in w.items()}
    want = pl.routed_ff(x.double(), wd, experts, top)
    gate_up = torch.stack([torch.cat((w[f"e{e}.gate"], w[f"e{e}.up"])) for e in range(experts)]).to(DEV)
    down = torch.stack([w[f"e{e}.down"] for e in range(experts)]).to(DEV)
    logits = ops.linear_f32(x.to(DEV), w["router"].to(DEV))
    close(logits, x.double() @ wd["router"].T, torch.float32, "router logits are exact products")
    ids, weights = ops.router_choose(logits, w["correction"].to(DEV), top)
    close(ops.experts_forward(x.to(DEV), gate_up, down, ids, weights, "silu"), want, dtype)


# ------------------------------------------------------------------ the engine

LENGTHS = {"P": [1, 7, 33, 150, 64, 300], "Q": [2, 19, 45, 260, 128], "R": [3, 40, 17, 270, 96]}
# float32: every position, against the largest logit of its request (a recurrent state carries its rounding along:
# 1e-7 is typical, 1e-5 happens).  bfloat16: an expert chosen by a hair may be another one after rounding, which
# changes that token and, through the state, the few after it; so tokens whose router margin is small are left
# to the float32 run, nearly all of the rest must be within rounding, and the typical error must be small.
F32_TOL = dict(max=1e-4, mean=2e-5)
BF16_TOL = dict(max=6e-2, mean=1e-2, over=0.08, median=5e-3)
CLOSE_CALL = 0.015


def _requests(which, seed=0):
    return {f"r{k}": lt.ids(which, n, seed * 100 + k) for k, n in enumerate(LENGTHS[which])}


def _check(steps, results, requests, which, dtype, what):
    rows = replay.collect(steps, results)
    errors, over = [], []
    for rid, tokens in requests.items():
        want = lt.oracle(which, tokens)
        margin = lt.router_margin(which, tokens)
        scale = float(want.abs().max())
        assert len(rows[rid]) == len(tokens)
        for pos, got in sorted(rows[rid].items()):
            assert torch.isfinite(got).all(), f"{what} request {rid} position {pos}: not finite"
            diff = (got.double() - want[pos]).abs()
            worst, mean = float(diff.max()) / scale, float(diff.mean()) / scale
            if dtype == "float32":
                assert worst <= F32_TOL["max"] and mean <= F32_TOL["mean"], \
                    f"{what} request {rid} position {pos}: max {worst:.3e} mean {mean:.3e} of the largest logit"
                continue
            if margin is not None and float(margin[pos]) < CLOSE_CALL:
                continue
            errors.append(mean)
            if worst > BF16_TOL["max"] or mean > BF16_TOL["mean"]:
                over.append((rid, pos, worst, mean))
    if dtype == "bfloat16":
        assert len(errors) >= 0.5 * sum(len(t) for t in requests.values()), "too few tokens are judged"
        assert len(over) <= max(1, BF16_TOL["over"] * len(errors)), f"{what}: {len(over)} of {len(errors)} over: {over[:5]}"
        assert sorted(errors)[len(errors) // 2] <= BF16_TOL["median"], f"{what}: typical error {sorted(errors)[len(errors) // 2]:.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["P", "Q", "R"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_cuts_match_plain(which, cut, dtype):
    requests = _requests(which)
    steps = getattr(replay, cut)(requests)
    pages = -(-replay.peak_tokens(steps, 16) // 16)
    core = lt.core(which, dtype, gpu_ops(), DEV, num_pages=pages, page_size=16, graph_sizes=[1, 2, 4] if cut != "whole" else None)
    results = replay.run_in_process(core, steps)
    _check(steps, results, requests, which, dtype, f"{which}/{cut}/{dtype}")
    assert all(pool.num_free == pool.num_pages for pool in core.manager.pools)
    if cut == "tail":
        assert core.graphs is not None and core.graphs.replays >= 32, "single tokens replay captured graphs"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_small_pages_slots_used_again_and_long_decoding(dtype):
    """Pages of 4 tokens, two state slots for five requests, and 150 tokens decoded one by one across the
    attention kernel's chunk of 256 keys, every one of them compared."""
    requests = {"long": lt.ids("P", 330, 1), "b": lt.ids("P", 23, 2), "c": lt.ids("P", 50, 3), "d": lt.ids("P", 9, 4),
                "e": lt.ids("P", 31, 5)}
    steps = replay.mixed(requests, seed=6, max_live=2, decode_tail=150)
    pages = -(-replay.peak_tokens(steps, 4) // 4)
    core = lt.core("P", dtype, gpu_ops(), DEV, num_pages=pages, page_size=4, max_num_seqs=2, graph_sizes=[1, 2])
    results = replay.run_in_process(core, steps)
    _check(steps, results, requests, "P", dtype, f"P/page4/{dtype}")


def test_logits_do_not_depend_on_the_batch_or_the_cut():
    """float32: a request's logits alone, cut in portions, and beside others differ by rounding of sums only."""
    requests = _requests("R")
    runs = []
    for cut in ("whole", "portions", "mixed"):
        steps = getattr(replay, cut)(requests)
        core = lt.core("R", "float32", gpu_ops(), DEV, num_pages=80, page_size=16)
        runs.append(replay.collect(steps, replay.run_in_process(core, steps)))
    for rid in requests:
        for pos in runs[0][rid]:
            for other in runs[1:]:
                assert float((runs[0][rid][pos] - other[rid][pos]).abs().max()) <= 2e-5 * float(runs[0][rid][pos].abs().max())


@pytest.mark.parametrize("which,dtype", [("P", "fp32"), ("Q", "fp32"), ("R", "fp32"), ("R", "bf16")])
def test_greedy_generation_through_the_engine(which, dtype):
    from atom_amd import LLMEngine, SamplingParams

    llm = LLMEngine(lt.folder(which), dtype=dtype, ops=gpu_ops(), kv_cache_block_size=16, num_kvcache_blocks=64,
                    max_num_seqs=4, max_num_batched_tokens=64, max_model_len=512)
    prompts = [lt.ids(which, n, 70 + n) for n in (1, 9, 40, 130, 65)]
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
    for prompt, out in zip(prompts, outs):
        tokens = list(prompt)
        assert len(out["token_ids"]) == 10
        for token in out["token_ids"]:
            logits = lt.oracle(which, tokens)[-1]
            best = int(logits.argmax())
            slack = 0.0 if dtype == "fp32" else 0.06 * float(logits.abs().max())
            margin = lt.router_margin(which, tokens)
            sure = dtype == "fp32" or margin is None or float(margin[-1]) >= CLOSE_CALL
            assert token == best or float(logits[best] - logits[token]) <= slack or not sure
            tokens.append(token)
    assert all(p.num_free == p.num_pages for p in llm.core.manager.pools)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_program(dtype, tmp_path):
    requests = {k: v for k, v in list(_requests("Q").items())[:4]}
    steps = replay.mixed(requests, seed=2, max_live=3)
    results = replay.run_program(lt.folder("Q"), dtype, steps, str(tmp_path / "out"), replay.peak_tokens(steps, 64),
                                 lt.CONFIGS["Q"]["vocab"])
    _check(steps, results, requests, "Q", dtype, f"program/{dtype}")


def test_command_line():
    """``python -m atom_amd.examples.simple_inference`` on a Lotorax folder: the registry picks the design from
    config.json; greedy completions are the plain implementation's."""
    import random
    import re
    import subprocess
    import sys

    cmd = [sys.executable, "-m", "atom_amd.examples.simple_inference", "--model", lt.folder("Q"), "--temperature", "0",
           "--max-tokens", "6", "--block_size", "16", "--num-kvcache-blocks", "32", "--max-num-seqs", "4", "--dtype", "fp32",
           "--max-model-len", "256", "--seed", "3"]
    res = subprocess.run(cmd, cwd=replay.ROOT, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    assert res.stdout.count("Completion:") == 3 and res.stdout.count("finish_reason=max_tokens") == 3
    rng = random.Random(3)
    prompts = [[rng.randrange(lt.CONFIGS["Q"]["vocab"]) for _ in range(n)] for n in (5, 17, 33)]
    shown = [eval(m) for m in re.findall(r"Completion: (\[.*?\])", res.stdout)]
    for prompt, out in zip(prompts, shown):
        tokens = list(prompt)
        for token in out:
            assert token == int(lt.oracle("Q", tokens)[-1].argmax())
            tokens.append(token)
