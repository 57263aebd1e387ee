"""Ralitar without a GPU: the plain implementation against itself (whole prompts against continuation, mechanisms
that must show, chunk edges), the configuration reader, the weights' names and the sizes only a tensor's shape
says, and the engine's bookkeeping (pages of chunked attention given back, state slots with the previous token,
batches) with plain stand-ins for the kernels."""

import copy

import pytest
import torch

import plain_ralitar as pr
import ralitar_tiny as rt
import replay
from plain_kernels import PlainKernels
from atom_amd.config import ConfigError, RalitarConfig, build_model, model_config_from_dict
from atom_amd.engine.core import StepEntry, load_model
from atom_amd.weights.loader import expected_tensors

LENGTHS = {"U": [1, 7, 33, 70], "V": [2, 19, 45, 64], "W": [3, 52]}


def _requests(which, seed=0):
    return {f"r{k}": rt.ids(which, n, seed * 100 + k) for k, n in enumerate(LENGTHS[which])}


# ------------------------------------------------------------------ the plain implementation


@pytest.mark.parametrize("which", ["U", "V"])
def test_plain_whole_equals_continuation(which):
    tokens = rt.ids(which, 41, 5)
    full = rt.oracle(which, tokens)
    carried, rows = None, []
    for cut in [9, 1, 1, 2, 13, 1, 14]:
        at = sum(r.shape[0] for r in rows)
        logits, carried = pr.forward(rt.CONFIGS[which], rt.tensors(which), tokens[at:at + cut], carried=carried)
        rows.append(logits)
    assert float((torch.cat(rows) - full).abs().max()) < 1e-9


def test_plain_mechanisms_show():
    """Dropping or misplacing a mechanism's tensor changes the logits."""
    tokens = rt.ids("U", 30, 2)
    base = rt.oracle("U", tokens)
    flip = lambda t: torch.flip(t, dims=[0])  # noqa: E731
    for name, change in [("bigram", lambda t: t * 0), ("side.embed", lambda t: torch.roll(t, 5, dims=1)),
                         ("l0.mix.dt_bias", flip), ("l0.mix.a2", lambda t: t * 0), ("l0.mix.g2", lambda t: -t),
                         ("l0.mix.k.conv", lambda t: torch.cat((t[:, :1] * 0, t[:, 1:]), 1)),
                         ("l1.mix.q.norm", flip), ("l1.mix.k.b", lambda t: t * 0), ("l1.mix.g", lambda t: t * 0),
                         ("l2.mix.lam", lambda t: t + 3), ("l2.mix.conv.b", lambda t: t + 1),
                         ("l2.mix.ri.b", lambda t: t - 4), ("l2.side.norm", lambda t: t * 0), ("l1.norm1", flip)]:
        changed = dict(rt.tensors("U"))
        changed[name] = change(changed[name].float())
        other = pr.forward(rt.CONFIGS["U"], changed, tokens)[0]
        assert float((other - base).abs().max()) > 1e-3 * float(base.abs().max()), name
    for key, value in [("softcap", 0.5), ("scale", 0.1)]:
        cfg = copy.deepcopy(rt.CONFIGS["U"])
        cfg["layers"][1]["mixer"][key] = value
        other = pr.forward(cfg, rt.tensors("U"), tokens)[0]
        assert float((other - base).abs().max()) > 1e-3 * float(base.abs().max()), key


def test_plain_chunks_are_counted_from_position_zero():
    """A query sees its own chunk only: the first position of a chunk sees itself alone, the last sees all of it."""
    assert pr.visible(13, 7, 7) and not pr.visible(14, 13, 7) and pr.visible(14, 14, 7) and not pr.visible(6, 7, 7)
    # a change of the token at the last position of a chunk moves the attention layer's output there and nowhere in
    # the next chunk (the layer alone, its input rows drawn at random)
    m = rt.CONFIGS["U"]["layers"][1]["mixer"]
    w = pr.sub({k: v.double() for k, v in rt.tensors("U").items()}, "l1.mix.")
    g = torch.Generator().manual_seed(3)
    h = torch.randn(21, 40, dtype=torch.float64, generator=g)
    base = pr.chunk_attention_mixer(h, torch.arange(21), w, m, 2e-5)[0]
    h2 = h.clone()
    h2[13] += 1.0
    moved = (pr.chunk_attention_mixer(h2, torch.arange(21), w, m, 2e-5)[0] - base).abs().amax(dim=1)
    assert float(moved[13]) > 1e-3 and float(moved[14:].max()) == 0 and float(moved[:13].max()) == 0


def test_plain_bands_of_frequencies():
    f = pr.banded_frequencies(6, 300.0, rt.BANDS)
    plain = pr.banded_frequencies(6, 300.0, None)
    assert float(f[0]) == pytest.approx(float(plain[0]))                 # short waves turn as they did
    assert float(f[2]) == pytest.approx(float(plain[2]) / 8.0)           # long waves eight times slower
    assert float(plain[1]) / 8.0 < float(f[1]) < float(plain[1])         # between: a mixture
    x = torch.zeros(1, 1, 10, dtype=torch.float64)
    x[0, 0, 0] = 1
    turned = pr.rotate_pairs(x, torch.tensor([3]), f)
    assert abs(float(turned[0, 0, 1])) > 0.1 and float(turned[0, 0, 5]) == 0 and float(turned[0, 0, 6]) == 0


def test_plain_first_token_takes_the_last_pair_row():
    bigram = rt.CONFIGS["U"]["embedding"]["bigram"]
    assert pr.bigram_rows([4, 9, 9], None, bigram) == [53, (4 * 31 + 9 * 5) % 53, (9 * 31 + 9 * 5) % 53]
    assert pr.bigram_rows([9], 4, bigram) == [(4 * 31 + 9 * 5) % 53]


# ------------------------------------------------------------------ configuration and weights


def test_config_reads_every_size_and_round_trips():
    cfg = model_config_from_dict(rt.RALI_U)
    assert isinstance(cfg, RalitarConfig) and cfg.vocab_size == 97 and cfg.hidden_size == 40
    assert cfg.bigram == (53, 31, 5) and cfg.side_dim == 5 and cfg.norm_eps == 2e-5
    assert model_config_from_dict(cfg.to_dict()) == cfg
    model = build_model(cfg)
    delta, attn, rec = (model.blocks[i].mixer for i in range(3))
    assert (delta.num_heads, delta.num_kv_heads, delta.head_dim, delta.value_dim, delta.conv_taps) == (4, 2, 8, 12, 3)
    assert delta.decay == "channel" and delta.gate_activation == "sigmoid" and delta.decay_rank is None
    assert (attn.num_heads, attn.num_kv_heads, attn.head_dim, attn.chunk, attn.softcap, attn.scale) == (6, 2, 10, 7, 3.0, 0.6)
    assert attn.rope.dims == 6 and attn.rope.scaling == (8.0, 1.0, 4.0, 64.0)
    assert (rec.width, rec.blocks, rec.conv_taps) == (24, 3, 2)
    assert model.blocks[1].ffn is None and model.blocks[0].side.layer == 0 and model.blocks[2].side.layer == 2
    bare = build_model(model_config_from_dict(rt.RALI_W))
    assert bare.blocks[0].side is None and not bare.tables and bare.embedding.cache_need() is None
    assert bare.blocks[3].mixer.softcap is None and bare.blocks[3].mixer.rope.scaling is None


@pytest.mark.parametrize("which", ["U", "V", "W"])
def test_names_and_shapes_are_the_designs(which):
    """The engine's list of checkpoint tensors, once the checkpoint's shapes have said the inner sizes of the
    low-rank projections, is the design's list."""
    model, _ = load_model(rt.folder(which), dtype=torch.float32, device="cpu")
    names = {name: tuple(shape) for name, (shape, _) in expected_tensors(model).items()}
    assert names == {k: tuple(v) for k, v in rt.shapes(which).items()}
    for block in model.blocks:
        if hasattr(block.mixer, "decay_rank"):
            assert (block.mixer.decay_rank, block.mixer.gate_rank) == (rt.RANKS[which]["a1"], rt.RANKS[which]["g1"])


def test_rank_without_a_checkpoint_must_be_named():
    model = build_model(model_config_from_dict(rt.RALI_U))
    with pytest.raises(ValueError, match="decay_rank|gate_rank"):
        expected_tensors(model)


@pytest.mark.parametrize("path,value", [(("layers", 0, "type"), "mamba"), (("layers", 0, "mixer", "kv_heads"), 3),
                                        (("layers", 1, "mixer", "vdim"), 12), (("layers", 1, "mixer", "rot", "dims"), 5),
                                        (("layers", 2, "mixer", "blocks"), 5), (("norm", "eps"), None),
                                        (("layers", 1, "mixer", "mask", "size"), 0), (("token_side", "dim"), -1),
                                        (("layers", 0, "mlp", "kind"), "moe")])
def test_config_refuses_what_does_not_fit(path, value):
    raw = copy.deepcopy(rt.RALI_U)
    at = raw
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(ConfigError):
        model_config_from_dict(raw)


# ------------------------------------------------------------------ the engine's bookkeeping


@pytest.mark.parametrize("which", ["U", "V", "W"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_cuts_match_plain(which, cut):
    requests = _requests(which)
    oracle = {rid: rt.oracle(which, tokens) for rid, tokens in requests.items()}
    steps = getattr(replay, cut)(requests, **({"last": 9} if cut == "tail" else {}))
    pages = -(-replay.peak_tokens(steps, 8) // 8)
    core = rt.core(which, "float32", PlainKernels(), "cpu", num_pages=pages, page_size=8)
    results = replay.run_in_process(core, steps)
    replay.check(steps, results, requests, oracle, "float32", f"{which}/{cut}")
    assert not core.manager.live_requests()
    assert all(pool.num_free == pool.num_pages for pool in core.manager.pools)


def test_pages_behind_the_chunk_go_back():
    """Runs with the same chunk share block tables; a page wholly before the chunk of the next position is free again."""
    core = rt.core("V", "float32", PlainKernels(), "cpu", num_pages=12, page_size=8)
    groups = core.manager.groups
    assert sorted((g.window, g.chunk) for g in groups) == [(None, 16), (None, 40)]
    a = rt.ids("V", 90, 1)
    got = core.step([StepEntry("a", a[:50], [49])])
    by_chunk = {g.chunk: i for i, g in enumerate(groups)}
    table16, table40 = (core.manager.block_table("a", by_chunk[c]) for c in (16, 40))
    assert [p >= 0 for p in table16] == [False] * 6 + [True]          # position 50 begins at 48: page 6 on
    assert [p >= 0 for p in table40] == [False] * 5 + [True, True]    # its chunk of 40 begins at 40: page 5 on
    more = core.step([StepEntry("a", a[50:], list(range(40)))])
    want = rt.oracle("V", a)
    assert replay.first_bad({49: got[0]}, want, "float32") is None
    assert replay.first_bad({50 + i: more[i] for i in range(40)}, want, "float32") is None
    core.close("a")
    assert all(pool.num_free == pool.num_pages for pool in core.manager.pools)


def test_slot_reuse_starts_from_nothing():
    """A slot that is used again holds no state, no convolution inputs and no previous token."""
    core = rt.core("U", "float32", PlainKernels(), "cpu", num_pages=24, page_size=8, max_num_seqs=2)
    assert core.storage.embedding_binding.state.shape == (2, 1)
    a, b, c = rt.ids("U", 30, 1), rt.ids("U", 12, 2), rt.ids("U", 21, 3)
    core.step([StepEntry("a", a[:20], []), StepEntry("b", b, [])])
    slot_b = core.manager.state_slot("b")
    assert int(core.storage.embedding_binding.state[slot_b, 0]) == b[-1] + 1
    assert all(float(t[slot_b].abs().max()) > 0 for t in core.storage.state_tensors)
    core.close("b")
    got = core.step([StepEntry("c", c, list(range(21))), StepEntry("a", a[20:], list(range(10)))])
    assert core.manager.state_slot("c") == slot_b
    assert replay.first_bad({i: got[i] for i in range(21)}, rt.oracle("U", c), "float32") is None
    assert replay.first_bad({20 + i: got[21 + i] for i in range(10)}, rt.oracle("U", a), "float32") is None


def test_greedy_generation_through_the_engine():
    from atom_amd import LLMEngine, SamplingParams

    llm = LLMEngine(rt.folder("V"), dtype="fp32", ops=PlainKernels(), device="cpu", kv_cache_block_size=8,
                    num_kvcache_blocks=40, max_num_seqs=3, max_num_batched_tokens=16, max_model_len=128,
                    enforce_eager=True)
    prompts = [rt.ids("V", n, 60 + n) for n in (1, 9, 30, 17)]
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True))
    for prompt, out in zip(prompts, outs):
        tokens = list(prompt)
        for token in out["token_ids"]:
            assert token == int(rt.oracle("V", tokens)[-1].argmax())
            tokens.append(token)
    assert all(p.num_free == p.num_pages for p in llm.core.manager.pools)


def test_prefix_cache_stays_off_where_the_embedding_keeps_a_token():
    """A request that took over cached pages would start without its previous token: the prefix cache is on only
    where nothing but pages is kept, and the pair embedding keeps a token per request."""
    import torch
    from atom_amd.engine.core import build_core

    raw = copy.deepcopy(rt.RALI_W)
    raw["layers"] = [layer for layer in raw["layers"] if layer["type"] == "attention"]
    for layer in raw["layers"]:
        layer["mixer"].pop("mask")
    bare = build_model(model_config_from_dict(raw))
    assert build_core(bare, PlainKernels(), dtype=torch.float32, device="cpu", num_pages=4, prefix_caching=True).prefix_caching
    raw["embedding"] = {"bigram": {"buckets": 7, "mul_prev": 3, "mul_cur": 5}}
    paired = build_model(model_config_from_dict(raw))
    assert not build_core(paired, PlainKernels(), dtype=torch.float32, device="cpu", num_pages=4, prefix_caching=True).prefix_caching
