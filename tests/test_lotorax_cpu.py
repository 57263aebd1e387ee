"""Lotorax without a GPU: the plain implementation against itself (whole prompts against token-by-token
continuation, mechanisms that must show), the configuration reader, the weights' names, and the engine's
bookkeeping (pages of latents, state slots, looped layers, batches) with plain stand-ins for the kernels."""

import copy
import math

import pytest
import torch

import lotorax_tiny as lt
import plain_lotorax as pl
import replay
from plain_kernels import PlainKernels
from atom_amd.config import ConfigError, LotoraxConfig, build_model, model_config_from_dict
from atom_amd.engine.core import StepEntry
from atom_amd.weights.loader import expected_tensors

LENGTHS = {"P": [1, 7, 33, 70], "Q": [2, 19, 45, 64], "R": [3, 40, 17]}


def _requests(which, seed=0):
    return {f"r{k}": lt.ids(which, n, seed * 100 + k) for k, n in enumerate(LENGTHS[which])}


# ------------------------------------------------------------------ the plain implementation


@pytest.mark.parametrize("which", ["P", "Q", "R"])
def test_plain_whole_equals_token_by_token(which):
    tokens = lt.ids(which, 26, 5)
    full = lt.oracle(which, tokens)
    carried, rows = None, []
    for cut in ([9, 1, 1, 2, 13] if which != "R" else [1] * 26):
        at = sum(r.shape[0] for r in rows)
        logits, carried = pl.forward(lt.CONFIGS[which], lt.tensors(which), tokens[at:at + cut], carried=carried)
        rows.append(logits)
    assert float((torch.cat(rows) - full).abs().max()) < 1e-9


def test_plain_rotation_is_relative_and_stretched():
    x = torch.randn(1, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(0))
    y = torch.randn(1, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    dot = lambda p, q, s: float((pl.rotate_pairs(x, torch.tensor([p]), 8, 100.0, s) *
                                 pl.rotate_pairs(y, torch.tensor([q]), 8, 100.0, s)).sum())  # noqa: E731
    assert abs(dot(5, 3, None) - dot(45, 43, None)) < 1e-9
    assert abs(dot(5, 3, lt.YARN) - dot(45, 43, lt.YARN)) < 1e-9
    f, mult = pl.yarn_frequencies(8, 100.0, lt.YARN)
    plain, _ = pl.yarn_frequencies(8, 100.0, None)
    assert mult == pytest.approx(0.1 * math.log(4.0) + 1)
    assert float(f[0]) == pytest.approx(float(plain[0])) and float(f[-1]) == pytest.approx(float(plain[-1]) / 4.0)
    # the pairs are neighbours: turning entry 0 moves entry 1, not entry 4
    e0 = torch.zeros(1, 8, dtype=torch.float64)
    e0[0, 0] = 1
    turned = pl.rotate_pairs(e0, torch.tensor([3]), 8, 100.0, None)
    assert abs(float(turned[0, 1])) > 0.1 and float(turned[0, 4]) == 0


def test_plain_mechanisms_show():
    """Dropping the sink, the gate, the correction, a convolution tap or the decay changes the logits."""
    tokens = lt.ids("P", 20, 2)
    base = lt.oracle("P", tokens)
    for name, change in [("l0.mix.sink", lambda t: t - 30), ("l0.mix.g", lambda t: t * 0), ("l1.mlp.correction", lambda t: -t),
                         ("l1.mix.k.conv", lambda t: torch.cat((t[:, :1] * 0, t[:, 1:]), 1)), ("l1.mix.A_log", lambda t: t - 20),
                         ("l1.norm1b.b", lambda t: t + 1), ("loop.in", lambda t: torch.cat((t[:, :48], t[:, 48:] * 0), 1))]:
        changed = dict(lt.tensors("P"))
        changed[name] = change(changed[name].float())
        other = pl.forward(lt.CONFIGS["P"], changed, tokens)[0]
        assert float((other - base).abs().max()) > 1e-3 * float(base.abs().max()), name


# ------------------------------------------------------------------ configuration and weights


def test_config_reads_every_size_and_round_trips():
    cfg = model_config_from_dict(lt.LOTO_P)
    assert isinstance(cfg, LotoraxConfig) and cfg.vocab_size == 131 and cfg.hidden_size == 48
    assert cfg.loop == (1, 3, 3) and cfg.norm_eps == 2e-5 and cfg.embedding_scale == 3.5
    assert model_config_from_dict(cfg.to_dict()) == cfg
    model = build_model(cfg)
    assert [(r.layer, r.enters) for r in model.order] == [(0, False)] + [(1, True), (2, False)] * 3
    mixer = model.blocks[0].mixer
    assert (mixer.num_heads, mixer.head_dim, mixer.rot_dim, mixer.value_dim, mixer.kv_rank) == (3, 8, 4, 12, 24)
    assert mixer.rope.scaling == (4.0, 64.0, 16.0, 2.0) and model.blocks[2].mixer.rope.scaling is None
    names = expected_tensors(model)
    assert names["l1.mix.v.conv"][0] == (48, 3) and names["l2.mlp.e3.down"][0] == (48, 24)
    assert names["loop.in"][0] == (48, 96) and names["l0.norm2b.b"][0] == (48,) and "head" in names
    plain = build_model(model_config_from_dict(lt.LOTO_Q))
    assert plain.join is None and "loop.in" not in expected_tensors(plain)
    assert plain.blocks[0].ffn is None and "l0.norm2" not in expected_tensors(plain)


@pytest.mark.parametrize("path,value", [(("layers", 0, "type"), "mamba"), (("layers", 1, "mixer", "kv_heads"), 3),
                                        (("layers", 2, "mlp", "router", "top"), 9), (("loop", "stop"), 7),
                                        (("layers", 0, "mixer", "rot", "dims"), 6), (("norm", "eps"), None)])
def test_config_refuses_what_does_not_fit(path, value):
    raw = copy.deepcopy(lt.LOTO_P)
    at = raw
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(ConfigError):
        model_config_from_dict(raw)


# ------------------------------------------------------------------ the engine's bookkeeping


@pytest.mark.parametrize("which", ["P", "Q", "R"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_cuts_match_plain(which, cut):
    requests = _requests(which)
    oracle = {rid: lt.oracle(which, tokens) for rid, tokens in requests.items()}
    steps = getattr(replay, cut)(requests, **({"last": 9} if cut == "tail" else {}))
    pages = -(-replay.peak_tokens(steps, 8) // 8)
    core = lt.core(which, "float32", PlainKernels(), "cpu", num_pages=pages, page_size=8)
    results = replay.run_in_process(core, steps)
    replay.check(steps, results, requests, oracle, "float32", f"{which}/{cut}")
    assert not core.manager.live_requests()
    assert all(pool.num_free == pool.num_pages for pool in core.manager.pools)


def test_memory_per_run_and_slot_reuse():
    """Every run of a looped layer has memory of its own; a slot that is used again starts from zero."""
    core = lt.core("P", "float32", PlainKernels(), "cpu", num_pages=24, page_size=8, max_num_seqs=2)
    assert len(core.storage.bindings) == 7 and len(core.storage.state_tensors) == 3
    assert len({b.state.data_ptr() for b in core.storage.bindings if hasattr(b, "state")}) == 3
    assert len({b.pages.data_ptr() for b in core.storage.bindings if hasattr(b, "pages")}) == 4
    m = core.model.blocks[1].mixer
    assert core.storage.state_tensors[0].shape == (2, (3 - 1) * (2 * 2 * 8 + 4 * 12) + 4 * 8 * 12) and m.conv_floats == 160
    a, b, c = lt.ids("P", 30, 1), lt.ids("P", 12, 2), lt.ids("P", 21, 3)
    core.step([StepEntry("a", a[:20], []), StepEntry("b", b, [])])
    slot_b = core.manager.state_slot("b")
    assert float(core.storage.state_tensors[0][slot_b].abs().max()) > 0
    core.close("b")
    got = core.step([StepEntry("c", c, list(range(21))), StepEntry("a", a[20:], list(range(10)))])
    assert core.manager.state_slot("c") == slot_b
    assert replay.first_bad({i: got[i] for i in range(21)}, lt.oracle("P", c), "float32") is None
    assert replay.first_bad({20 + i: got[21 + i] for i in range(10)}, lt.oracle("P", a), "float32") is None


def test_greedy_generation_through_the_engine():
    from atom_amd import LLMEngine, SamplingParams

    llm = LLMEngine(lt.folder("Q"), dtype="fp32", ops=PlainKernels(), device="cpu", kv_cache_block_size=8,
                    num_kvcache_blocks=40, max_num_seqs=3, max_num_batched_tokens=16, max_model_len=128,
                    enforce_eager=True)
    prompts = [lt.ids("Q", n, 60 + n) for n in (1, 9, 30, 17)]
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True))
    for prompt, out in zip(prompts, outs):
        tokens = list(prompt)
        for token in out["token_ids"]:
            assert token == int(lt.oracle("Q", tokens)[-1].argmax())
            tokens.append(token)
    assert all(p.num_free == p.num_pages for p in llm.core.manager.pools)
