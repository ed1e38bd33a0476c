"""Leduvik without a GPU: the plain implementation against itself (whole prompts against continuation, mechanisms
that must show, window edges, the first tokens), the configuration reader, the weights' names and the size only a
tensor's shape says, and the engine's bookkeeping (joint memory of mixers side by side, pages behind a window given
back, state slots used again, passes over repeated layers with memory of their own, batches) with plain stand-ins
for the kernels."""

import copy

import pytest
import torch

import leduvik_tiny as lt
import plain_leduvik as pl
import replay
from plain_kernels import PlainKernels
from atom_amd.config import ConfigError, build_model, model_config_from_dict
from atom_amd.config.model_config import LeduvikConfig
from atom_amd.engine.core import StepEntry, load_model
from atom_amd.weights.loader import expected_tensors

LENGTHS = {"A": [1, 7, 33, 70], "B": [2, 19, 45, 64], "C": [3, 52], "D": [1, 30, 66]}


def _requests(which, seed=0):
    return {f"r{k}": lt.ids(which, n, seed * 100 + k) for k, n in enumerate(LENGTHS[which])}


# ------------------------------------------------------------------ the plain implementation


@pytest.mark.parametrize("which", ["A", "B"])
def test_plain_whole_equals_continuation(which):
    tokens = lt.ids(which, 41, 5)
    full = lt.oracle(which, tokens)
    carried, rows = None, []
    for cut in [9, 1, 1, 2, 13, 1, 14]:
        at = sum(r.shape[0] for r in rows)
        logits, carried = pl.forward(lt.CONFIGS[which], lt.tensors(which), tokens[at:at + cut], carried=carried)
        rows.append(logits)
    assert float((torch.cat(rows) - full).abs().max()) < 1e-9


def test_plain_mechanisms_show():
    """Dropping or misplacing a mechanism's tensor or constant changes the logits."""
    tokens = lt.ids("A", 30, 2)
    base = lt.oracle("A", tokens)
    flip = lambda t: torch.flip(t, dims=[0])  # noqa: E731
    for name, change in [("pos", lambda t: t * 0), ("l0.mix.right.u", lambda t: t * 0), ("l0.mix.right.w0", flip),
                         ("l0.mix.right.mu.k", lambda t: t * 0), ("l0.mix.right.mu.w", lambda t: 1 - t),
                         ("l0.mix.right.w2", lambda t: t * 0), ("l0.mix.right.norm", flip), ("l0.mix.left.out", flip),
                         ("l0.mix.right.out", lambda t: t * 0), ("l1.mix.D", lambda t: t * 0), ("l1.mix.dt_bias", flip),
                         ("l1.mix.A_log", flip), ("l1.mix.conv.b", lambda t: t + 1),
                         ("l1.mix.conv", lambda t: torch.cat((t[:, :1] * 0, t[:, 1:]), 1)), ("l1.mix.norm", flip),
                         ("l2.mix.k", lambda t: torch.roll(t, 6, dims=0)), ("l1.norm1", flip)]:
        changed = dict(lt.tensors("A"))
        changed[name] = change(changed[name])
        other = pl.forward(lt.CONFIGS["A"], changed, tokens)[0]
        assert float((other - base).abs().max()) > 1e-3 * float(base.abs().max()), name
    for path, value in [(("logit_scale",), 1.0), (("loop", "times"), 2), (("loop", "stop"), 1),
                        (("layers", 2, "mixer", "mask", "size"), 8), (("layers", 2, "mixer", "scale"), 0.1),
                        (("layers", 0, "mixer", "left", "q_temp", "coef"), 0.0),
                        (("layers", 0, "mixer", "left", "q_temp", "every"), 8), (("layers", 1, "mixer", "norm_groups"), 1),
                        (("norm", "eps"), 1e-2)]:
        cfg = copy.deepcopy(lt.CONFIGS["A"])
        at = cfg
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        other = pl.forward(cfg, lt.tensors("A"), tokens)[0]
        assert float((other - base).abs().max()) > 1e-4 * float(base.abs().max()), path


def test_plain_window_holds_the_token_itself_and_the_ones_before():
    assert pl.may_see(20, 12, 9) and not pl.may_see(20, 11, 9) and pl.may_see(20, 20, 9) and not pl.may_see(20, 21, 9)
    assert pl.may_see(300, 0, None)
    # the attention layer alone on random rows: a change at position 4 moves positions 4 .. 12 and no other
    m = lt.CONFIGS["A"]["layers"][2]["mixer"]
    w = pl.sub(lt.tensors("A"), "l2.mix")
    h = torch.randn(21, 40, dtype=torch.float64, generator=torch.Generator().manual_seed(3))
    run = lambda rows: pl.attention_mixer(rows, torch.arange(21), w, m, 3e-5, unit_qk=True, window=9)[0]  # noqa: E731
    h2 = h.clone()
    h2[4] += 1.0
    moved = (run(h2) - run(h)).abs().amax(dim=1)
    assert float(moved[4:13].min()) > 1e-6 and float(moved[13:].max()) == 0 and float(moved[:4].max()) == 0


def test_plain_query_temperature_steps():
    t = pl.query_temperature(torch.tensor([0, 5, 6, 13, 14]), 0.25, 7)
    assert float(t[0]) == 1.0 and float(t[1]) == 1.0            # floor((p + 1) / 7) is 0 up to position 5
    assert float(t[2]) == pytest.approx(1 + 0.25 * 0.6931471805599453) and float(t[3]) > float(t[2])
    assert float(t[4]) == pytest.approx(1 + 0.25 * 1.0986122886681098)


def test_plain_first_token_has_zeros_before_it():
    """The time-mixing branch's first token mixes with zeros, the state-space mixer's convolution starts on zeros,
    and both states start at zero: a one-token request's mixers depend on nothing else."""
    w = pl.sub(lt.tensors("A"), "l0.mix.right")
    m = lt.CONFIGS["A"]["layers"][0]["mixer"]["right"]
    h = torch.randn(1, 40, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    out, (last, S) = pl.time_mix_mixer(h, w, m, 3e-5)
    mix_k = h * (1 - w["mu.k"])
    assert torch.allclose(S[0], torch.outer((mix_k @ w["k"].T)[0, :8], ((h * (1 - w["mu.v"])) @ w["v"].T)[0, :8]))
    assert torch.equal(last, h[0])


# ------------------------------------------------------------------ configuration and weights


def test_config_reads_every_size_and_round_trips():
    cfg = model_config_from_dict(lt.LEDU_A)
    assert isinstance(cfg, LeduvikConfig) and cfg.vocab_size == 101 and cfg.hidden_size == 40
    assert cfg.loop == (0, 2, 3) and cfg.logit_scale == 0.7 and cfg.norm_eps == 3e-5 and cfg.max_position_embeddings == 400
    assert model_config_from_dict(cfg.to_dict()) == cfg
    model = build_model(cfg)
    side, ssm, attn = (model.blocks[i].mixer for i in range(3))
    left, right = side.branches
    assert (left.num_heads, left.num_kv_heads, left.key_dim, left.value_dim, left.scale) == (4, 2, 10, 6, 0.4)
    assert left.temperature == (0.25, 7) and left.window is None and not left.unit_norm and left.padded_dim == 16
    assert (right.num_heads, right.head_dim, right.decay_rank) == (5, 8, None)
    assert (ssm.num_heads, ssm.value_dim, ssm.state_size, ssm.groups, ssm.conv_taps, ssm.norm_groups) == (4, 6, 5, 2, 2, 2)
    assert (attn.num_heads, attn.num_kv_heads, attn.key_dim, attn.value_dim, attn.window) == (6, 3, 6, 10, 9)
    assert attn.unit_norm and attn.temperature is None
    assert model.blocks[1].ffn is None and model.head.scale == 0.7 and model.embedding.max_positions == 400
    assert [(r.layer, r.enters) for r in model.order] == [(0, False), (1, False), (0, True), (1, False), (0, True),
                                                          (1, False), (2, False)]
    bare = build_model(model_config_from_dict(lt.LEDU_C))
    assert bare.join is None and [r.layer for r in bare.order] == [0, 1, 2]
    once = copy.deepcopy(lt.LEDU_B)
    once["loop"]["times"] = 1
    assert build_model(model_config_from_dict(once)).join is None


@pytest.mark.parametrize("which", ["A", "B", "C", "D"])
def test_names_and_shapes_are_the_designs(which):
    """The engine's list of checkpoint tensors, once the checkpoint's shapes have said the inner size of the decay's
    two products, is the design's list."""
    model, _ = load_model(lt.folder(which), dtype=torch.float32, device="cpu")
    names = {name: tuple(shape) for name, (shape, _) in expected_tensors(model).items()}
    assert names == {k: tuple(v) for k, v in lt.shapes(which).items()}
    for block in model.blocks:
        for branch in getattr(block.mixer, "branches", []):
            if hasattr(branch, "decay_rank"):
                assert branch.decay_rank == lt.RANKS[which]


def test_sizes_left_out_take_their_obvious_values():
    """No kv_heads: as many as heads; no vdim: the keys' size; no groups or norm_groups: one; a loop over no layers
    or of one pass repeats nothing."""
    raw = copy.deepcopy(lt.LEDU_B)
    full = model_config_from_dict(raw)
    del raw["layers"][0]["mixer"]["kv_heads"], raw["layers"][0]["mixer"]["vdim"], raw["layers"][1]["mixer"]["groups"]
    assert model_config_from_dict(raw).layers == full.layers
    raw["layers"][1]["mixer"].pop("norm_groups")
    assert model_config_from_dict(raw).layers[1]["mixer"]["norm_groups"] == 1
    for loop in ({"start": 2, "stop": 2, "times": 3}, {"start": 0, "stop": 3, "times": 1}):
        raw["loop"] = loop
        cfg = model_config_from_dict(raw)
        assert cfg.loop is None and [r.layer for r in build_model(cfg).order] == [0, 1, 2, 3]


def test_rank_without_a_checkpoint_must_be_named():
    with pytest.raises(ValueError, match="decay_rank"):
        expected_tensors(build_model(model_config_from_dict(lt.LEDU_A)))
    named = copy.deepcopy(lt.LEDU_A)
    named["layers"][0]["mixer"]["right"]["decay_rank"] = 3
    assert "l0.mix.right.w1" in expected_tensors(build_model(model_config_from_dict(named)))


@pytest.mark.parametrize("path,value", [(("layers", 0, "type"), "mamba"), (("layers", 0, "mixer", "left", "kv_heads"), 3),
                                        (("layers", 1, "mixer", "groups"), 3), (("layers", 1, "mixer", "norm_groups"), 5),
                                        (("layers", 2, "mixer", "mask", "size"), 0), (("norm", "eps"), None),
                                        (("layers", 0, "mixer", "left", "q_temp", "every"), 0), (("max_positions",), None),
                                        (("layers", 0, "mlp", "kind"), "moe"), (("loop", "stop"), 4),
                                        (("layers", 0, "mixer", "right", "dim"), 0)])
def test_config_refuses_what_does_not_fit(path, value):
    raw = copy.deepcopy(lt.LEDU_A)
    at = raw
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(ConfigError):
        model_config_from_dict(raw)


# ------------------------------------------------------------------ the engine's bookkeeping


@pytest.mark.parametrize("which", ["A", "B", "C", "D"])
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


def test_joint_memory_and_pages_behind_the_window():
    """Mixers side by side keep pages and a state; every pass over repeated layers has memory of its own; pages
    wholly behind a window go back to the pool while the request lives."""
    core = lt.core("A", "float32", PlainKernels(), "cpu", num_pages=12, page_size=8)
    assert {(g.window, g.chunk) for g in core.manager.groups} == {(9, None), (None, None)}
    bindings = core.storage.bindings
    assert len(bindings) == 7 and len({id(b) for b in bindings}) == 7
    sides = [b for b in bindings if hasattr(b, "parts")]
    assert len(sides) == 3 and all(b.parts[0].k_cache.shape[-1] == 16 and b.parts[1].state.shape[1] == 40 + 5 * 64 for b in sides)
    assert len(core.storage.state_tensors) == 6
    a = lt.ids("A", 60, 1)
    got = core.step([StepEntry("a", a[:50], [49])])
    windowed = [i for i, g in enumerate(core.manager.groups) if g.window == 9][0]
    table = core.manager.block_table("a", windowed)
    assert [p >= 0 for p in table] == [False] * 5 + [True, True]     # position 50 sees 42 on: page 5 on
    more = core.step([StepEntry("a", a[50:], list(range(10)))])
    want = lt.oracle("A", a)
    assert replay.first_bad({49: got[0]}, want, "float32") is None
    assert replay.first_bad({50 + i: more[i] for i in range(10)}, want, "float32") is None
    core.close("a")
    assert all(pool.num_free == pool.num_pages for pool in core.manager.pools)


def test_slot_reuse_starts_from_nothing():
    """A slot that is used again holds no state, no convolution inputs and no previous token's input."""
    core = lt.core("A", "float32", PlainKernels(), "cpu", num_pages=24, page_size=8, max_num_seqs=2)
    a, b, c = lt.ids("A", 30, 1), lt.ids("A", 12, 2), lt.ids("A", 21, 3)
    core.step([StepEntry("a", a[:20], []), StepEntry("b", b, [])])
    slot_b = core.manager.state_slot("b")
    assert all(float(t[slot_b].abs().max()) > 0 for t in core.storage.state_tensors)
    core.close("b")
    got = core.step([StepEntry("c", c, list(range(21))), StepEntry("a", a[20:], list(range(10)))])
    assert core.manager.state_slot("c") == slot_b
    assert replay.first_bad({i: got[i] for i in range(21)}, lt.oracle("A", c), "float32") is None
    assert replay.first_bad({20 + i: got[21 + i] for i in range(10)}, lt.oracle("A", a), "float32") is None


def test_positions_beyond_the_table_are_refused():
    core = lt.core("A", "float32", PlainKernels(), "cpu", num_pages=64, page_size=8)
    with pytest.raises(ValueError, match="positions"):
        core.step([StepEntry("a", lt.ids("A", 401, 1), [])])


def test_greedy_generation_through_the_engine():
    from atom_amd import LLMEngine, SamplingParams

    llm = LLMEngine(lt.folder("B"), dtype="fp32", ops=PlainKernels(), device="cpu", kv_cache_block_size=8,
                    num_kvcache_blocks=40, max_num_seqs=3, max_num_batched_tokens=16, max_model_len=128,
                    enforce_eager=True)
    prompts = [lt.ids("B", n, 60 + n) for n in (1, 9, 30, 17)]
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True))
    for prompt, out in zip(prompts, outs):
        tokens = list(prompt)
        for token in out["token_ids"]:
            assert token == int(lt.oracle("B", tokens)[-1].argmax())
            tokens.append(token)
    assert all(p.num_free == p.num_pages for p in llm.core.manager.pools)


def test_prefix_cache_stays_off_where_a_state_is_kept():
    from atom_amd.engine.core import build_core

    model, _ = load_model(lt.folder("A"), dtype=torch.float32, device="cpu")
    assert not build_core(model, PlainKernels(), dtype=torch.float32, device="cpu", num_pages=4, prefix_caching=True).prefix_caching
