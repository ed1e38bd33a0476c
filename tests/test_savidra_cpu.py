"""Savidra without a GPU: the plain implementation against itself (whole prompts against continuation, mechanisms
that must show, a sink and head mixing on weights made by hand, the first tokens), the configuration reader, the
weights' names and the sizes only a tensor's shape says, and the engine's bookkeeping (the shift's row, the carried
convolution inputs and the delta rule's state bound beside the pages of one layer, values handed from one layer to
another within a step, state slots and pages used again, batches) with plain stand-ins for the kernels."""

import copy
import math

import pytest
import torch

import plain_savidra as ps
import replay
import savidra_tiny as st
from plain_kernels import PlainKernels
from atom_amd.config import ConfigError, build_model, model_config_from_dict
from atom_amd.config.model_config import SavidraConfig
from atom_amd.engine.core import StepEntry, load_model
from atom_amd.weights.loader import expected_tensors

LENGTHS = {"A": [1, 7, 33, 70], "B": [2, 19, 45, 64], "C": [3, 52], "D": [1, 30, 66], "E": [1, 2, 40]}


def _requests(which, seed=0):
    return {f"r{k}": st.ids(which, n, seed * 100 + k) for k, n in enumerate(LENGTHS[which])}


# ------------------------------------------------------------------ the plain implementation


@pytest.mark.parametrize("which", ["A", "B", "D"])
def test_plain_whole_equals_continuation(which):
    tokens = st.ids(which, 41, 5)
    full = st.oracle(which, tokens)
    model = ps.PlainSavidra(st.CONFIGS[which], st.tensors(which))
    rows, at = [], 0
    for cut in [9, 1, 1, 2, 13, 1, 14]:
        rows.append(model.forward(tokens[at:at + cut]))
        at += cut
    assert float((torch.cat(rows) - full).abs().max()) < 1e-9


def test_plain_mechanisms_show():
    """Dropping or misplacing a mechanism's tensor or constant changes the logits."""
    tokens = st.ids("A", 30, 2)
    base = st.oracle("A", tokens)
    flip = lambda t: torch.flip(t, dims=[0])  # noqa: E731
    zero = lambda t: t * 0  # noqa: E731
    for name, change in [("l0.shift", zero), ("l1.shift", lambda t: 1 - t), ("l0.mix.sink", lambda t: t - 30), ("l0.mix.sink", flip),
                         ("l2.mix.vmix", zero), ("l0.mix.q.norm", flip), ("l0.mix.k.norm", flip),
                         ("l1.mix.left.talk", lambda t: torch.eye(t.shape[0], dtype=t.dtype)),
                         ("l1.mix.left.talk", lambda t: t.T.contiguous()), ("l1.mix.left.temp", flip),
                         ("l1.mix.left.q.b", zero), ("l1.mix.left.v.b", zero), ("l1.mix.left.o.b", zero),
                         ("l1.mix.left.k.conv", lambda t: torch.flip(t, dims=[1])),
                         ("l1.mix.left.v.conv", lambda t: torch.cat((t[:, :1] * 0, t[:, 1:]), 1)),
                         ("l1.mix.right.q.conv", lambda t: torch.flip(t, dims=[1])), ("l1.mix.right.dt_bias", flip),
                         ("l1.mix.right.A_log", flip), ("l1.mix.right.a2", zero), ("l1.mix.right.g2", zero),
                         ("l1.mix.right.b", zero), ("l1.mix.right.norm", flip), ("l0.norm1", zero), ("l0.norm2", flip),
                         ("final.norm", zero)]:
        changed = dict(st.tensors("A"))
        changed[name] = change(changed[name])
        other = ps.PlainSavidra(st.CONFIGS["A"], changed).forward(tokens)
        assert float((other - base).abs().max()) > 1e-3 * float(base.abs().max()), name
    for path, value in [(("postln_alpha",), 1.0), (("norm", "eps"), 1e-1), (("layers", 0, "mixer", "scale"), 0.1),
                        (("layers", 0, "mixer", "rot", "dims"), 4), (("layers", 0, "mixer", "rot", "base"), 10.0),
                        (("layers", 1, "mixer", "left", "rot", "scaling", "factor"), 1.0),
                        (("layers", 1, "mixer", "left_scale"), 0.0), (("layers", 1, "mixer", "right_scale"), 0.0),
                        (("layers", 2, "mixer", "v_mix"), False), (("layers", 0, "mixer", "v_mix"), False)]:
        cfg = copy.deepcopy(st.CONFIGS["A"])
        at = cfg
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        other = ps.PlainSavidra(cfg, st.tensors("A")).forward(tokens)
        assert float((other - base).abs().max()) > 1e-4 * float(base.abs().max()), path


def test_plain_sink_counts_once_and_has_no_value():
    """One key with score 0 and a sink of 0 share the denominator: the key's weight is a half; a sink far below
    every score changes nothing; a sink is not scaled."""
    q = torch.zeros(1, 2, 4, dtype=torch.float64)
    k = torch.zeros(1, 1, 4, dtype=torch.float64)
    at = torch.tensor([0])
    w = ps.softmax_weights(q, k, at, at, 0.5, sink=torch.tensor([0.0, -50.0], dtype=torch.float64))
    assert float(w[0, 0, 0]) == pytest.approx(0.5) and float(w[1, 0, 0]) == pytest.approx(1.0, abs=1e-12)
    q[0, 0, 0], k[0, 0, 0] = 2.0, 3.0          # score 6 * scale
    w = ps.softmax_weights(q, k, at, at, 0.5, sink=torch.tensor([3.0, 3.0], dtype=torch.float64))
    assert float(w[0, 0, 0]) == pytest.approx(0.5)           # exp(3) against exp(sink = 3): the sink was not scaled


def test_plain_mixed_heads_read_their_own_values():
    """Head 0 takes all of head 1's weights: it then looks where head 1 looks, but reads its own value head."""
    T = 5
    g = torch.Generator().manual_seed(4)
    q = torch.randn(T, 2, 3, dtype=torch.float64, generator=g)
    k = torch.randn(T, 2, 3, dtype=torch.float64, generator=g)
    v = torch.randn(T, 2, 2, dtype=torch.float64, generator=g)
    at = torch.arange(T)
    w = ps.softmax_weights(q, k, at, at, 1.0)
    swap = torch.tensor([[0.0, 1.0], [0.0, 1.0]], dtype=torch.float64)
    mixed = torch.einsum("hg,gij->hij", swap, w)
    out = ps.apply_weights(mixed, v, 2).view(T, 2, 2)
    assert torch.allclose(out[:, 0], w[1] @ v[:, 0]) and torch.allclose(out[:, 1], w[1] @ v[:, 1])


def test_plain_rotation_pairs_and_stretch():
    x = torch.zeros(1, 1, 6, dtype=torch.float64)
    x[0, 0, 0] = 1.0                                    # entry 0 pairs with entry 2 when four entries turn
    y = ps.rotate_half(x, torch.tensor([3]), 4, 100.0)
    assert float(y[0, 0, 0]) == pytest.approx(math.cos(3.0)) and float(y[0, 0, 2]) == pytest.approx(math.sin(3.0))
    assert float(y[0, 0, 1]) == 0 and float(y[0, 0, 4]) == 0
    y = ps.rotate_half(x, torch.tensor([3]), 4, 100.0, factor=6.0)
    assert float(y[0, 0, 0]) == pytest.approx(math.cos(0.5))
    x[0, 0, 0], x[0, 0, 1] = 0.0, 1.0                   # entry 1 pairs with entry 3 and turns at base^(-2/4)
    y = ps.rotate_half(x, torch.tensor([10]), 4, 100.0)
    assert float(y[0, 0, 3]) == pytest.approx(math.sin(1.0)) and float(y[0, 0, 5]) == 0


def test_plain_first_token_has_zeros_before_it():
    mu = torch.tensor([0.25, 1.0], dtype=torch.float64)
    x = torch.tensor([[4.0, 4.0], [8.0, 2.0]], dtype=torch.float64)
    h, kept = ps.token_shift(x, mu, torch.zeros(2, dtype=torch.float64))
    assert h.tolist() == [[3.0, 0.0], [7.0, 4.0]] and kept.tolist() == [8.0, 2.0]
    w = torch.tensor([[1.0, 10.0, 100.0]], dtype=torch.float64)
    y, kept = ps.short_conv(torch.tensor([[1.0], [2.0]], dtype=torch.float64), w, torch.zeros(2, 1, dtype=torch.float64))
    assert y.flatten().tolist() == [100.0, 210.0] and kept.flatten().tolist() == [1.0, 2.0]


def test_plain_delta_rule_reads_its_own_write():
    k = torch.tensor([[[1.0, 0.0]]], dtype=torch.float64)
    v = torch.tensor([[[5.0]]], dtype=torch.float64)
    one = torch.ones(1, 1, dtype=torch.float64)
    o, S = ps.delta_rule(k, k, v, one, torch.ones(1, 1, 2, dtype=torch.float64), torch.zeros(1, 2, 1, dtype=torch.float64))
    assert float(o[0, 0, 0]) == 5.0 and S.flatten().tolist() == [5.0, 0.0]
    # the decay acts on the rows of S that belong to key channels, before the write
    g = torch.tensor([[[0.5, 1.0]]], dtype=torch.float64)
    o, S2 = ps.delta_rule(k, k, v, one, g, S)
    assert float(o[0, 0, 0]) == pytest.approx(5.0) and float(S2[0, 0, 0]) == pytest.approx(5.0)   # 2.5 + 1 * (5 - 2.5)


# ------------------------------------------------------------------ configuration and weights


def test_config_reads_every_size_and_round_trips():
    cfg = model_config_from_dict(st.SAVI_A)
    assert isinstance(cfg, SavidraConfig) and cfg.vocab_size == 97 and cfg.hidden_size == 40
    assert cfg.postln_alpha == 1.5 and cfg.norm_eps == 3e-5
    assert model_config_from_dict(cfg.to_dict()) == cfg
    model = build_model(cfg)
    assert all(b.alpha == 1.5 for b in model.blocks) and model.blocks[1].ffn is None
    assert all(b.mixer_norm.one_plus and b.mixer_norm.eps == 3e-5 for b in model.blocks) and model.final_norm.one_plus
    first, side, third, fourth = (b.mixer.inner for b in model.blocks)
    assert (first.num_heads, first.num_kv_heads, first.head_dim, first.value_dim, first.scale) == (4, 2, 10, 6, 0.4)
    assert first.sink and not first.talk and first.value_mix == "source" and first.conv_taps is None
    assert (first.rope.dims, first.rope.base, first.rope.factor) == (6, 1000.0, 1.0)
    assert third.value_mix == "blend" and fourth.value_mix is None
    left, right = side.branches
    assert side.combine == "weighted_sum" and side.scales == [0.7, 1.2]
    assert (left.num_heads, left.num_kv_heads, left.head_dim, left.value_dim, left.conv_taps) == (6, 3, 6, 4, 2)
    assert left.talk and left.head_temperature and left.qkv_bias and left.out_bias and not left.sink
    assert left.rope.factor == 4.0
    assert (right.num_heads, right.num_kv_heads, right.head_dim, right.value_dim, right.conv_taps) == (4, 2, 5, 7, 3)
    assert right.decay == "channel" and right.gate_activation == "sigmoid"
    # the first layer that blends values is the source wherever it stands
    later = build_model(model_config_from_dict(st.SAVI_B))
    assert [b.mixer.inner.value_mix for b in later.blocks if hasattr(b.mixer.inner, "value_mix")] == ["source", "blend"]


@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E"])
def test_names_and_shapes_are_the_designs(which):
    model, _ = load_model(st.folder(which), dtype=torch.float32, device="cpu")
    names = {name: tuple(shape) for name, (shape, _) in expected_tensors(model).items()}
    assert names == {k: tuple(v) for k, v in st.shapes(which).items()}
    for block in model.blocks:
        for branch in getattr(block.mixer.inner, "branches", []):
            if hasattr(branch, "decay_rank"):
                assert (branch.decay_rank, branch.gate_rank) == st.RANKS[which]


def test_sizes_left_out_take_their_obvious_values():
    raw = copy.deepcopy(st.SAVI_B)
    full = model_config_from_dict(raw)
    del raw["layers"][2]["mixer"]["left"]["kv_heads"], raw["layers"][2]["mixer"]["left"]["vdim"]
    del raw["layers"][0]["mixer"]["right"]["kv_heads"]
    assert model_config_from_dict(raw).layers == full.layers
    del raw["postln_alpha"]
    assert model_config_from_dict(raw).postln_alpha == 1.0


def test_ranks_without_a_checkpoint_must_be_named():
    with pytest.raises(ValueError, match="rank"):
        expected_tensors(build_model(model_config_from_dict(st.SAVI_A)))
    named = copy.deepcopy(st.SAVI_A)
    named["layers"][1]["mixer"]["right"].update(decay_rank=3, gate_rank=5)
    assert "l1.mix.right.a1" in expected_tensors(build_model(model_config_from_dict(named)))


@pytest.mark.parametrize("path,value", [(("layers", 0, "type"), "mamba"), (("layers", 1, "mixer", "left", "kv_heads"), 4),
                                        (("layers", 0, "mixer", "rot", "dims"), 5), (("layers", 0, "mixer", "rot", "dims"), 12),
                                        (("layers", 1, "mixer", "left", "rot", "scaling", "factor"), 0.0),
                                        (("norm", "eps"), None), (("layers", 0, "mlp", "kind"), "moe"),
                                        (("layers", 1, "mixer", "right", "dim"), 0), (("layers", 1, "mixer", "right_scale"), None),
                                        (("layers", 1, "mixer", "right", "conv"), 0), (("layers", 0, "mixer", "scale"), None),
                                        (("layers", 2, "mixer", "vdim"), 5)])
def test_config_refuses_what_does_not_fit(path, value):
    raw = copy.deepcopy(st.SAVI_A)
    at = raw
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(ConfigError):
        model_config_from_dict(raw)


# ------------------------------------------------------------------ the engine's bookkeeping


def test_a_second_norm_without_feed_forward_and_single_taps():
    """A checkpoint that holds ``norm2`` for a layer without feed-forward gets ``x <- norm2(alpha x)`` there; without
    the tensor the step is left out.  Convolutions of one tap carry nothing."""
    model, _ = load_model(st.folder("E"), dtype=torch.float32, device="cpu")
    assert model.blocks[1].ffn is None and model.blocks[1].ffn_norm is not None
    assert "l1.norm2" in expected_tensors(model)
    assert build_model(model_config_from_dict(st.SAVI_E)).blocks[1].ffn_norm is None
    tokens = st.ids("E", 20, 1)
    without = {k: v for k, v in st.tensors("E").items() if k != "l1.norm2"}
    other = ps.PlainSavidra(st.CONFIGS["E"], without).forward(tokens)
    assert float((other - st.oracle("E", tokens)).abs().max()) > 1e-3


@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_cuts_match_plain(which, cut):
    requests = _requests(which)
    oracle = {rid: st.oracle(which, tokens) for rid, tokens in requests.items()}
    steps = getattr(replay, cut)(requests, **({"last": 9} if cut == "tail" else {}))
    pages = -(-replay.peak_tokens(steps, 8) // 8)
    core = st.core(which, "float32", PlainKernels(), "cpu", num_pages=pages, page_size=8)
    results = replay.run_in_process(core, steps)
    replay.check(steps, results, requests, oracle, "float32", f"{which}/{cut}")
    assert not core.manager.live_requests()
    assert all(pool.num_free == pool.num_pages for pool in core.manager.pools)


def test_memory_of_a_layer_is_bound_together():
    """A layer of mixers side by side keeps the shift's row, pages of keys and values of different sizes, the carried
    convolution inputs of the attention branch and the delta branch's row; all attention layers share block tables."""
    core = st.core("A", "float32", PlainKernels(), "cpu", num_pages=9, page_size=8, max_num_seqs=3)
    assert len(core.plan.groups) == 1 and core.plan.run_group == [0, 0, 0, 0]
    shift, inner = core.storage.bindings[1].parts
    assert tuple(shift.state.shape) == (3, 40)
    left, right = inner.parts
    pages, carried = left.parts
    assert tuple(pages.k_cache.shape) == (9, 3, 8, 6) and tuple(pages.v_cache.shape) == (9, 3, 4, 8)
    assert tuple(carried.state.shape) == (3, (2 - 1) * (6 * 6 + 3 * 6 + 3 * 4))
    assert tuple(right.state.shape) == (3, (3 - 1) * (2 * 2 * 5 + 4 * 7) + 4 * 5 * 7)
    plain = core.storage.bindings[0].parts[1]
    assert tuple(plain.k_cache.shape) == (9, 2, 8, 10) and tuple(plain.v_cache.shape) == (9, 2, 6, 8)


def test_slots_and_pages_used_again_start_clean():
    """A request that takes over the slot and the pages of a finished one sees nothing of it: not its shift row, not
    its convolution inputs, not its state, not its keys."""
    core = st.core("B", "float32", PlainKernels(), "cpu", num_pages=10, page_size=8, max_num_seqs=1)
    first, second = st.ids("B", 37, 1), st.ids("B", 29, 2)
    for rid, tokens in (("x", first), ("y", second), ("z", first)):
        got = core.step([StepEntry(rid, tokens[:11], list(range(11)))])
        got = torch.cat((got, core.step([StepEntry(rid, tokens[11:], list(range(len(tokens) - 11)))])))
        core.close(rid)
        want = st.oracle("B", tokens)
        assert float((got.double() - want).abs().max()) < 3e-5 * float(want.abs().max()), rid


def test_batches_of_unequal_requests_match_each_alone():
    core = st.core("A", "float32", PlainKernels(), "cpu", num_pages=40, page_size=8, max_num_seqs=4)
    reqs = {"a": st.ids("A", 50, 7), "b": st.ids("A", 3, 8), "c": st.ids("A", 21, 9)}
    core.step([StepEntry("a", reqs["a"][:40], []), StepEntry("c", reqs["c"][:20], [])])
    got = core.step([StepEntry("c", reqs["c"][20:], [0]), StepEntry("b", reqs["b"], [0, 1, 2]),
                     StepEntry("a", reqs["a"][40:], list(range(10)))]).double()
    want = torch.cat((st.oracle("A", reqs["c"])[20:], st.oracle("A", reqs["b"]), st.oracle("A", reqs["a"])[40:]))
    assert float((got - want).abs().max()) < 3e-5 * float(want.abs().max())
