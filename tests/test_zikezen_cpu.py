"""Zikezen on the CPU: the config reader and the plan it gives, the tensors the parts declare, what the layers
keep in the cache, and the plain implementation pinned by closed forms and by invariants (so that the oracle
the GPU tests compare with is itself checked)."""

import copy
import math

import pytest
import torch

import paged_attention_engine_amd as pae
from paged_attention_engine_amd.config import ConfigError
from tests import zikezen_models as M
from tests.plain import zikezen_plain as plain


# ----------------------------------------------------------------------------- configuration


def test_the_reader_is_chosen_by_the_architecture_key_and_round_trips():
    for cfg in M.CONFIGS.values():
        typed = pae.read_config_dict(cfg)
        assert type(typed).__name__ == "ZikezenConfig"
        assert pae.read_config_dict(typed.to_json_dict()) == typed


def test_every_size_and_constant_comes_from_the_config():
    plan = pae.read_config_dict(M.P).plan()
    assert (plan.hidden_size, plan.vocab_size, plan.head_name, plan.embedding_name) == (64, 300, "head", "embed")
    assert (plan.position_table_name, plan.max_positions, plan.embedding_scale, plan.logit_softcap) == ("pos", 256, 0.7, 20.0)
    # layers 1 and 2 twice; the embedding's output joins again before the second pass and nowhere else
    assert [(e.layer, e.add_embedding) for e in plan.schedule] == [(0, False), (1, False), (2, False), (1, True), (2, False), (3, False)]
    first, second, third, fourth = plan.layers
    assert all(layer.arrangement == "sandwich" for layer in plan.layers)
    for norm, name in ((first.mixer_norm, "norm1"), (first.mixer_out_norm, "norm1b"), (first.feed_forward_norm, "norm2"),
                       (first.feed_forward_out_norm, "norm2b"), (plan.final_norm, "final.norm")):
        assert (norm.weight_name, norm.eps, norm.weight_offset, norm.size) == (name, 2e-6, 0.0, 64)
    side = first.mixer
    assert (side.kind, side.left_scale, side.right_scale) == ("side_by_side", 0.7, 1.2)
    a = side.left
    assert (a.kind, a.num_heads, a.num_kv_heads, a.head_dim, a.v_dim, a.scale, a.window, a.qkv_bias, a.bias_suffix) == (
        "attention", 4, 2, 16, 24, 0.3, 11, True, ".b")
    assert (a.qk_norm, a.qk_norm_eps, a.q_norm_name, a.k_norm_name, a.fixed_sink, a.sinks) == ("per_head", 2e-6, "q.norm", "k.norm", 0.0, False)
    assert (a.position.kind, a.position.rotary_dim, a.position.theta) == ("interleaved_rope", 8, 500.0)
    assert (a.position.ramp.factor, a.position.ramp.low, a.position.ramp.high, a.position.ramp.original) == (8.0, 1.0, 4.0, 64.0)
    assert second.mixer.left.position.ramp is None and second.mixer.left.position.rotary_dim == 16
    g = side.right
    assert (g.kind, g.num_heads, g.key_dim, g.value_dim, g.decay_rank, g.decay_temperature, g.norm_eps, g.gate_activation) == (
        "gated_linear_attention", 2, 16, 24, 8, 4.0, 2e-6, "silu")
    d = first.feed_forward
    assert (d.kind, d.intermediate_size, d.activation, d.gate_name, d.weight_suffix) == ("swiglu", 40, "silu", "gate", "")
    e = second.feed_forward
    assert (e.kind, e.intermediate_size, e.num_experts, e.top, e.groups, e.groups_kept, e.route_scale, e.choice_bias_name) == (
        "experts", 24, 6, 2, 1, 1, 1.0, "correction")
    assert third.feed_forward is None and third.feed_forward_norm is None and third.feed_forward_out_norm is None
    t = third.token_side
    assert (t.table_name, t.table_width, t.first_column, t.dim, t.vocab_size, t.activation, t.eps) == ("side.embed", 32, 16, 8, 300, "gelu_tanh", 2e-6)
    # a checkpoint may hold the norms of a feed-forward that the layer does not have
    assert set(plan.optional_names) == {"l2.norm2", "l2.norm2b"}
    # no mask: every earlier key; no rotation: none; no table, no cap, no loop, no scale: none
    q = pae.read_config_dict(M.Q).plan()
    assert q.layers[2].mixer.left.window is None and q.layers[2].mixer.left.position is None
    assert q.layers[0].token_side is None and q.logit_softcap is None and q.embedding_scale == 1.0
    assert [(e.layer, e.add_embedding) for e in q.schedule] == [(0, False), (1, False), (0, True), (1, False), (0, True), (1, False), (2, False)]
    assert [(e.layer, e.add_embedding) for e in pae.read_config_dict(M.S).plan().schedule] == [(0, False), (1, False)]


def test_the_narrow_products_width_comes_from_the_tensors_shapes(tmp_path):
    """A config.json as the design writes it names no width for the decay's narrow products: the checkpoint's shapes do."""
    import json
    import os
    folder = M.make_folder(tmp_path, "P")
    with open(os.path.join(folder, "config.json")) as handle:
        cfg = json.load(handle)
    for layer in cfg["layers"]:
        layer["mixer"]["right"].pop("decay_rank", None)
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(cfg, handle)
    typed = pae.read_config(folder)
    assert [layer.decay_rank for layer in typed.layers] == [8, 4, 5, 8]
    assert typed == pae.read_config_dict(M.P)
    with pytest.raises(ConfigError, match="narrow product"):
        pae.read_config_dict(cfg)


def test_declared_tensors_carry_the_designs_names_and_shapes():
    shapes = pae.expected_tensors(pae.read_config_dict(M.P).plan())
    assert shapes["embed"] == (300, 64) and shapes["pos"] == (256, 64) and shapes["head"] == (300, 64)
    assert shapes["side.embed"] == (300, 32) and tuple(shapes["final.norm"]) == (64,)
    for name in ("norm1", "norm1b", "norm2", "norm2b"):
        assert tuple(shapes[f"l0.{name}"]) == (64,)
    assert "l2.norm2" not in shapes and "l2.norm2b" not in shapes and tuple(shapes["l2.norm1b"]) == (64,)
    assert shapes["l0.mix.left.q"] == (64, 64) and shapes["l0.mix.left.k"] == (32, 64) and shapes["l0.mix.left.v"] == (48, 64)
    assert shapes["l0.mix.left.q.b"] == (64,) and shapes["l0.mix.left.v.b"] == (48,) and shapes["l0.mix.left.o"] == (64, 96)
    assert tuple(shapes["l0.mix.left.q.norm"]) == (16,) and tuple(shapes["l0.mix.left.k.norm"]) == (16,)
    assert shapes["l0.mix.right.q"] == (32, 64) and shapes["l0.mix.right.k"] == (32, 64) and shapes["l0.mix.right.v"] == (48, 64)
    assert shapes["l0.mix.right.g"] == (48, 64) and shapes["l0.mix.right.o"] == (64, 48) and tuple(shapes["l0.mix.right.norm"]) == (24,)
    assert shapes["l0.mix.right.a1"] == (8, 64) and shapes["l0.mix.right.a2"] == (32, 8) and shapes["l0.mix.right.a2.b"] == (32,)
    assert shapes["l0.mlp.gate"] == (40, 64) and shapes["l0.mlp.up"] == (40, 64) and shapes["l0.mlp.down"] == (64, 40)
    assert shapes["l1.mlp.router"] == (6, 64) and shapes["l1.mlp.correction"] == (6,)
    assert shapes["l1.mlp.e5.gate"] == (24, 64) and shapes["l1.mlp.e0.down"] == (64, 24) and "l1.mlp.gate" not in shapes
    assert shapes["l2.side.gate"] == (8, 64) and shapes["l2.side.proj"] == (64, 8) and tuple(shapes["l2.side.norm"]) == (64,)
    assert not any(name.startswith("l2.mlp.") for name in shapes)
    assert not any("side" in name for name in pae.expected_tensors(pae.read_config_dict(M.Q).plan()))


def _damaged(path, value):
    cfg = copy.deepcopy(M.P)
    at = cfg
    for key in path[:-1]:
        at = at[key]
    if value is None:
        at.pop(path[-1])
    else:
        at[path[-1]] = value
    return cfg


@pytest.mark.parametrize("damage, needle", [
    ((("layers", 0, "type"), "windowed"), "unknown layer type"),
    ((("layers", 0, "mixer", "left", "kv_heads"), 3), "not a multiple"),
    ((("layers", 0, "mixer", "right", "tau"), None), "tau"),
    ((("layers", 0, "mixer", "right", "tau"), 0.0), "tau"),
    ((("layers", 0, "mixer", "left", "rot", "dims"), 18), "rot.dims"),
    ((("layers", 0, "mixer", "left", "rot", "scaling", "factor"), 0.0), "scaling.factor"),
    ((("layers", 0, "mixer", "left_scale"), None), "left_scale"),
    ((("layers", 1, "mlp", "router", "top"), 7), "top 7 of 6"),
    ((("layers", 1, "mlp", "kind"), "sparse"), "unknown kind"),
    ((("layers", 0, "mlp", "ff"), None), "ff"),
    ((("norm",), None), "norm"),
    ((("max_positions",), None), "max_positions"),
    ((("loop", "stop"), 5), "loop"),
    ((("loop", "times"), 0), "loop"),
    ((("token_side", "dim"), 0), "token_side.dim"),
    ((("logit_softcap",), -1.0), "logit_softcap"),
])
def test_a_config_the_engine_cannot_compute_is_refused_with_its_key(damage, needle):
    with pytest.raises(ConfigError, match=needle):
        pae.read_config_dict(_damaged(*damage))


def test_what_the_layers_keep():
    """Every run of a layer has pages and state of its own; the attention's windows give pages back; the linear
    attention keeps one float32 matrix per head; nothing else is kept."""
    from paged_attention_engine_amd.engine.model import Model

    model = Model(pae.read_config_dict(M.P).plan(), torch.float32, "meta")
    paged, states = model.cache_specs()
    assert len(paged) == len(states) == 6
    assert [spec.window for spec in paged] == [11, 20, 5, 20, 5, 11]
    assert paged[1] == paged[3] and paged[1] is not None
    keys, values = paged[0].tensors
    assert (keys.name, keys.page_shape, values.name, values.page_shape) == ("k", (2, "page", 16), "v", (2, 24, "page"))
    for run, layer in enumerate((0, 1, 2, 1, 2, 3)):
        (state,) = states[run]
        right = M.P["layers"][layer]["mixer"]["right"]
        assert (state.name, state.shape, state.dtype) == ("matrices", (right["heads"], right["vdim"], right["dim"]), torch.float32)
    cache = model.new_cache(16, 8, 2)
    # the runs of one layer share a group (equal pages) and still have pools of their own
    assert cache.group_of(1) == cache.group_of(3) and cache.group_of(0) == cache.group_of(5) != cache.group_of(1)
    assert model.graph_safe


def test_a_layer_that_runs_twice_is_one_set_of_tensors():
    plan = pae.read_config_dict(M.Q).plan()
    assert len(plan.layers) == 3 and len(plan.schedule) == 7
    shapes = pae.expected_tensors(plan)
    assert sum(1 for name in shapes if name.startswith("l0.norm1")) == 2  # norm1 and norm1b, once each


def test_the_bench_shape_is_a_config_the_reader_takes():
    """`bench.py --design zikezen` builds its model from a config of its own making: as many layer runs as asked for."""
    import bench

    for runs in (2, 8):
        plan = pae.read_config_dict(bench.zikezen_shape(bench.QWEN25_1P5B, runs)).plan()
        assert len(plan.schedule) == runs and plan.hidden_size == 1536
    plan = pae.read_config_dict(bench.zikezen_shape(bench.QWEN25_1P5B, 8)).plan()
    assert [e.layer for e in plan.schedule] == [0, 1, 2, 1, 2, 3, 4, 5] and [e.add_embedding for e in plan.schedule].count(True) == 1
    assert {type(layer.feed_forward).__name__ for layer in plan.layers} == {"FeedForwardSpec", "ExpertsSpec"}


# ----------------------------------------------------------------------------- the plain implementation, pinned


def test_norm_and_activations_by_closed_forms():
    x = torch.tensor([[3.0, -4.0]], dtype=torch.float64)
    got = plain.rms_norm(x, torch.tensor([2.0, 0.5], dtype=torch.float64), 0.5)
    root = math.sqrt(12.5 + 0.5)
    assert torch.allclose(got, torch.tensor([[6.0 / root, -2.0 / root]], dtype=torch.float64))
    z = torch.tensor([0.0, 1.0, -2.0], dtype=torch.float64)
    assert torch.allclose(plain.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))
    assert torch.allclose(plain.silu(z), torch.nn.functional.silu(z))


def test_the_order_of_the_layers():
    assert plain.layer_order({"layers": [0] * 4, "loop": {"start": 1, "stop": 4, "times": 2}}) == [
        (0, False), (1, False), (2, False), (3, False), (1, True), (2, False), (3, False)]
    assert plain.layer_order({"layers": [0] * 3, "loop": {"start": 0, "stop": 1, "times": 3}}) == [
        (0, False), (0, True), (0, True), (1, False), (2, False)]
    assert plain.layer_order({"layers": [0] * 2}) == [(0, False), (1, False)]


def test_stretched_frequencies_by_hand():
    """dims 8, base 500: frequencies 1, 500^-1/4, 500^-1/2, 500^-3/4, wavelengths 6.3, 29.7, 140, 664; with original 64,
    low 1 and high 4 the first is kept (below 16), the second blended, the last two divided by the factor."""
    rot = {"dims": 8, "base": 500.0, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}}
    f = [500.0 ** (-i / 4.0) for i in range(4)]
    share = (64 * f[1] / (2 * math.pi) - 1.0) / 3.0
    want = [f[0], (1 - share) * f[1] / 8.0 + share * f[1], f[2] / 8.0, f[3] / 8.0]
    assert torch.allclose(plain.stretched_frequencies(rot), torch.tensor(want, dtype=torch.float64), rtol=1e-12)
    assert 0.0 < share < 1.0
    plain_rot = {"dims": 8, "base": 500.0}
    assert torch.allclose(plain.stretched_frequencies(plain_rot), torch.tensor(f, dtype=torch.float64), rtol=1e-12)
    # the product's own frequencies are these
    from paged_attention_engine_amd.config.model_config import WavelengthRamp
    from paged_attention_engine_amd.parts.rope import ramped_frequencies
    got, magnitude = ramped_frequencies(8, 500.0, WavelengthRamp(factor=8.0, original=64.0, low=1.0, high=4.0))
    assert magnitude == 1.0 and torch.allclose(got.double(), torch.tensor(want, dtype=torch.float64), rtol=1e-6)


def test_a_rotated_pair_by_hand():
    x = torch.zeros((3, 1, 6), dtype=torch.float64)
    x[:, 0, 2], x[:, 0, 3], x[:, 0, 4] = 1.0, 2.0, 7.0
    got = plain.rotate_pairs(x, torch.tensor([0.3, 0.5], dtype=torch.float64))
    for t in range(3):
        c, s = math.cos(0.5 * t), math.sin(0.5 * t)
        assert torch.allclose(got[t, 0], torch.tensor([0.0, 0.0, c - 2 * s, 2 * c + s, 7.0, 0.0], dtype=torch.float64))


def test_a_window_and_the_one_more_in_the_denominator_on_flat_scores():
    """Scores of zero: a query that sees n keys weighs each by 1 / (n + 1)."""
    T, W = 7, 3
    q = torch.zeros((T, 4), dtype=torch.float64)
    k = torch.randn((T, 4), dtype=torch.float64)
    v = torch.arange(T, dtype=torch.float64)[:, None] + 1.0
    got = plain.window_softmax_one_more(q, k, v, 0.5, W)
    for i in range(T):
        seen = list(range(max(0, i - W + 1), i + 1))
        assert math.isclose(float(got[i, 0]), sum(j + 1.0 for j in seen) / (len(seen) + 1.0), rel_tol=1e-12)
    whole = plain.window_softmax_one_more(q, k, v, 0.5, None)
    assert math.isclose(float(whole[6, 0]), 28.0 / 8.0, rel_tol=1e-12)


def test_two_steps_of_the_decaying_state_by_hand():
    q = torch.tensor([[1.0, 0.0], [1.0, 1.0]], dtype=torch.float64)
    k = torch.tensor([[2.0, 1.0], [0.0, 3.0]], dtype=torch.float64)
    v = torch.tensor([[5.0], [7.0]], dtype=torch.float64)
    decay = torch.tensor([[0.5, 0.5], [0.5, 0.25]], dtype=torch.float64)
    got = plain.decaying_state_readout(q, k, v, decay)
    # S1 = k1 v1 = [10, 5]; o1 = 10.  S2 = [0.5 * 10, 0.25 * 5] + [0, 21] = [5, 22.25]; o2 = 27.25
    assert torch.allclose(got, torch.tensor([[10.0], [27.25]], dtype=torch.float64))


def test_a_routing_in_which_the_correction_changes_the_choice_and_not_the_weight():
    W = {"r.router": torch.eye(4, dtype=torch.float64), "r.correction": torch.tensor([0.0, 0.0, 0.5, 0.0], dtype=torch.float64)}
    h = torch.tensor([[2.0, 1.0, 0.0, -1.0]], dtype=torch.float64)
    s = torch.softmax(h, dim=-1)
    margins = []
    chosen, weights = plain.route(W, "r.", {"router": {"experts": 4, "top": 2}}, h, torch.float64, margins)
    assert chosen.tolist() == [[0, 2]]          # score + correction: 0.64, 0.24, 0.59, 0.03; the scores alone choose 0 and 1
    assert torch.allclose(weights, s[:, [0, 2]])  # and the weights are the scores alone, not renormalised
    assert math.isclose(float(margins[0][0]), float(s[0, 2] + 0.5 - s[0, 1]), rel_tol=1e-12)
    W["r.correction"] = torch.zeros(4, dtype=torch.float64)
    assert plain.route(W, "r.", {"router": {"experts": 4, "top": 2}}, h, torch.float64)[0].tolist() == [[0, 1]]


# ----------------------------------------------------------------------------- a mechanism left out shows


@pytest.fixture(scope="module")
def model_p(tmp_path_factory):
    cfg, weights = M.read_folder(M.make_folder(tmp_path_factory.mktemp("zikezen_cpu"), "P"))
    tokens = M.tokens_for("P", 40)
    return cfg, weights, tokens, plain.forward(weights, cfg, tokens, torch.float64)


def _moved(model_p, change) -> float:
    """How far the logits move, in units of the float32 tests' bound, under a changed config or changed weights."""
    cfg, weights, tokens, want = model_p
    cfg2, weights2 = copy.deepcopy(cfg), dict(weights)
    change(cfg2, weights2)
    got = plain.forward(weights2, cfg2, tokens, torch.float64)
    return float((got - want).abs().max()) / (1e-4 * float(want.abs().max()))


@pytest.mark.parametrize("what, change", [
    ("a window one longer", lambda c, w: c["layers"][2]["mixer"]["left"]["mask"].update(size=6)),
    ("no rotation", lambda c, w: c["layers"][0]["mixer"]["left"].pop("rot")),
    ("frequencies not stretched", lambda c, w: c["layers"][0]["mixer"]["left"]["rot"].pop("scaling")),
    ("another temperature", lambda c, w: c["layers"][1]["mixer"]["right"].update(tau=8.0)),
    ("one pass only", lambda c, w: c["loop"].update(times=1)),
    ("the loop one layer on", lambda c, w: c["loop"].update(start=2)),
    ("no second token table", lambda c, w: c.pop("token_side")),
    ("another logit cap", lambda c, w: c.update(logit_softcap=10.0)),
    ("the embedding not scaled", lambda c, w: c["embedding"].update(scale=1.0)),
    ("no positions", lambda c, w: w.update(pos=torch.zeros_like(w["pos"]))),
    ("no correction", lambda c, w: w.update({"l1.mlp.correction": torch.zeros_like(w["l1.mlp.correction"])})),
    ("no bias on the keys", lambda c, w: w.update({"l0.mix.left.k.b": torch.zeros_like(w["l0.mix.left.k.b"])})),
    ("no bias in the decay", lambda c, w: w.update({"l0.mix.right.a2.b": torch.zeros_like(w["l0.mix.right.a2.b"])})),
    ("the other side's factor", lambda c, w: c["layers"][0]["mixer"].update(left_scale=1.2, right_scale=0.7)),
    ("the norm after the mixer left at one", lambda c, w: w.update({"l0.norm1b": torch.ones_like(w["l0.norm1b"])})),
])
def test_a_mechanism_left_out_or_a_constant_off_moves_the_logits(model_p, what, change):
    assert _moved(model_p, change) > 10.0, what


def test_the_embedding_joins_before_the_second_pass_and_only_there(model_p):
    """The stream after the first layer of the second pass differs from a pass without the join by what the
    embedding's output does to it; the runs before are untouched."""
    cfg, weights, tokens, _ = model_p
    taps = []
    plain.forward(weights, cfg, tokens, torch.float64, taps=taps)
    x0 = plain.embed(weights, cfg, tokens, torch.float64)
    original = plain.layer_order
    plain.layer_order = lambda c: [(i, False) for i, _ in original(c)]
    try:
        bare = []
        plain.forward(weights, cfg, tokens, torch.float64, taps=bare)
    finally:
        plain.layer_order = original
    for run in range(3):
        assert torch.equal(taps[run], bare[run])
    assert float((taps[3] - bare[3]).abs().max()) > 0.1 * float(x0.abs().max())


def test_a_sink_of_zero_bounds_what_attention_adds():
    """With one more in the denominator the weights add up to less than one: a lone key's value is halved at score 0."""
    q = torch.zeros((1, 4), dtype=torch.float64)
    got = plain.window_softmax_one_more(q, torch.ones((1, 4), dtype=torch.float64), torch.tensor([[6.0]], dtype=torch.float64), 1.0, 1)
    assert math.isclose(float(got[0, 0]), 3.0, rel_tol=1e-12)
