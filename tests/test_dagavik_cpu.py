"""Dagavik on the CPU: the config reader and the plan it gives, the tensors the parts declare, what the layers
keep in the cache, and the plain implementation pinned by closed forms and by invariants (so that the oracle
the GPU tests compare with is itself checked)."""

import copy
import math

import pytest
import torch

import paged_attention_engine_amd as pae
from paged_attention_engine_amd.config import ConfigError
from tests import dagavik_models as M
from tests.plain import dagavik_plain as plain


# ----------------------------------------------------------------------------- configuration


def test_the_reader_is_chosen_by_the_architecture_key_and_round_trips():
    for cfg in M.CONFIGS.values():
        typed = pae.read_config_dict(cfg)
        assert type(typed).__name__ == "DagavikConfig"
        assert pae.read_config_dict(typed.to_json_dict()) == typed


def test_every_size_and_constant_comes_from_the_config():
    plan = pae.read_config_dict(M.U).plan()
    assert (plan.hidden_size, plan.vocab_size, plan.head_name, plan.embedding_name) == (64, 300, "head", "embed")
    assert (plan.pair_embedding.name, plan.pair_embedding.buckets, plan.pair_embedding.mul_prev, plan.pair_embedding.mul_cur) == ("bigram", 101, 13, 5)
    assert [(e.layer, e.cache_from) for e in plan.schedule] == [(0, None), (1, None), (2, None), (3, 1)]
    first, second, third, fourth = plan.layers
    assert all(layer.arrangement == "parallel" for layer in plan.layers)
    assert first.mixer_norm.weight_offset == 1.0 and first.mixer_norm.eps == 2e-6 and plan.final_norm.weight_offset == 1.0
    side = first.mixer
    assert (side.kind, side.left_scale, side.right_scale) == ("side_by_side", 0.7, 1.2)
    a = side.left
    assert (a.kind, a.num_heads, a.num_kv_heads, a.head_dim, a.v_dim, a.scale, a.window, a.qkv_bias, a.bias_suffix) == (
        "attention", 4, 2, 16, 24, 0.3, 11, True, ".b")
    assert (a.position.kind, a.position.rotary_dim, a.position.theta) == ("neox_rope", 8, 500.0) and not a.sinks and not a.convolved
    m = side.right
    assert (m.kind, m.num_heads, m.key_dim, m.value_dim, m.gate_cap, m.norm_eps, m.readout_floor) == ("matrix_memory", 2, 16, 24, 8.0, 2e-6, 1e-6)
    e = first.feed_forward
    assert (e.kind, e.intermediate_size, e.num_experts, e.top, e.groups, e.groups_kept, e.route_scale, e.activation) == (
        "experts", 24, 6, 2, 2, 1, 1.7, "silu")
    l = second.mixer
    assert (l.kind, l.num_heads, l.nope_dim, l.rope_dim, l.value_dim, l.kv_rank, l.scale, l.window, l.sinks, l.own_kv) == (
        "latent_attention", 4, 16, 0, 8, 32, 0.3, None, True, True)
    assert (second.feed_forward.groups, second.feed_forward.groups_kept, second.feed_forward.top) == (1, 1, 1)  # no groups named: one
    d = third.mixer
    assert (d.kind, d.num_heads, d.num_kv_heads, d.key_dim, d.value_dim, d.conv_taps, d.decay, d.decay_rank, d.gate_rank,
            d.gate_activation, d.unit_eps) == ("gated_delta", 4, 2, 16, 24, 3, "channel", 8, 16, "sigmoid", 1e-6)
    assert not fourth.mixer.own_kv and fourth.feed_forward is None and fourth.feed_forward_norm is None
    # no mask: every earlier key; no rotation: none; no bigram table: none
    x = pae.read_config_dict(M.X).plan()
    assert x.layers[0].mixer.left.window is None and x.layers[0].mixer.left.position is None and x.pair_embedding is None


def test_the_narrow_products_widths_come_from_the_tensors_shapes(tmp_path):
    """A config.json as the design writes it names no width for the delta rule's narrow products: the checkpoint's shapes do."""
    import json
    import os
    folder = M.make_folder(tmp_path, "U")
    with open(os.path.join(folder, "config.json")) as handle:
        cfg = json.load(handle)
    for layer in cfg["layers"]:
        layer["mixer"].pop("decay_rank", None)
        layer["mixer"].pop("gate_rank", None)
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(cfg, handle)
    typed = pae.read_config(folder)
    assert (typed.layers[2].decay_rank, typed.layers[2].gate_rank) == (8, 16)
    with pytest.raises(ConfigError, match="narrow product"):
        pae.read_config_dict(cfg)


def test_declared_tensors_carry_the_designs_names_and_shapes():
    shapes = pae.expected_tensors(pae.read_config_dict(M.U).plan())
    assert shapes["embed"] == (300, 64) and shapes["bigram"] == (102, 64) and shapes["head"] == (300, 64)
    assert tuple(shapes["final.norm"]) == (64,) and tuple(shapes["l0.norm2"]) == (64,) and "l3.norm2" not in shapes
    assert shapes["l0.mix.left.q"] == (64, 64) and shapes["l0.mix.left.k"] == (32, 64) and shapes["l0.mix.left.v"] == (48, 64)
    assert shapes["l0.mix.left.q.b"] == (64,) and shapes["l0.mix.left.v.b"] == (48,) and shapes["l0.mix.left.o"] == (64, 96)
    assert shapes["l0.mix.right.q"] == (32, 64) and shapes["l0.mix.right.v"] == (48, 64) and shapes["l0.mix.right.g"] == (48, 64)
    assert shapes["l0.mix.right.i"] == (2, 64) and shapes["l0.mix.right.f.b"] == (2,) and tuple(shapes["l0.mix.right.norm"]) == (48,)
    assert shapes["l0.mix.right.o"] == (64, 48)
    assert shapes["l0.mlp.router"] == (6, 64) and shapes["l0.mlp.e5.gate"] == (24, 64) and shapes["l0.mlp.e0.down"] == (64, 24)
    assert shapes["l1.mix.q"] == (64, 64) and shapes["l1.mix.dkv"] == (32, 64) and tuple(shapes["l1.mix.dkv.norm"]) == (32,)
    assert shapes["l1.mix.uk"] == (64, 32) and shapes["l1.mix.uv"] == (32, 32) and shapes["l1.mix.sink"] == (4,)
    assert shapes["l2.mix.q"] == (32, 64) and shapes["l2.mix.v"] == (96, 64) and shapes["l2.mix.v.conv"] == (96, 3)
    assert shapes["l2.mix.b"] == (4, 64) and shapes["l2.mix.A_log"] == (4,) and shapes["l2.mix.dt_bias"] == (64,)
    assert shapes["l2.mix.a1"] == (8, 64) and shapes["l2.mix.a2"] == (64, 8) and shapes["l2.mix.g1"] == (16, 64)
    assert shapes["l2.mix.g2"] == (96, 16) and tuple(shapes["l2.mix.norm"]) == (24,)
    assert "l3.mix.dkv" not in shapes and "l3.mix.dkv.norm" not in shapes and shapes["l3.mix.uk"] == (48, 32)


def _damaged(path, value):
    cfg = copy.deepcopy(M.U)
    at = cfg
    for key in path[:-1]:
        at = at[key]
    if value is None:
        at.pop(path[-1])
    else:
        at[path[-1]] = value
    return cfg


@pytest.mark.parametrize("damage, needle", [
    ((("layers", 0, "type"), "windowed"), "unknown mixer type"),
    ((("layers", 0, "mixer", "left", "kv_heads"), 3), "not a multiple"),
    ((("layers", 0, "mixer", "right", "gate_cap"), None), "gate_cap"),
    ((("layers", 0, "mixer", "left", "rot", "dims"), 18), "rot.dims"),
    ((("layers", 3, "mixer", "kv_from"), 2), "not a latent attention layer"),
    ((("layers", 3, "mixer", "kv_rank"), 16), "kv_rank differs"),
    ((("layers", 0, "mlp", "router", "top"), 4), "exceeds"),
    ((("layers", 0, "mlp", "router", "groups", "count"), 4), "groups"),
    ((("layers", 0, "mlp", "kind"), "dense"), "unknown kind"),
    ((("norm",), None), "norm"),
    ((("embedding", "bigram", "buckets"), 0), "buckets"),
])
def test_a_faulty_config_is_refused_with_the_key_named(damage, needle):
    with pytest.raises(ConfigError, match=needle):
        pae.read_config_dict(_damaged(*damage))


def test_random_weights_make_a_folder_the_loader_accepts(tmp_path):
    folder = M.make_folder(tmp_path, "W")
    cfg, tensors = M.read_folder(folder)
    declared = pae.expected_tensors(pae.read_config(folder).plan())
    assert cfg["architecture"] == "Dagavik" and set(tensors) == set(declared)
    got = pae.load_weights(folder, declared)
    assert torch.equal(got["l0.mix.a2"], tensors["l0.mix.a2"]) and got["l0.mix.a2"].shape == (60, 12)
    # norm weights are stored around zero
    assert float(tensors["l0.norm1"].float().abs().mean()) < 0.5


# ----------------------------------------------------------------------------- what the layers keep


def test_pages_state_and_borrowed_rows():
    """The attention half keeps keys and values behind its window, the memory half its matrix (with the key sum as one
    more column) and its maximum; a latent layer one row per token for ever, a reader of it nothing; the delta rule its
    matrices and the convolutions' last inputs; the embedding the last token."""
    model = pae.Model(pae.read_config_dict(M.U).plan(), torch.float32, "cpu")
    paged, states = model.cache_specs()
    assert len(paged) == 5 and paged[4] is None and states[4].name == "last_token" and states[4].dtype == torch.int32
    assert [t.name for t in paged[0].tensors] == ["k", "v"] and paged[0].window == 11
    assert paged[0].tensors[0].shape(16) == (2, 16, 16) and paged[0].tensors[1].shape(16) == (2, 24, 16)
    assert {s.name: s.shape for s in states[0]} == {"memory": (2, 25, 16), "memory_max": (2,)}
    assert [t.name for t in paged[1].tensors] == ["latent"] and paged[1].tensors[0].shape(16) == (16, 32) and paged[1].window is None
    assert states[1] is None and paged[3] is None and states[3] is None
    assert paged[2] is None and {s.name: s.shape for s in states[2]} == {"matrices": (4, 24, 16), "conv_tail": (2, 2 * 32 + 96)}
    cache = model.new_cache(16, 8, 2)
    assert cache.group_of(3) is None and cache.state_of(4).shape == (3,) and cache.state_of(0)["memory"].shape == (3, 2, 25, 16)
    assert cache.create_sequence(1) and cache.reserve(1, 100).ok
    free_before = cache.free_blocks()
    assert cache.release_passed(1) > 0  # the window's pages come back, the latent rows stay
    assert cache.free_blocks()[cache.group_of(0)] > free_before[cache.group_of(0)]
    assert cache.free_blocks()[cache.group_of(1)] == free_before[cache.group_of(1)]
    # a model of recurrent layers and a full attention: one group, nothing comes back
    model = pae.Model(pae.read_config_dict(M.X).plan(), torch.float32, "cpu")
    paged, states = model.cache_specs()
    assert len(paged) == 3 and paged[0].window is None and paged[1] is None  # no bigram table: no state behind the last stop
    assert {s.name: s.shape for s in states[1]} == {"matrices": (2, 16, 72), "conv_tail": (0, 2 * 72 + 32)}


# ----------------------------------------------------------------------------- the plain implementation


def test_the_offset_norm_and_the_bigram_rows_by_hand():
    x = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    got = plain.offset_norm(x, torch.tensor([0.5, -1.0], dtype=torch.float64), 0.5)
    root = math.sqrt(12.5 + 0.5)
    assert torch.allclose(got, torch.tensor([[3.0 / root * 1.5, 0.0]], dtype=torch.float64))
    assert plain.bigram_rows([4, 9, 9, 0], {"buckets": 7, "mul_prev": 3, "mul_cur": 5}) == [7, (12 + 45) % 7, (27 + 45) % 7, 27 % 7]


def test_the_rotation_turns_the_halves_and_leaves_the_rest():
    x = torch.arange(1.0, 7.0, dtype=torch.float64).view(1, 1, 6)
    got = plain.rotate_halves(x.repeat(2, 1, 1), torch.tensor([0, 3]), 4, 100.0)
    assert torch.equal(got[0], x[0])  # position 0
    a0, a1 = 3.0, 3.0 * 100.0 ** -0.5
    want = [1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
            3 * math.cos(a0) + 1 * math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 5.0, 6.0]
    assert torch.allclose(got[1, 0], torch.tensor(want, dtype=torch.float64))


def test_the_window_and_the_sink_by_hand():
    """Flat scores: a token sees itself and size - 1 before it; a sink of ln 2 counts as two more keys without a value."""
    T = 6
    q = torch.zeros((T, 1, 2), dtype=torch.float64)
    k = torch.zeros((T, 1, 2), dtype=torch.float64)
    v = torch.arange(T, dtype=torch.float64).view(T, 1, 1)
    got = plain.softmax_attend(q, k, v, 1.0, 3)[:, 0, 0]
    assert torch.allclose(got, torch.tensor([0.0, 0.5, 1.0, 2.0, 3.0, 4.0], dtype=torch.float64))
    got = plain.softmax_attend(q, k, v, 1.0, None, torch.tensor([math.log(2.0)], dtype=torch.float64))[:, 0, 0]
    assert torch.allclose(got, torch.tensor([sum(range(t + 1)) / (t + 3) for t in range(T)], dtype=torch.float64))


def test_two_steps_of_the_matrix_memory_by_hand():
    q = torch.tensor([[[1.0, 0.0]], [[0.0, 2.0]]], dtype=torch.float64)
    k = torch.tensor([[[1.0, 1.0]], [[0.0, 1.0]]], dtype=torch.float64)
    v = torch.tensor([[[2.0]], [[-4.0]]], dtype=torch.float64)
    log_in = torch.tensor([[-1.0], [0.5]], dtype=torch.float64)
    log_keep = torch.tensor([[-0.2], [-0.3]], dtype=torch.float64)
    got = plain.matrix_memory_recurrence(q, k, v, log_in, log_keep)
    # step 1: m = max(-0.2 + 0, -1) = -0.2; take = e^-0.8; C = take k v^T; n = take k; o = C^T q / (max(|n.q|, e^0.2) + 1e-6)
    take1 = math.exp(-0.8)
    assert math.isclose(float(got[0, 0, 0]), take1 * 2.0 / (max(take1, math.exp(0.2)) + 1e-6), rel_tol=1e-12)
    # step 2: m = max(-0.3 - 0.2, 0.5) = 0.5; keep = e^-1.0; take = 1
    keep2 = math.exp(-1.0)
    c_row2 = keep2 * take1 * 2.0 + 1.0 * -4.0   # row 2 of C (key feature 2)
    n2 = keep2 * take1 + 1.0
    assert math.isclose(float(got[1, 0, 0]), 2 * c_row2 / (max(abs(2 * n2), math.exp(-0.5)) + 1e-6), rel_tol=1e-12)
    # (step 1 is also the proof that the maximum starts at 0 and not below: from minus infinity it would be -1)


def test_two_steps_of_the_delta_rule_with_channel_decays_by_hand():
    q = torch.tensor([[[1.0, 0.0]], [[1.0, 1.0]]], dtype=torch.float64)
    k = torch.tensor([[[1.0, 0.0]], [[1.0, 1.0]]], dtype=torch.float64)
    v = torch.tensor([[[3.0]], [[5.0]]], dtype=torch.float64)
    beta = torch.tensor([[0.5], [1.0]], dtype=torch.float64)
    decay = torch.tensor([[[0.9, 0.8]], [[0.5, 0.25]]], dtype=torch.float64)
    got = plain.channel_delta_recurrence(q, k, v, beta, decay)
    # step 1: S = 0; u = 0.5 * 3; S = k u^T = [1.5, 0]; o = 1.5
    assert math.isclose(float(got[0, 0, 0]), 1.5)
    # step 2: S = [0.5 * 1.5, 0.25 * 0] = [0.75, 0]; u = 5 - 0.75 = 4.25; S = [5, 4.25]; o = 9.25: the read-out sees the write
    assert math.isclose(float(got[1, 0, 0]), 9.25)


def test_the_convolution_is_causal_and_its_last_tap_is_the_current_token():
    x = torch.tensor([[1.0], [2.0], [4.0]], dtype=torch.float64)
    got = plain.causal_conv_silu(x, torch.tensor([[100.0, 10.0, 1.0]], dtype=torch.float64))
    want = plain.silu(torch.tensor([[1.0], [12.0], [124.0]], dtype=torch.float64))
    assert torch.allclose(got, want)


def test_routing_by_hand():
    z = torch.log(torch.tensor([[0.30, 0.05, 0.05, 0.25, 0.24, 0.11]], dtype=torch.float64))
    router = {"top": 2, "scale": 2.0, "groups": {"count": 2, "keep": 1}}
    margins = []
    chosen, weights = plain.route(z, router, margins)
    assert chosen.tolist() == [[0, 1]] or chosen.tolist() == [[0, 2]]  # the first group wins by its best expert; 0.25 and 0.24 stay out
    assert math.isclose(float(weights[0, 0]), 0.6) and math.isclose(float(weights[0, 1]), 0.1)  # not renormalised
    assert math.isclose(float(margins[0][0]), 0.0, abs_tol=1e-12)  # experts 1 and 2 tie
    chosen, _ = plain.route(z, {"top": 2, "scale": 1.0}, None)
    assert chosen.tolist() == [[0, 3]]


def test_the_folded_query_scores_what_the_heads_keys_score():
    gen = torch.Generator().manual_seed(0)
    q, c = torch.randn(5, dtype=torch.float64, generator=gen), torch.randn(7, dtype=torch.float64, generator=gen)
    w_uk = torch.randn((5, 7), dtype=torch.float64, generator=gen)
    assert math.isclose(float(q @ (w_uk @ c)), float((w_uk.T @ q) @ c), rel_tol=1e-12)


def test_the_test_models_show_mistakes(tmp_path):
    """Leaving a mechanism out, or getting a constant one off, moves a test model's logits far beyond the tests' bounds."""
    folder = M.make_folder(tmp_path, "U")
    cfg, weights = M.read_folder(folder)
    tokens = M.tokens_for("U", 40)
    right = plain.forward(weights, cfg, tokens, torch.float64)
    top = float(right.abs().max())

    def moved(cfg2=None, weights2=None, patch=None):
        saved = {}
        for name, fn in (patch or {}).items():
            saved[name] = getattr(plain, name)
            setattr(plain, name, fn)
        try:
            other = plain.forward(weights2 or weights, cfg2 or cfg, tokens, torch.float64)
        finally:
            for name, fn in saved.items():
                setattr(plain, name, fn)
        return float((other - right).abs().max()) / top

    def with_key(path, value):
        out = copy.deepcopy(cfg)
        at = out
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        return out

    bound = 1e-3
    assert moved(with_key(("layers", 0, "mixer", "left", "mask", "size"), 12)) > bound     # a window one token longer
    assert moved(with_key(("layers", 0, "mixer", "left", "rot", "dims"), 0)) > bound       # no rotation
    assert moved(with_key(("layers", 0, "mixer", "right", "gate_cap"), 2.0)) > bound       # another cap
    assert moved(with_key(("layers", 0, "mixer", "left_scale"), 1.0)) > bound
    assert moved(with_key(("layers", 0, "mlp", "router", "groups"), {"count": 1, "keep": 1})) > bound   # no groups
    assert moved(with_key(("layers", 0, "mlp", "router", "scale"), 1.0)) > bound
    assert moved(with_key(("embedding", "bigram", "mul_prev"), 14)) > bound
    assert moved(with_key(("layers", 3, "mixer", "kv_from"), None), {**weights, "l3.mix.dkv": weights["l1.mix.dkv"], "l3.mix.dkv.norm": weights["l1.mix.dkv.norm"]}) > bound  # its own rows from its own input
    no_sink = {**weights, "l1.mix.sink": torch.full_like(weights["l1.mix.sink"], -60.0)}
    assert moved(weights2=no_sink) > bound
    no_bias = {**weights, "l0.mix.left.k.b": torch.zeros_like(weights["l0.mix.left.k.b"]), "l0.mix.left.q.b": torch.zeros_like(weights["l0.mix.left.q.b"])}
    assert moved(weights2=no_bias) > bound
    assert moved(patch={"offset_norm": lambda x, w, eps: plain.rms(x, eps) * w}) > bound          # the weight without its one
    assert moved(patch={"unit": lambda x: x}) > bound
    assert moved(patch={"READOUT_FLOOR": 1.0}) > bound
    reversed_taps = {**weights, **{n: t.flip(-1) for n, t in weights.items() if n.endswith(".conv")}}
    assert moved(weights2=reversed_taps) > bound
    head_decay = {**weights, "l2.mix.dt_bias": weights["l2.mix.dt_bias"].view(4, 16)[:, :1].expand(4, 16).reshape(-1).contiguous(),
                  "l2.mix.a2": weights["l2.mix.a2"].view(4, 16, 8)[:, :1].expand(4, 16, 8).reshape(64, 8).contiguous()}
    assert moved(weights2=head_decay) > bound  # one decay per head instead of one per channel
