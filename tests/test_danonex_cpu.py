"""Danonex on the CPU: the config reader and the plan it gives, the tensors the parts declare,
per-request state with several named tensors, and the plain implementation pinned by closed forms
and by invariants (so that the oracle the GPU tests compare with is itself checked)."""

import math

import pytest
import torch

import paged_attention_engine_amd as pae
from paged_attention_engine_amd.cache.manager import CacheManager, StateSpec, attention_pages
from paged_attention_engine_amd.config import ConfigError
from paged_attention_engine_amd.parts.rope import ramped_frequencies
from tests import danonex_models as M
from tests.plain import danonex_plain as plain


# ----------------------------------------------------------------------------- configuration


def test_the_reader_is_chosen_by_the_architecture_key_and_round_trips():
    for name, cfg in M.CONFIGS.items():
        typed = pae.read_config_dict(cfg)
        assert type(typed).__name__ == "DanonexConfig"
        assert pae.read_config_dict(typed.to_json_dict()) == typed


def test_every_size_and_constant_comes_from_the_config():
    plan = pae.read_config_dict(M.Q).plan()
    assert (plan.hidden_size, plan.vocab_size, plan.logit_scale, plan.head_name) == (100, 211, 3.0, None)
    first, second, third = plan.layers
    assert first.arrangement == "branchnorm" and first.residual_scale == 0.4
    a = first.mixer
    assert (a.kind, a.num_heads, a.num_kv_heads, a.head_dim, a.v_dim, a.scale, a.softcap) == ("attention", 3, 1, 48, 80, 0.35, 20.0)
    assert a.sinks and a.qk_norm == "projection" and a.qk_norm_eps == 1e-5 and not a.qkv_bias and not a.plain
    assert (a.position.kind, a.position.rotary_dim, a.position.theta) == ("interleaved_rope", 24, 2000.0)
    assert a.position.ramp.factor == 2.5 and a.position.ramp.original == 512
    d = second.mixer
    assert (d.kind, d.num_heads, d.num_kv_heads, d.key_dim, d.value_dim, d.conv_taps, d.norm_eps) == ("gated_delta", 3, 3, 20, 36, 4, 1e-5)
    assert first.feed_forward.kind == "dense" and first.feed_forward.intermediate_size == 130
    assert third.feed_forward is None and third.feed_forward_norm is None
    assert third.mixer.position is None and third.mixer.softcap == 5.0


def test_declared_tensors_carry_the_designs_names_and_shapes():
    shapes = pae.expected_tensors(pae.read_config_dict(M.P).plan())
    assert shapes["embed"] == (300, 64) and tuple(shapes["final.norm"]) == (64,)
    assert shapes["l0.mix.q"] == (2 * 16, 64) and shapes["l0.mix.v"] == (4 * 24, 64) and shapes["l0.mix.g"] == (4 * 24, 64)
    assert shapes["l0.mix.q.conv"] == (32, 3) and shapes["l0.mix.v.conv"] == (96, 3)
    assert shapes["l0.mix.b"] == (4, 64) and shapes["l0.mix.a"] == (4, 64) and shapes["l0.mix.o"] == (64, 96)
    assert shapes["l0.mix.A_log"] == (4,) and shapes["l0.mix.dt_bias"] == (4,) and tuple(shapes["l0.mix.norm"]) == (24,)
    assert shapes["l1.mix.q"] == (6 * 32, 64) and shapes["l1.mix.k"] == (2 * 32, 64) and shapes["l1.mix.v"] == (2 * 16, 64)
    assert shapes["l1.mix.o"] == (64, 6 * 16) and shapes["l1.mix.sink"] == (6,)
    assert tuple(shapes["l1.mix.q.norm"]) == (192,) and tuple(shapes["l1.mix.k.norm"]) == (64,)
    assert shapes["l0.mlp.up"] == (96, 64) and shapes["l0.mlp.down"] == (64, 96)
    assert "l1.mlp.up" not in shapes and "l1.norm2" not in shapes and "l1.norm1" in shapes and "l0.norm2" in shapes


@pytest.mark.parametrize("damage,needle", [
    (lambda c: c["layers"][0].update(type="conv"), "unknown mixer type"),
    (lambda c: c["layers"][1]["mixer"].pop("vdim"), "vdim"),
    (lambda c: c["layers"][1]["mixer"].update(heads=5), "not a multiple"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=34), "rot.dims"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "unknown kind"),
    (lambda c: c.pop("residual_mult"), "residual_mult"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_a_faulty_config_is_refused_with_the_key_named(damage, needle):
    import copy
    cfg = copy.deepcopy(M.P)
    damage(cfg)
    with pytest.raises(ConfigError, match=needle):
        pae.read_config_dict(cfg)


def test_random_weights_make_a_folder_the_loader_accepts(tmp_path):
    folder = M.make_folder(tmp_path, "R")
    cfg, tensors = M.read_folder(folder)
    assert cfg["architecture"] == "Danonex" and set(tensors) == set(pae.expected_tensors(pae.read_config_dict(cfg).plan()))
    got = pae.load_weights(folder, pae.expected_tensors(pae.read_config_dict(cfg).plan()))
    assert torch.equal(got["l0.mix.A_log"], tensors["l0.mix.A_log"])


# ----------------------------------------------------------------------------- cache and state


def test_a_stop_may_keep_several_named_state_tensors_and_a_model_without_pages_runs():
    states = [(StateSpec((2, 3, 4), torch.float32, "matrices"), StateSpec((1, 10), torch.float32, "tail")), None,
              StateSpec((5,))]
    cache = CacheManager([None, attention_pages(2, 8, None, 4), None], states, 16, 4, 2, torch.float32, "cpu")
    assert set(cache.state_of(0)) == {"matrices", "tail"} and cache.state_of(0)["tail"].shape == (3, 1, 10)
    assert cache.state_of(2).shape == (3, 5)
    assert cache.pages_of(1)["v"].shape == (5, 2, 4, 16) and cache.pages_of(1)["k"].shape == (5, 2, 16, 8)
    assert cache.create_sequence(7) and cache.create_sequence(8) and not cache.create_sequence(9)
    slot = cache.slot_of(7)
    cache.state_of(0)["matrices"][slot] += 1.0
    cache.state_of(2)[slot] += 1.0
    cache.free_sequence(7)
    assert cache.create_sequence(9) and cache.slot_of(9) == slot      # the slot is used again, and is zero again
    assert float(cache.state_of(0)["matrices"][slot].abs().sum()) == 0.0 and float(cache.state_of(2)[slot].abs().sum()) == 0.0
    with pytest.raises(ValueError, match="distinct names"):
        CacheManager([None], [(StateSpec((1,), name="x"), StateSpec((2,), name="x"))], 16, 1, 1, torch.float32, "cpu")
    # state alone: no groups, nothing to reserve, sequences bounded by the slots
    only_state = CacheManager([None], [StateSpec((3,))], 16, 4, 2, torch.float32, "cpu")
    assert only_state.groups == [] and only_state.create_sequence(0) and only_state.reserve(0, 100).ok
    assert only_state.num_tokens(0) == 100 and only_state.fits_now(10_000, 1)


# ----------------------------------------------------------------------------- the plain implementation


def test_stretched_frequencies_by_their_closed_form():
    rot = {"base": 100.0, "dims": 8, "scaling": {"factor": 4.0, "original": 64, "fast": 4.0, "slow": 1.0}}
    freq, mult = plain.yarn_frequencies(rot)
    # index(t) = 8 ln(64 / (2 pi t)) / (2 ln 100): index(4) = 0.81 -> low 0; index(1) = 2.02 -> high 3
    base = torch.tensor([100.0 ** (-2 * i / 8) for i in range(4)], dtype=torch.float64)
    blend = torch.tensor([0.0, 1 / 3, 2 / 3, 1.0], dtype=torch.float64)
    assert torch.allclose(freq, base / 4 * blend + base * (1 - blend), rtol=1e-12)
    assert mult == pytest.approx(0.1 * math.log(4.0) + 1.0)
    got, got_mult = ramped_frequencies(8, 100.0, pae.config.FrequencyRamp(4.0, 64, 4.0, 1.0))
    assert torch.allclose(got.double(), freq, rtol=1e-6) and got_mult == pytest.approx(mult)
    plain_freq, one = plain.yarn_frequencies({"base": 100.0, "dims": 8, "scaling": None})
    assert torch.allclose(plain_freq, base) and one == 1.0


def test_the_rotation_turns_interleaved_pairs_and_leaves_the_rest():
    rot = {"base": 10.0, "dims": 4, "scaling": None}
    x = torch.arange(1.0, 13.0, dtype=torch.float64).view(2, 1, 6)
    out = plain.rotate_interleaved(x, torch.tensor([0, 3]), rot)
    assert torch.equal(out[0], x[0])                      # position 0: nothing turns
    assert torch.equal(out[1, 0, 4:], x[1, 0, 4:])        # beyond rot.dims: unchanged
    a0, a1 = 3.0, 3.0 * 10.0 ** -0.5
    u, v = x[1, 0, 0], x[1, 0, 1]
    assert out[1, 0, 0] == pytest.approx(u * math.cos(a0) - v * math.sin(a0))
    assert out[1, 0, 1] == pytest.approx(v * math.cos(a0) + u * math.sin(a0))
    u, v = x[1, 0, 2], x[1, 0, 3]
    assert out[1, 0, 2] == pytest.approx(u * math.cos(a1) - v * math.sin(a1))
    # scores depend on the distance alone
    q = torch.randn(1, 1, 6, dtype=torch.float64)
    k = torch.randn(1, 1, 6, dtype=torch.float64)
    s = [float((plain.rotate_interleaved(q, torch.tensor([p + 5]), rot) * plain.rotate_interleaved(k, torch.tensor([p]), rot)).sum())
         for p in (0, 40)]
    assert s[0] == pytest.approx(s[1])


def test_the_sink_joins_the_denominator_once_and_the_cap_bounds_the_scores():
    q = torch.zeros(2, 1, 4, dtype=torch.float64)
    k = torch.zeros(2, 1, 4, dtype=torch.float64)
    v = torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]]], dtype=torch.float64)
    # all scores 0: weights 1 / (n + e^sink) each; without a sink 1 / n
    out = plain.attend(q, k, v, 1.0, None, torch.tensor([math.log(2.0)], dtype=torch.float64))
    assert torch.allclose(out[0, 0], torch.tensor([1 / 3, 0.0], dtype=torch.float64))
    assert torch.allclose(out[1, 0], torch.tensor([1 / 4, 1 / 4], dtype=torch.float64))
    assert torch.allclose(plain.attend(q, k, v, 1.0, None, None)[1, 0], torch.tensor([0.5, 0.5], dtype=torch.float64))
    # a score of 1000 capped at 2 weighs e^2 against e^0 (the sink is neither scaled nor capped)
    q[1, 0, 0], k[1, 0, 0] = 100.0, 10.0
    out = plain.attend(q, k, v, 1.0, 2.0, torch.tensor([0.0], dtype=torch.float64))
    e = math.exp(2.0 * math.tanh(500.0))
    assert out[1, 0, 1] == pytest.approx(e / (e + 2.0))


def test_the_delta_rule_by_hand_and_its_invariants():
    # one head, D = 2, V = 1: follow two tokens by hand
    q = torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]]], dtype=torch.float64)
    k = torch.tensor([[[1.0, 0.0]], [[0.6, 0.8]]], dtype=torch.float64)
    v = torch.tensor([[[2.0]], [[5.0]]], dtype=torch.float64)
    beta = torch.tensor([[0.5], [1.0]], dtype=torch.float64)
    decay = torch.tensor([[0.9], [0.5]], dtype=torch.float64)
    out = plain.delta_recurrence(q, k, v, beta, decay)
    # t0: S = 0; u = 0.5 * 2 = 1; S = [1, 0]^T; o = S^T q = 1
    # t1: S = [0.5, 0]; S^T k = 0.3; u = 5 - 0.3 = 4.7; S = [0.5 + 0.6 * 4.7, 0.8 * 4.7]; o = S^T q = 3.76
    assert out[0, 0, 0] == pytest.approx(1.0) and out[1, 0, 0] == pytest.approx(3.76)
    # with beta = 1 and unit k, the state returns v exactly when asked with the key just written
    gen = torch.Generator().manual_seed(0)
    k = plain.unit(torch.randn(6, 1, 8, generator=gen, dtype=torch.float64) * 50)
    v = torch.randn(6, 2, 3, generator=gen, dtype=torch.float64)
    out = plain.delta_recurrence(k, k, v, torch.ones(6, 2, dtype=torch.float64), torch.rand(6, 2, generator=gen, dtype=torch.float64))
    assert torch.allclose(out, v, atol=1e-6)


def test_the_convolution_is_causal_and_its_last_tap_is_the_current_token():
    x = torch.tensor([[1.0], [10.0], [100.0]], dtype=torch.float64)
    taps = torch.tensor([[0.5, 0.0, 2.0]], dtype=torch.float64)
    y = plain.causal_conv_silu(x, taps)
    assert torch.allclose(y, plain.silu(torch.tensor([[2.0], [20.0], [200.5]], dtype=torch.float64)))


def test_a_layer_adds_the_normed_branch_times_the_multiplier():
    """One attention layer, one token: x1 = x0 + m * norm1(W_o v * p) with p = 1 / (1 + e^(sink - s))."""
    cfg = {"architecture": "Danonex", "vocab": 3, "width": 4, "norm": {"eps": 1e-6}, "residual_mult": 0.25,
           "logit_scale": 2.0, "layers": [M.layer(M.attention(1, 1, 2, 2, 1.0, softcap=None, rot_dims=None))]}
    gen = torch.Generator().manual_seed(1)
    w = {name: torch.randn(*shape, generator=gen, dtype=torch.float64)
         for name, shape in pae.expected_tensors(pae.read_config_dict(cfg).plan()).items()}
    logits, layers = plain.forward(w, cfg, [2], torch.float64, keep_layers=True)
    x0 = w["embed"][2]
    q = plain.rms_norm(w["l0.mix.q"] @ x0, w["l0.mix.q.norm"], 1e-6)
    k = plain.rms_norm(w["l0.mix.k"] @ x0, w["l0.mix.k.norm"], 1e-6)
    p = 1.0 / (1.0 + torch.exp(w["l0.mix.sink"][0] - q @ k))
    x1 = x0 + 0.25 * plain.rms_norm(w["l0.mix.o"] @ (p * (w["l0.mix.v"] @ x0)), w["l0.norm1"], 1e-6)
    assert torch.allclose(layers[0][0], x1, atol=1e-12)
    assert torch.allclose(logits[0], 2.0 * (w["embed"] @ plain.rms_norm(x1, w["final.norm"], 1e-6)), atol=1e-12)


def test_the_touchy_models_show_mistakes():
    """Leaving out a mechanism moves the logits of the test models far beyond the comparison bounds:
    the sink, the cap, the stretched frequencies, the decay."""
    tmp_cfg, length = M.P, 40
    gen = torch.Generator().manual_seed(3)
    shapes = pae.expected_tensors(pae.read_config_dict(tmp_cfg).plan())
    w = {}
    for name, shape in shapes.items():
        centre = float(getattr(shape, "centre", 0.0))
        std = next((v for end, v in M.STD.items() if end and name.endswith(end)), M.STD[""])
        w[name] = centre + (0.2 if centre else std) * torch.randn(*tuple(shape), generator=gen, dtype=torch.float64)
    tokens = M.tokens_for("P", length)
    base = plain.forward(w, tmp_cfg, tokens)
    top = float(base.abs().max())

    def moved(change):
        import copy
        cfg, w2 = copy.deepcopy(tmp_cfg), dict(w)
        change(cfg, w2)
        return float((plain.forward(w2, cfg, tokens) - base).abs().max()) / top

    assert moved(lambda c, w2: w2.update({"l1.mix.sink": w2["l1.mix.sink"] - 30.0})) > 0.01
    assert moved(lambda c, w2: c["layers"][1]["mixer"].update(softcap=None)) > 0.01
    assert moved(lambda c, w2: c["layers"][1]["mixer"]["rot"].update(scaling=None)) > 0.01
    assert moved(lambda c, w2: w2.update({"l0.mix.A_log": w2["l0.mix.A_log"] - 30.0})) > 0.01
    assert moved(lambda c, w2: c.update(residual_mult=0.9)) > 0.01
