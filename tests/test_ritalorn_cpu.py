"""Ritalorn on the CPU: the config reader and the plan it gives, the tensors the parts declare, what
the layers keep in the cache, and the plain implementation pinned by closed forms and by invariants
(so that the oracle the GPU tests compare with is itself checked)."""

import copy
import math

import pytest
import torch

import paged_attention_engine_amd as pae
from paged_attention_engine_amd.config import ConfigError
from tests import ritalorn_models as M
from tests.plain import ritalorn_plain as plain


# ----------------------------------------------------------------------------- configuration


def test_the_reader_is_chosen_by_the_architecture_key_and_round_trips():
    for name, cfg in M.CONFIGS.items():
        typed = pae.read_config_dict(cfg)
        assert type(typed).__name__ == "RitalornConfig"
        assert pae.read_config_dict(typed.to_json_dict()) == typed


def test_every_size_and_constant_comes_from_the_config():
    plan = pae.read_config_dict(M.A).plan()
    assert (plan.hidden_size, plan.vocab_size, plan.streams, plan.logit_softcap, plan.head_name) == (64, 301, 3, 12.0, "head")
    assert [(e.layer, e.cache_from) for e in plan.schedule] == [(0, None), (1, None), (2, 1), (3, None)]
    first, second, third, fourth = plan.layers
    assert first.arrangement == "hyper" and first.streams == 3 and first.layer_scale_names == ("ls1", "ls2")
    m = first.mixer
    assert (m.kind, m.num_heads, m.nope_dim, m.rope_dim, m.value_dim, m.kv_rank, m.scale, m.window, m.mask, m.norm_eps) == (
        "latent_attention", 3, 16, 8, 24, 40, 0.3, 20, "window", 2e-6)
    assert (m.position.kind, m.position.rotary_dim, m.position.theta) == ("interleaved_rope", 8, 1000.0)
    a = second.mixer
    assert (a.kind, a.num_heads, a.num_kv_heads, a.head_dim, a.v_dim, a.scale, a.window, a.mask, a.conv_taps) == (
        "attention", 6, 2, 32, 16, 0.4, 50, "chunk", 4)
    assert a.qkv_bias and a.out_bias and a.qk_norm == "head" and a.qk_norm_eps == 2e-6 and a.gate_name == "g"
    assert a.distance_slope_base == 8.0 and a.position is None and a.own_kv and a.convolved and not a.plain
    b = third.mixer
    assert not b.own_kv and (b.window, b.conv_taps, b.scale) == (33, 2, 0.25)
    assert third.feed_forward is None and third.feed_forward_norm is None
    assert first.feed_forward.kind == "swiglu" and first.feed_forward.activation == "gelu_tanh"
    assert fourth.mixer.position.rotary_dim == 8 and fourth.mixer.rope_dim == 16
    # no mask: every earlier key; no cap: none
    assert pae.read_config_dict(M.C).plan().layers[3].mixer.window is None
    assert pae.read_config_dict(M.E).plan().layers[2].mixer.window is None
    assert pae.read_config_dict(M.B).plan().logit_softcap is None and pae.read_config_dict(M.B).plan().streams == 1


def test_declared_tensors_carry_the_designs_names_and_shapes():
    shapes = pae.expected_tensors(pae.read_config_dict(M.A).plan())
    assert shapes["embed"] == (301, 64) and shapes["head"] == (301, 64) and tuple(shapes["final.norm"]) == (64,)
    assert shapes["l0.mix.q"] == (3 * 24, 64) and shapes["l0.mix.dkv"] == (48, 64) and tuple(shapes["l0.mix.dkv.norm"]) == (40,)
    assert shapes["l0.mix.uk"] == (48, 40) and shapes["l0.mix.uv"] == (72, 40) and shapes["l0.mix.o"] == (64, 72)
    assert shapes["l1.mix.q"] == (192, 64) and shapes["l1.mix.k"] == (64, 64) and shapes["l1.mix.v"] == (32, 64)
    assert shapes["l1.mix.q.b"] == (192,) and shapes["l1.mix.v.b"] == (32,) and shapes["l1.mix.o.b"] == (64,)
    assert shapes["l1.mix.q.conv"] == (192, 4) and shapes["l1.mix.k.conv"] == (64, 4) and shapes["l1.mix.v.conv"] == (32, 4)
    assert shapes["l1.mix.g"] == (96, 64) and shapes["l1.mix.o"] == (64, 96) and "l1.mix.g.b" not in shapes
    # a layer that reads another's keys and values has the query side only
    assert shapes["l2.mix.q"] == (192, 64) and shapes["l2.mix.q.conv"] == (192, 2) and shapes["l2.mix.g"] == (96, 64)
    assert not any(name.startswith("l2.mix.k") or name.startswith("l2.mix.v") for name in shapes)
    for q in ("hc1", "hc2"):
        assert shapes[f"l0.{q}.in"] == (3,) and shapes[f"l0.{q}.out"] == (3,) and shapes[f"l0.{q}.mix"] == (3, 3)
    assert tuple(shapes["l0.ls1"]) == (64,) and tuple(shapes["l0.ls2"]) == (64,)
    assert shapes["l0.mlp.gate"] == (96, 64) and shapes["l0.mlp.up"] == (96, 64) and shapes["l0.mlp.down"] == (64, 96)
    assert "l2.mlp.up" not in shapes and "l2.norm2" not in shapes and "l2.hc2.in" not in shapes and "l2.ls2" not in shapes
    assert "l2.hc1.in" in shapes and "l2.ls1" in shapes


@pytest.mark.parametrize("damage,needle", [
    (lambda c: c["layers"][0].update(type="conv"), "unknown mixer type"),
    (lambda c: c["layers"][1]["mixer"].pop("vdim"), "vdim"),
    (lambda c: c["layers"][1]["mixer"].update(heads=5), "not a multiple"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10), "rot.dims"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "unknown kind"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "earlier layer"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=0), "keys and values of its own"),
    (lambda c: c["layers"][2]["mixer"].update(dim=16), "differs from that of layer"),
    (lambda c: c.pop("streams"), "streams"),
    (lambda c: c.update(streams=9), "up to 8"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_a_faulty_config_is_refused_with_the_key_named(damage, needle):
    cfg = copy.deepcopy(M.A)
    damage(cfg)
    with pytest.raises(ConfigError, match=needle):
        pae.read_config_dict(cfg)


def test_random_weights_make_a_folder_the_loader_accepts(tmp_path):
    folder = M.make_folder(tmp_path, "D")
    cfg, tensors = M.read_folder(folder)
    declared = pae.expected_tensors(pae.read_config_dict(cfg).plan())
    assert cfg["architecture"] == "Ritalorn" and set(tensors) == set(declared)
    got = pae.load_weights(folder, declared)
    assert torch.equal(got["l0.hc1.mix"], tensors["l0.hc1.mix"]) and got["l0.hc1.mix"].shape == (4, 4)


# ----------------------------------------------------------------------------- what the layers keep


def test_pages_state_and_borrowed_pages():
    """Latent layers keep one row per token and give pages back behind their window; attention layers keep keys and
    values and the convolutions' last inputs, a reader of another layer's pages only those of its queries."""
    model = pae.Model(pae.read_config_dict(M.A).plan(), torch.float32, "cpu")
    paged, states = model.cache_specs()
    assert [t.name for t in paged[0].tensors] == ["latent"] and paged[0].tensors[0].shape(16) == (16, 48) and paged[0].window == 20
    assert [t.name for t in paged[1].tensors] == ["k", "v"] and paged[1].window is None  # a reader may have another mask
    assert paged[2] is None and paged[3].window == 7
    assert states[0] is None and states[3] is None
    assert states[1].shape == (3, 192 + 64 + 32) and states[2].shape == (1, 192)
    cache = model.new_cache(16, 8, 2)
    assert cache.group_of(2) is None and cache.state_of(2).shape == (3, 1, 192) and cache.state_of(1).shape == (3, 3, 288)
    # one tap: nothing to remember
    model = pae.Model(pae.read_config_dict(M.B).plan(), torch.float32, "cpu")
    assert model.cache_specs()[1][0] is None and model.cache_specs()[1][2].shape == (2, 144)
    # a window's pages come back, a chunked layer's do not
    assert cache.create_sequence(1) and cache.reserve(1, 100).ok
    free_before = cache.free_blocks()
    assert cache.release_passed(1) > 0
    latent_group, kv_group = cache.group_of(0), cache.group_of(1)
    assert cache.free_blocks()[latent_group] > free_before[latent_group] and cache.free_blocks()[kv_group] == free_before[kv_group]


# ----------------------------------------------------------------------------- the plain implementation


def test_the_tanh_gelu_and_the_norm_by_hand():
    z = torch.tensor([-2.0, 0.0, 0.5, 3.0], dtype=torch.float64)
    want = [0.5 * v * (1 + math.tanh(math.sqrt(2 / math.pi) * (v + 0.044715 * v ** 3))) for v in z.tolist()]
    assert torch.allclose(plain.gelu_tanh(z), torch.tensor(want, dtype=torch.float64), atol=1e-15)
    x = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    assert torch.allclose(plain.rms_norm(x, None, 0.5), x / math.sqrt(12.5 + 0.5))  # eps inside the root
    assert torch.allclose(plain.rms_norm(x, torch.tensor([2.0, 0.5], dtype=torch.float64), 0.5), x / math.sqrt(13.0) * torch.tensor([2.0, 0.5]))


def test_the_convolution_is_causal_and_its_last_tap_is_the_current_token():
    u = torch.arange(1.0, 7.0, dtype=torch.float64).view(6, 1)
    taps = torch.tensor([[100.0, 10.0, 1.0]], dtype=torch.float64)
    assert plain.causal_conv(u, taps).view(-1).tolist() == [1.0, 12.0, 123.0, 234.0, 345.0, 456.0]
    assert torch.equal(plain.causal_conv(u, torch.tensor([[2.0]], dtype=torch.float64)), 2 * u)


def test_the_rotation_turns_interleaved_pairs_and_leaves_the_rest():
    x = torch.tensor([[[1.0, 0.0, 0.0, 2.0, 9.0, 8.0]]], dtype=torch.float64)
    out = plain.rotate_pairs(x, torch.tensor([3]), 10.0, 4)
    f1 = 10.0 ** (-2.0 / 4)
    want = [math.cos(3.0), math.sin(3.0), -2 * math.sin(3 * f1), 2 * math.cos(3 * f1), 9.0, 8.0]
    assert torch.allclose(out[0, 0], torch.tensor(want, dtype=torch.float64))
    assert torch.equal(plain.rotate_pairs(x, torch.tensor([0]), 10.0, 4), x)  # position 0 turns nothing


def test_masks_slopes_and_the_softmax_by_hand():
    assert [plain.visible(7, j, "chunk", 4) for j in range(9)] == [False] * 4 + [True] * 4 + [False]
    assert [plain.visible(8, j, "chunk", 4) for j in range(9)] == [False] * 8 + [True]       # a chunk's first token sees itself alone
    assert [plain.visible(7, j, "window", 3) for j in range(9)] == [False] * 5 + [True] * 3 + [False]
    assert all(plain.visible(7, j, "window", None) for j in range(8))
    assert plain.distance_slopes(4) == [2.0 ** -2, 2.0 ** -4, 2.0 ** -6, 2.0 ** -8] and plain.distance_slopes(1) == [2.0 ** -8]
    # equal keys: the weights are softmax(-slope * distance) over the visible ones
    q = torch.ones(6, 2, dtype=torch.float64)
    k = torch.ones(6, 2, dtype=torch.float64)
    v = torch.eye(6, dtype=torch.float64)
    out = plain.attend(q, k, v, 0.5, "chunk", 4, slope=0.3)
    w = torch.softmax(torch.tensor([-0.9, -0.6, -0.3, 0.0], dtype=torch.float64), 0)
    assert torch.allclose(out[3, :4], w) and float(out[3, 4:].abs().sum()) == 0.0
    w = torch.softmax(torch.tensor([-0.3, 0.0], dtype=torch.float64), 0)
    assert torch.allclose(out[5, 4:], w) and float(out[5, :4].abs().sum()) == 0.0


def test_the_copies_of_the_stream_by_hand():
    X = torch.tensor([[[1.0, 2.0]], [[10.0, 20.0]]], dtype=torch.float64)  # two copies, one token, width 2
    w = {"p.in": torch.tensor([0.5, -1.0], dtype=torch.float64), "p.out": torch.tensor([2.0, 3.0], dtype=torch.float64),
         "p.mix": torch.tensor([[1.0, 2.0], [0.0, -1.0]], dtype=torch.float64)}  # [from, to]
    seen = []
    new = plain.hyper_sublayer(X, w, "p.", lambda u: (seen.append(u), torch.tensor([[1.0, 1.0]], dtype=torch.float64))[1])
    assert torch.equal(seen[0], torch.tensor([[-9.5, -19.0]], dtype=torch.float64))
    assert torch.equal(new[0], torch.tensor([[1.0 + 2.0, 2.0 + 2.0]], dtype=torch.float64))                  # mix[0, 0] x0 + mix[1, 0] x1 + out[0] y
    assert torch.equal(new[1], torch.tensor([[2.0 - 10.0 + 3.0, 4.0 - 20.0 + 3.0]], dtype=torch.float64))    # mix[0, 1] x0 + mix[1, 1] x1 + out[1] y


def test_the_folded_query_scores_what_the_heads_keys_score():
    """q . (W c) = (W^T q) . c: the identity the engine's latent attention rests on, in the oracle's numbers."""
    gen = torch.Generator().manual_seed(0)
    W, c, q = (torch.randn(*s, generator=gen, dtype=torch.float64) for s in ((6, 9), (9,), (6,)))
    assert abs(float(q @ (W @ c)) - float((W.T @ q) @ c)) < 1e-12


def test_the_test_models_show_mistakes(tmp_path):
    """Leaving a mechanism out of the plain implementation moves the test models' logits far beyond the
    tolerances of the GPU tests: the random weights hide nothing."""
    folder = M.make_folder(tmp_path, "A")
    cfg, weights = M.read_folder(folder)
    tokens = M.tokens_for("A", 80)
    want = plain.forward(weights, cfg, tokens)
    top = float(want.abs().max())

    def moved(change):
        c, w = copy.deepcopy(cfg), dict(weights)
        change(c, w)
        return float((plain.forward(w, c, tokens) - want).abs().max()) / top

    assert moved(lambda c, w: c["layers"][1]["mixer"]["mask"].update(size=51)) > 1e-3          # a chunk one token longer
    assert moved(lambda c, w: c["layers"][0]["mixer"]["mask"].update(size=19)) > 1e-3          # a window one token shorter
    assert moved(lambda c, w: c["layers"][2]["mixer"]["mask"].update(size=50)) > 1e-3          # the reader under its source's mask
    assert moved(lambda c, w: w.update({"l1.mix.q.conv": torch.roll(w["l1.mix.q.conv"], 1, 1)})) > 1e-2   # taps in the wrong order
    assert moved(lambda c, w: w.update({"l1.mix.k.b": torch.zeros_like(w["l1.mix.k.b"])})) > 1e-3         # a bias left out
    assert moved(lambda c, w: w.update({"l2.mix.g": torch.zeros_like(w["l2.mix.g"])})) > 1e-3             # the gate left out
    assert moved(lambda c, w: c["layers"][0]["mixer"]["rot"].update(base=10.0)) > 1e-3                    # another rotation
    assert moved(lambda c, w: w.update({"l0.hc1.mix": w["l0.hc1.mix"].T.contiguous()})) > 1e-2            # [to, from] for [from, to]
    assert moved(lambda c, w: w.update({"l0.ls1": torch.ones_like(w["l0.ls1"])})) > 1e-3                  # the scale left out
    assert moved(lambda c, w: c.update(logit_softcap=None)) > 1e-3
    old = plain.SLOPE_BASE
    try:
        plain.SLOPE_BASE = 0.0
        assert float((plain.forward(weights, cfg, tokens) - want).abs().max()) / top > 1e-3          # the distance bias left out
    finally:
        plain.SLOPE_BASE = old
