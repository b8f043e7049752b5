"""The Pikesun configuration as data (no GPU): which class config.json selects, the tensors the
model declares, layers that run another layer's tensors, what is refused; and pins of the plain
implementation's pieces against library routines."""
import math

import pytest
import torch

from axon_amd.config import ConfigError, PikesunConfig, config_from_dict
from axon_amd.models import build_model_description
from pikesun_models import MODELS, att, config, dense, draw_weights, layer, moe, rec
from plain import pikesun_plain as P


def test_config_json_selects_the_class_and_describes_the_layers():
    cfg = MODELS["P"]["cfg"]
    c = config_from_dict(cfg)
    assert isinstance(c, PikesunConfig) and c.to_dict() == cfg
    spec = c.model_spec()
    # four entries, two with tensors of their own; the others run those with a cache or state of their own
    assert [l.prefix for l in spec.layers] == ["l0.", "l1."]
    assert [(r.layer, r.cache) for r in spec.order] == [(0, 0), (1, 1), (1, 2), (0, 3)]
    assert [l.block for l in spec.layers] == ["sublayer_norm"] * 2
    assert spec.embedding.params["scale"] == 4.0 and spec.layers[0].norm.params["residual_mult"] == 0.5
    m = spec.layers[0].mixer.params
    assert (m["window"], m["kv_rank"], m["rot_dim"], m["position"].params["theta"]) == (9, 20, 4, 100.0)
    model = build_model_description(c)
    plan = model.cache_plan
    assert [(s.entries, s.heads, s.head_dim, s.window, n) for s, n in zip(plan.group_specs, plan.group_layers)] == [(1, 1, 44, 9, 2)]
    assert plan.state_elems == [(2 * 3 * 72, "float32")] * 2
    assert [(b.group, b.index, b.state_index) for b in plan.bindings] == [(0, 0, -1), (-1, -1, 0), (-1, -1, 1), (0, 1, -1)]


@pytest.mark.parametrize("name", sorted(MODELS))
def test_the_declared_tensors_are_the_checkpoints(name):
    cfg = MODELS[name]["cfg"]
    declared = {d.name: tuple(d.shape) for d in build_model_description(config_from_dict(cfg)).tensors()}
    assert declared == {k: tuple(v.shape) for k, v in draw_weights(cfg, 0).items()}


def test_two_attention_layers_of_other_sizes_get_pools_of_their_own():
    plan = build_model_description(config_from_dict(MODELS["R"]["cfg"])).cache_plan
    assert [(s.head_dim, s.window) for s in plan.group_specs] == [(56, 0), (26, 33)] and plan.state_elems == [(2 * 64, "float32")]


def test_a_model_of_recurrences_alone_has_no_pages():
    plan = build_model_description(config_from_dict(MODELS["S"]["cfg"])).cache_plan
    assert plan.group_specs == [] and [e for e, _ in plan.state_elems] == [2 * 4 * 96, 2 * 2 * 160, 2 * 4 * 96]


def test_a_layer_without_a_feed_forward_and_defaults():
    cfg = config(32, 50, [layer(rec(32, 2, 2), None)])
    del cfg["embedding"], cfg["residual_mult"]
    c = config_from_dict(cfg)
    assert c.embedding_scale == 1.0 and c.residual_mult == 1.0
    model = build_model_description(c)
    assert model.blocks[0].feed_forward is None and model.blocks[0].norm2 is None
    assert sorted(d.name for d in model.tensors() if d.name.startswith("l0.norm")) == ["l0.norm1"]


@pytest.mark.parametrize("breaker,message", [
    (lambda c: c["layers"][0].update(type="mamba"), "is not a mixer of this design"),
    (lambda c: c["layers"][1]["mixer"].update(blocks=5), "does not split into 5 equal blocks"),
    (lambda c: c["layers"][2].update(weights_of=0), "does not name a layer of type rglru"),
    (lambda c: c["layers"][2].update(weights_of=2), "does not name a layer"),
    (lambda c: c["layers"][0]["mlp"].update(kind="glu"), "is not a feed-forward of this design"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=7), "7 of 6 experts"),
    (lambda c: c.pop("vocab"), "missing vocab"),
    (lambda c: c["norm"].pop("eps"), "missing eps"),
])
def test_what_cannot_run_is_refused_with_its_key(breaker, message):
    import copy
    cfg = copy.deepcopy(MODELS["P"]["cfg"])
    breaker(cfg)
    with pytest.raises(ConfigError, match=message):
        build_model_description(config_from_dict(cfg))


# --------------------------------------------------------------------------- pins of the plain implementation
def test_plain_pieces_reduce_to_library_routines():
    g = torch.Generator().manual_seed(0)
    z = torch.randn(50, generator=g, dtype=torch.float64) * 3
    assert torch.allclose(P.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"), atol=1e-12)
    assert torch.allclose(P.sigma(z), torch.sigmoid(z), atol=1e-12)
    x = torch.randn(4, 10, generator=g, dtype=torch.float64)
    assert torch.allclose(P.rms(x, torch.ones(10, dtype=torch.float64), 0.0).pow(2).mean(-1), torch.ones(4, dtype=torch.float64))
    # the rotation of pair (k, k + half) is a complex product by exp(i p f_k)
    v = torch.randn(6, 3, 8, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 7, 100, 1000])
    got = P.rotate(v, pos, 6, 50.0)
    f = torch.tensor([50.0 ** (-2.0 * k / 6) for k in range(3)], dtype=torch.float64)
    turned = torch.complex(v[..., :3], v[..., 3:6]) * torch.polar(torch.ones(6, 3, dtype=torch.float64), pos[:, None].double() * f)[:, None, :]
    assert torch.allclose(got[..., :3], turned.real) and torch.allclose(got[..., 3:6], turned.imag)
    assert torch.equal(got[..., 6:], v[..., 6:]) and torch.equal(got[0], v[0])
    # the convolution is the library's, with its taps in the same order
    xs, taps, bias = torch.randn(9, 5, generator=g, dtype=torch.float64), torch.randn(5, 3, generator=g, dtype=torch.float64), torch.randn(5, generator=g, dtype=torch.float64)
    lib = torch.nn.functional.conv1d(torch.nn.functional.pad(xs.T[None], (2, 0)), taps[:, None, :], bias, groups=5)[0].T
    assert torch.allclose(P.causal_conv(xs, taps, bias), lib)


def test_plain_mixers_behave_as_the_design_says():
    cfg = config(16, 20, [layer(att(heads=2, dim=4, rot_dim=4, vdim=6, kv_rank=8, q_rank=6, window=5), moe(4, 4, 8, 1.0)),
                          layer(rec(24, 2, 3), dense(12))])
    W = {k: v.double() for k, v in draw_weights(cfg, 1).items()}
    g = torch.Generator().manual_seed(1)
    h = torch.randn(12, 16, generator=g, dtype=torch.float64)
    c = cfg["layers"][0]["mixer"]
    full = P.latent_attention(W, "l0.mix.", c, h, 1e-6)
    # a window reaches back size - 1 positions: rows before that do not feel it, a row does not feel what lies further back
    assert torch.allclose(full[:5], P.latent_attention(W, "l0.mix.", c, h, 1e-6, window_override=0)[:5])
    far = h.clone()
    far[2] += 1.0
    moved = P.latent_attention(W, "l0.mix.", c, far, 1e-6)
    assert torch.allclose(moved[7:], full[7:]) and not torch.allclose(moved[6], full[6])
    # every expert chosen: the softmax over all logits weighs them all
    m = cfg["layers"][0]["mlp"]
    z = torch.softmax(h @ W["l0.mlp.router"].T, -1)
    mix = sum(z[:, e:e + 1] * P.clamped_unit(W, f"l0.mlp.e{e}.", h, 1.0) for e in range(4))
    assert torch.allclose(P.routed_ff(W, "l0.mlp.", m, h), mix)
    # the recurrence: a later token does not move an earlier row; from its state, the second half continues the first
    r = cfg["layers"][1]["mixer"]
    out = P.gated_recurrence(W, "l1.mix.", r, h)
    later = h.clone()
    later[9] += 1.0
    assert torch.allclose(P.gated_recurrence(W, "l1.mix.", r, later)[:9], out[:9])
    a = torch.exp(-8.0 * torch.log1p(torch.exp(W["l1.mix.lam"])))        # r = 1: the fastest decay
    assert float(a.min()) > 0 and float(a.max()) < 1


def test_the_command_line_writes_and_describes_a_model_of_the_design(tmp_path, capsys):
    import json
    from axon_amd.cli import main
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(MODELS["R"]["cfg"]))
    out = tmp_path / "model"
    assert main(["random-weights", str(cfg_path), str(out), "--seed", "3"]) == 0
    assert main(["info", str(out)]) == 0
    text = capsys.readouterr().out
    assert "architecture: Pikesun" in text and "cache group: 1 layers x 1 x 1 heads x 56" in text and "window 33" in text
    from safetensors.torch import load_file
    names = set(load_file(str(out / "model.safetensors")))
    assert names == set(draw_weights(MODELS["R"]["cfg"], 0))
