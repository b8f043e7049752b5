"""The Figalorn configuration on the CPU: what config.json becomes, and what is refused."""
import copy

import pytest

from axon_amd.config import ConfigError, config_from_dict
from axon_amd.config.figalorn import FigalornConfig
from axon_amd.models import build_model_description
from figalorn_models import MODELS, config, diff, draw_weights, keyed, layer
from plain import figalorn_plain as P


def test_the_registry_finds_the_design_by_its_name():
    assert isinstance(config_from_dict(MODELS["A"]["cfg"]), FigalornConfig)


@pytest.mark.parametrize("name", sorted(MODELS))
def test_the_declared_tensors_are_the_checkpoints(name):
    cfg = MODELS[name]["cfg"]
    model = build_model_description(config_from_dict(cfg))
    declared = {d.name: tuple(d.shape) for d in model.tensors()}
    drawn = {k: tuple(v.shape) for k, v in draw_weights(cfg, 1).items()}
    assert declared == drawn


@pytest.mark.parametrize("name", sorted(MODELS))
def test_the_order_of_runs_is_the_plain_implementations(name):
    cfg = MODELS[name]["cfg"]
    model = build_model_description(config_from_dict(cfg))
    want = P.layer_order(cfg)
    assert [(r.layer, r.enter is not None) for r in model.order] == want
    assert len({r.cache for r in model.order}) == len(want)          # every run a cache of its own
    assert len(model.entries) == (1 if "loop" in cfg else 0)


def test_a_loop_of_no_passes_and_one_over_nothing():
    cfg = copy.deepcopy(MODELS["A"]["cfg"])
    cfg["loop"] = {"start": 1, "stop": 3, "times": 0}
    assert [r.layer for r in build_model_description(config_from_dict(cfg)).order] == [0, 3]
    cfg["loop"] = {"start": 2, "stop": 2, "times": 5}
    order = build_model_description(config_from_dict(cfg)).order
    assert [r.layer for r in order] == [0, 1, 2, 3] and all(r.enter is None for r in order)


def test_the_mixers_parameters_come_from_the_configuration():
    cfg = MODELS["A"]["cfg"]
    model = build_model_description(config_from_dict(cfg))
    keyed_mixer, diff_mixer = model.blocks[0].mixer, model.blocks[1].mixer
    assert (keyed_mixer.maps, keyed_mixer.values, keyed_mixer.mask, keyed_mixer.mask_size) == (1, "keys", "window", 24)
    assert keyed_mixer.qk_norm and not keyed_mixer.gate and not keyed_mixer.bias and keyed_mixer.softcap == 30.0
    assert keyed_mixer.position.pairing == "halves" and keyed_mixer.position.magnitude > 1.0
    assert (diff_mixer.maps, diff_mixer.values, diff_mixer.mask, diff_mixer.mask_size) == (2, "projected", "chunk", 40)
    assert diff_mixer.gate and diff_mixer.bias and not diff_mixer.qk_norm and diff_mixer.softcap == 0.0
    assert diff_mixer.position.pairing == "neighbours" and diff_mixer.position.magnitude == 1.0
    assert model.blocks[2].feed_forward is None and model.blocks[2].norm2 is None
    # caches: one row a position holds the keys of every kv head and map, and the values
    assert keyed_mixer.cache_spec().head_dim == 2 * 16 + 2 * 16 and keyed_mixer.cache_spec().window == 24
    assert diff_mixer.cache_spec().head_dim == 2 * 2 * 8 + 2 * 32 and diff_mixer.cache_spec().window == 40


def test_the_frequencies_are_the_plain_implementations():
    model = build_model_description(config_from_dict(MODELS["B"]["cfg"]))
    for block, entry in zip(model.blocks, MODELS["B"]["cfg"]["layers"]):
        rot, sc = entry["mixer"]["rot"], entry["mixer"]["rot"].get("scaling")
        got = block.mixer.position.frequencies().tolist()
        if entry["type"] == "attention":
            want = P.stretched_frequencies(rot["dims"], rot["base"], sc["factor"], sc["low"], sc["high"], sc["original"])
            assert block.mixer.position.magnitude == 1.0
        else:
            want, magnitude = P.ramped_frequencies(rot["dims"], rot["base"], sc["factor"], sc["original"], sc["fast"], sc["slow"])
            assert block.mixer.position.magnitude == pytest.approx(magnitude, rel=1e-15)
        assert got == pytest.approx(want, rel=1e-14)
        assert got != pytest.approx(P.base_frequencies(rot["dims"], rot["base"]), rel=1e-3)      # the scaling does something


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][0].update(type="attention_3"), "not a mixer"),
    (lambda c: c["layers"][1]["mixer"].pop("diff"), "diff"),
    (lambda c: c["layers"][0]["mixer"].update(vdim=8), "values that are the keys"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "not a multiple"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "not a feed-forward"),
    (lambda c: c["loop"].update(stop=9), "loop"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=40), "rotary_dim 40"),
])
def test_what_is_refused(change, message):
    cfg = copy.deepcopy(MODELS["A"]["cfg"])
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        build_model_description(config_from_dict(cfg))


def test_a_mixer_without_mask_rotation_or_bend():
    entry = keyed(heads=2, kv_heads=1, dim=8, window=5, rot_dims=4)
    for key in ("mask", "rot", "softcap"):
        entry["mixer"].pop(key)
    mixer = build_model_description(config_from_dict(config(16, 20, [layer(entry, None)]))).blocks[0].mixer
    assert (mixer.mask, mixer.position, mixer.softcap, mixer.cache_spec().window) == ("causal", None, 0.0, 0)
    entry = diff(heads=2, kv_heads=1, dim=8, vdim=4, chunk=5, rot_dims=4, scaling=None)
    mixer = build_model_description(config_from_dict(config(16, 20, [layer(entry, 8)]))).blocks[0].mixer
    assert mixer.position.scaling is None and mixer.position.frequencies().tolist() == pytest.approx(P.base_frequencies(4, 10000.0))


# --------------------------------------------------------------------------- pins of the plain implementation
def test_plain_pieces_reduce_to_library_routines():
    import torch
    g = torch.Generator().manual_seed(0)
    z = torch.randn(50, generator=g, dtype=torch.float64) * 3
    assert torch.allclose(P.gelu_erf(z), torch.nn.functional.gelu(z), atol=1e-12)
    assert torch.allclose(P.sigma(z), torch.sigmoid(z), atol=1e-12)
    x = torch.randn(4, 10, generator=g, dtype=torch.float64)
    assert torch.allclose(P.rms(x, 0.0).pow(2).mean(-1), torch.ones(4, dtype=torch.float64))
    assert torch.allclose(P.norm(x, torch.zeros(10, dtype=torch.float64), 1e-5), P.rms(x, 1e-5))      # a stored 0 is a gain of 1
    # either pairing is a complex product by exp(i p f_k), on its own places; the rest passes
    v = torch.randn(6, 3, 8, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 7, 100, 1000])
    f = [0.9, 0.05, 0.003]
    turn = torch.polar(torch.full((6, 3), 1.5, dtype=torch.float64), pos[:, None].double() * torch.tensor(f, dtype=torch.float64))[:, None, :]
    halves = P.turn(v, pos, f, "halves", 1.5)
    want = torch.complex(v[..., :3], v[..., 3:6]) * turn
    assert torch.allclose(halves[..., :3], want.real) and torch.allclose(halves[..., 3:6], want.imag)
    assert torch.equal(halves[..., 6:], v[..., 6:])
    near = P.turn(v, pos, f, "neighbours", 1.5)
    want = torch.complex(v[..., 0:6:2], v[..., 1:6:2]) * turn
    assert torch.allclose(near[..., 0:6:2], want.real) and torch.allclose(near[..., 1:6:2], want.imag)
    assert torch.equal(near[..., 6:], v[..., 6:]) and not torch.allclose(near, halves)
    # the masks, place by place
    assert P.window_mask(5, 2).int().tolist() == [[1, 0, 0, 0, 0], [1, 1, 0, 0, 0], [0, 1, 1, 0, 0], [0, 0, 1, 1, 0], [0, 0, 0, 1, 1]]
    assert P.chunk_mask(5, 2).int().tolist() == [[1, 0, 0, 0, 0], [1, 1, 0, 0, 0], [0, 0, 1, 0, 0], [0, 0, 1, 1, 0], [0, 0, 0, 0, 1]]


def test_plain_frequencies_at_their_corners():
    # stretched by wavelength: short waves kept, long ones divided, the blend continuous at both ends
    f = P.stretched_frequencies(64, 10000.0, 8.0, 1.0, 4.0, 512)
    base = P.base_frequencies(64, 10000.0)
    import math
    for got, b in zip(f, base):
        wave = 2 * math.pi / b
        if wave < 512 / 4.0:
            assert got == b
        elif wave > 512 / 1.0:
            assert got == b / 8.0
        else:
            assert b / 8.0 <= got <= b
    assert f[0] == base[0] and f[-1] == base[-1] / 8.0
    # ramped by pair index: the first pairs kept, the last divided by the factor, in between monotone
    f, magnitude = P.ramped_frequencies(64, 10000.0, 4.0, 2048, 32.0, 1.0)
    ratio = [b / g for g, b in zip(f, base)]
    assert ratio[0] == 1.0 and ratio[-1] == pytest.approx(4.0) and all(a <= b + 1e-12 for a, b in zip(ratio, ratio[1:]))
    assert magnitude == pytest.approx(0.1 * math.log(4.0) + 1.0)


def test_plain_mixers_behave_as_the_design_says():
    import torch
    cfg = config(16, 20, [layer(keyed(heads=2, kv_heads=1, dim=4, window=3, rot_dims=2), 8),
                          layer(diff(heads=2, kv_heads=2, dim=4, vdim=6, chunk=4, rot_dims=4), None)], loop=(0, 1, 2))
    W = {k: v.double() for k, v in draw_weights(cfg, 1).items()}
    g = torch.Generator().manual_seed(1)
    h = torch.randn(12, 16, generator=g, dtype=torch.float64)
    k, d = cfg["layers"][0]["mixer"], cfg["layers"][1]["mixer"]
    full = P.key_value_attention(h, W, "l0.mix.", k, 1e-5)
    # a window of 3 reaches back two positions: row 5 feels row 3 and not row 2
    far = h.clone()
    far[2] += 1.0
    moved = P.key_value_attention(far, W, "l0.mix.", k, 1e-5)
    assert torch.allclose(moved[5:], full[5:]) and not torch.allclose(moved[4], full[4])
    # chunks of 4: row 4 starts a chunk and feels nothing before it, row 3 ends one and feels row 0
    full = P.differential_attention(h, W, "l1.mix.", d, 1e-5)
    first = h.clone()
    first[0] += 1.0
    moved = P.differential_attention(first, W, "l1.mix.", d, 1e-5)
    assert torch.allclose(moved[4:], full[4:]) and not torch.allclose(moved[3], full[3])
    # a bend far above the scores changes nothing, one near them does
    loose = P.key_value_attention(h, W, "l0.mix.", dict(k, softcap=1e6), 1e-5)
    assert torch.allclose(loose, P.key_value_attention(h, W, "l0.mix.", dict(k, softcap=None), 1e-5))
    assert not torch.allclose(P.key_value_attention(h, W, "l0.mix.", dict(k, softcap=0.5), 1e-5), loose)
    # the loop: two passes of layer 0, each behind the rewrite of the stream; then layer 1
    assert P.layer_order(cfg) == [(0, True), (0, True), (1, False)]
    streams = []
    P.forward(cfg, W, list(range(7)), streams)
    x0 = W["embed"][torch.arange(7)]
    entered = torch.cat([x0, x0], dim=-1) @ W["loop.in"].T
    once = entered + P.key_value_attention(P.norm(entered, W["l0.norm1"], 1e-5), W, "l0.mix.", k, 1e-5)
    once = once + P.feed_forward(P.norm(once, W["l0.norm2"], 1e-5), W, "l0.mlp.")
    assert torch.allclose(streams[0], once)
    again = torch.cat([once, x0], dim=-1) @ W["loop.in"].T
    assert not torch.allclose(streams[1], streams[0])
    twice = again + P.key_value_attention(P.norm(again, W["l0.norm1"], 1e-5), W, "l0.mix.", k, 1e-5)
    twice = twice + P.feed_forward(P.norm(twice, W["l0.norm2"], 1e-5), W, "l0.mlp.")
    assert torch.allclose(streams[1], twice)


def test_the_command_line_writes_and_describes_a_model_of_the_design(tmp_path, capsys):
    import json
    from axon_amd.cli import main
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(MODELS["B"]["cfg"]))
    out = tmp_path / "model"
    assert main(["random-weights", str(cfg_path), str(out), "--seed", "3"]) == 0
    assert main(["info", str(out)]) == 0
    text = capsys.readouterr().out
    assert "architecture: Figalorn" in text and "window 7" in text and "window 13" in text
    from safetensors.torch import load_file
    names = set(load_file(str(out / "model.safetensors")))
    assert names == set(draw_weights(MODELS["B"]["cfg"], 0))
