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
