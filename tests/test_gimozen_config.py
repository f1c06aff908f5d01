"""The Gimozen configuration, its registry entry and the tensors its model declares (no GPU)."""

import copy

import numpy as np
import pytest

import plain_gimozen as plain
from gimozen_cases import CASES, attention_layer, latent_layer, model
from mini_llm_amd.config import ConfigError, GimozenConfig, config_from_dict
from mini_llm_amd.engine.loading import build_model


@pytest.mark.parametrize("name", list(CASES))
def test_round_trip_and_tensor_names(name):
    raw = CASES[name]
    config = config_from_dict(raw)
    assert isinstance(config, GimozenConfig) and config_from_dict(config.to_dict()) == config
    built = build_model(config, "float32")
    specs = {n: tuple(s.shape) for n, s in built.named_tensor_specs().items()}
    assert specs == plain.tensor_shapes(raw)
    calls = built.schedule
    for index, layer in enumerate(raw["layers"]):
        source = layer["mixer"].get("kv_from")
        assert calls[index].cache == (index if source is None else source) and calls[index].write_cache == (source is None)
    # a borrowed latent has no pages of its own; latent layers keep one plane
    latent = [g for g in built.cache_groups() if g.planes == 1]
    own = [i for i, layer in enumerate(raw["layers"]) if layer["type"] == "latent_attention" and "kv_from" not in layer["mixer"]]
    assert sorted(l for g in latent for l in g.layers) == own


def test_what_the_configuration_refuses():
    bad = copy.deepcopy(CASES["mixed"])
    bad["layers"][2]["mixer"]["kv_from"] = 1          # an attention layer keeps no latent
    with pytest.raises(ConfigError, match="kv_from"):
        config_from_dict(bad)
    bad = copy.deepcopy(CASES["mixed"])
    bad["layers"][2]["mixer"]["kv_rank"] += 8          # the borrowed rows have another size
    with pytest.raises(ConfigError, match="differ"):
        config_from_dict(bad)
    bad = copy.deepcopy(CASES["mixed"])
    bad["layers"][0]["mixer"]["kv_from"] = 0           # not an earlier layer
    with pytest.raises(ConfigError, match="kv_from"):
        config_from_dict(bad)
    bad = copy.deepcopy(CASES["attention"])
    bad["layers"][0]["mixer"]["kv_heads"] = 2
    with pytest.raises(ConfigError, match="divide"):
        config_from_dict(bad)
    bad = copy.deepcopy(CASES["attention"])
    bad["layers"][0]["type"] = "recurrence"
    with pytest.raises(ConfigError, match="unknown type"):
        config_from_dict(bad)
    bad = copy.deepcopy(CASES["latent"])
    bad["layers"][0]["mixer"]["rot"]["dims"] = 18
    with pytest.raises(ConfigError, match="rot.dims"):
        config_from_dict(bad)
    with pytest.raises(ConfigError):
        config_from_dict({"architecture": "Gimozen", "layers": []})


def test_the_plain_implementation_holds_its_own_invariants():
    config = model([latent_layer(), attention_layer(), latent_layer(kv_from=0)])
    weights = plain.random_weights(config, 1)
    tokens = list(np.random.default_rng(0).integers(0, config["vocab"], 40))
    whole = plain.forward(config, weights, tokens)
    np.testing.assert_allclose(plain.forward(config, weights, tokens[:17]), whole[:17], atol=1e-10)   # causal
    # the sink only shrinks the weights: with a sink far below every score the softmax is the ordinary one
    scores = np.random.default_rng(1).normal(0, 1, (3, 5))
    visible = plain.causal_mask(3, 5, first_position=2)
    np.testing.assert_allclose(plain.softmax_rows(scores, visible, sink=-80.0), plain.softmax_rows(scores, visible), atol=1e-12)
    assert (plain.softmax_rows(scores, visible, sink=0.0).sum(axis=1) < 1).all()
    # a rotation keeps lengths up to its magnitude, and position 0 is the identity times the magnitude
    rot = {"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0}}
    x = np.random.default_rng(2).normal(0, 1, (6, 8))
    turned = plain.rotate_half(x, np.arange(6), rot)
    magnitude = plain.rotary_frequencies(rot)[1]
    np.testing.assert_allclose(np.linalg.norm(turned, axis=1), np.linalg.norm(x, axis=1) * magnitude, rtol=1e-12)
    np.testing.assert_allclose(turned[0], x[0] * magnitude, rtol=1e-12)
    # relative positions: the score of a rotated pair depends on the distance alone
    a, b = x[:1], x[1:2]
    near = plain.rotate_half(a, [3], rot) @ plain.rotate_half(b, [1], rot).T
    far = plain.rotate_half(a, [10], rot) @ plain.rotate_half(b, [8], rot).T
    np.testing.assert_allclose(near, far, rtol=1e-10)
