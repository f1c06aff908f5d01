"""The Ketolix configuration, its registry entry, the tensors, cache groups and state its model declares, and the plain
implementation's own mechanisms against each other (no GPU)."""

import copy

import numpy as np
import pytest

import plain_ketolix as plain
from ketolix_cases import CASES, attention_layer, mlstm_layer, model, parallel_layer, rot
from mini_llm_amd.config import ConfigError, KetolixConfig, config_from_dict
from mini_llm_amd.engine.loading import build_model


@pytest.mark.parametrize("name", list(CASES))
def test_round_trip_tensor_names_cache_and_state(name):
    raw = CASES[name]
    config = config_from_dict(raw)
    assert isinstance(config, KetolixConfig) and config_from_dict(config.to_dict()) == config
    built = build_model(config, "float32")
    assert {n: tuple(s.shape) for n, s in built.named_tensor_specs().items()} == plain.tensor_shapes(raw)
    paged = sorted(layer for group in built.cache_groups() for layer in group.layers)
    assert paged == [i for i, layer in enumerate(raw["layers"]) if layer["type"] != "mlstm"]   # attention, alone or beside a recurrence
    for group in built.cache_groups():
        for layer in group.layers:
            mixer = raw["layers"][layer]["mixer"]
            mixer = mixer.get("left", mixer)
            assert group.window == (mixer.get("mask") or {}).get("size") and group.n_kv_heads == mixer["kv_heads"]
            assert group.head_size == -(-max(mixer["dim"], mixer["vdim"]) // 16) * 16
    state = built.state_needs()
    for index, layer in enumerate(raw["layers"]):
        m = layer["mixer"]
        if layer["type"] == "mlstm":
            assert state[index].shape == (m["heads"] * (m["dim"] * m["vdim"] + m["dim"] + 1),)
        elif layer["type"] == "parallel":
            left, right = m["left"], m["right"]
            kept = (left.get("conv", 1) - 1) * (left["heads"] + left["kv_heads"]) * left["dim"] if left.get("conv") else 0
            assert state[index].shape == (kept + right["heads"] * right["dim"] * right["vdim"],)
        else:
            assert index not in state
    assert built.all_graph_safe() and built.max_positions() is None


def test_what_the_configuration_refuses():
    def broken(change, match):
        bad = copy.deepcopy(CASES["mixed"])
        change(bad)
        with pytest.raises(ConfigError, match=match):
            config_from_dict(bad)

    broken(lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "divide")
    broken(lambda c: c["layers"][0].update(type="convolution"), "unknown type")
    broken(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "rot.dims")
    broken(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "not even")
    broken(lambda c: c["layers"][2]["mixer"].update(vdim=8), "mixed")              # values of another size cannot be mixed with the first layer's
    broken(lambda c: c["layers"][3]["mixer"]["right"].update(decay=[0.5]), "decay")   # one number a head
    broken(lambda c: c["layers"][3]["mixer"]["left"].update(vdim=8), "values are the keys")
    broken(lambda c: c["layers"][3]["mixer"]["left"].update(conv=40), "taps")
    broken(lambda c: c["layers"][1]["mixer"].update(dim=4096, vdim=64), "recurrence")
    broken(lambda c: c["layers"][1]["mixer"].update(gate_cap=0.0), "gate_cap")
    broken(lambda c: c["layers"][0]["mixer"].update(softcap=-1.0), "softcap")
    broken(lambda c: c["layers"][1].update(mlp={"kind": "routed", "ff": 8}), "mlp.kind")
    broken(lambda c: c.update(norm={"eps": 0.0}), "eps")
    with pytest.raises(ConfigError):
        config_from_dict({"architecture": "Ketolix", "layers": []})


def test_rotation_frequencies_of_the_part_are_the_plain_ones():
    for raw in CASES.values():
        built = build_model(config_from_dict(raw), "float32")
        for index, layer in enumerate(raw["layers"]):
            mixer = built.blocks[index].mixer
            mixer = getattr(mixer, "left", mixer)
            described = layer["mixer"].get("left", layer["mixer"]).get("rot")
            if layer["type"] == "mlstm":
                continue
            if described:
                assert mixer.rotary.pairing == "neighbours"
                np.testing.assert_allclose(mixer.rotary.values, plain.rotary_frequencies(described), rtol=1e-13)
            else:
                assert mixer.rotary is None


# -- the plain implementation's mechanisms against each other ---------------------------------------------------------------
def test_the_matrix_memory_is_attention_with_decaying_weights():
    # unrolled, the recurrence says: o_t = sum_s exp(F_t - F_s + i_s - m_t) (q_t . k_s) v_s / (max(|same with v = 1|, exp(-m_t)) + 1e-6) with F the
    # running sum of the log forget gates and m_t = max(F_t, max_s (F_t - F_s + i_s))
    rng = np.random.default_rng(0)
    T, dim, vdim = 40, 6, 5
    q, k, v = rng.normal(0, 1, (T, 1, dim)), rng.normal(0, 1, (T, 1, dim)), rng.normal(0, 1, (T, 1, vdim))
    gi, gf = rng.normal(0, 2, (T, 1)), plain.log_sigmoid(rng.normal(2, 2, (T, 1)))
    got = plain.mlstm_recurrence(q, k, v, gi, gf)[:, 0]
    F = np.cumsum(gf[:, 0])
    for t in range(T):
        reach = F[t] - F[: t + 1] + gi[: t + 1, 0]
        m = max(F[t], reach.max())
        w = np.exp(reach - m) * (k[: t + 1, 0] @ q[t, 0])
        np.testing.assert_allclose(got[t], (w @ v[: t + 1, 0]) / (max(abs(w.sum()), np.exp(-m)) + 1e-6), rtol=1e-9, atol=1e-12)


def test_the_decayed_recurrence_is_attention_with_powers_of_the_decay():
    rng = np.random.default_rng(1)
    T, dim, vdim = 30, 4, 3
    q, k, v = rng.normal(0, 1, (T, 2, dim)), rng.normal(0, 1, (T, 2, dim)), rng.normal(0, 1, (T, 2, vdim))
    decay = np.array([0.5, 0.99])
    got = plain.decayed_recurrence(q, k, v, decay)
    for h in range(2):
        for t in range(T):
            w = decay[h] ** (t - np.arange(t + 1)) * (k[: t + 1, h] @ q[t, h])
            np.testing.assert_allclose(got[t, h], w @ v[: t + 1, h], rtol=1e-9, atol=1e-12)


def test_rotation_window_sink_and_convolution_of_the_plain_implementation():
    rng = np.random.default_rng(2)
    x = rng.normal(0, 1, (5, 2, 8))
    turned = plain.rotate_pairs(x, [0, 1, 2, 3, 100], rot(4, 100.0))
    np.testing.assert_allclose(turned[0], x[0])                                        # position 0 turns nothing
    np.testing.assert_allclose(turned[..., 4:], x[..., 4:])                            # beyond rot.dims nothing turns
    np.testing.assert_allclose((turned[..., :2] ** 2).sum(-1), (x[..., :2] ** 2).sum(-1))   # a pair keeps its length: elements 0 and 1 are one
    a = plain.rotate_pairs(x[:1], [7], rot(8, 50.0))[0, 0] @ plain.rotate_pairs(x[1:2], [4], rot(8, 50.0))[0, 0]
    b = plain.rotate_pairs(x[:1], [13], rot(8, 50.0))[0, 0] @ plain.rotate_pairs(x[1:2], [10], rot(8, 50.0))[0, 0]
    np.testing.assert_allclose(a, b)                                                   # scores depend on the distance alone
    q, k, v = rng.normal(0, 1, (9, 1, 4)), rng.normal(0, 1, (9, 1, 4)), rng.normal(0, 1, (9, 1, 3))
    seen = plain.windowed_attention(q, k, v, 1.0, window=3)
    k2, v2 = k.copy(), v.copy()
    k2[:6], v2[:6] = 9.0, 9.0
    np.testing.assert_allclose(plain.windowed_attention(q, k2, v2, 1.0, window=3)[8], seen[8])   # position 8 sees 6, 7, 8
    assert np.abs(plain.windowed_attention(q, k2, v2, 1.0, window=4)[8] - seen[8]).max() > 1e-3
    plain_out = plain.windowed_attention(q, k, v, 1.0)
    with_sink = plain.windowed_attention(q, k, v, 1.0, sinks=np.array([0.0]))
    np.testing.assert_allclose(with_sink[0], plain_out[0] * np.exp(k[0, 0] @ q[0, 0]) / (np.exp(k[0, 0] @ q[0, 0]) + 1.0))
    u, w = rng.normal(0, 1, (6, 2)), rng.normal(0, 1, (2, 3))
    y = plain.short_convolution(u, w)
    np.testing.assert_allclose(y[0], w[:, 2] * u[0])
    np.testing.assert_allclose(y[4], w[:, 0] * u[2] + w[:, 1] * u[3] + w[:, 2] * u[4])


def test_the_plain_model_reads_the_stream_itself_and_norms_each_branch():
    raw = model([mlstm_layer(heads=1, dim=4, vdim=4, ff=8), attention_layer(heads=1, kv_heads=1, dim=4, vdim=4, window=None, ff=None),
                 parallel_layer(heads=1, kv_heads=1, dim=4, conv=2, right_heads=1, right_dim=4, right_vdim=4, decay=(0.9,), ff=8)], width=8, vocab=11)
    weights = plain.as_float64(plain.random_weights(raw, 3))
    layers = []
    logits = plain.forward(raw, weights, [1, 2, 3, 4], layers_out=layers)
    assert logits.shape == (4, 11) and len(layers) == 3
    # a later token changes nothing before it; every branch enters with the size its norm's gains give it
    again = plain.forward(raw, weights, [1, 2, 3, 9])
    np.testing.assert_allclose(again[:3], logits[:3])
    x0 = weights["embed"][[1, 2, 3, 4]]
    branch = plain.mlstm_mixer(x0, {n[len("l0.mix."):]: t for n, t in weights.items() if n.startswith("l0.mix.")}, raw["layers"][0]["mixer"], 1e-5)
    x1 = x0 + plain.rms_unit(branch, 1e-5) * weights["l0.norm1"]
    mlp = {n[len("l0.mlp."):]: t for n, t in weights.items() if n.startswith("l0.mlp.")}
    np.testing.assert_allclose(layers[0], x1 + plain.rms_unit(plain.dense_feed_forward(x1, mlp), 1e-5) * weights["l0.norm2"])
    assert plain.greedy(raw, weights, [1, 2], 3)[:2] == plain.greedy(raw, weights, [1, 2], 2)
