"""Host-side checks of the Dezudra design: its configuration and tensor names, what its parts keep between steps,
and the plain implementation's own mechanisms on cases worked out by hand."""
import copy
import math

import numpy as np
import pytest

import plain_dezudra as pd
import tiny_dezudra as td


def test_configuration_is_read_layer_by_layer():
    from inferx_amd.config import ConfigError, config_from_dict
    cfg = config_from_dict(copy.deepcopy(td.B))
    assert cfg.architecture == "Dezudra" and cfg.vocab == 131 and cfg.width == 72 and cfg.logit_scale == 1.0
    assert [l.type for l in cfg.layers] == ["delta", "attention", "attention", "delta"]
    assert [l.mixer.conv for l in cfg.layers] == [5, 1, 3, 1]
    assert cfg.layers[1].mlp is None and cfg.layers[0].mlp.ff == 36 and cfg.layers[0].mlp.groups == 1
    assert (cfg.layers[2].mlp.groups, cfg.layers[2].mlp.groups_keep, cfg.layers[2].mlp.top) == (3, 1, 3)
    assert (cfg.layers[1].mixer.mask_size, cfg.layers[1].mixer.rot_dims) == (0, 0)
    assert (cfg.layers[2].mixer.mask_size, cfg.layers[2].mixer.keep_first, cfg.layers[2].mixer.rot_base) == (17, 5, 100.0)
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    for breaker, text in [
        (lambda c: c["layers"][0].update(type="convolution"), "not a mixer"),
        (lambda c: c["layers"][2]["mixer"].update(heads=4, kv_heads=3), "multiple"),
        (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "not known"),
        (lambda c: c["layers"][1]["mixer"].pop("scale"), "lacks 'scale'"),
        (lambda c: c["layers"][1]["mixer"].pop("diff"), "lacks 'diff'"),
        (lambda c: c["layers"][0]["mixer"].pop("conv"), "lacks 'conv'"),
        (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=7), "even"),
        (lambda c: c["layers"][2]["mlp"]["router"]["groups"].update(count=4), "divide"),
        (lambda c: c["layers"][2]["mlp"]["router"].update(top=4), "fit into the kept groups"),
        (lambda c: c.update(layers=[]), "at least one layer"),
        (lambda c: c["layers"][0]["mixer"].update(dim=True), "must be int"),
    ]:
        raw = copy.deepcopy(td.B)
        breaker(raw)
        with pytest.raises(ConfigError, match=text):
            config_from_dict(raw)


def test_tensor_names_and_what_keeps_what():
    from inferx_amd.config import config_from_dict
    from inferx_amd.parts import build_model
    model = build_model(config_from_dict(copy.deepcopy(td.B)).model_spec())
    names = model.expected_tensors()
    shape = lambda n: tuple(names[n].shape)
    assert shape("l0.mix.q") == (20, 72) and shape("l0.mix.v") == (36, 72) and shape("l0.mix.q.conv") == (20, 5)
    assert shape("l0.mix.b") == (3, 72) and shape("l0.mix.A_log") == (3,) and shape("l0.mix.norm") == (12,)
    assert shape("l0.mix.g") == (36, 72) and shape("l0.mix.o") == (72, 36) and shape("l0.mlp.e4.up") == (36, 72)
    assert shape("l2.mix.q") == (6 * 2 * 20, 72) and shape("l2.mix.k") == (3 * 2 * 20, 72) and shape("l2.mix.v") == (36, 72)
    assert shape("l2.mix.q.b") == (240,) and shape("l2.mix.v.conv") == (36, 3) and shape("l2.mix.lk2") == (20,)
    assert shape("l2.mix.o") == (72, 72) and shape("l2.mlp.router") == (9, 72) and shape("l2.mlp.e8.down") == (72, 52)
    assert shape("l1.norm1b") == (72,) and shape("final.norm") == (72,) and shape("head") == (131, 72)
    assert "l1.norm2" not in names and "l1.mlp.router" not in names and "l0.mlp.e0.gate" not in names
    plan = model.cache_plan()
    assert plan[0][0]["mixer"][0] is None and plan[0][0]["mixer"][1].shape == (3 * 20 * 12 + 4 * (20 + 20 + 36),)
    need, state = plan[2][0]["mixer"]
    assert [(a.name, a.heads, a.width, a.transposed) for a in need.arrays] == [("k", 6, 20, False), ("v", 3, 12, True)]
    assert (need.window, need.keep_first) == (17, 5) and state.shape == (2 * (240 + 120 + 36),)
    need, state = plan[1][0]["mixer"]
    assert (need.window, need.keep_first) == (0, 0) and state.dtype == "float32"
    assert model.graph_safe()


def test_plain_short_convolution_and_window_by_hand():
    u = np.array([[1.0], [2.0], [4.0]])
    w = np.array([[0.5, -1.0, 2.0]])  # last column: the current token's
    assert np.allclose(pd.short_conv(u, w)[:, 0], [2.0, 4.0 - 1.0, 8.0 - 2.0 + 0.5])
    see = pd.visible(8, 3, 2)
    assert see[7].tolist() == [True, True, False, False, False, True, True, True]
    assert see[2].tolist() == [True, True, True] + [False] * 5 and see[4].tolist()[:5] == [True, True, True, True, True]
    assert pd.visible(5, 1, 0)[4].tolist() == [False, False, False, False, True]


def test_plain_rotation_by_hand():
    x = np.zeros((1, 1, 6))
    x[0, 0] = [1.0, 2.0, 3.0, 4.0, 5.0, 6.0]
    y = pd.rotate(x, np.array([3]), 4, 100.0)[0, 0]  # pairs (0, 2) and (1, 3); elements 4 and 5 pass
    a0, a1 = 3.0, 3.0 * 100.0 ** -0.5
    assert np.allclose(y, [math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
                           3 * math.cos(a0) + math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 5.0, 6.0])


def test_plain_routing_among_groups_by_hand():
    # six experts in three groups; logits chosen so that the best expert of all sits in a group that is kept, and
    # the second best expert of all in a group that is dropped
    h = np.eye(1)
    w = np.array([[2.0], [0.1], [1.9], [-3.0], [1.0], [1.5]])  # groups (0, 1), (2, 3), (4, 5)
    s, ids, wts = pd.route(h, {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 1}}, w)
    assert ids.tolist() == [[0, 1]] and np.allclose(wts, s[:, [0, 1]]) and abs(s.sum() - 1.0) < 1e-12
    _, ids, _ = pd.route(h, {"experts": 6, "top": 3, "groups": {"count": 3, "keep": 2}}, w)
    assert ids.tolist() == [[0, 2, 1]]
    _, ids, _ = pd.route(h, {"experts": 6, "top": 3}, w)
    assert ids.tolist() == [[0, 2, 5]]


def test_plain_delta_rule_first_steps_by_hand():
    # one head of one key element: S is a row vector; with k a unit "vector" +-1 the write replaces what was there
    m = {"heads": 1, "kv_heads": 1, "dim": 1, "vdim": 2, "conv": 1}
    W = {"q": np.array([[1.0]]), "k": np.array([[1.0]]), "v": np.array([[1.0], [2.0]]), "g": np.array([[0.0], [0.0]]),
         "a": np.array([[0.0]]), "b": np.array([[0.0]]), "A_log": np.array([0.0]), "dt_bias": np.array([0.0]),
         "norm": np.ones(2), "o": np.eye(2), "q.conv": np.ones((1, 1)), "k.conv": np.ones((1, 1)),
         "v.conv": np.ones((2, 1))}
    out = pd.delta_mixer(np.array([[1.0]]), m, W, 1e-6)
    # the gate's logit is 0, and silu(0) = 0: nothing passes
    assert np.allclose(out, 0.0)
    W["g"] = np.array([[50.0], [50.0]])  # silu(50) = 50
    out = pd.delta_mixer(np.array([[1.0]]), m, W, 0.0)
    # q = k = silu(1) -> unit; beta = 1/2; S = 1/2 * silu(v); o = S * q: a head whose rms norm makes it (a, 2a)/rms
    sv = np.array([1.0, 2.0]) / (1 + np.exp(-np.array([1.0, 2.0])))
    o = 0.5 * sv
    assert np.allclose(out[0], o / np.sqrt(np.mean(o * o)) * 50.0, rtol=1e-5)
