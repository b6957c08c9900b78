"""Host-side checks of the Pelalix design: its configuration and tensor names, the parts it is put together from,
and the plain implementation's own mechanisms on cases worked out by hand."""
import copy
import math

import pytest
import torch

import plain_pelalix as pp
import tiny_pelalix as tp

F64 = torch.float64


def test_configuration_is_read_layer_by_layer():
    from inferx_amd.config import ConfigError, config_from_dict
    cfg = config_from_dict(copy.deepcopy(tp.Q))
    assert cfg.architecture == "Pelalix" and cfg.vocab == 131 and cfg.width == 72
    assert [l.mixer.heads for l in cfg.layers] == [4, 4, 2, 8]
    assert cfg.layers[1].mlp_kind is None and cfg.layers[0].ff == 100
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    for breaker, text in [
        (lambda c: c["layers"][0].update(type="convolution"), "not a mixer"),
        (lambda c: c["layers"][0]["mixer"].update(heads=3, kv_heads=2), "multiple"),
        (lambda c: c["layers"][0]["mlp"].update(kind="sparse"), "not known"),
        (lambda c: c["layers"][3]["mixer"].update(vdim=24), "value size differ"),
        (lambda c: c["layers"][0]["mixer"].pop("scale"), "lacks 'scale'"),
        (lambda c: c.update(layers=[]), "at least one layer"),
        (lambda c: c["layers"][0]["mixer"].update(dim=True), "must be int"),
    ]:
        raw = copy.deepcopy(tp.Q)
        breaker(raw)
        with pytest.raises(ConfigError, match=text):
            config_from_dict(raw)
    with pytest.raises(ConfigError, match="unknown architecture"):
        config_from_dict({"architecture": "Nobody"})


def test_tensor_names_and_what_keeps_what():
    from inferx_amd.config import config_from_dict
    from inferx_amd.parts import build_model
    model = build_model(config_from_dict(copy.deepcopy(tp.Q)).model_spec())
    names = model.expected_tensors()
    assert tuple(names["l0.mix.q"].shape) == (96, 72) and tuple(names["l0.mix.v"].shape) == (40, 72)
    assert tuple(names["l3.mix.talk"].shape) == (8, 8) and tuple(names["l3.mix.g"].shape) == (8, 72)
    assert tuple(names["l2.mix.q.norm"].shape) == (96,) and tuple(names["l2.mix.k.norm"].shape) == (96,)
    assert tuple(names["final.norm.alpha"].shape) == () and tuple(names["l1.ls1"].shape) == (72,)
    assert "l1.mlp.gate" not in names and "l1.norm2" not in names and "l1.ls2" not in names  # no feed-forward there
    assert "l0.mix.vmix" not in names and "l1.mix.vmix" in names and "l3.mix.vmix" in names
    kinds = [model.blocks[i].mixer.value_mix for i in range(4)]
    assert kinds == ["none", "source", "none", "mix"]
    plan = model.cache_plan()
    for i, (keeps, _) in enumerate(plan):
        need, _ = keeps["mixer"]
        m = tp.Q["layers"][i]["mixer"]
        assert [(a.heads, a.width) for a in need.arrays] == [(m["kv_heads"], m["dim"]), (m["kv_heads"], m["vdim"])]
        assert keeps["mixer_shift"][1].shape == (72,) and keeps["mixer_shift"][1].dtype == "float32"
    assert model.graph_safe()


def test_token_shift_by_hand():
    x = torch.tensor([[1.0, 10.0], [2.0, 20.0], [4.0, 40.0]], dtype=F64)
    mix = torch.tensor([0.0, 1.0], dtype=F64)
    got = pp.token_shift(x, mix)
    assert torch.equal(got, torch.tensor([[1.0, 0.0], [2.0, 10.0], [4.0, 20.0]], dtype=F64))
    half = pp.token_shift(x, torch.full((2,), 0.5, dtype=F64))
    assert torch.equal(half[2], torch.tensor([3.0, 30.0], dtype=F64))  # from the ORIGINAL row 1, not the blended one
    # cut in two with the row before handed over
    again = torch.cat([pp.token_shift(x[:1], mix), pp.token_shift(x[1:], mix, before=x[0])])
    assert torch.equal(again, got)


def test_sink_and_mixing_by_hand():
    # one head, two keys with equal scores, sink equal to them: the weights are a third each and add up to two thirds
    s = torch.zeros(1, 2, 2, dtype=F64)
    p = pp.softmax_with_sink(s, torch.zeros(1, dtype=F64))
    assert torch.allclose(p[0, 1], torch.tensor([1 / 3, 1 / 3], dtype=F64)) and float(p[0, 0, 0]) == 0.5 and float(p[0, 0, 1]) == 0.0
    # a sink far below every score is the usual softmax
    g = torch.Generator().manual_seed(0)
    s = torch.randn(3, 5, 5, generator=g, dtype=F64)
    usual = pp.softmax_with_sink(s, None)
    assert torch.allclose(pp.softmax_with_sink(s, torch.full((3,), -1e3, dtype=F64)), usual)
    assert torch.allclose(usual.sum(-1), torch.ones(3, 5, dtype=F64))
    # mixing with the identity changes nothing; a row of the matrix picks and weighs heads
    assert torch.equal(pp.mix_heads(s, torch.eye(3, dtype=F64)), s)
    talk = torch.tensor([[0.0, 2.0, 0.0], [1.0, 0.0, 0.0], [0.5, 0.0, 0.5]], dtype=F64)
    m = pp.mix_heads(s, talk)
    assert torch.allclose(m[0], 2 * s[1]) and torch.allclose(m[1], s[0]) and torch.allclose(m[2], 0.5 * (s[0] + s[2]))


def test_whole_projection_norm_and_grouping():
    x = torch.tensor([[3.0, 4.0, 0.0, 0.0]], dtype=F64)  # mean square 25 / 4
    got = pp.rms_norm_whole(x, torch.ones(4, dtype=F64), 0.0)
    assert torch.allclose(got, x / 2.5)
    # four query heads on two key heads: heads 0, 1 read key head 0, heads 2, 3 key head 1
    q = torch.ones(1, 4, 2, dtype=F64)
    k = torch.tensor([[[1.0, 0.0], [0.0, 5.0]]], dtype=F64)
    assert pp.raw_scores(q, k, 2.0)[:, 0, 0].tolist() == [2.0, 2.0, 10.0, 10.0]


def test_attention_options_off_is_the_usual_attention():
    import plain_model as pm
    g = torch.Generator().manual_seed(1)
    T, H, G, d = 9, 4, 2, 8
    q, k, v = (torch.randn(T, n, d, generator=g, dtype=F64) for n in (H, G, G))
    s = pp.raw_scores(q, k, 0.3)
    got = pp.weighted_values(pp.softmax_with_sink(s, None), v)
    want = pm.attention(q, k, v, torch.arange(T), 0.3)
    assert torch.allclose(got, want)
