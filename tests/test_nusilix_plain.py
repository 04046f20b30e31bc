"""The Nusilix configuration reader and model description (no GPU), and the plain
implementation's own consistency: identities that hold for the equations whatever the
weights, so that the oracle the GPU tests lean on is itself pinned."""

import copy
import math

import pytest
import torch

import nusilix_tiny as T
import plain_nusilix as P
from kllm_amd.config import ConfigError, NusilixConfig, config_from_dict
from kllm_amd.config.registry import resolve_architecture
from kllm_amd.engine.model import collect_weight_specs

F64 = torch.float64


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_configuration_round_trip_and_tensor_list(name):
    raw = T.CONFIGS[name]
    cfg = config_from_dict(raw)
    assert isinstance(cfg, NusilixConfig) and cfg.to_dict() == config_from_dict(cfg.to_dict()).to_dict()
    assert [l.type for l in cfg.layers] == [l["type"] for l in raw["layers"]]
    assert cfg.norm_groups == raw["norm"]["groups"] and cfg.residual_mult == raw["residual_mult"]
    spec = resolve_architecture(raw).build(cfg)
    wanted = {s.name: tuple(s.shape) for s in collect_weight_specs(spec)}
    assert wanted == P.tensor_shapes(raw)
    assert spec.layers[0].norm_feed_forward is None
    assert [l.feed_forward is None for l in spec.layers] == [l["mlp"] is None for l in raw["layers"]]


def test_a_width_the_configuration_does_not_name_is_left_to_the_checkpoint():
    raw = copy.deepcopy(T.CONFIGS["N1"])
    raw["layers"][1]["mixer"].pop("rank")
    spec = resolve_architecture(raw).build(config_from_dict(raw))
    shapes = {s.name: tuple(s.shape) for s in collect_weight_specs(spec)}
    assert shapes["l1.mix.w1"] == (-1, 64) and shapes["l1.mix.w2"] == (32, -1)


@pytest.mark.parametrize("change,text", [
    (lambda c: c["layers"][0].update(type="convolution"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(vdim=8), "vdim"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "kind"),
    (lambda c: c["norm"].update(groups=5), "groups"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_configurations_that_are_refused(change, text):
    raw = copy.deepcopy(T.CONFIGS["N1"])
    change(raw)
    with pytest.raises(ConfigError, match=text):
        config_from_dict(raw)


def test_sinusoid_channels():
    p = P.sinusoid([0, 1, 7], 6)
    assert torch.allclose(p[0], torch.tensor([0., 1., 0., 1., 0., 1.], dtype=F64))
    assert math.isclose(p[2, 0], math.sin(7.0)) and math.isclose(p[2, 1], math.cos(7.0))
    assert math.isclose(p[2, 4], math.sin(7.0 * 10000 ** (-4 / 6)))


def test_one_group_is_the_rms_norm_and_groups_do_not_see_each_other():
    g = torch.Generator().manual_seed(0)
    x, w = torch.randn(3, 12, generator=g, dtype=F64), torch.randn(12, generator=g, dtype=F64)
    assert torch.allclose(P.group_norm(x, w, 1, 1e-5), P.rms(x, 1e-5) * w)
    y = x.clone()
    y[:, 6:] *= 100.0
    assert torch.allclose(P.group_norm(x, w, 2, 1e-5)[:, :6], P.group_norm(y, w, 2, 1e-5)[:, :6])


def test_xielu_is_continuous_with_slope_one_half_at_zero():
    z = torch.tensor([-1e-6, 0.0, 1e-6], dtype=F64)
    a = P.xielu(z, 0.3, -0.2)
    assert abs(a[1]) == 0 and abs((a[2] - a[0]) / 2e-6 - 0.5) < 1e-6
    assert math.isclose(P.xielu(torch.tensor([2.0], dtype=F64), 0.3, 0.0)[0], math.log1p(math.exp(0.3)) * 4 + 1)


def test_the_distance_bias_may_be_written_by_key_position():
    """slope * (i - j) and -slope * j differ by a constant of the row, which a softmax drops."""
    g = torch.Generator().manual_seed(1)
    q, k = torch.randn(9, 2, 4, generator=g, dtype=F64), torch.randn(9, 1, 4, generator=g, dtype=F64)
    pos = list(range(20, 29))
    a = P.attention_scores_to_output(q, k, k, 0.7, [0.25, 0.0625], pos)
    b = P.attention_scores_to_output(q, k, k, 0.7, [0.25, 0.0625], list(range(9)))
    assert torch.allclose(a, b)          # only distances matter
    assert not torch.allclose(a, P.attention_scores_to_output(q, k, k, 0.7, [0.0, 0.0], pos))


def test_the_recurrence_in_pieces_equals_the_recurrence_at_once():
    g = torch.Generator().manual_seed(2)
    n, H, d = 11, 2, 5
    r, k, v = (torch.randn(n, H, d, generator=g, dtype=F64) for _ in range(3))
    decay, rate = (torch.rand(n, H, d, generator=g, dtype=F64) for _ in range(2))
    whole, S = P.delta_recurrence(r, k, v, decay, rate)
    state, outs = None, []
    for a, b in ((0, 1), (1, 4), (4, 6), (6, 11)):
        o, state = P.delta_recurrence(r[a:b], k[a:b], v[a:b], decay[a:b], rate[a:b], state)
        outs.append(o)
    assert torch.allclose(torch.cat(outs), whole) and torch.allclose(state, S)
    # with full removal and no decay, a key's old value is replaced: reading with the unit key returns v
    kk = torch.randn(1, 1, d, generator=g, dtype=F64)
    one, zero = torch.ones(1, 1, d, dtype=F64), torch.zeros(1, 1, d, dtype=F64)
    _, S1 = P.delta_recurrence(kk, kk, v[:1, :1], one, one)
    o2, _ = P.delta_recurrence(kk / (kk * kk).sum(), kk, v[1:2, :1], one, one, S1)
    assert torch.allclose(o2[0, 0], v[1, 0], atol=1e-5)


def test_prefix_logits_do_not_depend_on_what_follows():
    cfg = T.CONFIGS["N4"]
    w = P.random_weights(cfg, 5)
    ids = T.tokens(cfg, 20, 1)
    full, part = P.forward(w, cfg, ids), P.forward(w, cfg, ids[:13])
    assert torch.allclose(full[:13], part, atol=1e-9)
    layers = []
    P.forward(w, cfg, ids, layers_out=layers)
    assert len(layers) == len(cfg["layers"]) and layers[0].shape == (20, cfg["width"])
