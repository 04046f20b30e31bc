"""The plain Ribovik (tests/plain_ribovik.py) pinned by identities of its own, and the
configuration reader and model builder, without a GPU."""

import json
import math

import pytest
import torch

import plain_ribovik as P
import ribovik_tiny as T

F64 = torch.float64


def weights(name, seed=3):
    return {k: v.double() for k, v in P.random_weights(T.CONFIGS[name], seed).items()}


def test_sink_is_a_key_with_score_zero_and_no_value():
    g = torch.Generator().manual_seed(0)
    s = 3.0 * torch.randn(7, 11, generator=g, dtype=F64)
    s[2, 4:] = float("-inf")
    p = P.softmax_with_sink(s)
    full = torch.softmax(torch.cat([s, torch.zeros(7, 1, dtype=F64)], dim=1), dim=1)
    assert torch.allclose(p, full[:, :-1], atol=1e-15)
    assert (p.sum(1) < 1).all()
    one = P.softmax_with_sink(torch.tensor([[0.0]], dtype=F64))
    assert abs(float(one) - 0.5) < 1e-15           # a lone key with score 0 shares the weight with the sink


def test_chunks_are_counted_from_position_zero():
    assert [j for j in range(12) if P.visible(9, j, 4)] == [8, 9]
    assert [j for j in range(12) if P.visible(8, j, 4)] == [8]
    assert [j for j in range(12) if P.visible(7, j, 4)] == [4, 5, 6, 7]
    assert [j for j in range(5) if P.visible(3, j, 0)] == [0, 1, 2, 3]


def test_a_token_depends_on_its_own_chunk_only():
    cfg, w = T.CONFIGS["R5"], weights("R5")          # chunks of 16 on every layer
    a = T.tokens(cfg, 40, 1)
    b = T.tokens(cfg, 16, 2) + a[16:]
    la, lb = P.forward(cfg, w, a), P.forward(cfg, w, b)
    assert torch.allclose(la[16:], lb[16:], atol=1e-12)
    assert not torch.allclose(la[:16], lb[:16], atol=1e-3)
    c = a[:31] + [(a[31] + 1) % cfg["vocab"]] + a[32:]          # the last token of a chunk
    lc = P.forward(cfg, w, c)
    assert torch.allclose(la[32:], lc[32:], atol=1e-12) and torch.allclose(la[:31], lc[:31], atol=1e-12)


def test_stretched_frequencies():
    plain, one = P.yarn_frequencies({"dims": 32, "base": 10000.0})
    assert one == 1.0 and abs(float(plain[3]) - 10000.0 ** (-6 / 32)) < 1e-15
    rot = {"dims": 32, "base": 10000.0, "scaling": {"factor": 4.0, "original": 256, "fast": 32.0, "slow": 1.0}}
    f, mag = P.yarn_frequencies(rot)
    assert abs(mag - (0.1 * math.log(4.0) + 1)) < 1e-15
    assert float(f[0]) == 1.0                              # the fastest pair is left alone
    assert abs(float(f[-1]) - float(plain[-1]) / 4.0) < 1e-18   # the slowest is stretched by the whole factor
    ratio = plain / f
    assert ((ratio[1:] - ratio[:-1]) >= -1e-12).all() and float(ratio.max()) <= 4.0 + 1e-12
    same, _ = P.yarn_frequencies({"dims": 32, "base": 10000.0, "scaling": {"factor": 1.0, "original": 256, "fast": 32.0, "slow": 1.0}})
    assert torch.allclose(same, plain, rtol=1e-15)


def test_rotation_keeps_lengths_and_relative_positions():
    rot = {"dims": 8, "base": 100.0}
    g = torch.Generator().manual_seed(1)
    q, k = torch.randn(1, 1, 12, generator=g, dtype=F64), torch.randn(1, 1, 12, generator=g, dtype=F64)
    for shift in (0, 5, 1000):
        a = P.rotate_neighbours(q, [7 + shift], rot)
        b = P.rotate_neighbours(k, [3 + shift], rot)
        assert abs(float(a.norm()) - float(q.norm())) < 1e-12
        assert torch.equal(a[..., 8:], q[..., 8:])         # what lies behind rot.dims passes
        if shift == 0:
            dot = float((a * b).sum())
        assert abs(float((a * b).sum()) - dot) < 1e-9


def test_identity_experts_and_weights_without_the_correction():
    cfg = T.CONFIGS["R3"]
    mlp = cfg["layers"][0]["mlp"]
    w = {k: v.double() for k, v in P.random_weights(cfg, 2).items()}
    h = torch.randn(9, cfg["width"], generator=torch.Generator().manual_seed(4), dtype=F64)
    idx, wt = P.route(h, w, "l0.mlp", mlp["router"]["top"])
    assert torch.allclose(wt.sum(1), torch.ones(9, dtype=F64), atol=1e-12)
    s = torch.softmax(h @ w["l0.mlp.router"].T, -1)
    assert torch.allclose(wt, torch.gather(s, 1, idx) / torch.gather(s, 1, idx).sum(1, keepdim=True), atol=1e-12)
    # a router that only ever chooses identity experts, and no shared expert: the layer hands its input on
    only = dict(mlp, router={"experts": 2, "identity": 3, "top": 3})
    only.pop("shared")
    w2 = dict(w)
    w2["l0.mlp.correction"] = torch.tensor([-9.0, -9.0, 0.0, 0.0, 0.0], dtype=F64)
    assert torch.allclose(P.moe_ff(h, w2, "l0.mlp", only), h, atol=1e-12)


def test_clamped_expert_by_hand():
    w = {"e.gate": torch.tensor([[1.0]], dtype=F64), "e.up": torch.tensor([[1.0]], dtype=F64), "e.down": torch.tensor([[1.0]], dtype=F64)}
    for x, limit in ((0.5, 2.0), (5.0, 2.0), (-5.0, 2.0)):
        g, u = min(x, limit), max(-limit, min(x, limit))
        want = g / (1 + math.exp(-1.702 * g)) * (u + 1)
        assert abs(float(P.clamped_expert(torch.tensor([[x]], dtype=F64), w, "e", limit)) - want) < 1e-12


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_configuration_reader_and_builder(name):
    from kllm_amd.config.registry import config_from_dict, resolve_architecture
    from kllm_amd.engine.model import collect_weight_specs
    raw = T.CONFIGS[name]
    cfg = config_from_dict(raw)
    assert cfg.to_dict() == json.loads(json.dumps(raw))
    spec = resolve_architecture(raw).build(cfg)
    got = {s.name: tuple(s.shape) for s in collect_weight_specs(spec)}
    assert got == {k: tuple(v) for k, v in P.tensor_shapes(raw).items()}


def test_configuration_errors_name_the_key():
    from kllm_amd.config.base import ConfigError
    from kllm_amd.config.registry import config_from_dict
    good = json.loads(json.dumps(T.CONFIGS["R1"]))
    for path, value, word in ((("layers", 0, "type"), "conv", "type"), (("layers", 0, "mixer", "kv_heads"), 3, "kv_heads"),
                              (("layers", 1, "mlp", "kind"), "sparse", "kind"), (("layers", 0, "mixer", "rot", "dims"), 7, "rot.dims"),
                              (("layers", 1, "mlp", "router", "top"), 9, "top"), (("norm", "eps"), -1, "eps")):
        bad = json.loads(json.dumps(good))
        at = bad
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ConfigError, match=word):
            config_from_dict(bad)


def test_frequencies_of_the_package_are_the_plain_ones():
    from kllm_amd.parts.rotary import scaled_frequencies
    for name in ("R1", "R5", "R6", "R3"):
        rot = T.CONFIGS[name]["layers"][0]["mixer"]["rot"]
        sc = rot.get("scaling")
        f, mag = scaled_frequencies(rot["dims"], rot["base"], (sc["factor"], sc["original"], sc["fast"], sc["slow"]) if sc else None)
        wf, wmag = P.yarn_frequencies(rot)
        assert torch.allclose(torch.tensor(f, dtype=F64), wf, rtol=1e-14) and abs(mag - wmag) < 1e-15
