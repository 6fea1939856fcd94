"""The Zivovik design on the host: its configuration and what it becomes (run order, parts, tensor names, cache units,
state), and the plain implementation's mechanisms against direct sums."""
import copy

import numpy as np
import pytest

import braidinfer_amd as B
import plain_zivovik as P
from braidinfer_amd.config import config_from_dict, spec_of
from braidinfer_amd.engine.model import DecoderModel
from braidinfer_amd.errors import ConfigError


def moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def small():
    att = {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 8, "scale": 0.3, "q_temp": {"coef": 0.25, "every": 4}}
    left = {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 12, "scale": 0.4, "q_temp": {"coef": 0.1, "every": 6}}
    right = {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 10, "conv": 3}
    return {"architecture": "Zivovik", "vocab": 40, "width": 24, "max_positions": 64, "norm": {"eps": 1e-5},
            "embedding": {"scale": 1.5}, "residual_mult": 0.8, "loop": {"start": 1, "stop": 3, "times": 2}, "layers": [
                {"type": "attention", "mixer": copy.deepcopy(att), "mlp": moe(8, 3, 2)},
                {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": moe(8, 3, 2)},
                {"type": "lightning", "mixer": {"heads": 3, "dim": 4, "vdim": 6, "decay": [0.5, 0.9, 0.99]}, "mlp": None},
                {"type": "attention", "mixer": copy.deepcopy(att), "mlp": moe(8, 4, 4)}]}


def test_configuration_round_trip_and_registry():
    d = small()
    cfg = config_from_dict(d)
    assert isinstance(cfg, B.ZivovikConfig) and cfg.to_dict() == d
    assert "Zivovik" in B.registered_architectures()
    assert B.any_preset("zivovik-tiny").width == 96
    for name in ("zivovik-1b", "zivovik-7b"):
        assert len(spec_of(B.any_preset(name)).schedule) == 8


@pytest.mark.parametrize("change,what", [
    (lambda d: d["layers"][0]["mixer"].__setitem__("vdim", 6), "values are the keys"),
    (lambda d: d["layers"][0]["mixer"].__setitem__("kv_heads", 3), "multiple"),
    (lambda d: d["layers"][1]["mixer"].pop("right"), "left.*right"),
    (lambda d: d["layers"][1]["mixer"]["right"].pop("conv"), "conv"),
    (lambda d: d["layers"][2]["mixer"].__setitem__("decay", [0.5, 0.9]), "decay"),
    (lambda d: d["layers"][3]["mlp"]["router"].__setitem__("top", 5), "chooses"),
    (lambda d: d["layers"][0]["mlp"].__setitem__("kind", "dense"), "kind"),
    (lambda d: d["layers"][0].__setitem__("type", "wkv"), "type"),
    (lambda d: d["loop"].__setitem__("stop", 5), "loop"),
    (lambda d: d["loop"].__setitem__("start", 4), "loop"),
    (lambda d: d.pop("max_positions"), "max_positions"),
    (lambda d: d["layers"][0]["mixer"]["q_temp"].__setitem__("every", 0), "every"),
])
def test_configurations_that_are_refused(change, what):
    d = small()
    change(d)
    with pytest.raises(ConfigError, match=what):
        config_from_dict(d)


@pytest.mark.parametrize("loop,order", [
    ({"start": 1, "stop": 3, "times": 2}, [(0, False), (1, False), (2, False), (1, True), (2, False), (3, False)]),
    ({"start": 0, "stop": 2, "times": 3}, [(0, False), (1, False), (0, True), (1, False), (0, True), (1, False), (2, False), (3, False)]),
    ({"start": 0, "stop": 4, "times": 2}, [(0, False), (1, False), (2, False), (3, False), (0, True), (1, False), (2, False), (3, False)]),
    ({"start": 2, "stop": 3, "times": 1}, [(0, False), (1, False), (2, False), (3, False)]),
    ({"start": 3, "stop": 4, "times": 2}, [(0, False), (1, False), (2, False), (3, False), (3, True)]),
    ({"start": 2, "stop": 2, "times": 5}, [(0, False), (1, False), (2, False), (3, False)]),
    (None, [(0, False), (1, False), (2, False), (3, False)]),
])
def test_run_order(loop, order):
    d = small()
    if loop is None:
        d.pop("loop")
    else:
        d["loop"] = loop
    cfg = config_from_dict(d)
    assert cfg.run_order() == order == P.run_order(d)
    spec = spec_of(cfg)
    assert [(e.layer, e.adds_embedding) for e in spec.schedule] == order
    assert [e.cache for e in spec.schedule] == list(range(len(order)))          # a cache unit of its own for every run


def test_parts_units_state_and_tensor_names():
    d = small()
    cfg = config_from_dict(d)
    spec = spec_of(cfg)
    assert [l.block for l in spec.layers] == ["prenorm_residual", "prenorm_side_by_side", "prenorm_residual", "prenorm_residual"]
    model = DecoderModel(spec)
    needs = model.cache_needs()
    # attention runs 0 and 5, the parallel layers' left sides at runs 1 and 3; nothing for the lightning runs
    assert sorted(needs) == [0, 1, 3, 5]
    assert needs[0].kv_heads == 2 and needs[0].head_dim == 8 and needs[0].val_dim == 8 and needs[0].first_live(1000) == 0
    assert needs[1].kv_heads == 1 and needs[1].head_dim == 8 and needs[1].val_dim == 12
    states = model.state_needs()
    assert sorted(states, key=str) == sorted([("entry", 1, "right"), ("entry", 3, "right"), ("entry", 2), ("entry", 4)], key=str)
    conv_channels = 2 * 2 * 6 + 4 * 10
    assert states[("entry", 1, "right")].shape[0] >= 4 * 6 * 10 + 2 * conv_channels
    names = {s.name: tuple(s.shape) for s in model.weight_specs()}
    w = P.random_weights(d, seed=1)
    assert set(names) == set(w) and all(names[n] == w[n].shape for n in names)
    assert "l2.norm2" in model.optional_names()
    att = model.layers[0].mixer
    assert att.full and att.values_from_keys and att.gate == "element" and att.q_temp == (0.25, 4) and att.out_scale == 0.8
    left = model.layers[1].mixer
    assert left.gate == "head" and left.qk_norm_eps is None and not left.values_from_keys and left.out_scale == 1.0
    assert model.layers[1].norms["mixer_out"].scale == 0.4 and model.layers[1].norms["mixer_out.right"].offset == 0.0
    assert model.layers[0].norms["mixer"].offset == 1.0 and model.final_norm.offset == 1.0
    assert model.graph_safe()


# ------------------------------------------------ the plain mechanisms against direct sums -------
def test_plain_delta_rule_against_its_unrolled_form():
    """Without decay and with beta = 1 and orthonormal keys the state stores exactly v_t under k_t: reading with k_j
    returns v_j; with a decay g the stored value fades by the product of the later decays."""
    rng = np.random.default_rng(0)
    d, e, T = 6, 4, 5
    keys = np.linalg.qr(rng.standard_normal((d, d)))[0][:T]
    v = rng.standard_normal((T, e))
    o = P.delta_rule(keys, keys, v, np.ones(T), np.ones(T))
    assert np.allclose(o, v)
    g = rng.uniform(0.5, 1.0, T)
    q = np.tile(keys[0], (T, 1))
    o = P.delta_rule(q, keys, v, np.ones(T), g)
    assert np.allclose(o, [v[0] * np.prod(g[1:t + 1]) for t in range(T)])
    # a repeated key is corrected, not added: beta = 1 replaces what lies under it
    k2 = np.stack([keys[0], keys[0]])
    o = P.delta_rule(k2, k2, v[:2], np.ones(2), np.ones(2))
    assert np.allclose(o[1], v[1])


def test_plain_decayed_sum_convolution_and_temperature():
    rng = np.random.default_rng(1)
    T, d, e = 7, 3, 2
    q, k, v = rng.standard_normal((T, d)), rng.standard_normal((T, d)), rng.standard_normal((T, e))
    o = P.decayed_outer_sum(q, k, v, 0.8)
    want = [sum(0.8 ** (t - j) * (q[t] @ k[j]) * v[j] for j in range(t + 1)) for t in range(T)]
    assert np.allclose(o, want)
    x, taps = rng.standard_normal((T, 2)), rng.standard_normal((2, 3))
    y = P.short_convolution(x, taps)
    assert np.allclose(y[0], taps[:, 2] * x[0]) and np.allclose(y[3], taps[:, 0] * x[1] + taps[:, 1] * x[2] + taps[:, 2] * x[3])
    t = P.query_temperature(np.arange(10), 0.5, 4)
    assert np.allclose(t[:3], 1.0) and np.allclose(t[3:7], 1 + 0.5 * np.log(2.0)) and np.allclose(t[7:], 1 + 0.5 * np.log(3.0))


def test_plain_routing_is_softmax_over_the_chosen():
    """Scores over all experts divided by the chosen ones' sum equal the softmax over the chosen logits."""
    rng = np.random.default_rng(2)
    W, E, top, F = 6, 5, 2, 3
    w = {"router": rng.standard_normal((E, W))}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = rng.standard_normal((F, W)), rng.standard_normal((F, W)), rng.standard_normal((W, F))
    h = rng.standard_normal((4, W))
    got = P.routed_ff(h, w, "", moe(F, E, top))
    for t in range(4):
        z = h[t] @ w["router"].T
        ch = np.argsort(-z)[:top]
        a = np.exp(z[ch] - z[ch].max())
        a /= a.sum()
        want = sum(ai * ((P.silu(h[t] @ w[f"e{e}.gate"].T) * (h[t] @ w[f"e{e}.up"].T)) @ w[f"e{e}.down"].T) for ai, e in zip(a, ch))
        assert np.allclose(got[t], want)
