"""The Ladadra design on the host: configuration, run order and parts, tensor names, what the cache keeps, and the
plain implementation's mechanisms against direct sums."""
import copy
import math

import numpy as np
import pytest

import plain_ladadra as P


def tiny():
    return {"architecture": "Ladadra", "vocab": 90, "width": 40, "norm": {"eps": 1e-5}, "layers": [
        {"type": "attention_2", "mixer": {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 12, "scale": 0.3, "diff": 0.25,
                                          "mask": {"size": 9, "keep_first": 3}}, "mlp": {"kind": "dense", "ff": 56}},
        {"type": "attention", "mixer": {"heads": 6, "kv_heads": 3, "dim": 8, "vdim": 4, "scale": 0.4, "softcap": 12.0, "mask": {"size": 11},
                                        "rot": {"base": 100.0, "dims": 4, "scaling": {"factor": 3.0, "low": 1.0, "high": 2.0, "original": 16}}},
         "mlp": {"kind": "moe", "expert": {"ff": 16}, "shared": {"ff": 24}, "router": {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}}}},
        {"type": "retention", "mixer": {"heads": 2, "dim": 6, "vdim": 10, "decay": [0.9, 0.97], "rot": {"base": 50.0, "dims": 6}}, "mlp": None}]}


def test_configuration_is_read_and_checked():
    import braidinfer_amd as B
    from braidinfer_amd.errors import ConfigError
    cfg = B.config_from_dict(tiny())
    assert type(cfg).__name__ == "LadadraConfig" and cfg.to_dict()["layers"][1]["mixer"]["softcap"] == 12.0
    assert B.config_from_dict(cfg.to_dict()) == cfg

    def broken(change):
        d = tiny()
        change(d)
        with pytest.raises(ConfigError):
            B.config_from_dict(d)
    broken(lambda d: d["layers"][0].__setitem__("type", "attention_3"))
    broken(lambda d: d["layers"][0]["mixer"].__setitem__("kv_heads", 3))
    broken(lambda d: d["layers"][0]["mixer"].pop("diff"))
    broken(lambda d: d["layers"][1]["mixer"]["rot"].__setitem__("dims", 10))
    broken(lambda d: d["layers"][1]["mixer"]["rot"].__setitem__("dims", 3))
    broken(lambda d: d["layers"][1]["mixer"].__setitem__("softcap", 0.0))
    broken(lambda d: d["layers"][1]["mlp"]["router"].__setitem__("top", 7))
    broken(lambda d: d["layers"][1]["mlp"]["router"]["groups"].__setitem__("count", 4))
    broken(lambda d: d["layers"][1]["mlp"]["router"]["groups"].__setitem__("keep", 0))
    broken(lambda d: d["layers"][1]["mlp"]["router"].__setitem__("groups", {"count": 3, "keep": 1}) or
           d["layers"][1]["mlp"]["router"].__setitem__("top", 3))
    broken(lambda d: d["layers"][2]["mixer"].__setitem__("decay", [0.9]))
    broken(lambda d: d["layers"][2]["mixer"]["rot"].__setitem__("scaling", {"factor": 2.0, "low": 1.0, "high": 2.0, "original": 8}))
    broken(lambda d: d["layers"][1]["mlp"].__setitem__("kind", "wide"))
    broken(lambda d: d.pop("norm"))


def test_parts_tensor_names_units_and_state():
    import braidinfer_amd as B
    from braidinfer_amd.engine.model import DecoderModel
    d = tiny()
    model = DecoderModel(B.spec_of(B.config_from_dict(d)))
    assert {s.name: tuple(s.shape) for s in model.weight_specs()} == P.tensor_shapes(d)
    assert model.graph_safe()
    needs = model.cache_needs()
    assert sorted(needs) == [0, 1]                        # the retention layer keeps no rows
    assert (needs[0].kv_heads, needs[0].key_dim, needs[0].val_dim, needs[0].keep_first) == (2, 16, 12, 3)      # both maps' keys side by side
    assert (needs[1].kv_heads, needs[1].key_dim, needs[1].val_dim, needs[1].keep_first) == (3, 8, 4, 0)
    # a window of 9: at length 20 the next query (position 20) sees from 12 on; runs of 11: from 11 on
    assert needs[0].first_live(20) == 12 and needs[1].first_live(20) == 11 and needs[1].first_live(22) == 22 and needs[1].first_live(10) == 0
    assert list(model.state_needs()) == [("entry", 2)]
    assert [sorted(l.norms) for l in model.layers] == [["feed_forward", "feed_forward_out", "mixer", "mixer_out"]] * 2 + [["mixer", "mixer_out"]]
    assert model.optional_names() == ["l2.norm2", "head.weight"]
    # every key a mixer may leave out
    d2 = copy.deepcopy(d)
    for k in ("kv_heads", "vdim", "mask"):
        d2["layers"][0]["mixer"].pop(k)
    for k in ("softcap", "mask", "rot", "vdim"):
        d2["layers"][1]["mixer"].pop(k)
    d2["layers"][1]["mlp"]["router"].pop("groups")
    d2["layers"][1]["mlp"].pop("shared")
    d2["layers"][2]["mixer"].pop("rot")
    m2 = DecoderModel(B.spec_of(B.config_from_dict(d2)))
    assert {s.name: tuple(s.shape) for s in m2.weight_specs()} == P.tensor_shapes(d2)
    n2 = m2.cache_needs()
    assert n2[0].live_from is None and n2[1].live_from is None and (n2[0].kv_heads, n2[0].key_dim, n2[0].val_dim) == (4, 16, 8)
    assert m2.positions == {}


def test_presets_are_configurations():
    import braidinfer_amd as B
    from braidinfer_amd.engine.model import DecoderModel
    for name in ("ladadra-tiny", "ladadra-1b", "ladadra-7b"):
        cfg = B.any_preset(name)
        model = DecoderModel(B.spec_of(cfg))
        assert {s.name: tuple(s.shape) for s in model.weight_specs()} == P.tensor_shapes(cfg.to_dict())


def test_pages_of_kept_first_tokens_stay():
    from braidinfer_amd.cache import CacheNeed, SequenceCache
    from braidinfer_amd.parts.pooled_attention import window_and_open_block
    window = CacheNeed(kv_heads=1, head_dim=4, live_from=window_and_open_block(100, 0), keep_first=70)      # two pages of kept tokens
    runs = CacheNeed(kv_heads=1, head_dim=4, live_from=window_and_open_block(1 << 30, 0, 150))
    cache = SequenceCache({0: window, 1: runs}, {}, max_tokens=64 * 12, dtype=None)
    s = cache.alloc_slot()
    g_window, g_runs = cache.unit_group(0), cache.unit_group(1)
    for new in (130, 1, 200, 1, 1, 300):
        cache.reserve([s], [new])
        cache.commit([s], [new])
        n = cache.length(s)
        live = lambda g: [i for i, p in enumerate(g.pages[s]) if p >= 0]
        first = (n - 100 + 1) // 64
        assert live(g_window) == sorted(set([0, 1]) | set(range(max(first, 0), -(-n // 64))))
        assert live(g_runs) == list(range(((n // 150) * 150) // 64, -(-n // 64)))
    cache.free_slot(s)
    assert g_window.pool.free_count == g_window.pool.n_pages and g_runs.pool.free_count == g_runs.pool.n_pages


# ------------------------------------------------------------------ the plain mechanisms against direct sums -------
def test_plain_masks():
    T = 23
    for size, keep in ((5, 0), (5, 3), (1, 2), (40, 0)):
        m = P.window_mask(T, size, keep)
        for i in range(T):
            for j in range(T):
                assert m[i, j] == (j <= i and (i - j < size or j < keep))
    for size in (1, 4, 7, 50):
        m = P.chunk_mask(T, size)
        for i in range(T):
            for j in range(T):
                assert m[i, j] == (j <= i and i // size == j // size)


def test_plain_attention_with_sink_and_bounded_scores():
    rng = np.random.default_rng(0)
    T, H, G, d, e = 9, 4, 2, 5, 3
    q, k, v = rng.standard_normal((T, H, d)), rng.standard_normal((T, G, d)), rng.standard_normal((T, G, e))
    sinks = rng.standard_normal(H)
    visible = P.chunk_mask(T, 4)
    got = P.masked_attention(q, k, v, 0.7, visible, softcap=2.0, sinks=sinks)
    for t in range(T):
        for h in range(H):
            g = h // (H // G)
            num, den = np.zeros(e), math.exp(sinks[h])
            for j in range(T):
                if visible[t, j]:
                    s = 2.0 * math.tanh(float(q[t, h] @ k[j, g]) * 0.7 / 2.0)
                    num += math.exp(s) * v[j, g]
                    den += math.exp(s)
            assert np.abs(got[t, h] - num / den).max() < 1e-12
    # without a sink the weights sum to one; a very large sink takes all the weight
    one = P.masked_attention(q, k, np.ones((T, G, e)), 0.7, P.causal(T))
    assert np.abs(one - 1.0).max() < 1e-12
    assert np.abs(P.masked_attention(q, k, v, 0.7, P.causal(T), sinks=np.full(H, 80.0))).max() < 1e-20


def test_plain_rotation_and_stretched_frequencies():
    f = P.rotary_frequencies(8, 100.0)
    assert np.allclose(f, [1.0, 100 ** -0.25, 100 ** -0.5, 100 ** -0.75])
    sc = {"factor": 5.0, "low": 1.0, "high": 4.0, "original": 40}
    g = P.rotary_frequencies(8, 100.0, sc)
    for fi, gi in zip(f, g):
        wl = 2 * math.pi / fi
        if wl < 10:
            assert gi == fi
        elif wl > 40:
            assert gi == fi / 5
        else:
            s = (40 / wl - 1.0) / 3.0
            assert 0 <= s <= 1 and abs(gi - ((1 - s) * fi / 5 + s * fi)) < 1e-15
    assert g[0] == f[0] and g[-1] == f[-1] / 5 and f[1] / 5 < g[1] < f[1]      # one of each kind
    # a rotation keeps lengths, passes the elements behind the rotated ones, and scores depend on distances only
    rng = np.random.default_rng(1)
    x, y = rng.standard_normal((1, 1, 10)), rng.standard_normal((1, 1, 10))
    a, b = P.rotate_half(x, [7], f), P.rotate_half(y, [3], f)
    a2, b2 = P.rotate_half(x, [107], f), P.rotate_half(y, [103], f)
    assert np.allclose(a[..., 8:], x[..., 8:]) and abs(np.linalg.norm(a) - np.linalg.norm(x)) < 1e-12
    assert abs(float((a * b).sum()) - float((a2 * b2).sum())) < 1e-9
    assert np.allclose(P.rotate_half(x, [0], f), x)
    u, v = x[0, 0, 1], x[0, 0, 5]                      # element 1 pairs with element 1 + 4
    ang = 7 * f[1]
    assert abs(a[0, 0, 1] - (u * math.cos(ang) - v * math.sin(ang))) < 1e-12 and abs(a[0, 0, 5] - (v * math.cos(ang) + u * math.sin(ang))) < 1e-12


def test_plain_choice_of_experts():
    rng = np.random.default_rng(2)
    T, E, top = 40, 12, 3
    z = rng.standard_normal((T, E)) * 2
    corr = rng.standard_normal(E) - 1.0                      # negative choice scores happen
    chosen, weights = P.choose_experts(z, corr, top, {"count": 4, "keep": 2})
    s = 1 / (1 + np.exp(-z))
    for t in range(T):
        c = s[t] + corr
        gs = [sum(sorted(c[g * 3:g * 3 + 3])[-2:]) for g in range(4)]
        best = sorted(range(4), key=lambda g: (-gs[g], g))[:2]
        allowed = [e for e in range(E) if e // 3 in best]
        want = sorted(allowed, key=lambda e: (-c[e], e))[:top]
        assert list(chosen[t]) == want
        assert np.allclose(weights[t], s[t][want] / s[t][want].sum())
    plain_top, _ = P.choose_experts(z, np.zeros(E), top)
    assert all(list(plain_top[t]) == list(np.argsort(-z[t], kind="stable")[:top]) for t in range(T))


def test_plain_retention_is_a_decayed_sum():
    rng = np.random.default_rng(3)
    T, d, e = 12, 4, 3
    q, k, v = rng.standard_normal((T, d)), rng.standard_normal((T, d)), rng.standard_normal((T, e))
    o, S = P.decayed_outer_sum(q, k, v, 0.8, return_state=True)
    for t in range(T):
        want = sum(0.8 ** (t - j) * float(q[t] @ k[j]) * v[j] for j in range(t + 1))
        assert np.abs(o[t] - want).max() < 1e-12
    assert np.allclose(S, sum(0.8 ** (T - 1 - j) * np.outer(k[j], v[j]) for j in range(T)))


def test_plain_model_is_causal_and_differential_factor():
    d = tiny()
    w = P.random_weights(d, 5)
    toks = [int(t) for t in np.random.default_rng(4).integers(0, d["vocab"], 30)]
    whole, rows = P.forward(d, w, toks, return_layers=True)
    assert rows.shape == (3, 30, d["width"])
    assert np.abs(P.forward(d, w, toks[:17]) - whole[:17]).max() < 1e-9
    # with equal maps and a factor of one the two maps cancel: the head's output is zero before the norm
    w2 = dict(w)
    for n in ("lq1", "lk1", "lq2", "lk2"):
        w2["l0.mix." + n] = np.zeros(8)
    d2 = copy.deepcopy(d)
    d2["layers"][0]["mixer"]["diff"] = 1.0                 # exp(0) - exp(0) + 1
    q = w2["l0.mix.q"].reshape(4, 2, 8, -1).copy()
    q[:, 1] = q[:, 0]
    k = w2["l0.mix.k"].reshape(2, 2, 8, -1).copy()
    k[:, 1] = k[:, 0]
    w2["l0.mix.q"], w2["l0.mix.k"] = q.reshape(64, -1), k.reshape(32, -1)
    x = w2["embed"][toks]
    assert np.abs(P.differential_mixer(x, w2, "l0.mix.", d2["layers"][0]["mixer"], 1e-5, np.arange(30))).max() < 1e-9
