"""The Ladadra design in the engine against the plain implementation (`plain_ladadra`): each mechanism's kernels alone,
whole prompts, portions, single tokens, batches, slots and pages used again, keys at the edges of windows, of runs of
positions, of the kept first tokens and of pages, and greedy generation through the engine's own entry point.
Configurations and weights are made here; where random weights would hide a fault (one far key among hundreds, an
edge that is one token off, a sink) the inputs are made so that it shows."""
import copy
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_ladadra as P

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def runs(heads, kv, dim, vdim, size=None, rot=None, softcap=None, scale=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else 1.2 / math.sqrt(dim)}
    if size is not None:
        m["mask"] = {"size": size}
    if rot is not None:
        m["rot"] = rot
    if softcap is not None:
        m["softcap"] = softcap
    return {"type": "attention", "mixer": m, "mlp": mlp}


def two_maps(heads, kv, dim, vdim, size=None, keep=0, diff=0.3, scale=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "diff": diff, "scale": scale if scale is not None else 1.2 / math.sqrt(dim)}
    if size is not None:
        m["mask"] = {"size": size, "keep_first": keep}
    return {"type": "attention_2", "mixer": m, "mlp": mlp}


def ret(heads, dim, vdim, decay, rot_dims=None, base=10000.0, mlp=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
    return {"type": "retention", "mixer": m, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, groups=None, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if groups is not None:
        m["router"]["groups"] = {"count": groups[0], "keep": groups[1]}
    if shared is not None:
        m["shared"] = {"ff": shared}
    return m


def model(width, vocab, layers, eps=1e-5):
    return {"architecture": "Ladadra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


STRETCH = {"factor": 3.0, "low": 1.0, "high": 3.0, "original": 64}
CONFIGS = {
    # the usual stack: two maps in a window with kept first tokens, runs of positions with part of every head rotated by
    # stretched frequencies, retention; dense units and routed experts with groups and a shared expert
    "a": model(64, 211, [two_maps(4, 2, 16, 24, size=40, keep=6, mlp=dense(96)),
                         runs(6, 2, 16, 16, size=48, rot={"base": 10000.0, "dims": 8, "scaling": STRETCH}, softcap=20.0, mlp=moe(32, 8, 3, (4, 2), 40)),
                         ret(3, 16, 24, (0.9, 0.97, 0.995), rot_dims=16, mlp=dense(96)),
                         runs(6, 2, 16, 16, size=48, rot={"base": 10000.0, "dims": 8, "scaling": STRETCH}, softcap=20.0, mlp=dense(96)),
                         two_maps(4, 2, 16, 24, size=40, keep=6, mlp=moe(32, 8, 3, (4, 2), 40))]),
    # sizes the usual shapes make equal or 1, and odd ones: one head, as many kv heads as heads, head sizes that are no
    # multiples of 4 or 8, a window of one token with kept first tokens, kept tokens beyond the window, runs of one
    # position, every element of a head rotated, no stretch, no score bound, a decay of 1 (a plain sum) and a short
    # memory, no rotation in a retention layer, all experts chosen, one chosen of one kept group, no groups, no shared
    # expert, layers without feed-forward
    "b": model(50, 97, [ret(1, 6, 20, (1.0,), mlp=moe(20, 3, 3)),
                        two_maps(1, 1, 6, 10, size=1, keep=3, diff=0.5, mlp=moe(24, 6, 1, (3, 1))),
                        runs(3, 3, 10, 6, size=1, rot={"base": 30.0, "dims": 10}),
                        two_maps(3, 3, 10, 5, size=7, keep=12, diff=0.1, mlp=dense(30)),
                        runs(2, 1, 12, 9, size=33, rot={"base": 1000.0, "dims": 2}, softcap=1.5, mlp=moe(12, 4, 2, (2, 2), 7)),
                        ret(2, 9, 5, (0.3, 0.97), rot_dims=4, base=77.0)], eps=1e-6),
    # sizes that the matrix-core attention kernels, the products' wide tiles and the grouped experts' kernels take;
    # windows, runs and kept tokens that cross page borders
    "c": model(256, 1000, [two_maps(4, 2, 64, 128, size=70, keep=10, mlp=dense(512)),
                           runs(8, 2, 64, 64, size=100, rot={"base": 500000.0, "dims": 32, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 256}},
                                softcap=30.0, mlp=moe(128, 12, 2, (3, 1), 192)),
                           ret(4, 64, 64, (0.9, 0.97, 0.99, 0.999), rot_dims=64, mlp=moe(128, 12, 2, (3, 1), 192)),
                           two_maps(8, 8, 32, 64, size=130, keep=65, mlp=dense(512))]),
    # retention only: no cache unit at all
    "d": model(64, 101, [ret(2, 16, 16, (0.8, 0.99), rot_dims=8, mlp=moe(16, 4, 2, (2, 1), 16)), ret(4, 8, 12, (0.5, 0.7, 0.9, 0.999), mlp=dense(64))]),
    # attention only, nothing masked (every earlier token is seen), a scale of 1, wide windows
    "e": model(32, 64, [runs(2, 2, 16, 16, scale=1.0, mlp=dense(48)), two_maps(2, 1, 16, 16, scale=1.0, mlp=moe(16, 2, 1)),
                        two_maps(2, 2, 8, 16, size=5000, keep=2, mlp=dense(48))]),
}
GAINS = {"a": 1.0, "b": 1.0, "c": 1.0, "d": 1.0, "e": 0.6}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    """(name, dtype) -> (folder, configuration, weights).  The bfloat16 runs get routers whose choice is clear (a token
    that takes another expert than the plain implementation differs by far more than rounding): the experts'
    corrections lie further apart than the scores' whole range; float32 holds the lively ones."""
    out = {}
    for name, cfg in CONFIGS.items():
        for dtype, spread in (("float32", 0.0), ("bfloat16", 2.5)):
            w = P.random_weights(cfg, seed=500 + ord(name), router_spread=spread, gain=GAINS[name])
            d = str(tmp_path_factory.mktemp(f"ladadra_{name}_{dtype}"))
            P.write_model(d, cfg, w)
            out[(name, dtype)] = (d, copy.deepcopy(cfg), w)
    return out


@pytest.fixture(scope="module")
def engines(folders):
    import braidinfer_amd as B
    made = {}

    def get(name, dtype, max_tokens=4096):
        if (name, dtype) not in made:
            made[(name, dtype)] = B.Engine.from_folder(folders[(name, dtype)][0], dtype=dtype, max_tokens=max_tokens)
        return made[(name, dtype)]
    return get


_plain = {}


def plain(name, dtype, cfg, w, toks):
    key = (name, dtype, json.dumps(cfg, sort_keys=True), tuple(toks))
    if key not in _plain:
        _plain[key] = P.forward(cfg, w, toks)
    return _plain[key]


def close(got, want, dtype, what=""):
    """Logits against the plain ones: centred difference over the vocabulary, relative to the logits' spread."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want)
    assert got.shape == want.shape, f"{what}: {got.shape} against {want.shape}"
    d = got - want
    d = d - d.mean(axis=-1, keepdims=True)
    err = np.sqrt((d * d).mean(axis=-1)) / want.std()
    if dtype == "float32":
        assert err.max() < 2e-4, f"{what}: row {err.argmax()} differs by {err.max():.3g}"
        return
    tol = 6e-2
    assert (err > tol).sum() <= max(1, len(err) // 25) and err.max() < 4 * tol, \
        f"{what}: {int((err > tol).sum())} rows of {len(err)} over {tol}, the worst (row {err.argmax()}) by {err.max():.3g}"


def run(eng, tokens, portions):
    """One sequence in the given portions; logits of every place."""
    import braidinfer_amd as B
    s = eng.alloc_slot()
    out, at = [], 0
    try:
        for n in portions:
            out.append(eng.step([B.StepEntry(s, tokens[at:at + n], list(range(n)))]).cpu().numpy())
            at += n
    finally:
        eng.free_slot(s)
    assert at == len(tokens)
    return np.concatenate(out)


def tokens_of(cfg, n, seed):
    return [int(t) for t in np.random.default_rng(seed).integers(0, cfg["vocab"], n)]


def dev_i(a):
    return torch.tensor(np.asarray(a), dtype=torch.int32).cuda()


def dev_f(a):
    return torch.tensor(np.asarray(a, dtype=np.float32)).cuda()


def f32(a):
    """Float64 values that float32 holds exactly."""
    return np.asarray(a, dtype=np.float32).astype(np.float64)


def bf(a):
    return P.to_bf16_values(a)


# ------------------------------------------------------------ mechanisms alone -------
def test_rows_as_they_are_and_the_norm_that_adds_behind_a_half():
    """The part in front of a half that reads the residual rows themselves, and the norm behind a half that also leaves
    the new rows for such a reader in the same kernel."""
    from braidinfer_amd.parts import Runtime, build_part
    from braidinfer_amd.config import PartSpec
    rng = np.random.default_rng(1)
    for T, W in ((7, 50), (3, 256), (2, 2050)):
        x = rng.standard_normal((T, W)).astype(np.float32)
        y = (rng.standard_normal((T, W)) * 0.03).astype(np.float32)        # small rows: eps inside the root matters
        wn = bf(1 + 0.2 * rng.standard_normal(W))
        want = f32(x) + P.rms_norm(f32(y), wn, 1e-3)
        for dtype in (torch.float32, torch.bfloat16):
            rt = Runtime(torch.device("cuda"), dtype)
            rows = build_part("norm", PartSpec("rows", {"size": W}))
            rows.load({}, "", rt)
            assert rows.weight_specs("x") == []
            out = torch.zeros((T, W), dtype=dtype, device="cuda")
            rows.forward(dev_f(x), out)
            assert np.array_equal(out.float().cpu().numpy(), x if dtype == torch.float32 else bf(x).astype(np.float32))
            n = build_part("norm", PartSpec("rmsnorm", {"size": W, "eps": 1e-3, "tensor": ""}))
            n.load({"n": torch.tensor(wn, dtype=torch.float32)}, "n", rt)
            acc, nxt = dev_f(x), torch.zeros((T, W), dtype=dtype, device="cuda")
            assert n.add_normed(dev_f(y), acc, rows, nxt)
            assert np.abs(acc.cpu().numpy() - want).max() < 2e-6
            got = nxt.float().cpu().numpy()
            assert np.array_equal(got, acc.cpu().numpy() if dtype == torch.float32 else bf(acc.cpu().numpy()).astype(np.float32))


def test_frequencies_stretched_by_wavelength():
    from braidinfer_amd.parts import Runtime, build_part
    from braidinfer_amd.config import PartSpec
    from braidinfer_amd import kernels as K
    rt = Runtime(torch.device("cuda"), torch.float32)
    for dims, base, sc in ((8, 100.0, {"factor": 3.0, "low": 1.0, "high": 5.0, "original": 40}), (32, 1e6, {"factor": 8.0, "low": 0.5, "high": 3.0, "original": 300}),
                           (6, 50.0, None)):
        params = {"rotary_dim": dims, "theta": base, "frequencies_from_float64": True}
        if sc:
            params.update(scaling=sc, scaling_rule="wavelength")
        enc = build_part("position", PartSpec("rope", params))
        enc.load({}, "", rt)
        want = P.rotary_frequencies(dims, base, sc)
        assert np.array_equal(enc.inv_freq.cpu().numpy(), want.astype(np.float32))
        if sc:
            kinds = {("same" if g == f else "slow" if g == f / sc["factor"] else "between") for f, g in zip(P.rotary_frequencies(dims, base), want)}
            assert kinds == {"same", "slow", "between"}, "the test's numbers leave a branch out"
        pos = np.array([0, 1, 63, 64, 700, 5])
        cos, sin = torch.zeros((6, dims // 2), device="cuda"), torch.zeros((6, dims // 2), device="cuda")
        K.rope_table(dev_i(pos), enc.inv_freq, cos, sin)
        ang = pos[:, None].astype(np.float64) * want.astype(np.float32).astype(np.float64)[None, :]
        assert np.abs(cos.cpu().numpy() - np.cos(ang)).max() < 1e-4 and np.abs(sin.cpu().numpy() - np.sin(ang)).max() < 1e-4


def shuffled_table(n_pages, n_slots, slot, seed):
    """A block table whose pages of `slot` lie in no order among pages that belong to nobody."""
    rng = np.random.default_rng(seed)
    table = np.full((n_slots, n_pages), -1, dtype=np.int32)
    table[slot] = rng.permutation(n_pages + 3)[:n_pages]
    return table


@pytest.mark.parametrize("H,G,d,e,rd,maps", [(4, 2, 16, 24, 8, 1), (3, 3, 10, 6, 10, 1), (1, 1, 6, 20, 0, 1), (8, 2, 64, 64, 32, 1),
                                             (4, 2, 16, 24, 0, 2), (1, 1, 6, 10, 0, 2), (3, 3, 10, 5, 4, 2), (4, 2, 64, 128, 0, 2)])
def test_prepare_norm_over_the_projection_maps_and_rotation(H, G, d, e, rd, maps):
    """Bias, the norm over a token's whole projection (or over every map of every head), rotation of part of a head,
    the query rows and the cache rows, in two portions at positions that are not the rows' numbers."""
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(H * 7 + d)
    T, eps = 70, 1e-3
    whole = maps == 1
    kw = maps * d
    width = (H + G) * kw + G * e + 3
    raw = (rng.standard_normal((T, width)) * 0.05).astype(np.float32)           # small sums: eps inside the root matters
    bias = (rng.standard_normal((H + G) * kw + G * e) * 0.05).astype(np.float32) if whole else None
    qn = (1 + 0.3 * rng.standard_normal(H * kw if whole else d)).astype(np.float32)
    kn = (1 + 0.3 * rng.standard_normal(G * kw if whole else d)).astype(np.float32)
    pos = np.arange(T) + 60                                                      # the pages' border inside
    freqs = P.rotary_frequencies(rd, 100.0).astype(np.float32).astype(np.float64) if rd else None
    x = f32(raw[:, :(H + G) * kw + G * e]) + (f32(bias) if whole else 0.0)
    q, k, v = x[:, :H * kw], x[:, H * kw:(H + G) * kw], x[:, (H + G) * kw:].reshape(T, G, e)
    if whole:
        q, k = P.rms_norm(q, f32(qn), eps).reshape(T, H, d), P.rms_norm(k, f32(kn), eps).reshape(T, G, d)
    else:
        q, k = P.rms_norm(q.reshape(T, H * maps, d), f32(qn), eps), P.rms_norm(k.reshape(T, G * maps, d), f32(kn), eps)
    if rd:
        q, k = P.rotate_half(q, pos, freqs), P.rotate_half(k, pos, freqs)
    n_pages = -(-int(pos[-1] + 1) // 64)
    table = shuffled_table(n_pages, 3, 1, d)
    for dtype, tol in ((torch.float32, 3e-5), (torch.bfloat16, 1e-2)):
        unit = torch.zeros((n_pages + 3, G * 64 * (kw + e)), dtype=dtype, device="cuda")
        got_q = []
        cos = sin = None
        for lo, hi in ((0, 41), (41, T)):
            n = hi - lo
            if rd:
                cos, sin = torch.zeros((n, rd // 2), device="cuda"), torch.zeros((n, rd // 2), device="cuda")
                K.rope_table(dev_i(pos[lo:hi]), dev_f(freqs), cos, sin)
            qo = torch.full((n, H * maps * kw), 9.0, dtype=dtype, device="cuda")
            K.pwa_prepare(dev_f(raw[lo:hi]), dev_f(bias) if whole else None, dev_f(qn), dev_f(kn), eps, cos, sin, rd, dev_i(pos[lo:hi]),
                          dev_i(np.zeros(n)), dev_i([1]), dev_i(table), qo, unit, None, None, 0, H, G, d, e, 64, True,
                          maps=maps, row_ss=torch.zeros((n, 2), device="cuda") if whole else None)
            got_q.append(qo.float().cpu().numpy())
        got_q = np.concatenate(got_q).reshape(T, H * maps, kw)
        scale_q = max(1.0, np.abs(q).max())
        for m in range(maps):
            mine = got_q[:, m::maps] if maps > 1 else got_q
            assert np.abs(mine[..., m * d:(m + 1) * d] - (q[:, m::maps] if maps > 1 else q)).max() < tol * scale_q
            other = np.delete(mine, np.s_[m * d:(m + 1) * d], axis=2)
            assert other.size == 0 or np.abs(other).max() == 0                   # zeros where the other map's keys lie
        pages = unit.float().cpu().numpy()
        for t in range(T):
            pg = pages[table[1, pos[t] // 64]]
            keys = pg[:G * 64 * kw].reshape(G, 64, kw)[:, pos[t] % 64]
            vals = pg[G * 64 * kw:].reshape(G, e, 64)[:, :, pos[t] % 64]
            assert np.abs(keys.reshape(G * maps, d) - k[t]).max() < tol * max(1.0, np.abs(k).max()), f"keys of token {t}"
            assert np.abs(vals - v[t]).max() < tol * max(1.0, np.abs(v).max())
        used = set(table[1].tolist())
        assert all(float(np.abs(pages[p]).max()) == 0 for p in range(n_pages + 3) if p not in used)


def attend(q, k, v, portions, dtype, matrix, size=None, chunk=0, keep=0, softcap=0.0, scale=1.0, sinks=None, first=0):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv] of one sequence whose first token stands at position `first` of a slot
    whose pages lie shuffled: the rows go into the cache portion by portion (no norm, no rotation), each portion's
    queries through the float kernel, or the matrix-core kernels for prompts and for single tokens."""
    from braidinfer_amd import kernels as K
    T, H, dk = q.shape
    G, dv = k.shape[1], v.shape[2]
    assert first == 0
    n_pages = -(-T // 64)
    table = shuffled_table(n_pages, 4, 2, T + H)
    unit = torch.zeros((n_pages + 3, G * 64 * (dk + dv)), dtype=dtype, device="cuda")
    rows = np.concatenate([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], axis=1).astype(np.float32)
    window = size if size is not None else (1 << 30)
    sk = dev_f(sinks) if sinks is not None else None
    mask = dict(chunk=chunk, keep=keep, softcap=softcap)
    out, at = [], 0
    for n in portions:
        pos, sot, slots = dev_i(np.arange(at, at + n)), dev_i(np.zeros(n)), dev_i([2])
        qo = torch.zeros((n, H * dk), dtype=dtype, device="cuda")
        K.pwa_prepare(dev_f(rows[at:at + n]), None, None, None, 0.0, None, None, 0, pos, sot, slots, dev_i(table), qo, unit, None, None, 0,
                      H, G, dk, dv, 64, True)
        o = torch.full((n, H * dv), 5.0, dtype=dtype, device="cuda")
        if not matrix:
            K.pwa_attend(qo, o, pos, sot, slots, dev_i(table), unit, None, None, H, G, dk, dv, 64, window, 0, scale, sinks is not None, sk, **mask)
        elif n > 1:
            K.pwa_prefill_bf16(qo, o, dev_i([0, n]), slots, dev_i([at + n]), dev_i(table), unit, None, None, 1, n, H, G, dk, dv, 64, window, 0,
                               scale, sinks is not None, sk, **mask)
        else:
            K.pwa_decode_bf16(qo, o, slots, dev_i([at + n]), dev_i(table), unit, None, None, 1, H, G, dk, dv, 64, window, 0, scale,
                              sinks is not None, sk, **mask)
        out.append(o.float().cpu().numpy())
        at += n
    return np.concatenate(out).reshape(T, H, dv)


def visible_of(T, size, chunk, keep):
    """Window and run of positions together; the kept first tokens are seen whatever the two say."""
    m = P.window_mask(T, size) if size is not None else P.causal(T)
    if chunk:
        m = m & P.chunk_mask(T, chunk)
    return m | (P.causal(T) & (np.arange(T)[None, :] < keep))


MASKS = [dict(size=40, keep=6), dict(size=1, keep=3), dict(size=7, keep=12), dict(size=70, keep=65), dict(size=130, keep=0), dict(chunk=48),
         dict(chunk=1), dict(chunk=100, softcap=3.0), dict(chunk=64), dict(size=50, chunk=30, keep=2), dict()]


@pytest.mark.parametrize("mask", MASKS, ids=lambda m: "-".join(f"{k}{v}" for k, v in m.items()) or "all")
def test_attention_kernels_with_windows_runs_and_kept_tokens(mask):
    """The three attention kernels on shuffled pages against the plain attention: whole, in portions down to single
    tokens; with a learnt sink, bounded scores, kept first tokens."""
    rng = np.random.default_rng(len(mask) + sum(int(v) for v in mask.values()))
    T, H, G, dk, dv = 215, 4, 2, 16, 24
    q, k, v = rng.standard_normal((T, H, dk)), rng.standard_normal((T, G, dk)), rng.standard_normal((T, G, dv))
    sinks = rng.standard_normal(H) if "chunk" in mask else None
    vis = visible_of(T, mask.get("size"), mask.get("chunk", 0), mask.get("keep", 0))
    want = P.masked_attention(f32(q), f32(k), f32(v), 0.4, vis, mask.get("softcap"), f32(sinks) if sinks is not None else None)
    for portions in ([T], [2, 3, 59, 1, 63, 2, 64, 21], [150] + [1] * 65):
        got = attend(q, k, v, portions, torch.float32, False, scale=0.4, sinks=sinks, **mask)
        assert np.abs(got - want).max() < 3e-5, f"float kernel, {portions[:3]}"
    want16 = P.masked_attention(bf(q), bf(k), bf(v), 0.4, vis, mask.get("softcap"), f32(sinks) if sinks is not None else None)
    for portions in ([T], [150, 2, 33] + [1] * 30, [20] + [1] * 195):
        got = attend(q, k, v, portions, torch.bfloat16, True, scale=0.4, sinks=sinks, **mask)
        assert np.abs(got - want16).max() < 0.03, f"matrix-core kernels, {portions[:3]}"
    got = attend(q, k, v, [100, 115], torch.bfloat16, False, scale=0.4, sinks=sinks, **mask)          # the float kernel on bfloat16 rows
    assert np.abs(got - want16).max() < 0.03


@pytest.mark.parametrize("H,G,dk,dv", [(8, 2, 128, 64), (2, 2, 32, 128), (16, 1, 64, 64), (3, 1, 24, 20)])
def test_attention_kernels_at_other_sizes(H, G, dk, dv):
    """Key rows as wide as two maps' keys, many query heads to a kv head, widths the matrix cores take in part."""
    rng = np.random.default_rng(dk)
    T = 300
    q, k, v = rng.standard_normal((T, H, dk)) * 0.5, rng.standard_normal((T, G, dk)), rng.standard_normal((T, G, dv))
    sinks = rng.standard_normal(H)
    for mask in (dict(size=75, keep=21), dict(chunk=110, softcap=8.0)):
        vis = visible_of(T, mask.get("size"), mask.get("chunk", 0), mask.get("keep", 0))
        want = P.masked_attention(bf(q), bf(k), bf(v), 0.2, vis, mask.get("softcap"), f32(sinks))
        got = attend(q, k, v, [2, 250] + [1] * 48, torch.bfloat16, True, scale=0.2, sinks=sinks, **mask)
        assert np.abs(got - want).max() < 0.03
        got = attend(q, k, v, [140, 160], torch.float32, False, scale=0.2, sinks=sinks, **mask)
        assert np.abs(got - P.masked_attention(f32(q), f32(k), f32(v), 0.2, vis, mask.get("softcap"), f32(sinks))).max() < 5e-5


def test_edges_that_random_inputs_would_hide():
    """One key made loud (its score stands out) just inside and just outside every edge: the window's first position,
    the kept tokens' last, a run's first position, page borders, a far key among hundreds; asked for in a prompt and
    by a single token.  The loud key's value is marked, so the output says whether it was seen."""
    rng = np.random.default_rng(9)
    T, H, G, dk, dv = 330, 2, 1, 16, 8
    cases = []            # (mask, query position, loud key, seen?)
    for size, keep in ((75, 21), (64, 64), (65, 1), (128, 0)):
        for p in (size + 30, 255, 256, 329):
            cases += [(dict(size=size, keep=keep), p, p - size + 1, True), (dict(size=size, keep=keep), p, p - size, p - size < keep)]
            if keep:
                cases += [(dict(size=size, keep=keep), p, keep - 1, True), (dict(size=size, keep=keep), p, keep, p - keep < size)]
    for chunk in (110, 64, 63, 100):
        for p in (chunk, chunk + 5, 2 * chunk - 1, 2 * chunk, 329):
            lo = (p // chunk) * chunk
            cases += [(dict(chunk=chunk), p, lo, True)] + ([(dict(chunk=chunk), p, lo - 1, False)] if lo else [])
    cases += [(dict(), 329, 0, True), (dict(), 329, 63, True), (dict(), 329, 64, True), (dict(), 300, 301, False)]
    for dtype, matrix in ((torch.float32, False), (torch.bfloat16, True)):
        for mask, p, loud, seen in cases:
            if not 0 <= loud < T:
                continue
            q, k, v = rng.standard_normal((T, H, dk)) * 0.3, rng.standard_normal((T, G, dk)) * 0.3, rng.standard_normal((T, G, dv)) * 0.1
            k[loud, 0] = 0.0
            k[loud, 0, 3] = 8.0
            q[p, :, 3] = 8.0                      # a score of 64 where the others stay below 2
            v[loud, 0] = 100.0
            for portions in ([T], [p] + [1] * (T - p)):
                got = attend(q, k, v, portions, dtype, matrix, **mask)[p]
                if seen:
                    assert got.min() > 99.0, f"{mask}: the query at {p} does not see key {loud} ({portions[:2]}, {dtype})"
                else:
                    assert np.abs(got).max() < 5.0, f"{mask}: the query at {p} sees key {loud} ({portions[:2]}, {dtype})"


def test_a_sink_that_takes_all_the_weight_and_one_that_takes_none():
    rng = np.random.default_rng(10)
    T, H, G, dk, dv = 90, 4, 2, 16, 16
    q, k, v = rng.standard_normal((T, H, dk)), rng.standard_normal((T, G, dk)), rng.standard_normal((T, G, dv)) + 3.0
    sinks = np.array([60.0, -60.0, 0.0, 1.5])
    want = P.masked_attention(f32(q), f32(k), f32(v), 0.3, P.chunk_mask(T, 70), 5.0, sinks)
    no_sink = P.masked_attention(f32(q), f32(k), f32(v), 0.3, P.chunk_mask(T, 70), 5.0)
    assert np.abs(want[:, 0]).max() < 1e-15 and np.abs(want[:, 1] - no_sink[:, 1]).max() < 1e-12 and np.abs(want[:, 2] - no_sink[:, 2]).min() > 1e-4
    for dtype, matrix, tol in ((torch.float32, False, 3e-5), (torch.bfloat16, True, 0.05)):
        got = attend(q, k, v, [60] + [1] * 30, dtype, matrix, chunk=70, softcap=5.0, scale=0.3, sinks=sinks)
        assert np.abs(got - want).max() < tol
        # a score bound holds the scores below the sink's reach: without it head 3 would differ
        unbounded = attend(q * 6, k, v, [T], dtype, matrix, chunk=70, scale=0.3, sinks=sinks)
        bounded = attend(q * 6, k, v, [T], dtype, matrix, chunk=70, softcap=5.0, scale=0.3, sinks=sinks)
        assert np.abs(bounded - P.masked_attention(f32(q * 6), f32(k), f32(v), 0.3, P.chunk_mask(T, 70), 5.0, sinks)).max() < tol * 2
        assert np.abs(unbounded - bounded).max() > 0.1


@pytest.mark.parametrize("H,G,d,e,T", [(4, 2, 16, 24, 150), (2, 2, 64, 128, 300), (8, 1, 32, 64, 100), (1, 1, 8, 12, 70)])
def test_two_maps_through_the_matrix_core_kernels(H, G, d, e, T):
    """Prompts on the matrix cores take the maps as workgroups of their own (query rows of d, reading their map's part
    of the key rows); single tokens and the float kernel see every map as a query head over whole key rows (zeros outside
    the map).  Both against the plain attention of every map, whole and behind an earlier portion."""
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(T + d)
    raw = rng.standard_normal((T, (H + G) * 2 * d + G * e)).astype(np.float32)
    q, k = bf(raw[:, :H * 2 * d]).reshape(T, H * 2, d), bf(raw[:, H * 2 * d:(H + G) * 2 * d]).reshape(T, G, 2, d)
    v = bf(raw[:, (H + G) * 2 * d:]).reshape(T, G, e)
    vis = P.window_mask(T, 70, 9)
    want = np.zeros((T, H * 2, e))
    for m in range(2):
        want[:, m::2] = P.masked_attention(q[:, m::2], k[:, :, m], v, 0.3, vis)
    n_pages = -(-T // 64)
    table = shuffled_table(n_pages, 4, 2, T)
    for padded in (True, False):
        unit = torch.zeros((n_pages + 3, G * 64 * (2 * d + e)), dtype=torch.bfloat16, device="cuda")
        got, at = [], 0
        for n in (T - 40, 38, 1, 1):
            pos, sot, slots = dev_i(np.arange(at, at + n)), dev_i(np.zeros(n)), dev_i([2])
            pad = padded or n == 1
            qo = torch.zeros((n, H * 2 * (2 * d if pad else d)), dtype=torch.bfloat16, device="cuda")
            K.pwa_prepare(dev_f(raw[at:at + n]), None, None, None, 0.0, None, None, 0, pos, sot, slots, dev_i(table), qo, unit, None, None, 0,
                          H, G, d, e, 64, True, maps=2, pad_queries=pad)
            o = torch.full((n, H * 2 * e), 5.0, dtype=torch.bfloat16, device="cuda")
            if n == 1:
                K.pwa_decode_bf16(qo, o, slots, dev_i([at + 1]), dev_i(table), unit, None, None, 1, H * 2, G, 2 * d, e, 64, 70, 0, 0.3, False, None, keep=9)
            elif pad:
                K.pwa_prefill_bf16(qo, o, dev_i([0, n]), slots, dev_i([at + n]), dev_i(table), unit, None, None, 1, n, H * 2, G, 2 * d, e, 64, 70, 0,
                                   0.3, False, None, keep=9)
            else:
                K.pwa_prefill_bf16(qo, o, dev_i([0, n]), slots, dev_i([at + n]), dev_i(table), unit, None, None, 1, n, H * 2, G, d, e, 64, 70, 0,
                                   0.3, False, None, keep=9, maps=2)
            got.append(o.float().cpu().numpy())
            at += n
        assert np.abs(np.concatenate(got).reshape(T, H * 2, e) - want).max() < 0.03, f"padded {padded}"


def test_two_maps_into_one_head():
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(11)
    for T, H, e in ((9, 4, 24), (5, 1, 10), (3, 3, 128), (2, 2, 5)):
        a = rng.standard_normal((T, H, 2, e)).astype(np.float32)
        for eps, factor, scale in ((1e-5, 0.37, 0.7), (None, -0.2, 1.0), (0.5, 1.0, 0.25)):
            d = f32(a[:, :, 0]) - np.float32(factor).astype(np.float64) * f32(a[:, :, 1])
            want = (P.rms_divide(d, eps) if eps is not None else d) * scale
            o = torch.zeros((T, H * e), device="cuda")
            K.pwa_pair_combine(dev_f(a.reshape(T, -1)), o, H, e, factor, eps, scale)
            assert np.abs(o.cpu().numpy().reshape(T, H, e) - want).max() < 1e-5
        ob = torch.zeros((T, H * e), dtype=torch.bfloat16, device="cuda")
        K.pwa_pair_combine(dev_f(a.reshape(T, -1)).to(torch.bfloat16), ob, H, e, 0.37, 1e-5, 0.7)
        want = P.rms_divide(bf(a[:, :, 0]) - np.float32(0.37).astype(np.float64) * bf(a[:, :, 1]), 1e-5) * 0.7
        assert np.abs(ob.float().cpu().numpy().reshape(T, H, e) - want).max() < 0.02


@pytest.mark.parametrize("H,d,e,rd", [(3, 16, 24, 16), (1, 6, 20, 0), (2, 9, 5, 4), (4, 64, 64, 64), (2, 128, 256, 32)])
def test_retention_rotation_sum_and_head_norm(H, d, e, rd):
    """q and k turned in place and the key scaled, the decayed sum in portions with the state in a slot, every head's
    output over its root mean square times silu of the gate."""
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(d + e)
    T, eps = 75, 1e-5
    decay = np.array([1.0, 0.3, 0.97, 0.999][:H], dtype=np.float32)
    width = 2 * H * d + 2 * H * e
    raw = rng.standard_normal((T, width)).astype(np.float32)
    freqs = P.rotary_frequencies(rd, 77.0).astype(np.float32).astype(np.float64) if rd else None
    x = f32(raw)
    q, k = x[:, :H * d].reshape(T, H, d), x[:, H * d:2 * H * d].reshape(T, H, d)
    if rd:
        q, k = P.rotate_half(q, np.arange(T), freqs), P.rotate_half(k, np.arange(T), freqs)
    k = k * d ** -0.5
    v, gate = x[:, 2 * H * d:2 * H * d + H * e].reshape(T, H, e), x[:, 2 * H * d + H * e:]
    o = np.stack([P.decayed_outer_sum(q[:, h], k[:, h], v[:, h], float(decay[h])) for h in range(H)], axis=1)
    want = P.rms_divide(o, eps).reshape(T, H * e) * P.silu(gate)
    shape = K.glr_state_shape(H, d, e)
    state = torch.zeros((4,) + tuple(shape), device="cuda")
    got, at = [], 0
    for n in (40, 1, 1, 2, 31):
        rows = dev_f(raw[at:at + n])
        cos = sin = None
        if rd:
            cos, sin = torch.zeros((n, rd // 2), device="cuda"), torch.zeros((n, rd // 2), device="cuda")
            K.rope_table(dev_i(np.arange(at, at + n)), dev_f(freqs), cos, sin)
        K.dr_rotate_rows(rows[:, :H * d], rows[:, H * d:2 * H * d], cos, sin, rd, H, d, 1.0, d ** -0.5)
        oo = torch.zeros((n, H * e), device="cuda")
        K.dr_scan(rows[:, :H * d], rows[:, H * d:2 * H * d], rows[:, 2 * H * d:2 * H * d + H * e], None, dev_f(decay), oo, state, dev_i([0, n]),
                  dev_i([2]), 1, H, H, d, e, silu=False)
        y = torch.zeros((n, H * e), device="cuda")
        K.head_norm_gate(oo, None, rows[:, 2 * H * d + H * e:], y, H, e, eps)
        got.append(y.cpu().numpy())
        at += n
    assert np.abs(np.concatenate(got) - want).max() < 2e-4 * max(1.0, np.abs(want).max())
    assert float(state[[0, 1, 3]].abs().max()) == 0


def test_choice_of_experts_by_corrected_sigmoid_scores_in_groups():
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(12)
    for T, E, top, groups in ((40, 8, 3, (2, 1)), (30, 12, 3, (4, 2)), (9, 6, 1, (3, 1)), (9, 6, 6, None), (20, 70, 5, (10, 3)), (7, 4, 2, (4, 2)),
                              (11, 130, 8, (65, 9)), (5, 3, 3, (1, 1)), (6, 2, 1, None)):
        z = (rng.standard_normal((T, E)) * 2).astype(np.float32)
        corr = (rng.standard_normal(E) - 1.0).astype(np.float32)                 # choice scores below zero happen
        z[:, 1] = z[:, 0]
        corr[1] = corr[0]                                                         # two experts that always tie: the lower number first
        g = {"count": groups[0], "keep": groups[1]} if groups else None
        want_c, want_w = P.choose_experts(f32(z), f32(corr), top, g)
        chosen = torch.zeros((T, top), dtype=torch.int32, device="cuda")
        share = torch.zeros((T, top), dtype=torch.float32, device="cuda")
        K.route_sigmoid(dev_f(z), dev_f(corr), chosen, share, top, groups[0] if groups else 1, groups[1] if groups else 1, 1.0)
        got_c = chosen.cpu().numpy()
        s = 1 / (1 + np.exp(-f32(z)))
        c = s + f32(corr)
        for t in range(T):
            if list(got_c[t]) != list(want_c[t]):
                # float32 scores may order two experts otherwise than float64 ones only where they are equal to rounding
                a, b = np.sort(c[t][got_c[t]]), np.sort(c[t][want_c[t]])
                assert np.abs(a - b).max() < 1e-6, f"{E} experts, token {t}: {got_c[t]} against {want_c[t]}"
            else:
                assert np.abs(share[t].cpu().numpy() - want_w[t]).max() < 1e-6
        if g:           # nothing outside the kept groups, whatever its score
            per = E // groups[0]
            assert all(len({e // per for e in row}) <= groups[1] for row in got_c)


# ------------------------------------------------------------ whole models -----------
@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_against_plain(folders, engines, name, dtype):
    _, cfg, w = folders[(name, dtype)]
    toks = tokens_of(cfg, 150, 1)
    want = plain(name, dtype, cfg, w, toks)
    close(run(engines(name, dtype), toks, [150]), want, dtype, f"{name} {dtype}")
    close(run(engines(name, dtype), toks[:1], [1]), want[:1], dtype, "a sequence of one token")
    close(run(engines(name, dtype), toks[:3], [1, 1, 1]), want[:3], dtype, "the first tokens one by one")
    close(run(engines(name, dtype), toks[:5], [2, 3]), want[:5], dtype, "the first tokens in two portions")


@pytest.mark.parametrize("name", ["a", "b"])
def test_residual_rows_after_every_layer(folders, engines, name):
    import braidinfer_amd as B
    _, cfg, w = folders[(name, "float32")]
    toks = tokens_of(cfg, 60, 9)
    _, layers = P.forward(cfg, w, toks, return_layers=True)
    eng = engines(name, "float32")
    seen = {}
    s = eng.alloc_slot()
    eng.step([B.StepEntry(s, toks, [])], probe=lambda n, t: seen.__setitem__(n, t.float().cpu().numpy().copy()))
    eng.free_slot(s)
    for i in range(len(layers)):
        assert np.abs(seen[f"L{i}.post_ffn"] - layers[i]).max() < 2e-4 * np.abs(layers[i]).max(), f"layer {i}"


@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_and_single_tokens(folders, engines, name, dtype):
    """A prompt in portions down to two tokens, then token by token across pages' borders, windows' and runs' edges,
    against the plain logits and, in float32, against the whole prompt's own."""
    _, cfg, w = folders[(name, dtype)]
    n = 215
    toks = tokens_of(cfg, n, 2)
    want = plain(name, dtype, cfg, w, toks)
    eng = engines(name, dtype)
    whole = run(eng, toks, [n])
    for portions in ([2, 3, 59, 1, 63, 2, 64, 21], [17] + [1] * 198, [128, 2] + [1] * 85):
        got = run(eng, toks, portions)
        close(got, want, dtype, f"{name} {dtype} {portions[:4]}")
        if dtype == "float32":
            assert np.abs(got - whole).max() < 2e-4 * np.abs(whole).max()


@pytest.mark.parametrize("name", ["a", "b", "c"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batch_against_each_alone(folders, engines, name, dtype):
    import braidinfer_amd as B
    _, cfg, w = folders[(name, dtype)]
    eng = engines(name, dtype)
    lens = [1, 90, 33, 140, 7]
    prompts = [tokens_of(cfg, n + 20, 10 + n) for n in lens]
    slots = [eng.alloc_slot() for _ in lens]
    got = [[] for _ in lens]
    lg = eng.step([B.StepEntry(s, p[:n], list(range(n))) for s, p, n in zip(slots, prompts, lens)]).cpu().numpy()
    at = 0
    for i, n in enumerate(lens):
        got[i].append(lg[at:at + n])
        at += n
    live = list(range(len(lens)))
    for t in range(20):
        if t == 8:                                  # two requests end early; the batch goes on without them
            for i in (1, 4):
                eng.free_slot(slots[i])
                live.remove(i)
        lg = eng.step([B.StepEntry(slots[i], [prompts[i][lens[i] + t]], [0]) for i in live]).cpu().numpy()
        for r, i in enumerate(live):
            got[i].append(lg[r:r + 1])
    for i in live:
        eng.free_slot(slots[i])
    for i, p in enumerate(prompts):
        g = np.concatenate(got[i])
        close(g, plain(name, dtype, cfg, w, p)[:len(g)], dtype, f"request {i} of the batch")


def test_slots_and_pages_used_again(folders):
    """Requests come and go through a cache of few pages and slots: what a freed slot's state or a returned page held
    never shows, the kept first tokens' pages stay while the window's move on, and every page comes back."""
    import braidinfer_amd as B
    folder, cfg, w = folders[("a", "float32")]
    eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=448, max_seq_len=448, n_slots=2)
    free_before = [g.pool.free_count for g in eng.cache.groups]
    assert sorted(eng.cache.group_of_unit) == [0, 1, 3, 4]           # the retention layer keeps a state, no rows
    for r in range(5):
        toks = tokens_of(cfg, 120 + 67 * r, 50 + r)
        close(run(eng, toks, [len(toks) - 10] + [1] * 10), P.forward(cfg, w, toks), "float32", f"request {r}")
    assert [g.pool.free_count for g in eng.cache.groups] == free_before
    # a sequence longer than the pages a window holds at a time: pages behind the window have gone back, the first stays
    toks = tokens_of(cfg, 400, 77)
    s = eng.alloc_slot()
    got = [eng.step([B.StepEntry(s, toks[:380], [379])]).cpu().numpy()]
    windowed = eng.cache.unit_group(0)
    assert [i for i, p in enumerate(windowed.pages[s]) if p >= 0] == [0, 5]
    for t in range(380, 400):
        got.append(eng.step([B.StepEntry(s, [toks[t]], [0])]).cpu().numpy())
    eng.free_slot(s)
    close(np.concatenate(got), P.forward(cfg, w, toks)[379:], "float32", "behind returned pages")
    # two requests side by side whose slots have just been used, one of them a single token long
    a, b = tokens_of(cfg, 70, 90), tokens_of(cfg, 1, 91)
    sa, sb = eng.alloc_slot(), eng.alloc_slot()
    lg = eng.step([B.StepEntry(sa, a, [69]), B.StepEntry(sb, b, [0])]).cpu().numpy()
    eng.free_slot(sa)
    eng.free_slot(sb)
    close(lg, np.stack([P.forward(cfg, w, a)[69], P.forward(cfg, w, b)[0]]), "float32", "after the slots' earlier users")


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_long_decoding(folders, engines, name):
    """Three hundred single-token steps from a short prompt (recorded steps of the engine), past page borders, windows
    that move over decoded tokens and runs of positions that begin among them."""
    for dtype in ("float32", "bfloat16"):
        _, cfg, w = folders[(name, dtype)]
        toks = tokens_of(cfg, 330, 3)
        close(run(engines(name, dtype), toks, [30] + [1] * 300), plain(name, dtype, cfg, w, toks), dtype, f"{name} {dtype}")


def test_a_long_prompt(folders, engines):
    for dtype in ("float32", "bfloat16"):
        _, cfg, w = folders[("c", dtype)]
        toks = tokens_of(cfg, 700, 8)
        want = plain("c", dtype, cfg, w, toks)
        close(run(engines("c", dtype), toks, [700]), want, dtype, f"whole {dtype}")
        close(run(engines("c", dtype), toks, [100, 600]), want, dtype, f"behind a portion {dtype}")


def drawn_configuration(seed):
    """A configuration drawn at random: any order of layers, head counts and widths from lists that hold odd ones and
    such that the matrix-core kernels take, any window, run and number of kept tokens, keys left out."""
    rng = np.random.default_rng(seed)
    pick = lambda xs: xs[int(rng.integers(len(xs)))]

    def heads():
        H = pick([1, 2, 3, 4, 6, 8, 12])
        return H, pick([g for g in (1, 2, 3, 4, 6, 8, 12) if H % g == 0])

    def mlp():
        r = rng.random()
        if r < 0.15:
            return None
        if r < 0.5:
            return dense(pick([24, 40, 64]))
        E = pick([2, 4, 6, 8, 16])
        count = pick([c for c in (1, 2, 4, 8) if E % c == 0])
        keep = int(rng.integers(1, count + 1))
        top = pick([t for t in (1, 2, 3, 4, 8) if t <= keep * (E // count)])
        return moe(pick([8, 16, 24, 40]), E, top, (count, keep) if rng.random() < 0.8 else None, pick([None, 16, 24]))
    layers = []
    for _ in range(int(rng.integers(2, 6))):
        kind = pick(["attention", "attention_2", "retention"])
        if kind == "attention":
            H, G = heads()
            d = pick([8, 12, 16, 24, 32, 64])
            rot = None
            if rng.random() < 0.85:
                rot = {"base": pick([100.0, 10000.0, 1e6]), "dims": pick([r for r in (2, 4, 8, 12, 16, 32, 64) if r <= d])}
                if rng.random() < 0.6:
                    rot["scaling"] = {"factor": pick([2.0, 4.0, 8.0]), "low": pick([0.5, 1.0]), "high": pick([2.0, 4.0]), "original": pick([16, 64, 256])}
            layers.append(runs(H, G, d, pick([8, 12, 16, 32, 64]), size=pick([None, 1, 7, 33, 64, 100]), rot=rot, softcap=pick([None, 5.0, 30.0]), mlp=mlp()))
        elif kind == "attention_2":
            H, G = heads()
            layers.append(two_maps(H, G, pick([8, 12, 16, 32, 48]), pick([8, 12, 16, 32, 64]), size=pick([None, 1, 9, 40, 64, 90]),
                                   keep=pick([0, 1, 5, 20, 70]), diff=pick([0.1, 0.3, 0.5]), mlp=mlp()))
        else:
            H = pick([1, 2, 3, 4, 8])
            d = pick([4, 8, 16, 32, 40])
            layers.append(ret(H, d, pick([4, 8, 16, 32, 72]), [float(x) for x in rng.uniform(0.5, 1.0, H)],
                              rot_dims=pick([0] + [r for r in (2, 4, 8, 16, 32) if r <= d]), mlp=mlp()))
    return model(pick([32, 48, 64, 80]), int(rng.integers(40, 300)), layers, eps=pick([1e-6, 1e-5, 1e-3]))


@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_at_random(seed, tmp_path):
    """Whole, in portions and token by token in float32 against the plain implementation; bfloat16 whole and decoded."""
    import braidinfer_amd as B
    cfg = drawn_configuration(2000 + seed)
    what = f"seed {seed}: {json.dumps(cfg['layers'])}"
    toks = tokens_of(cfg, 110, seed)
    other = tokens_of(cfg, 45, seed + 50)
    folder = str(tmp_path / "m")
    w = P.random_weights(cfg, seed=seed, gain=0.9)
    P.write_model(folder, cfg, w)
    want, ow = P.forward(cfg, w, toks), P.forward(cfg, w, other)
    eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=512)
    close(run(eng, toks, [110]), want, "float32", what)
    close(run(eng, toks, [3, 62, 2, 1, 1] + [1] * 41), want, "float32", what + " in portions")
    sa, sb = eng.alloc_slot(), eng.alloc_slot()
    lg = eng.step([B.StepEntry(sa, toks[:70], [69]), B.StepEntry(sb, other[:44], [0, 43])]).cpu().numpy()
    lg2 = eng.step([B.StepEntry(sa, toks[70:71], [0]), B.StepEntry(sb, other[44:], [0])]).cpu().numpy()
    eng.free_slot(sa)
    eng.free_slot(sb)
    close(np.concatenate([lg, lg2]), np.stack([want[69], ow[0], ow[43], want[70], ow[44]]), "float32", what + " two requests")
    del eng
    w = P.random_weights(cfg, seed=seed, gain=0.9, router_spread=2.5)
    P.write_model(folder, cfg, w)
    eng = B.Engine.from_folder(folder, dtype="bfloat16", max_tokens=512)
    close(run(eng, toks, [60] + [1] * 50), P.forward(cfg, w, toks), "bfloat16", what + " bfloat16")


def test_greedy_generation_through_the_engine(folders, engines):
    _, cfg, w = folders[("a", "float32")]
    prompts = [tokens_of(cfg, n, 20 + n) for n in (3, 41, 12, 70)]
    want = [P.greedy(cfg, w, p, 12) for p in prompts]
    got = engines("a", "float32").generate(prompts, max_new_tokens=12, temperature=0.0, stop_token_ids=[])
    assert got == want
    _, cfg, w = folders[("a", "bfloat16")]
    want = [P.greedy(cfg, w, p, 12) for p in prompts]
    got16 = engines("a", "bfloat16").generate(prompts, max_new_tokens=12, temperature=0.0, stop_token_ids=[])
    for g, wnt, p in zip(got16, want, prompts):
        for i, (a, b) in enumerate(zip(g, wnt)):
            if a != b:                              # bfloat16 may take the runner-up where two logits are nearly tied
                l = P.forward(cfg, w, p + wnt[:i])[-1]
                assert abs(l[a] - l[b]) < 0.05 * np.abs(l).max()
                break


def test_the_command_line_generates_from_a_ladadra_folder(folders):
    """`bin/generate` on a Ladadra folder: the model class by config.json, greedy tokens as the plain implementation's;
    a sampled run ends and stays inside the vocabulary."""
    folder, cfg, w = folders[("a", "float32")]
    p = [7, 3, 200, 5, 11]
    want = P.greedy(cfg, w, p, 6)
    env = dict(os.environ, MODEL=folder, MAX_TOKENS="6")
    gen = [sys.executable, os.path.join(ROOT, "bin", "generate"), "--dtype", "float32", "--prompt-ids", ",".join(map(str, p))]
    r = subprocess.run(gen, env=env, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    assert [int(t) for t in r.stdout.split()] == want
    r = subprocess.run(gen + ["--temperature", "0.8", "--top-k", "20", "--seed", "5"], env=env, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    toks = [int(t) for t in r.stdout.split()]
    assert len(toks) == 6 and all(0 <= t < cfg["vocab"] for t in toks)


def test_presets_run(tmp_path):
    """The tiny preset as a random-weights folder of the library's own making, against the plain implementation."""
    import braidinfer_amd as B
    cfg = B.any_preset("ladadra-tiny")
    folder = B.Engine.write_random_folder(str(tmp_path / "m"), cfg, seed=3, std=0.2, vector_jitter=0.3)
    pc, pw = P.read_model(folder)
    toks = tokens_of(pc, 120, 4)
    eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=512)
    close(run(eng, toks, [90] + [1] * 30), P.forward(pc, pw, toks), "float32", "preset")


def test_replay_of_given_tokens_through_the_command(folders, tmp_path):
    """`bin/trace_run` as a child process on a Ladadra folder: requests whole, with their last tokens one by one, and two
    of unequal length in one batch, against the plain logits."""
    folder, cfg, w = folders[("b", "float32")]
    V = cfg["vocab"]
    seqs = [tokens_of(cfg, n, 60 + n) for n in (90, 41)]
    refs = [P.forward(cfg, w, s) for s in seqs]
    out = str(tmp_path / "out")
    p = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", out,
                          "--max-tokens", "512"], stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    n = [0]

    def step(entries, end=()):
        p.stdin.write(json.dumps({"step": n[0], "entries": entries, "end": list(end)}) + "\n")
        p.stdin.flush()
        line = p.stdout.readline().strip()
        assert line == f"done {n[0]}", f"trace_run said {line!r} (exit {p.poll()})"
        path = os.path.join(out, f"{n[0]}.f32")
        n[0] += 1
        return np.fromfile(path, dtype="<f4").reshape(-1, V) if os.path.exists(path) else None

    got = step([{"id": "w", "tokens": seqs[0], "want": [0, 63, 64, 89]}], end=["w"])
    close(got, refs[0][[0, 63, 64, 89]], "float32", "whole")
    assert step([{"id": "d", "tokens": seqs[0][:60], "want": []}]) is None
    for t in range(60, 90):
        got = step([{"id": "d", "tokens": [seqs[0][t]], "want": [0]}], end=["d"] if t == 89 else [])
        close(got, refs[0][t:t + 1], "float32", f"one by one at {t}")
    got = step([{"id": "a", "tokens": seqs[0][:80], "want": [79]}, {"id": "b", "tokens": seqs[1][:35], "want": [3, 34]}])
    close(got, np.stack([refs[0][79], refs[1][3], refs[1][34]]), "float32", "a batch's prompts")
    for t in range(6):
        ending = ["b"] if t == 5 else []
        got = step([{"id": "a", "tokens": [seqs[0][80 + t]], "want": [0]}, {"id": "b", "tokens": [seqs[1][35 + t]], "want": [0]}], end=ending)
        close(got, np.stack([refs[0][80 + t], refs[1][35 + t]]), "float32", f"a batch's token {t}")
    got = step([{"id": "a", "tokens": [seqs[0][86]], "want": [0]}], end=["a"])
    close(got, refs[0][86:87], "float32", "the batch's longer request alone")
    p.stdin.close()
    assert p.wait(timeout=60) == 0
