"""The Zivovik design in the engine against the plain implementation (`plain_zivovik`): each mechanism's kernels
alone, whole prompts, portions, single tokens, batches, slots used again, far keys, page borders, the edges of the
query temperature's steps, and greedy generation through the engine's own entry point.  Configurations and weights
are made here; where random weights would hide a fault (one far key among hundreds, a temperature's step) the inputs
are made so that it shows."""
import copy
import json
import math

import numpy as np
import pytest
import torch

import plain_zivovik as P

pytestmark = pytest.mark.gpu


def att(heads, kv, dim, coef=0.4, every=16, scale=None, mlp=None):
    return {"type": "attention", "mlp": mlp, "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim,
                                                        "scale": scale if scale is not None else 1.2 / math.sqrt(dim),
                                                        "q_temp": {"coef": coef, "every": every}}}


def par(left, right, mlp=None):
    """left (heads, kv, dim, vdim, coef, every), right (heads, kv, dim, vdim, taps)."""
    H, G, d, e, coef, every = left
    rh, rg, rd, re_, taps = right
    return {"type": "parallel", "mlp": mlp, "mixer": {
        "left": {"heads": H, "kv_heads": G, "dim": d, "vdim": e, "scale": 1.1 / math.sqrt(d), "q_temp": {"coef": coef, "every": every}},
        "right": {"heads": rh, "kv_heads": rg, "dim": rd, "vdim": re_, "conv": taps}}}


def lig(heads, dim, vdim, decay, mlp=None):
    return {"type": "lightning", "mlp": mlp, "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}}


def moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def model(width, vocab, layers, loop, eps=1e-5, emb=2.0, mult=0.7, positions=1024):
    d = {"architecture": "Zivovik", "vocab": vocab, "width": width, "max_positions": positions, "norm": {"eps": eps},
         "embedding": {"scale": emb}, "residual_mult": mult, "layers": layers}
    if loop is not None:
        d["loop"] = dict(zip(("start", "stop", "times"), loop))
    return d


CONFIGS = {
    # the usual stack: attention, then a parallel and a lightning layer passed four times, a closing attention layer
    "a": model(64, 211, [att(4, 2, 16, every=16, mlp=moe(32, 6, 2)), par((3, 1, 16, 24, 0.3, 24), (4, 2, 16, 24, 4), mlp=moe(32, 6, 2)),
                         lig(3, 16, 24, (0.6, 0.9, 0.995), mlp=moe(32, 6, 2)), att(4, 2, 16, every=16, mlp=moe(32, 6, 2))], (1, 3, 4)),
    # sizes the usual shapes make equal or 1, and odd ones: the whole model passed twice, as many key heads as heads and
    # one head, head sizes that are no multiples of 4 or 8, a convolution of one tap (none) and of two, a decay of 1
    # (a plain sum) and a short memory, all experts chosen, one expert chosen, layers without feed-forward, an
    # embedding scale and a residual multiplier of 1, a temperature that steps every 7 positions and one that never
    # steps inside the table
    "b": model(50, 97, [lig(1, 6, 20, (1.0,), mlp=moe(20, 3, 3)), att(3, 3, 10, coef=0.5, every=7, mlp=moe(24, 5, 1)),
                        par((1, 1, 12, 6, 0.2, 5000), (4, 2, 6, 10, 1)), par((4, 4, 6, 6, 0.3, 3), (3, 3, 5, 9, 2), mlp=moe(12, 2, 1)),
                        lig(2, 9, 5, (0.3, 0.97))], (0, 5, 2), eps=1e-6, emb=1.0, mult=1.0),
    # no repeated pass; a lightning layer first and a parallel layer last; heads wider than 64 channels in both
    # recurrences; more heads than a matrix-core workgroup serves at once; a convolution of five taps
    "c": model(96, 150, [lig(1, 80, 72, (0.9,), mlp=moe(40, 9, 4)), att(24, 8, 8, every=64, mlp=moe(24, 4, 2)),
                         par((2, 2, 32, 16, 0.5, 10), (2, 1, 72, 80, 5), mlp=moe(24, 4, 2))], None),
    # recurrent layers only, the last one passed three times: no cache unit at all
    "d": model(64, 101, [lig(2, 16, 16, (0.8, 0.99), mlp=moe(16, 4, 2)), lig(4, 8, 12, (0.5, 0.7, 0.9, 0.999), mlp=moe(16, 4, 2))], (1, 2, 3)),
    # attention only, the first layer passed twice; every width equal, a scale of 1, two experts
    "e": model(32, 64, [att(2, 2, 16, coef=0.25, every=1, scale=1.0, mlp=moe(16, 2, 1)), att(2, 1, 16, coef=0.0, every=9, scale=1.0, mlp=moe(16, 2, 2))],
               (0, 1, 2)),
    # sizes that the matrix-core attention kernels, the products' wide tiles and the grouped experts' kernels take
    "f": model(256, 1000, [par((4, 2, 64, 128, 0.3, 32), (4, 2, 64, 128, 4), mlp=moe(128, 8, 2)), att(8, 2, 64, every=48, mlp=moe(128, 8, 2)),
                           lig(4, 64, 64, (0.7, 0.9, 0.97, 0.999), mlp=moe(128, 8, 2))], (0, 2, 2)),
}

# The size of the random matrices: large enough for every layer to move the logits, small enough where a scale of 1
# or a head of few channels would otherwise make a softmax so sharp that it amplifies bfloat16 rounding a hundredfold.
GAINS = {"a": 1.3, "b": 1.0, "c": 1.3, "d": 1.3, "e": 0.7, "f": 1.0}


# One expert chosen in front of a state that never forgets (a decay of 1) and a model passed twice: a single close call of
# a router early in a prompt, which bfloat16 activations may turn the other way, moves every later row.  The bfloat16
# runs of this configuration choose all experts of every layer (the weights are the same); float32 runs it as it is.
ALL_EXPERTS_IN_BFLOAT16 = {"b"}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    """(name, dtype) -> (folder, configuration, weights)."""
    out = {}
    for name, cfg in CONFIGS.items():
        w = P.random_weights(cfg, seed=300 + ord(name), gain=GAINS[name])
        d = str(tmp_path_factory.mktemp(f"zivovik_{name}"))
        P.write_folder(d, cfg, w)
        out[(name, "float32")] = out[(name, "bfloat16")] = (d, copy.deepcopy(cfg), w)
        if name in ALL_EXPERTS_IN_BFLOAT16:
            calm = copy.deepcopy(cfg)
            for l in calm["layers"]:
                if l["mlp"] is not None:
                    l["mlp"]["router"]["top"] = l["mlp"]["router"]["experts"]
            d = str(tmp_path_factory.mktemp(f"zivovik_{name}_all"))
            P.write_folder(d, calm, w)
            out[(name, "bfloat16")] = (d, calm, w)
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


def plain(name, cfg, w, toks):
    """The plain logits, and per token whether every choice of experts on its way was a clear one: the distance
    between the last chosen router logit and the first one left out, smallest over the layer runs."""
    key = (name, json.dumps(cfg, sort_keys=True), tuple(toks))
    if key not in _plain:
        margins = []
        want = P.forward(cfg, w, toks, margins=margins)
        _plain[key] = (want, np.min(margins, axis=0) if margins else np.full(len(toks), np.inf))
    return _plain[key]


CLOSE_CALL = 0.05        # router logits closer than this may fall the other way once activations are rounded to bfloat16


def close(got, want, dtype, what="", margins=None, close_call=CLOSE_CALL, min_clear=0.3):
    """Logits against the plain ones: centred difference over the vocabulary, relative to the logits' spread.  In
    bfloat16 a token whose choice of experts was a close call in the plain implementation may have taken the other
    expert (the router has no bias that a test could set apart); such rows are left out, float32 holds them like all
    others."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want)
    d = got - want
    d = d - d.mean(axis=-1, keepdims=True)
    err = np.sqrt((d * d).mean(axis=-1)) / want.std()
    tol = 2e-4 if dtype == "float32" else 6e-2
    if dtype != "float32":
        if margins is not None:
            clear = np.asarray(margins)[:len(err)] >= close_call
            assert len(err) < 20 or clear.sum() >= min_clear * len(err), f"{what}: most choices of experts are close calls; the test's weights are at fault"
            err = err[clear]
            if not len(err):
                return
        assert (err > tol).sum() <= max(1, len(err) // 25) and err.max() < 4 * tol, \
            f"{what}: {int((err > tol).sum())} rows of {len(err)} over {tol}, the worst (row {err.argmax()}) by {err.max():.3g}"
        return
    assert err.max() < tol, f"{what}: row {err.argmax()} differs by {err.max():.3g} (tolerance {tol})"


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


# ------------------------------------------------------------ mechanisms alone -------
def test_learnt_positions_embedding_scale_and_the_sum_of_rows():
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(1)
    T, W, rows = 9, 50, 30
    table = P.to_bf16(rng.standard_normal((rows, W)))
    x0 = rng.standard_normal((T, W)).astype(np.float32)
    pos = np.array([0, 1, 29, 5, 5, 17, 28, 2, 3])
    for dtype in (torch.float32, torch.bfloat16):
        x = dev_f(x0)
        K.add_position_rows(x, torch.tensor(table, dtype=torch.float32).cuda().to(dtype), dev_i(pos))
        assert np.abs(x.cpu().numpy() - (x0 + table[pos])).max() < 1e-6
    emb = P.to_bf16(rng.standard_normal((20, W)))
    out = torch.zeros((T, W), device="cuda")
    toks = rng.integers(0, 20, T)
    K.embedding(torch.tensor(emb, dtype=torch.float32).cuda().to(torch.bfloat16), dev_i(toks), out, 3.5)
    assert np.abs(out.cpu().numpy() - emb[toks] * 3.5).max() < 1e-6
    y = rng.standard_normal((T, W)).astype(np.float32)
    x = dev_f(x0)
    K.residual_add(x, dev_f(y))
    assert np.array_equal(x.cpu().numpy(), x0 + y)


def test_norm_weights_around_zero_and_a_normed_branch_added():
    """The norm part with an offset (w = 1 + stored) and with a multiplier; the norm behind a branch adds into the rows."""
    from braidinfer_amd.parts import Runtime, build_part
    from braidinfer_amd.config import PartSpec
    rng = np.random.default_rng(2)
    T, W, eps = 7, 50, 1e-3
    rt = Runtime(torch.device("cuda"), torch.float32)
    stored = P.to_bf16(0.2 * rng.standard_normal(W))
    x = (rng.standard_normal((T, W)) * 0.02).astype(np.float32)          # small rows: eps inside the root matters
    n = build_part("norm", PartSpec("rmsnorm", {"size": W, "eps": eps, "tensor": "", "offset": 1.0, "scale": 1.0}))
    n.load({"n": torch.tensor(stored, dtype=torch.float32)}, "n", rt)
    out = torch.zeros((T, W), device="cuda")
    n.forward(dev_f(x), out)
    assert np.abs(out.cpu().numpy() - P.offset_norm(f32(x), stored, eps)).max() < 1e-6
    chosen = torch.zeros((2, W), device="cuda")
    n.forward(dev_f(x), chosen, rows=dev_i([5, 0]))
    assert np.abs(chosen.cpu().numpy() - P.offset_norm(f32(x), stored, eps)[[5, 0]]).max() < 1e-6
    m = build_part("norm", PartSpec("rmsnorm", {"size": W, "eps": eps, "tensor": "", "offset": 0.0, "scale": 0.35}))
    m.load({"n": torch.tensor(stored + 1.0, dtype=torch.float32)}, "n", rt)
    acc0 = rng.standard_normal((T, W)).astype(np.float32)
    acc = dev_f(acc0)
    m.add_normed(dev_f(x), acc)
    assert np.abs(acc.cpu().numpy() - (acc0 + 0.35 * P.plain_norm(f32(x), stored + 1.0, eps))).max() < 1e-6


@pytest.mark.parametrize("G,H,d,e,taps,by_four", [(2, 4, 6, 10, 3, False), (1, 1, 80, 72, 1, False), (2, 2, 16, 24, 4, False), (3, 6, 33, 7, 2, False),
                                                 (1, 2, 130, 8, 16, False), (2, 2, 16, 24, 4, True), (1, 1, 80, 72, 1, True), (2, 4, 128, 128, 4, True),
                                                 (1, 2, 300, 260, 3, True)])
def test_convolution_unit_vectors_decay_and_write_strength(G, H, d, e, taps, by_four):
    """The step in front of the delta rule: two sequences in unequal portions down to single tokens, the last inputs
    kept in slots that are not neighbours and lie inside wider rows, a padding sequence between them."""
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(G * 100 + taps)
    C = 2 * G * d + H * e
    width = C + 2 * H + (4 - (C + 2 * H) % 4 if by_four else 5)       # the projection's rows carry further columns behind
    lens = [41, 9]
    raw = [rng.standard_normal((n, width)).astype(np.float32) * 1.5 for n in lens]
    w_taps = (rng.standard_normal((C, taps)) * 0.6).astype(np.float32)
    a_log, dt_bias = rng.uniform(-3, 0.5, H).astype(np.float32), rng.uniform(-2, 25, H).astype(np.float32)
    want = []
    for r in raw:
        r = f32(r)
        c = P.silu(P.short_convolution(r[:, :C], f32(w_taps)))
        q = P.unit_vectors(c[:, :G * d].reshape(-1, G, d)) * d ** -0.5
        k = P.unit_vectors(c[:, G * d:2 * G * d].reshape(-1, G, d))
        beta = P.sigmoid(r[:, C:C + H])
        g = np.exp(-np.exp(f32(a_log)) * P.softplus(r[:, C + H:C + 2 * H] + f32(dt_bias)))
        want.append((q.reshape(-1, G * d), k.reshape(-1, G * d), c[:, 2 * G * d:], np.concatenate([g, beta], axis=1)))
    n_kept = (taps - 1) * C
    arena = torch.zeros((6, n_kept + (8 if by_four else 9)), dtype=torch.float32, device="cuda")
    kept = arena[:, 4:4 + n_kept] if taps > 1 else None
    taps_t = dev_f(np.ascontiguousarray(w_taps.T)) if by_four else None          # four channels a lane through 16-byte loads
    slots_of = [4, 1]
    got = [[[] for _ in range(4)] for _ in lens]
    at = [0, 0]
    for portion in ([20, 3], [1, 1], [1, 1], [2, 2], [17, 2]):
        pieces = [raw[0][at[0]:at[0] + portion[0]], np.full((1, width), 3.0, np.float32), raw[1][at[1]:at[1] + portion[1]]]
        rows = torch.tensor(np.concatenate(pieces)).cuda()
        T = rows.shape[0]
        new = [portion[0], 1, portion[1]]
        q, k = torch.zeros((T, G * d), device="cuda"), torch.zeros((T, G * d), device="cuda")
        v, gb = torch.zeros((T, H * e), device="cuda"), torch.zeros((T, 2 * H), device="cuda")
        K.dr_conv_prepare(rows, dev_f(w_taps), kept, dev_f(a_log), dev_f(dt_bias), dev_i(np.repeat(np.arange(3), new)),
                          dev_i(np.cumsum([0] + new)), dev_i([slots_of[0], -1, slots_of[1]]), q, k, v, gb, 3, G, H, d, e, taps_t=taps_t)
        for i, lo in ((0, 0), (1, portion[0] + 1)):
            for j, t in enumerate((q, k, v, gb)):
                got[i][j].append(t.cpu().numpy()[lo:lo + portion[i]])
            at[i] += portion[i]
    for i in range(2):
        for j, what in enumerate(("q", "k", "v", "g and beta")):
            g_ = np.concatenate(got[i][j])
            assert np.abs(g_ - want[i][j][:len(g_)]).max() < 2e-5 * max(1.0, np.abs(want[i][j]).max()), f"sequence {i}: {what}"
    if taps > 1:
        for i in range(2):                       # the slot keeps the sequence's last taps - 1 inputs, oldest first
            last = raw[i][at[i] - (taps - 1):at[i], :C] if at[i] >= taps - 1 else None
            if last is not None:
                assert np.array_equal(kept[slots_of[i]].cpu().numpy().reshape(taps - 1, C), last)
    assert float(arena[[0, 2, 3, 5]].abs().max()) == 0 and float(arena[:, :4].abs().max()) == 0 and float(arena[:, 4 + n_kept:].abs().max()) == 0


def scan_in_portions(q, k, v, gb, decay, H, G, d, e, portions, silu=False):
    """Two sequences (lists of arrays) through the scan in the given portions, a padding sequence between them, the
    states in slots 4 and 1 of an arena whose rows are wider than the state.  Returns outputs and dense final states."""
    from braidinfer_amd import kernels as K
    n_state = int(np.prod(K.glr_state_shape(H, d, e)))
    arena = torch.zeros((6, n_state + 24), dtype=torch.float32, device="cuda")
    state = arena[:, 8:8 + n_state].view((6,) + tuple(K.glr_state_shape(H, d, e)))
    slots_of = [4, 1]
    got, at = [[], []], [0, 0]
    for portion in portions:
        new = [portion[0], 1, portion[1]]

        def cut(seqs, width, fill):
            return torch.tensor(np.concatenate([seqs[0][at[0]:at[0] + portion[0]], np.full((1, width), fill, np.float32),
                                                seqs[1][at[1]:at[1] + portion[1]]]).astype(np.float32)).cuda()
        T = sum(new)
        o = torch.full((T, H * e), 7.0, dtype=torch.float32, device="cuda")
        K.dr_scan(cut(q, G * d, 1.0), cut(k, G * d, 1.0), cut(v, H * e, 1.0), cut(gb, 2 * H, 0.5) if gb is not None else None,
                  dev_f(decay) if decay is not None else None, o, state, dev_i(np.cumsum([0] + new)), dev_i([slots_of[0], -1, slots_of[1]]),
                  3, H, G, d, e, silu=silu)
        o = o.cpu().numpy()
        got[0].append(o[:portion[0]])
        got[1].append(o[portion[0] + 1:])
        at[0] += portion[0]
        at[1] += portion[1]
    dense = [K.glr_state_dense(state[s], H, d, e).cpu().numpy() for s in slots_of]
    assert float(arena[[0, 2, 3, 5]].abs().max()) == 0 and float(arena[:, :8].abs().max()) == 0 and float(arena[:, 8 + n_state:].abs().max()) == 0
    return [np.concatenate(g) for g in got], dense


PORTIONS = ([20, 3], [1, 1], [1, 1], [2, 1], [13, 0], [1, 2])


@pytest.mark.parametrize("H,G,d,e", [(4, 2, 16, 24), (1, 1, 80, 72), (3, 3, 5, 9), (6, 2, 33, 7), (2, 1, 130, 8), (2, 2, 128, 128)])
def test_gated_delta_rule_scan(H, G, d, e):
    rng = np.random.default_rng(H * 10 + d)
    lens = [38, 8]
    q = [f32(P.unit_vectors(rng.standard_normal((n, G, d))).reshape(n, -1)) for n in lens]
    k = [f32(P.unit_vectors(rng.standard_normal((n, G, d))).reshape(n, -1)) for n in lens]
    v = [f32(rng.standard_normal((n, H * e))) for n in lens]
    gb = [f32(np.concatenate([rng.uniform(0.3, 1.0, (n, H)), rng.uniform(0.0, 1.0, (n, H))], axis=1)) for n in lens]
    got, dense = scan_in_portions(q, k, v, gb, None, H, G, d, e, PORTIONS)
    for i, n in enumerate(lens):
        for h in range(H):
            kh = h // (H // G)
            o, S = P.delta_rule(q[i][:, kh * d:(kh + 1) * d], k[i][:, kh * d:(kh + 1) * d], v[i][:, h * e:(h + 1) * e], gb[i][:, H + h],
                                gb[i][:, h], return_state=True)
            assert np.abs(got[i][:, h * e:(h + 1) * e] - o).max() < 2e-5 * max(1.0, np.abs(o).max()), f"sequence {i} head {h}"
            assert np.abs(dense[i][h] - S).max() < 2e-5 * max(1.0, np.abs(S).max())


@pytest.mark.parametrize("H,d,e", [(3, 16, 24), (1, 80, 72), (2, 9, 5), (1, 6, 20), (2, 128, 128)])
def test_decayed_outer_sum_scan(H, d, e):
    """The fixed decay per head, with silu on the way in (the projections' sums go straight into the walk), among the
    decays 1 (a plain sum) and 0 (only the current token)."""
    rng = np.random.default_rng(H * 10 + e)
    lens = [38, 8]
    decay = np.array([1.0, 0.0, 0.9][:H] if H > 1 else [0.97], dtype=np.float32)
    q, k, v = ([f32(rng.standard_normal((n, H * w))) for n in lens] for w in (d, d, e))
    got, dense = scan_in_portions(q, k, v, None, decay, H, H, d, e, PORTIONS, silu=True)
    for i in range(2):
        for h in range(H):
            o, S = P.decayed_outer_sum(P.silu(q[i][:, h * d:(h + 1) * d]), P.silu(k[i][:, h * d:(h + 1) * d]), P.silu(v[i][:, h * e:(h + 1) * e]),
                                       float(decay[h]), return_state=True)
            assert np.abs(got[i][:, h * e:(h + 1) * e] - o).max() < 3e-5 * max(1.0, np.abs(o).max()), f"sequence {i} head {h}"
            assert np.abs(dense[i][h] - S).max() < 3e-5 * max(1.0, np.abs(S).max())


@pytest.mark.parametrize("H,d,e,pieces", [(3, 16, 24, 3), (1, 80, 72, 5), (2, 128, 128, 4), (2, 9, 5, 2)])
def test_decayed_outer_sum_in_pieces(H, d, e, pieces):
    """Long portions cut into pieces that are walked side by side: two sequences with states left by an earlier portion,
    a padding sequence between them, pieces of unequal length and an empty one."""
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(H + d + pieces)
    lens, first = [150, 61], [30, 5]
    decay = np.array([1.0, 0.0, 0.9][:H] if H > 1 else [0.97], dtype=np.float32)
    q, k, v = ([f32(rng.standard_normal((n, H * w))) for n in lens] for w in (d, d, e))
    shape = tuple(K.glr_state_shape(H, d, e))
    state = torch.zeros((6,) + shape, dtype=torch.float32, device="cuda")
    slots_of = [4, 1]
    got = [[], []]
    # the first portions by the plain walk
    new = [first[0], 1, first[1]]
    cat = lambda seqs, lo, n, width: torch.tensor(np.concatenate([seqs[0][lo[0]:lo[0] + n[0]], np.ones((1, width)),
                                                                   seqs[1][lo[1]:lo[1] + n[1]]]).astype(np.float32)).cuda()
    o = torch.zeros((sum(new), H * e), dtype=torch.float32, device="cuda")
    K.dr_scan(cat(q, [0, 0], first, H * d), cat(k, [0, 0], first, H * d), cat(v, [0, 0], first, H * e), None, dev_f(decay), o, state,
              dev_i(np.cumsum([0] + new)), dev_i([slots_of[0], -1, slots_of[1]]), 3, H, H, d, e, silu=True)
    got[0].append(o.cpu().numpy()[:first[0]])
    got[1].append(o.cpu().numpy()[first[0] + 1:])
    # the rest in pieces: runs of equal length, the last ones shorter or empty
    rest = [lens[0] - first[0], lens[1] - first[1]]
    new = [rest[0], 1, rest[1]]
    cu, numbers, at = [0], [], 0
    for b, n in enumerate(new):
        run = -(-(-(-n // pieces)) // 16) * 16
        for c in range(pieces):
            cu.append(at + min(n, (c + 1) * run))
            numbers.append(b * pieces + c if b != 1 else -1)
        at += n
    assert any(cu[i] == cu[i + 1] for i in range(len(cu) - 1))
    o = torch.full((sum(new), H * e), 7.0, dtype=torch.float32, device="cuda")
    scratch = torch.full((3 * pieces,) + shape, 5.0, dtype=torch.float32, device="cuda")
    K.dr_scan_pieces(cat(q, first, rest, H * d), cat(k, first, rest, H * d), cat(v, first, rest, H * e), dev_f(decay), o, state,
                     dev_i([slots_of[0], -1, slots_of[1]]), dev_i(cu), dev_i(numbers), scratch, 3, pieces, H, d, e, silu=True)
    got[0].append(o.cpu().numpy()[:rest[0]])
    got[1].append(o.cpu().numpy()[rest[0] + 1:])
    for i in range(2):
        g_ = np.concatenate(got[i])
        for h in range(H):
            want, S = P.decayed_outer_sum(P.silu(q[i][:, h * d:(h + 1) * d]), P.silu(k[i][:, h * d:(h + 1) * d]), P.silu(v[i][:, h * e:(h + 1) * e]),
                                          float(decay[h]), return_state=True)
            assert np.abs(g_[:, h * e:(h + 1) * e] - want).max() < 3e-5 * max(1.0, np.abs(want).max()), f"sequence {i} head {h}"
            dense = K.glr_state_dense(state[slots_of[i]], H, d, e).cpu().numpy()[h]
            assert np.abs(dense - S).max() < 3e-5 * max(1.0, np.abs(S).max())
    assert float(state[[0, 2, 3, 5]].abs().max()) == 0


def test_silu_of_some_columns_in_place():
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(11)
    for T, width, lo, n in ((9, 40, 0, 24), (5, 37, 3, 30), (1, 16, 4, 8), (300, 64, 8, 52)):
        x0 = (rng.standard_normal((T, width)) * 4).astype(np.float32)
        x = dev_f(x0)
        K.silu_rows(x[:, lo:lo + n])
        want = f32(x0).copy()
        want[:, lo:lo + n] = P.silu(want[:, lo:lo + n])
        assert np.abs(x.cpu().numpy() - want).max() < 1e-6 * np.abs(want).max()
        assert np.array_equal(x.cpu().numpy()[:, :lo], x0[:, :lo]) and np.array_equal(x.cpu().numpy()[:, lo + n:], x0[:, lo + n:])


def test_order_of_decay_correction_write_and_read():
    """Inputs that tell the order apart: the read-out sees the token's own write; the decay comes before the correction;
    a repeated key with full write strength replaces what lay under it; no write strength leaves the state alone."""
    H = G = 1
    d, e = 4, 4
    k0 = np.array([1.0, 0, 0, 0])
    k1 = np.array([0.0, 1, 0, 0])
    v = np.array([[1.0, -2, 0.5, 4], [3.0, 1, -1, 2], [0.5, 0.5, 8, -3]])
    # token 0 writes v0 under k0 and reads it at once; token 1 repeats k0 with decay 0.5 and beta 1: v1 replaces 0.5 v0;
    # token 2 has beta 0 and another key: it reads what lies under k0 after its decay 0.25
    q = [np.stack([k0, k0, k0]), np.zeros((1, 4))]
    k = [np.stack([k0, k0, k1]), np.zeros((1, 4))]
    vv = [v, np.zeros((1, 4))]
    gb = [np.array([[0.9, 1.0], [0.5, 1.0], [0.25, 0.0]]), np.ones((1, 2))]
    for portions in ([[3, 1]], [[1, 1], [1, 0], [1, 0]], [[2, 0], [1, 1]]):
        got, dense = scan_in_portions(q, k, vv, gb, None, H, G, d, e, portions)
        assert np.allclose(got[0][0], v[0], atol=1e-6) and np.allclose(got[0][1], v[1], atol=1e-6) and np.allclose(got[0][2], 0.25 * v[1], atol=1e-6)
        want = np.zeros((4, 4))
        want[0] = 0.25 * v[1]
        assert np.allclose(dense[0][0], want, atol=1e-6)


def test_head_norms_with_both_gates():
    """Every head normed alone with one weight for all heads and a silu gate; all heads normed together with a sigmoid
    gate; the gates read from inside wider rows."""
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(4)
    for T, H, e in ((7, 3, 33), (2, 1, 80), (5, 4, 16), (1, 6, 7), (3, 8, 128), (2, 2, 600)):       # rows of 512 channels and more take a workgroup each
        o = rng.standard_normal((T, H * e)).astype(np.float32) * 3
        o[0] *= 1e-3                                            # a row so small that eps inside the root matters
        w1 = (1 + 0.3 * rng.standard_normal(e)).astype(np.float32)
        wa = (1 + 0.3 * rng.standard_normal(H * e)).astype(np.float32)
        wide = rng.standard_normal((T, 3 * H * e)).astype(np.float32)
        gate = torch.tensor(wide).cuda()[:, H * e:2 * H * e]
        g = f32(wide[:, H * e:2 * H * e])
        for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
            y = torch.empty((T, H * e), dtype=dtype, device="cuda")
            K.head_norm_gate(dev_f(o), dev_f(np.tile(w1, H)), gate, y, H, e, 1e-5)
            want = (P.rms_divide(f32(o).reshape(T, H, e), 1e-5) * f32(w1)).reshape(T, H * e) * P.silu(g)
            assert np.abs(y.float().cpu().numpy() - want).max() < tol * max(1.0, np.abs(want).max())
            K.head_norm_gate(dev_f(o), dev_f(wa), gate, y, 1, H * e, 1e-5, gate_sigmoid=True)
            want = P.plain_norm(f32(o), f32(wa), 1e-5) * P.sigmoid(g)
            assert np.abs(y.float().cpu().numpy() - want).max() < tol * max(1.0, np.abs(want).max())


def test_output_gates_of_attention():
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(5)
    for T, H, e in ((6, 3, 24), (1, 4, 16), (9, 1, 7)):
        o0 = P.to_bf16(rng.standard_normal((T, H * e)))
        wide = rng.standard_normal((T, 11 + H * e + H)).astype(np.float32) * 2
        dev = torch.tensor(wide).cuda()
        for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 1e-2)):
            o = torch.tensor(o0, dtype=torch.float32).cuda().to(dtype)
            K.pwa_gate(o, dev[:, 11:11 + H * e], H, e, False, 0.7)
            assert np.abs(o.float().cpu().numpy() - o0 * P.sigmoid(f32(wide[:, 11:11 + H * e])) * np.float32(0.7)).max() < tol * np.abs(o0).max()
            o = torch.tensor(o0, dtype=torch.float32).cuda().to(dtype)
            K.pwa_gate(o, dev[:, 11 + H * e:], H, e, True, 1.0)
            want = (o0.reshape(T, H, e) * P.sigmoid(f32(wide[:, 11 + H * e:]))[:, :, None]).reshape(T, H * e)
            assert np.abs(o.float().cpu().numpy() - want).max() < tol * np.abs(o0).max()


class HandCache:
    """A cache unit with a block table of shuffled pages, for the attention kernels alone."""

    def __init__(self, G, dk, dv, dtype, n_pages=24, slots=3, seed=0):
        perm = np.random.default_rng(seed).permutation(n_pages)
        per = n_pages // slots
        self.G, self.dk, self.dv = G, dk, dv
        self.table = torch.tensor(perm[:per * slots].reshape(slots, per), dtype=torch.int32).cuda()
        self.unit = torch.full((n_pages, G * 64 * (dk + dv)), 1e4, dtype=dtype, device="cuda")     # stale rows would show

    def rows(self, slot, positions):
        """Keys [n, G, dk] and values [n, G, dv] as the cache holds them (values lie transposed in a page)."""
        unit, table = self.unit.float().cpu().numpy(), self.table.cpu().numpy()
        G, dk, dv = self.G, self.dk, self.dv
        ks = [unit[table[slot, p // 64]][:G * 64 * dk].reshape(G, 64, dk)[:, p % 64] for p in positions]
        vs = [unit[table[slot, p // 64]][G * 64 * dk:].reshape(G, dv, 64)[:, :, p % 64] for p in positions]
        return np.stack(ks), np.stack(vs)


NO_WINDOW = 1 << 30


def attend(rows, H, G, dk, dv, scale, portions, dtype=torch.float32, matrix=False, keys_as_values=False, eps=None, temp=(0.0, 0),
           start=0, cache=None, slot=1):
    """The projections' float sums [T, H dk + G dk (+ G dv)] through prepare and an attention kernel without window, in the
    given portions from position `start` on (`matrix`: the matrix-core kernels).  Returns the mixed values, the
    queries as prepared, and the cache."""
    from braidinfer_amd import kernels as K
    T = rows.shape[0]
    c = cache or HandCache(G, dk, dv, dtype)
    ones = torch.ones(dk, device="cuda") if eps is not None else None
    outs, qs, at = [], [], 0
    for n in portions:
        pos, sot = dev_i(np.arange(start + at, start + at + n)), dev_i(np.ones(n))     # the batch's second sequence; the first is padding
        slots, cu, ctx = dev_i([-1, slot]), dev_i([0, 0, n]), dev_i([0, start + at + n])
        qo = torch.empty((n, H * dk), dtype=dtype, device="cuda")
        K.pwa_prepare(dev_f(rows[at:at + n]), None, ones, ones, eps or 0.0, None, None, 0, pos, sot, slots, c.table, qo, c.unit, None, None, 0,
                      H, G, dk, dv, 64, True, keys_as_values, temp[0], temp[1])
        o = torch.empty((n, H * dv), dtype=dtype, device="cuda")
        if matrix and n == 1:
            o2 = torch.empty((2, H * dv), dtype=dtype, device="cuda")
            K.pwa_decode_bf16(qo[:1].repeat(2, 1), o2, slots, ctx, c.table, c.unit, None, None, 2, H, G, dk, dv, 64, NO_WINDOW, 0, scale, False)
            o = o2[1:]                    # row b of a single-token step is sequence b: the first is padding
        elif matrix:
            K.pwa_prefill_bf16(qo, o, cu, slots, ctx, c.table, c.unit, None, None, 2, n, H, G, dk, dv, 64, NO_WINDOW, 0, scale, False)
        else:
            K.pwa_attend(qo, o, pos, sot, slots, c.table, c.unit, None, None, H, G, dk, dv, 64, NO_WINDOW, 0, scale, False)
        outs.append(o.float().cpu().numpy())
        qs.append(qo.float().cpu().numpy())
        at += n
    assert at == T
    return np.concatenate(outs).reshape(T, H, dv), np.concatenate(qs).reshape(T, H, dk), c


def plain_attention(rows, H, G, dk, dv, scale, keys_as_values, eps, temp, start=0):
    T = rows.shape[0]
    q = rows[:, :H * dk].reshape(T, H, dk)
    k = rows[:, H * dk:(H + G) * dk].reshape(T, G, dk)
    v = k.copy() if keys_as_values else rows[:, (H + G) * dk:(H + G) * dk + G * dv].reshape(T, G, dv)
    if eps is not None:
        q, k = P.rms_divide(q, eps), P.rms_divide(k, eps)
    if temp[1]:
        q = q * P.query_temperature(np.arange(start, start + T), temp[0], temp[1])[:, None, None]
    return P.causal_softmax_attention(q, k, v, scale), q, k, v


@pytest.mark.parametrize("H,G,dk,dv,kav", [(4, 2, 16, 16, True), (3, 1, 16, 24, False), (3, 3, 10, 10, True), (1, 1, 12, 6, False),
                                           (24, 8, 8, 8, True), (2, 2, 32, 16, False), (8, 2, 48, 48, True), (6, 3, 48, 64, False)])
def test_attention_without_window(H, G, dk, dv, kav):
    """Keys that serve as values before their norm, the norm without weights, the query temperature, all earlier tokens
    seen: whole, in portions across page borders, token by token; in float and through the matrix-core kernels."""
    rng = np.random.default_rng(H * 100 + dk)
    T, every = 300, 24
    width = (H + G) * dk + (0 if kav else G * dv) + 3
    # without the norm the scores grow with the inputs: small ones, or the softmax is so sharp that it amplifies bfloat16 rounding
    rows = f32(rng.standard_normal((T, width)) * (1.5 if kav else 0.6))
    eps = 1e-5 if kav else None
    want, q, k, v = plain_attention(rows, H, G, dk, dv, 0.4, kav, eps, (0.6, every))
    whole, q_got, c = attend(rows, H, G, dk, dv, 0.4, [T], keys_as_values=kav, eps=eps, temp=(0.6, every))
    assert np.abs(q_got - q).max() < 1e-5 * np.abs(q).max()
    ck, cv = c.rows(1, range(T))
    assert np.abs(ck - k).max() < 1e-5 * np.abs(k).max() and np.abs(cv - v).max() < 1e-6 * np.abs(v).max()
    assert np.abs(whole - want).max() < 3e-5 * max(1.0, np.abs(want).max())
    cut, _, _ = attend(rows, H, G, dk, dv, 0.4, [61, 2, 1, 1, 64, 65, 3] + [1] * 40 + [63], keys_as_values=kav, eps=eps, temp=(0.6, every))
    assert np.array_equal(cut, whole), "portions and single tokens must give the bits of the whole prompt"
    plain16, _, _ = attend(rows, H, G, dk, dv, 0.4, [T], dtype=torch.bfloat16, keys_as_values=kav, eps=eps, temp=(0.6, every))
    assert np.abs(plain16 - want).max() < 0.03 * np.abs(want).max()
    from braidinfer_amd import kernels as K
    if K.pwa_prefill_takes(torch.bfloat16, dk, dv, 64):
        for portions in ([T], [33, 31, 2, 63, 65, 100, 6], [T - 45] + [1] * 45):
            if not K.pwa_decode_takes(torch.bfloat16, H, G, dk, dv, 64) and 1 in portions:
                continue
            fast, _, _ = attend(rows, H, G, dk, dv, 0.4, portions, dtype=torch.bfloat16, matrix=True, keys_as_values=kav, eps=eps, temp=(0.6, every))
            assert np.abs(fast - plain16).max() < 0.03 * np.abs(plain16).max()


def test_the_temperature_steps_where_it_should():
    """Queries of one fixed direction against two keys: the weight of the better key grows with the temperature, so the
    positions at which the factor steps show in the output: just below and at every multiple of the period, in a
    prompt, in portions that end at the step, and token by token."""
    H = G = 1
    dk = dv = 8
    every, coef, T = 6, 2.0, 40
    rows = np.zeros((T, (H + 2 * G) * dk))
    rows[:, 0] = 1.0                                      # every query: e0
    rows[0, dk] = 1.0                                     # the first key answers it; all others are orthogonal
    rows[1:, dk + 1] = 1.0
    rows[0, 2 * dk] = 1.0                                 # the first value: e0; the others e1
    rows[1:, 2 * dk + 1] = 1.0
    want, q, _, _ = plain_attention(rows, H, G, dk, dv, 1.0, False, None, (coef, every))
    f = 1.0 + coef * np.log(((np.arange(T) + 1) // every) + 1.0)
    assert np.allclose(q[:, 0, 0], f) and f[every - 2] == 1.0 and f[every - 1] > 2.0 and f[2 * every - 2] < f[2 * every - 1]
    share = np.exp(f) / (np.exp(f) + np.arange(T))        # the first key's weight among p orthogonal ones
    assert np.allclose(want[1:, 0, 0], share[1:])
    for portions in ([T], [every - 1, 1, every - 1, 1, T - 2 * every], [every, every, T - 2 * every], [3] + [1] * (T - 3)):
        got, qg, _ = attend(rows, H, G, dk, dv, 1.0, portions, temp=(coef, every))
        assert np.abs(qg[:, 0, 0] - f).max() < 1e-6
        assert np.abs(got - want).max() < 1e-6
    # a sequence that goes on far behind its start: the position counts, not the place in the step
    got, qg, _ = attend(rows[:4], H, G, dk, dv, 1.0, [2, 1, 1], temp=(coef, every), start=2 * every - 3)
    assert np.abs(qg[:, 0, 0] - (1.0 + coef * np.log(np.array([2, 2, 3, 3.0])))).max() < 1e-6


def test_a_far_key_shows():
    """One key made to stand out among hundreds: the first token, at a page's border, far back and the newest; in a
    prompt and token by token, in float and through the matrix-core kernels; with the keys serving as values the
    answer is the loud key itself as projected, not its normed form."""
    from braidinfer_amd import kernels as K
    H, G, dk, T = 2, 1, 8, 460
    rng = np.random.default_rng(5)
    for kav in (True, False):
        dv = dk if kav else 4
        for loud in (0, 5, 63, 64, 127, 128, 399, T - 1):
            rows = rng.standard_normal((T, (H + G) * dk + (0 if kav else G * dv))) * 0.3
            rows[:, :H * dk] = 0.0
            rows[:, 0] = rows[:, dk] = 1.0                              # both heads ask for the first channel
            rows[:, H * dk] = rng.uniform(-1.0, 0.0, T)                 # which no key but the loud one has
            rows[loud, H * dk:(H + G) * dk] *= 0.05
            rows[loud, H * dk] = 5.0
            rows = f32(rows)
            eps = 1e-6 if kav else None
            scale = 8.0 if kav else 3.0
            want, _, _, v = plain_attention(rows, H, G, dk, dv, scale, kav, eps, (0.0, 0))
            assert np.abs(want[T - 1, 0] - v[loud, 0]).max() < 2e-3 * np.abs(v[loud, 0]).max()     # the last query sees the loud token alone
            got, _, _ = attend(rows, H, G, dk, dv, scale, [T - 30] + [1] * 30, keys_as_values=kav, eps=eps)
            assert np.abs(got - want).max() < 3e-5 * np.abs(want).max()
            matrix = K.pwa_prefill_takes(torch.bfloat16, dk, dv, 64) and K.pwa_decode_takes(torch.bfloat16, H, G, dk, dv, 64)
            fast, _, _ = attend(rows, H, G, dk, dv, scale, [T - 30] + [1] * 30, dtype=torch.bfloat16, matrix=matrix, keys_as_values=kav, eps=eps)
            assert np.abs(fast[T - 1, 0] - v[loud, 0]).max() < 0.03 * np.abs(v[loud, 0]).max()
            if loud:                             # the query before it sees nothing loud
                assert np.abs(want[loud - 1, 0]).max() < 0.5 * np.abs(v[loud, 0]).max()


def test_scores_over_all_experts_divided_by_the_chosen_ones_sum():
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(6)
    for T, E, top in ((9, 7, 3), (4, 70, 5), (3, 2, 2), (6, 8, 1), (5, 5, 5)):
        z = rng.standard_normal((T, E)).astype(np.float32) * 3
        z[:, 1] = z[:, 0]                                      # two experts that always tie: the lower number goes first
        chosen = torch.zeros((T, top), dtype=torch.int32, device="cuda")
        share = torch.zeros((T, top), dtype=torch.float32, device="cuda")
        K.route_topk(dev_f(z), None, chosen, share, top, 0.6)
        s = np.exp(f32(z) - f32(z).max(axis=1, keepdims=True))
        s = s / s.sum(axis=1, keepdims=True)
        order = np.argsort(-s, axis=1, kind="stable")[:, :top]
        assert np.array_equal(chosen.cpu().numpy(), order)
        picked = np.take_along_axis(s, order, axis=1)
        assert np.abs(share.cpu().numpy() - 0.6 * picked / (picked.sum(axis=1, keepdims=True) + 1e-20)).max() < 1e-6


# ------------------------------------------------------------ whole models -----------
@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_against_plain(folders, engines, name, dtype):
    _, cfg, w = folders[(name, dtype)]
    toks = tokens_of(cfg, 150, 1)
    want, m = plain(name, cfg, w, toks)
    close(run(engines(name, dtype), toks, [150]), want, dtype, f"{name} {dtype}", m)
    close(run(engines(name, dtype), toks[:1], [1]), want[:1], dtype, "a sequence of one token", m)
    close(run(engines(name, dtype), toks[:3], [1, 1, 1]), want[:3], dtype, "the first tokens one by one", m)
    close(run(engines(name, dtype), toks[:5], [2, 3]), want[:5], dtype, "the first tokens in two portions", m)


@pytest.mark.parametrize("name", ["a", "b"])
def test_residual_rows_after_every_layer_run(folders, engines, name):
    import braidinfer_amd as B
    _, cfg, w = folders[(name, "float32")]
    toks = tokens_of(cfg, 40, 9)
    _, layers = P.forward(cfg, w, toks, return_layers=True)
    eng = engines(name, "float32")
    seen = {}
    s = eng.alloc_slot()
    eng.step([B.StepEntry(s, toks, [])], probe=lambda n, t: seen.__setitem__(n, t.float().cpu().numpy().copy()))
    eng.free_slot(s)
    assert len(layers) == len(P.run_order(cfg)) > len(cfg["layers"])
    for i in range(len(layers)):
        assert np.abs(seen[f"L{i}.post_ffn"] - layers[i]).max() < 2e-4 * np.abs(layers[i]).max(), f"layer run {i}"


@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_and_single_tokens(folders, engines, name, dtype):
    """A prompt in portions down to two tokens, then token by token across a page's border and the temperature's
    steps, against the plain logits and, in float32, against the whole prompt's own."""
    _, cfg, w = folders[(name, dtype)]
    n = 215
    toks = tokens_of(cfg, n, 2)
    want, m = plain(name, cfg, w, toks)
    eng = engines(name, dtype)
    whole = run(eng, toks, [n])
    for portions in ([2, 3, 59, 1, 63, 2, 64, 21], [17] + [1] * 198, [128, 2] + [1] * 85):
        got = run(eng, toks, portions)
        close(got, want, dtype, f"{name} {dtype} {portions[:4]}", m)
        if dtype == "float32":
            assert np.abs(got - whole).max() < 2e-4 * np.abs(whole).max()


@pytest.mark.parametrize("name", ["a", "b", "c", "f"])
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
        want, m = plain(name, cfg, w, p)
        close(g, want[:len(g)], dtype, f"request {i} of the batch", m)


def test_slots_and_pages_used_again(folders):
    """Requests come and go through a cache of few pages and slots: what a freed slot's state, its convolution's last
    inputs or a returned page held never shows."""
    import braidinfer_amd as B
    folder, cfg, w = folders[("a", "float32")]
    eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=704, max_seq_len=512, n_slots=2)
    free_before = [g.pool.free_count for g in eng.cache.groups]
    for r in range(6):
        toks = tokens_of(cfg, 100 + 37 * r, 50 + r)
        want = P.forward(cfg, w, toks)
        close(run(eng, toks, [len(toks) - 10] + [1] * 10), want, "float32", f"request {r}")
    assert [g.pool.free_count for g in eng.cache.groups] == free_before
    # a cache unit for every attention run and none for the lightning runs: runs 0 and 9, and the left sides at 1, 3, 5, 7
    assert sorted(eng.cache.group_of_unit) == [0, 1, 3, 5, 7, 9]
    # two requests side by side whose slots have just been used, one of them a single token long
    import braidinfer_amd as B
    a, b = tokens_of(cfg, 70, 90), tokens_of(cfg, 1, 91)
    sa, sb = eng.alloc_slot(), eng.alloc_slot()
    lg = eng.step([B.StepEntry(sa, a, [69]), B.StepEntry(sb, b, [0])]).cpu().numpy()
    eng.free_slot(sa)
    eng.free_slot(sb)
    close(lg, np.stack([P.forward(cfg, w, a)[69], P.forward(cfg, w, b)[0]]), "float32", "after the slots' earlier users")


@pytest.mark.parametrize("name", ["a", "b", "f"])
def test_long_decoding(folders, engines, name):
    """Three hundred single-token steps from a short prompt (recorded steps of the engine), past page borders and many
    steps of the temperature."""
    for dtype in ("float32", "bfloat16"):
        _, cfg, w = folders[(name, dtype)]
        toks = tokens_of(cfg, 330, 3)
        want, m = plain(name, cfg, w, toks)
        close(run(engines(name, dtype), toks, [30] + [1] * 300), want, dtype, f"{name} {dtype}", m)


def test_a_long_prompt(folders, engines):
    for dtype in ("float32", "bfloat16"):
        _, cfg, w = folders[("a", dtype)]
        toks = tokens_of(cfg, 700, 8)
        want, m = plain("a", cfg, w, toks)
        close(run(engines("a", dtype), toks, [700]), want, dtype, f"whole {dtype}", m)
        close(run(engines("a", dtype), toks, [100, 600]), want, dtype, f"behind a portion {dtype}", m)


def drawn_configuration(seed):
    """A configuration drawn at random: any order of layers, any repeated run, head counts and widths from lists that
    hold odd ones and such that the matrix-core kernels take."""
    rng = np.random.default_rng(seed)
    pick = lambda xs: xs[int(rng.integers(len(xs)))]

    def heads():
        H = pick([1, 2, 3, 4, 6, 8, 12])
        return H, pick([g for g in (1, 2, 3, 4, 6, 8, 12) if H % g == 0])

    def experts():
        if rng.random() < 0.2:
            return None
        E = pick([2, 3, 4, 8, 16])
        return moe(pick([8, 16, 24, 40]), E, pick([t for t in (1, 2, 4, 8) if t <= E]))
    layers = []
    for _ in range(int(rng.integers(2, 6))):
        kind = pick(["attention", "parallel", "lightning"])
        if kind == "attention":
            H, G = heads()
            layers.append(att(H, G, pick([8, 12, 16, 24, 32, 48, 64]), coef=pick([0.0, 0.2, 0.5]), every=pick([1, 5, 16, 64, 1000]), mlp=experts()))
        elif kind == "parallel":
            H, G = heads()
            rh, rg = heads()
            layers.append(par((H, G, pick([8, 16, 32, 48]), pick([8, 12, 16, 32, 64]), pick([0.1, 0.4]), pick([2, 9, 32])),
                              (rh, rg, pick([4, 8, 16, 32, 40]), pick([4, 8, 24, 32, 72]), pick([1, 2, 3, 4])), mlp=experts()))
        else:
            H = pick([1, 2, 3, 4, 8])
            layers.append(lig(H, pick([4, 8, 16, 32, 40]), pick([4, 8, 16, 32, 72]), [float(x) for x in rng.uniform(0.5, 1.0, H)], mlp=experts()))
    n = len(layers)
    loop = None
    if rng.random() < 0.8:
        a = int(rng.integers(0, n))
        b = int(rng.integers(a + 1, n + 1))
        loop = (a, b, int(rng.integers(1, 4)))
    return model(pick([32, 48, 64, 80]), int(rng.integers(40, 300)), layers, loop, eps=pick([1e-6, 1e-5, 1e-3]), emb=pick([1.0, 2.5, 0.5]),
                 mult=pick([1.0, 0.5, 0.3]), positions=128)


@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_at_random(seed, tmp_path):
    """Whole, in portions and token by token in float32 against the plain implementation; bfloat16 whole and decoded."""
    import braidinfer_amd as B
    cfg = drawn_configuration(1000 + seed)
    w = P.random_weights(cfg, seed=seed, gain=0.9)
    folder = str(tmp_path / "m")
    P.write_folder(folder, cfg, w)
    toks = tokens_of(cfg, 100, seed)
    want, m = plain(f"drawn{seed}", cfg, w, toks)
    eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=512)
    what = f"seed {seed}: {[l['type'] for l in cfg['layers']]} loop {cfg.get('loop')}"
    close(run(eng, toks, [100]), want, "float32", what)
    close(run(eng, toks, [3, 62, 2, 1, 1] + [1] * 31), want, "float32", what + " in portions")
    other = tokens_of(cfg, 45, seed + 50)
    sa, sb = eng.alloc_slot(), eng.alloc_slot()
    lg = eng.step([B.StepEntry(sa, toks[:70], [69]), B.StepEntry(sb, other[:44], [0, 43])]).cpu().numpy()
    lg2 = eng.step([B.StepEntry(sa, toks[70:71], [0]), B.StepEntry(sb, other[44:], [0])]).cpu().numpy()
    eng.free_slot(sa)
    eng.free_slot(sb)
    ow = P.forward(cfg, w, other)
    close(np.concatenate([lg, lg2]), np.stack([want[69], ow[0], ow[43], want[70], ow[44]]), "float32", what + " two requests")
    del eng
    # bfloat16 with all experts chosen: a drawn model may choose one expert in front of a recurrence, where a router's
    # close call that falls the other way moves the rows behind it too (the float32 runs above hold the choice)
    calm = copy.deepcopy(cfg)
    for l in calm["layers"]:
        if l["mlp"] is not None:
            l["mlp"]["router"]["top"] = l["mlp"]["router"]["experts"]
    P.write_folder(folder, calm, w)
    eng = B.Engine.from_folder(folder, dtype="bfloat16", max_tokens=512)
    close(run(eng, toks, [60] + [1] * 40), P.forward(calm, w, toks), "bfloat16", what + " bfloat16")


def test_beyond_the_learnt_positions_is_refused(folders, tmp_path):
    import braidinfer_amd as B
    from braidinfer_amd.errors import BraidError
    _, cfg, w = folders[("e", "float32")]
    short = dict(copy.deepcopy(cfg), max_positions=48)
    w2 = dict(w, pos=w["pos"][:48])
    P.write_folder(str(tmp_path / "m"), short, w2)
    eng = B.Engine.from_folder(str(tmp_path / "m"), dtype="float32", max_tokens=256)
    toks = tokens_of(short, 48, 1)
    close(run(eng, toks, [40] + [1] * 8), P.forward(short, w2, toks), "float32", "up to the last learnt position")
    s = eng.alloc_slot()
    with pytest.raises(BraidError):
        eng.step([B.StepEntry(s, tokens_of(short, 49, 2), [48])])
    eng.free_slot(s)


def test_greedy_generation_through_the_engine(folders, engines):
    _, cfg, w = folders[("a", "float32")]
    prompts = [tokens_of(cfg, n, 20 + n) for n in (3, 41, 12, 70)]
    want = [P.greedy_generate(cfg, w, p, 12) for p in prompts]
    got = engines("a", "float32").generate(prompts, max_new_tokens=12, temperature=0.0, stop_token_ids=[])
    assert got == want
    got16 = engines("a", "bfloat16").generate(prompts, max_new_tokens=12, temperature=0.0, stop_token_ids=[])
    for g, wnt, p in zip(got16, want, prompts):
        for i, (a, b) in enumerate(zip(g, wnt)):
            if a != b:                              # bfloat16 may take the runner-up where two logits are nearly tied
                l = P.forward(cfg, w, p + wnt[:i])[-1]
                assert abs(l[a] - l[b]) < 0.05 * np.abs(l).max()
                break


def test_the_command_line_generates_from_a_zivovik_folder(folders):
    """`bin/generate` on a Zivovik folder: the model class by config.json, greedy tokens as the plain implementation's;
    a sampled run ends and stays inside the vocabulary."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, cfg, w = folders[("a", "float32")]
    p = [7, 3, 200, 5, 11]
    want = P.greedy_generate(cfg, w, p, 6)
    env = dict(os.environ, MODEL=folder, MAX_TOKENS="6")
    gen = [sys.executable, os.path.join(root, "bin", "generate"), "--dtype", "float32", "--prompt-ids", ",".join(map(str, p))]
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
    cfg = B.any_preset("zivovik-tiny")
    folder = B.Engine.write_random_folder(str(tmp_path / "m"), cfg, seed=3, std=0.2, vector_jitter=0.3)
    pc, pw = P.read_folder(folder)
    toks = tokens_of(pc, 60, 4)
    eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=512)
    close(run(eng, toks, [40] + [1] * 20), P.forward(pc, pw, toks), "float32", "preset")


def test_replay_of_given_tokens_through_the_command(folders, tmp_path):
    """`bin/trace_run` as a child process on a Zivovik folder: requests whole, with their last tokens one by one, and two
    of unequal length in one batch, against the plain logits."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, cfg, w = folders[("b", "float32")]
    V = cfg["vocab"]
    seqs = [tokens_of(cfg, n, 60 + n) for n in (90, 41)]
    refs = [P.forward(cfg, w, s) for s in seqs]
    out = str(tmp_path / "out")
    p = subprocess.Popen([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", out,
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
