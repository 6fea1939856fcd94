"""A plain, slow implementation of the Zivovik design in NumPy float64, one function per
mechanism, written from the design's equations.  It shares no code with the library: the
tests hold the engine against it.

Notation: a sequence's tokens are rows; positions count from 0.  `cfg` is the model's
configuration as a dict (the keys of its config.json), `w` maps tensor names to float arrays.
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np


# ------------------------------------------------------------------ mechanisms ------
def rms_divide(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def offset_norm(x, weight, eps):
    """The layer norm: a weight kept around zero, applied as 1 + weight."""
    return rms_divide(x, eps) * (1.0 + weight)


def plain_norm(x, weight, eps):
    return rms_divide(x, eps) * weight


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def query_temperature(positions, coef, every):
    """The factor on a query at position p: 1 + coef ln(floor((p + 1) / every) + 1)."""
    p = np.asarray(positions, dtype=np.int64)
    return 1.0 + coef * np.log(((p + 1) // every) + 1.0)


def causal_softmax_attention(q, k, v, scale):
    """q [T, H, d], k [T, G, d], v [T, G, e] of one sequence from position 0 -> [T, H, e]; query head h reads
    key/value head h // (H / G); every position sees itself and all before it; an ordinary softmax."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = np.where(np.tril(np.ones((T, T), dtype=bool)), s, -np.inf)
        p = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, h] = (p / p.sum(axis=1, keepdims=True)) @ v[:, g]
    return out


def short_convolution(x, taps):
    """x [T, C], taps [C, n]: y_t[c] = sum_j taps[c, j] x_(t - n + 1 + j)[c], zeros before the start (the last
    column weighs the current token)."""
    T, C = x.shape
    n = taps.shape[1]
    padded = np.concatenate([np.zeros((n - 1, C)), x])
    y = np.zeros((T, C))
    for j in range(n):
        y += padded[j:j + T] * taps[:, j][None, :]
    return y


def unit_vectors(x):
    return x / np.sqrt((x * x).sum(axis=-1, keepdims=True) + 1e-6)


def delta_rule(q, k, v, beta, g, return_state=False):
    """One head: q, k [T, d], v [T, e], beta, g [T].  S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, d = q.shape
    S = np.zeros((d, v.shape[1]))
    o = np.zeros((T, v.shape[1]))
    for t in range(T):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + np.outer(k[t], u)
        o[t] = S.T @ q[t]
    return (o, S) if return_state else o


def decayed_outer_sum(q, k, v, decay, return_state=False):
    """One head with a fixed decay: S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t."""
    T, d = q.shape
    S = np.zeros((d, v.shape[1]))
    o = np.zeros((T, v.shape[1]))
    for t in range(T):
        S = decay * S + np.outer(k[t], v[t])
        o[t] = S.T @ q[t]
    return (o, S) if return_state else o


# ------------------------------------------------------------------ mixers ----------
def attention_mixer(h, w, p, m, eps, positions):
    """Keys double as values (taken before the norm); queries and keys divided by their root mean square per head;
    an elementwise output gate."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w[p + "q"].T).reshape(T, H, d)
    k = (h @ w[p + "k"].T).reshape(T, G, d)
    v = k.copy()
    q, k = rms_divide(q, eps), rms_divide(k, eps)
    q = q * query_temperature(positions, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None, None]
    o = causal_softmax_attention(q, k, v, m["scale"]).reshape(T, H * d)
    return (o * sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def left_mixer(h, w, p, m, positions):
    """Attention with values of their own, no norms, one gate number per head."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(T, H, d)
    k = (h @ w[p + "k"].T).reshape(T, G, d)
    v = (h @ w[p + "v"].T).reshape(T, G, e)
    q = q * query_temperature(positions, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None, None]
    o = causal_softmax_attention(q, k, v, m["scale"]) * sigmoid(h @ w[p + "g"].T)[:, :, None]
    return o.reshape(T, H * e) @ w[p + "o"].T


def right_mixer(h, w, p, m, eps):
    """The gated delta rule behind short convolutions."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_convolution(h @ w[p + "q"].T, w[p + "q.conv"])).reshape(T, G, d)
    k = silu(short_convolution(h @ w[p + "k"].T, w[p + "k.conv"])).reshape(T, G, d)
    v = silu(short_convolution(h @ w[p + "v"].T, w[p + "v.conv"])).reshape(T, H, e)
    q, k = unit_vectors(q) * d ** -0.5, unit_vectors(k)
    beta = sigmoid(h @ w[p + "b"].T)
    g = np.exp(-np.exp(w[p + "A_log"])[None, :] * softplus(h @ w[p + "a"].T + w[p + "dt_bias"][None, :]))
    o = np.zeros((T, H, e))
    for hd in range(H):
        kv = hd // (H // G)
        o[:, hd] = delta_rule(q[:, kv], k[:, kv], v[:, hd], beta[:, hd], g[:, hd])
    o = rms_divide(o, eps) * w[p + "norm"][None, None, :]
    o = o.reshape(T, H * e) * silu(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def parallel_mixer(h, w, p, m, eps, positions):
    a = left_mixer(h, w, p + "left.", m["left"], positions)
    b = right_mixer(h, w, p + "right.", m["right"], eps)
    return 0.5 * (plain_norm(a, w[p + "left.out"], eps) + plain_norm(b, w[p + "right.out"], eps))


def lightning_mixer(h, w, p, m, eps):
    T = h.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[p + "q"].T).reshape(T, H, d)
    k = silu(h @ w[p + "k"].T).reshape(T, H, d)
    v = silu(h @ w[p + "v"].T).reshape(T, H, e)
    o = np.stack([decayed_outer_sum(q[:, i], k[:, i], v[:, i], float(m["decay"][i])) for i in range(H)], axis=1)
    o = plain_norm(o.reshape(T, H * e), w[p + "norm"], eps) * sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def routed_ff(h, w, p, mlp, margins=None):
    """Scores are the softmax of the router's logits over all experts; the `top` largest are chosen and weighted by their
    scores over the chosen scores' sum.  `margins` (a list) receives, per token, the gap between the last chosen and the
    first left-out router logit."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ w[p + "router"].T
    s = np.exp(z - z.max(axis=1, keepdims=True))
    s = s / s.sum(axis=1, keepdims=True)
    order = np.argsort(-s, axis=1, kind="stable")
    if margins is not None and top < E:
        srt = np.take_along_axis(z, order, axis=1)
        margins.append(srt[:, top - 1] - srt[:, top])
    out = np.zeros((h.shape[0], w[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        chosen = order[t, :top]
        share = s[t, chosen] / (s[t, chosen].sum() + 1e-20)
        for e, a in zip(chosen, share):
            q = f"{p}e{e}."
            out[t] += a * ((silu(h[t] @ w[q + "gate"].T) * (h[t] @ w[q + "up"].T)) @ w[q + "down"].T)
    return out


# ------------------------------------------------------------------ the model -------
def run_order(cfg):
    """[(layer, first of a repeated pass)] : the layers start .. stop - 1 run `times` times in a row."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    out = [(i, False) for i in range(a)]
    for r in range(times):
        out += [(i, r > 0 and i == a) for i in range(a, b)]
    return out + [(i, False) for i in range(b, n)]


def forward(cfg, w, tokens, return_layers=False, margins=None):
    """Logits [T, vocab] of one sequence from position 0 (and the residual rows after every layer run)."""
    eps, mult = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    T = len(tokens)
    positions = np.arange(T)
    x = w["embed"][np.asarray(tokens)] * float(cfg["embedding"]["scale"]) + w["pos"][positions]
    x0 = x.copy()
    layers = []
    for i, again in run_order(cfg):
        l = cfg["layers"][i]
        p, m = f"l{i}.", l["mixer"]
        if again:
            x = x + x0
        h = offset_norm(x, w[p + "norm1"], eps)
        if l["type"] == "attention":
            y = attention_mixer(h, w, p + "mix.", m, eps, positions)
        elif l["type"] == "parallel":
            y = parallel_mixer(h, w, p + "mix.", m, eps, positions)
        elif l["type"] == "lightning":
            y = lightning_mixer(h, w, p + "mix.", m, eps)
        else:
            raise ValueError(l["type"])
        x = x + mult * y
        if l.get("mlp") is not None:
            x = x + mult * routed_ff(offset_norm(x, w[p + "norm2"], eps), w, p + "mlp.", l["mlp"], margins)
        layers.append(x.copy())
    logits = offset_norm(x, w["final.norm"], eps) @ w["head"].T
    return (logits, np.stack(layers)) if return_layers else logits


def greedy_generate(cfg, w, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(np.argmax(forward(cfg, w, toks)[-1])))
    return toks[len(prompt):]


# ------------------------------------------------------------------ files -----------
def read_folder(folder):
    """(config dict, float64 tensors by name) of a model folder; bfloat16 and float32 tensors."""
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    with open(os.path.join(folder, "model.safetensors"), "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        head = json.loads(f.read(n))
        data = f.read()
    for name, t in head.items():
        if name == "__metadata__":
            continue
        a, b = t["data_offsets"]
        raw = data[a:b]
        if t["dtype"] == "BF16":
            arr = (np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        elif t["dtype"] == "F32":
            arr = np.frombuffer(raw, dtype="<f4").astype(np.float64)
        elif t["dtype"] == "I32":
            arr = np.frombuffer(raw, dtype="<i4")
        else:
            raise ValueError(f"{name}: dtype {t['dtype']}")
        w[name] = arr.reshape(t["shape"])
    return cfg, w


def to_bf16(a):
    """Round float values to the nearest bfloat16 (ties to even), returned as float64."""
    u = np.ascontiguousarray(np.asarray(a, dtype=np.float32)).view(np.uint32)
    r = ((u + (((u >> 16) & 1) + 0x7FFF)) >> 16).astype(np.uint32) << 16
    return r.view(np.float32).astype(np.float64)


def write_folder(folder, cfg, w):
    """config.json and model.safetensors (bfloat16) of a configuration dict and float tensors."""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    head, blobs, off = {}, [], 0
    for name, a in w.items():
        a32 = np.asarray(a, dtype=np.float32)
        u = np.ascontiguousarray(a32).reshape(-1).view(np.uint32)
        raw = ((u + (((u >> 16) & 1) + 0x7FFF)) >> 16).astype("<u2").tobytes()
        head[name] = {"dtype": "BF16", "shape": list(a32.shape), "data_offsets": [off, off + len(raw)]}
        off += len(raw)
        blobs.append(raw)
    hj = json.dumps(head).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)) + hj + b"".join(blobs))


def random_weights(cfg, seed, gain=1.0, router_gain=1.0):
    """Random tensors (bfloat16 values) for a configuration dict: matrices N(0, gain^2 / fan-in), layer-norm weights
    around 0, plain norm weights around 1."""
    rng = np.random.default_rng(seed)
    W, w = cfg["width"], {}

    def mat(o, i, g=gain):
        return to_bf16(rng.standard_normal((o, i)) * g / math.sqrt(i))

    def vec(n, around=1.0, spread=0.2):
        return to_bf16(around + spread * rng.standard_normal(n))

    def attention(q, m, own_values, gate_rows):
        H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        g = gain if own_values else 2.0 * gain          # queries and keys that pass no norm set the softmax's sharpness themselves
        w[q + "q"], w[q + "k"] = mat(H * d, W, g), mat(G * d, W, g)
        if own_values:
            w[q + "v"] = mat(G * e, W)
        w[q + "g"], w[q + "o"] = mat(gate_rows, W), mat(W, H * e)

    w["embed"] = to_bf16(rng.standard_normal((cfg["vocab"], W)))
    w["pos"] = to_bf16(rng.standard_normal((cfg["max_positions"], W)) * 0.5)
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        w[p + "norm1"] = vec(W, 0.0)
        q = p + "mix."
        if l["type"] == "attention":
            attention(q, m, False, m["heads"] * m["dim"])
        elif l["type"] == "parallel":
            attention(q + "left.", m["left"], True, m["left"]["heads"])
            r, q = m["right"], q + "right."
            H, G, d, e, n = r["heads"], r["kv_heads"], r["dim"], r["vdim"], r["conv"]
            for s, rows in (("q", G * d), ("k", G * d), ("v", H * e)):
                w[q + s] = mat(rows, W, 2.0 * gain)
                w[q + s + ".conv"] = to_bf16(rng.standard_normal((rows, n)) * 0.6)
            w[q + "b"], w[q + "a"] = mat(H, W, 2.0), mat(H, W, 2.0)
            w[q + "A_log"] = to_bf16(rng.uniform(-3.0, 0.5, H))
            w[q + "dt_bias"] = to_bf16(rng.uniform(-2.0, 1.0, H))
            w[q + "norm"], w[q + "g"], w[q + "o"] = vec(e), mat(H * e, W), mat(W, H * e)
            w[p + "mix.left.out"], w[p + "mix.right.out"] = vec(W), vec(W)
        else:
            H, d, e = m["heads"], m["dim"], m["vdim"]
            w[q + "q"], w[q + "k"], w[q + "v"] = mat(H * d, W), mat(H * d, W), mat(H * e, W)
            w[q + "g"], w[q + "norm"], w[q + "o"] = mat(H * e, W), vec(H * e), mat(W, H * e)
        mlp = l.get("mlp")
        if mlp is not None:
            w[p + "norm2"] = vec(W, 0.0)
            q, F = p + "mlp.", mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                w[f"{q}e{e}.gate"], w[f"{q}e{e}.up"], w[f"{q}e{e}.down"] = mat(F, W), mat(F, W), mat(W, F)
            w[q + "router"] = mat(mlp["router"]["experts"], W, router_gain)
    w["final.norm"] = vec(W, 0.0)
    w["head"] = mat(cfg["vocab"], W)
    return w
