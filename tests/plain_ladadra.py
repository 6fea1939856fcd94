"""A plain, slow implementation of the Ladadra design in NumPy float64, one function per
mechanism, written from the design's equations.  It shares no code with the library: the
tests hold the engine against it.

Notation: a sequence's tokens are rows; positions count from 0.  `cfg` is the model's
configuration as a dict (the keys of its config.json), `w` maps tensor names to float arrays.
A layer is x += norm1(mixer(x)), x += norm2(feed_forward(x)): the halves read the residual
rows themselves and the norm stands behind each half.
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


def rms_norm(x, weight, eps):
    return rms_divide(x, eps) * weight


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def rotary_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims) for i < dims/2; with `scaling` {factor, low, high, original} a frequency whose
    wavelength is shorter than original/high stays, one longer than original/low is divided by the factor, and
    between the two the mix (1 - s) f/factor + s f with s = (original/wavelength - low) / (high - low)."""
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=np.float64)
    if not scaling:
        return f
    factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = f.copy()
    for i, fi in enumerate(f):
        wavelength = 2.0 * math.pi / fi
        if wavelength < original / high:
            out[i] = fi
        elif wavelength > original / low:
            out[i] = fi / factor
        else:
            s = (original / wavelength - low) / (high - low)
            out[i] = (1.0 - s) * fi / factor + s * fi
    return out


def rotate_half(x, positions, freqs):
    """x [T, heads, d]: element i of the first 2 len(freqs) is paired with element i + len(freqs) and the pair
    turned by position * f_i; the other elements pass."""
    n = len(freqs)
    a = np.asarray(positions, dtype=np.float64)[:, None, None] * freqs[None, None, :]
    c, s = np.cos(a), np.sin(a)
    y = x.copy()
    u, v = x[..., :n], x[..., n:2 * n]
    y[..., :n] = u * c - v * s
    y[..., n:2 * n] = v * c + u * s
    return y


def masked_attention(q, k, v, scale, visible, softcap=None, sinks=None):
    """q [T, H, d], k [T, G, d], v [T, G, e] of one sequence from position 0 -> [T, H, e].  Query head h reads
    key/value head h // (H / G).  visible [T, T] (row: query, column: key).  Scores (q . k) scale, then
    softcap tanh(score / softcap) if given.  With `sinks` [H] the denominator has one more term exp(sink_h)
    that brings no value."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap:
            s = softcap * np.tanh(s / softcap)
        s = np.where(visible, s, -np.inf)
        m = s.max(axis=1, keepdims=True)
        if sinks is not None:
            m = np.maximum(m, sinks[h])
        p = np.exp(s - m)
        den = p.sum(axis=1, keepdims=True)
        if sinks is not None:
            den = den + np.exp(sinks[h] - m)
        out[:, h] = (p / den) @ v[:, g]
    return out


def causal(T):
    return np.tril(np.ones((T, T), dtype=bool))


def chunk_mask(T, size):
    """Key j is seen by query i when j <= i and both lie in the same run of `size` positions counted from 0."""
    i = np.arange(T)
    return causal(T) & ((i[:, None] // size) == (i[None, :] // size))


def window_mask(T, size, keep_first=0):
    """Key j is seen by query i when j <= i and (i - j < size or j < keep_first)."""
    i = np.arange(T)
    return causal(T) & (((i[:, None] - i[None, :]) < size) | (i[None, :] < keep_first))


def decayed_outer_sum(q, k, v, decay, return_state=False):
    """One head with a fixed decay: S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t."""
    T, d = q.shape
    S = np.zeros((d, v.shape[1]))
    o = np.zeros((T, v.shape[1]))
    for t in range(T):
        S = decay * S + np.outer(k[t], v[t])
        o[t] = S.T @ q[t]
    return (o, S) if return_state else o


def gated_unit(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def choose_experts(z, correction, top, groups=None):
    """z [T, E] router logits.  Scores s = sigmoid(z); the choice is made on s + correction, the weights on s.
    With `groups` {count, keep} the experts form `count` runs of neighbours, a run's score is the sum of its two
    largest choice scores, and only experts of the `keep` best runs can be chosen.  -> (chosen [T, top], weights)."""
    T, E = z.shape
    s = sigmoid(z)
    c = s + correction[None, :]
    if groups and groups.get("count", 1) > 1:
        n, keep = int(groups["count"]), int(groups["keep"])
        per = E // n
        gs = np.sort(c.reshape(T, n, per), axis=2)[:, :, -2:].sum(axis=2) if per >= 2 else c.reshape(T, n, per).sum(axis=2)
        best = np.argsort(-gs, axis=1, kind="stable")[:, :keep]
        allowed = np.zeros((T, n), dtype=bool)
        np.put_along_axis(allowed, best, True, axis=1)
        c = np.where(np.repeat(allowed, per, axis=1), c, -np.inf)
    chosen = np.argsort(-c, axis=1, kind="stable")[:, :top]
    picked = np.take_along_axis(s, chosen, axis=1)
    return chosen, picked / (picked.sum(axis=1, keepdims=True) + 1e-20)


# ------------------------------------------------------------------ mixers ----------
def attention_mixer(h, w, p, m, eps, positions):
    """Grouped heads with biased projections, one norm over the whole query (key) projection, partial rotation with
    stretched frequencies, capped scores inside runs of positions, a sink in the softmax, a sigmoid gate a head."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q = h @ w[p + "q"].T + w[p + "q.b"]
    k = h @ w[p + "k"].T + w[p + "k.b"]
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, e)
    q = rms_norm(q, w[p + "q.norm"], eps).reshape(T, H, d)
    k = rms_norm(k, w[p + "k.norm"], eps).reshape(T, G, d)
    rot = m.get("rot")
    if rot:
        f = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate_half(q, positions, f), rotate_half(k, positions, f)
    size = (m.get("mask") or {}).get("size")
    visible = chunk_mask(T, size) if size else causal(T)
    o = masked_attention(q, k, v, m["scale"], visible, m.get("softcap"), w[p + "sink"])
    o = o * sigmoid(h @ w[p + "g"].T)[:, :, None]
    return o.reshape(T, H * e) @ w[p + "o"].T


def retention_mixer(h, w, p, m, eps, positions, state=None):
    """A decayed sum of key-value products per head, read by the rotated query, normed per head, gated."""
    T = h.shape[0]
    H, d, e = m["heads"], m["dim"], m.get("vdim", m["dim"])
    q = (h @ w[p + "q"].T).reshape(T, H, d)
    k = (h @ w[p + "k"].T).reshape(T, H, d)
    v = (h @ w[p + "v"].T).reshape(T, H, e)
    rot = m.get("rot")
    if rot:
        f = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate_half(q, positions, f), rotate_half(k, positions, f)
    k = k * d ** -0.5
    o = np.stack([decayed_outer_sum(q[:, i], k[:, i], v[:, i], m["decay"][i]) for i in range(H)], axis=1)
    o = rms_divide(o, eps).reshape(T, H * e)
    return (o * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def differential_mixer(h, w, p, m, eps, positions):
    """Two softmax maps a head over the same values inside a window that also keeps the first tokens; the second
    map is taken off the first with a learnt factor."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q = rms_norm((h @ w[p + "q"].T).reshape(T, H, 2, d), w[p + "q.norm"], eps)
    k = rms_norm((h @ w[p + "k"].T).reshape(T, G, 2, d), w[p + "k.norm"], eps)
    v = (h @ w[p + "v"].T).reshape(T, G, e)
    mask = m.get("mask") or {}
    visible = window_mask(T, mask["size"], mask.get("keep_first", 0)) if mask.get("size") else causal(T)
    a1 = masked_attention(q[:, :, 0], k[:, :, 0], v, m["scale"], visible)
    a2 = masked_attention(q[:, :, 1], k[:, :, 1], v, m["scale"], visible)
    diff = m["diff"]
    lam = math.exp(float(np.sum(w[p + "lq1"] * w[p + "lk1"]))) - math.exp(float(np.sum(w[p + "lq2"] * w[p + "lk2"]))) + diff
    o = rms_divide(a1 - lam * a2, eps) * (1.0 - diff)
    return o.reshape(T, H * e) @ w[p + "o"].T


MIXERS = {"attention": attention_mixer, "retention": retention_mixer, "attention_2": differential_mixer}


# ------------------------------------------------------------------ feed-forward ----
def feed_forward(h, w, p, f):
    if f["kind"] == "dense":
        return gated_unit(h, w[p + "gate"], w[p + "up"], w[p + "down"])
    r = f["router"]
    chosen, weights = choose_experts(h @ w[p + "router"].T, w[p + "correction"], r["top"], r.get("groups"))
    out = np.zeros((h.shape[0], w[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, share in zip(chosen[t], weights[t]):
            q = p + "e%d." % e
            out[t] += share * gated_unit(h[t:t + 1], w[q + "gate"], w[q + "up"], w[q + "down"])[0]
    if f.get("shared"):
        out += gated_unit(h, w[p + "shared.gate"], w[p + "shared.up"], w[p + "shared.down"])
    return out


# ------------------------------------------------------------------ the model -------
def forward(cfg, w, tokens, return_layers=False):
    """Logits [T, vocab] of one sequence from position 0 (and the residual rows after every layer)."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][np.asarray(tokens)]
    positions = np.arange(len(tokens))
    rows = []
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        x = x + rms_norm(MIXERS[layer["type"]](x, w, p + "mix.", layer["mixer"], eps, positions), w[p + "norm1"], eps)
        if layer.get("mlp"):
            x = x + rms_norm(feed_forward(x, w, p + "mlp.", layer["mlp"]), w[p + "norm2"], eps)
        rows.append(x)
    logits = rms_norm(x, w["final.norm"], eps) @ w["embed"].T
    return (logits, np.stack(rows)) if return_layers else logits


def greedy(cfg, w, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(np.argmax(forward(cfg, w, tokens)[-1])))
    return tokens[len(prompt):]


# ------------------------------------------------------------------ weights ---------
def tensor_shapes(cfg):
    """name -> shape of every tensor of a model of this configuration, in the order of its layers."""
    W, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, W)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = "l%d." % i, layer["mixer"]
        out[p + "norm1"] = (W,)
        if layer.get("mlp"):
            out[p + "norm2"] = (W,)
        p += "mix."
        if layer["type"] == "attention":
            H, G, d, e = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
            for n, rows in (("q", H * d), ("k", G * d), ("v", G * e)):
                out[p + n] = (rows, W)
                out[p + n + ".b"] = (rows,)
            out[p + "q.norm"], out[p + "k.norm"] = (H * d,), (G * d,)
            out[p + "sink"], out[p + "g"], out[p + "o"] = (H,), (H, W), (W, H * e)
        elif layer["type"] == "retention":
            H, d, e = m["heads"], m["dim"], m.get("vdim", m["dim"])
            out[p + "q"], out[p + "k"], out[p + "v"] = (H * d, W), (H * d, W), (H * e, W)
            out[p + "g"], out[p + "o"] = (H * e, W), (W, H * e)
        else:
            H, G, d, e = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
            out[p + "q"], out[p + "k"], out[p + "v"] = (H * 2 * d, W), (G * 2 * d, W), (G * e, W)
            for n in ("q.norm", "k.norm", "lq1", "lk1", "lq2", "lk2"):
                out[p + n] = (d,)
            out[p + "o"] = (W, H * e)
        f = layer.get("mlp")
        p = "l%d.mlp." % i
        if not f:
            continue
        if f["kind"] == "dense":
            out[p + "gate"], out[p + "up"], out[p + "down"] = (f["ff"], W), (f["ff"], W), (W, f["ff"])
            continue
        for e in range(f["router"]["experts"]):
            q, n = p + "e%d." % e, f["expert"]["ff"]
            out[q + "gate"], out[q + "up"], out[q + "down"] = (n, W), (n, W), (W, n)
        out[p + "router"], out[p + "correction"] = (f["router"]["experts"], W), (f["router"]["experts"],)
        if f.get("shared"):
            n = f["shared"]["ff"]
            out[p + "shared.gate"], out[p + "shared.up"], out[p + "shared.down"] = (n, W), (n, W), (W, n)
    out["final.norm"] = (W,)
    return out


def to_bf16_values(a):
    """Round float64 values to the nearest bfloat16 (ties to even), returned as float64."""
    u = np.asarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).astype(np.float64)


def random_weights(cfg, seed, router_spread=0.0, gain=1.0):
    """Weights that keep every activation of order one, already rounded to bfloat16.  `router_spread` puts the
    experts' correction that far apart, so that a bfloat16 run chooses as the float64 run does; `gain` sizes the
    matrices."""
    rng = np.random.default_rng(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        tail = name.split(".")[-1]
        if name.endswith("norm1") or name.endswith("norm2") or name == "final.norm" or name.endswith(".norm"):
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif tail == "b":
            a = 0.3 * rng.standard_normal(shape)
        elif tail == "sink":
            a = rng.standard_normal(shape)
        elif tail in ("lq1", "lk1", "lq2", "lk2"):
            a = 0.3 * rng.standard_normal(shape)
        elif tail == "correction":
            # apart by growing steps, so that no two experts and no two sums of a group's best two come close
            a = 0.2 * rng.standard_normal(shape) + router_spread * 1.6 ** rng.permutation(shape[0]) * (router_spread > 0)
        elif name == "embed":
            a = rng.standard_normal(shape)
        else:
            a = rng.standard_normal(shape) * (1.5 * gain / math.sqrt(shape[-1]))
        w[name] = to_bf16_values(a)
    return w


def write_safetensors(path, w, dtype="bfloat16"):
    """Write `w` as one safetensors file of bfloat16 (or float32) tensors."""
    header, blobs, at = {}, [], 0
    for name, a in w.items():
        a32 = np.ascontiguousarray(a, dtype=np.float32)
        if dtype == "bfloat16":
            blob = (a32.view(np.uint32) >> 16).astype(np.uint16).tobytes()
            tag = "BF16"
        else:
            blob, tag = a32.tobytes(), "F32"
        header[name] = {"dtype": tag, "shape": list(a32.shape), "data_offsets": [at, at + len(blob)]}
        blobs.append(blob)
        at += len(blob)
    text = json.dumps(header, separators=(",", ":")).encode()
    text += b" " * (-len(text) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for b in blobs:
            f.write(b)


def read_model(folder):
    """(configuration, weights as float64) of a folder with config.json and one model.safetensors."""
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    with open(os.path.join(folder, "model.safetensors"), "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        data = f.read()
    w = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        blob = data[info["data_offsets"][0]:info["data_offsets"][1]]
        if info["dtype"] == "BF16":
            a = (np.frombuffer(blob, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
        elif info["dtype"] == "F32":
            a = np.frombuffer(blob, dtype=np.float32)
        else:
            raise ValueError(f"{name}: dtype {info['dtype']}")
        w[name] = a.reshape(info["shape"]).astype(np.float64)
    return cfg, w


def write_model(folder, cfg, w, dtype="bfloat16"):
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), w, dtype)
