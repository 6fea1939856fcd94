"""Typed configuration of the `Zivovik` design and its translation into parts.

A Zivovik model is a stack of pre-norm layers, x += m mixer(norm(x)) and then x += m feed_forward(norm(x)) with a
residual multiplier m and RMS norms whose weights are stored around zero (w = 1 + stored).  A learnt vector per
position joins the scaled token embedding.  A run of layers may be passed several times with the same weights
(`loop`); every pass keeps a cache and state of its own, and before every pass but the first the embedding output is
added to the residual rows.  Mixers:

* `"attention"`: causal grouped-query attention without rotation; the values are the keys as projected; queries and
  keys are divided by their root mean square per head (no weights); the query carries a temperature that grows with
  the logarithm of the position; a sigmoid gate per output element.
* `"parallel"`: two mixers side by side on the same input, `left` an attention with values of their own, no
  query/key norm and one sigmoid gate per head, `right` a gated delta rule behind short convolutions; each output is
  RMS-normed over the model width with a plain weight, and the result is half their sum.
* `"lightning"`: linear attention with a fixed decay per head.

The feed-forward is a set of routed experts (softmax over all experts, the `top` largest chosen and weighted by their
scores over the chosen ones' sum) or absent.  The output head has a matrix of its own.  The reference has no such
model; its configuration is one flat struct (crates/braidinfer-runtime/src/config.rs:75-115), this one keeps the
nesting of the design's config.json:

    {"architecture": "Zivovik", "vocab": V, "width": W, "max_positions": P, "norm": {"eps": e},
     "embedding": {"scale": s}, "residual_mult": m, "loop": {"start": a, "stop": b, "times": n},
     "layers": [{"type": "attention",
                 "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "q_temp": {"coef", "every"}},
                 "mlp": {"kind": "moe", "expert": {"ff": F}, "router": {"experts": E, "top": k}} | null},
                {"type": "parallel", "mixer": {"left": {attention keys}, "right": {"heads", "kv_heads", "dim", "vdim", "conv"}}, ...},
                {"type": "lightning", "mixer": {"heads", "dim", "vdim", "decay": [one per head]}, ...}]}

Tensor names: `embed`, `pos`, `final.norm`, `head`, and under `l<i>.`: `norm1`, `norm2`, `mix.*` (`mix.left.*`,
`mix.right.*`, `mix.left.out`, `mix.right.out` in a parallel layer), `mlp.e<j>.gate|up|down`, `mlp.router`.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

from ..errors import ConfigError
from .kesitar import _num, _pos_int
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

ARCHITECTURE = "Zivovik"
MIXERS = ("attention", "parallel", "lightning")
NORM_OFFSET = 1.0          # the layers' and the model's norm weights are stored around zero


def _check_attention(m, where: str, own_values: bool) -> None:
    heads = _pos_int(m, "heads", where)
    kv = _pos_int(m, "kv_heads", where, required=False, default=heads)
    if heads % kv:
        raise ConfigError(f"config.json: {where}: {heads} heads are not a multiple of {kv} kv heads")
    dim = _pos_int(m, "dim", where)
    vdim = _pos_int(m, "vdim", where, required=False, default=dim)
    if not own_values and vdim != dim:
        raise ConfigError(f"config.json: {where}: the values are the keys, so vdim ({vdim}) must equal dim ({dim})")
    _num(m, "scale", where)
    qt = m.get("q_temp")
    if qt is not None:
        _num(qt, "coef", where + ".q_temp")
        _pos_int(qt, "every", where + ".q_temp")


def _check_delta(m, where: str) -> None:
    heads = _pos_int(m, "heads", where)
    kv = _pos_int(m, "kv_heads", where, required=False, default=heads)
    if heads % kv:
        raise ConfigError(f"config.json: {where}: {heads} heads are not a multiple of {kv} key heads")
    _pos_int(m, "dim", where)
    _pos_int(m, "vdim", where)
    _pos_int(m, "conv", where)


@dataclass(frozen=True)
class ZivovikConfig:
    vocab: int
    width: int
    max_positions: int
    norm_eps: float
    embedding_scale: float
    residual_mult: float
    loop: Optional[Tuple[int, int, int]]      # (start, stop, times) or None
    layers: Tuple[Dict[str, Any], ...]        # as in config.json, checked

    architecture = ARCHITECTURE

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ZivovikConfig":
        layers = d.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        loop = d.get("loop")
        if loop is not None:
            start = _num(loop, "start", "loop", kind=int)
            stop = _num(loop, "stop", "loop", kind=int)
            times = _num(loop, "times", "loop", kind=int, required=False, default=1)
            loop = (int(start), int(stop), int(times))
        cfg = cls(vocab=_pos_int(d, "vocab", "the model"), width=_pos_int(d, "width", "the model"),
                  max_positions=_pos_int(d, "max_positions", "the model"),
                  norm_eps=float(_num(d.get("norm"), "eps", "norm")),
                  embedding_scale=float(_num(d.get("embedding"), "scale", "embedding", required=False, default=1.0)),
                  residual_mult=float(_num(d, "residual_mult", "the model", required=False, default=1.0)),
                  loop=loop, layers=tuple(copy.deepcopy(l) for l in layers))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.norm_eps < 0:
            raise ConfigError(f"config.json: norm.eps must not be negative, found {self.norm_eps}")
        if self.loop is not None:
            start, stop, times = self.loop
            if not 0 <= start <= stop <= len(self.layers) or times < 0:
                raise ConfigError(f"config.json: loop runs layers {start}..{stop - 1} {times} times; the model has "
                                  f"{len(self.layers)} layers")
        for i, l in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(l, dict) or l.get("type") not in MIXERS:
                raise ConfigError(f"config.json: {where}.type must be one of {MIXERS}, found {l.get('type') if isinstance(l, dict) else l!r}")
            m = l.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"config.json: {where} has no 'mixer'")
            if l["type"] == "attention":
                _check_attention(m, where + ".mixer", own_values=False)
            elif l["type"] == "parallel":
                if not isinstance(m.get("left"), dict) or not isinstance(m.get("right"), dict):
                    raise ConfigError(f"config.json: {where}.mixer needs 'left' and 'right'")
                _check_attention(m["left"], where + ".mixer.left", own_values=True)
                _check_delta(m["right"], where + ".mixer.right")
            else:
                heads = _pos_int(m, "heads", where + ".mixer")
                _pos_int(m, "dim", where + ".mixer")
                _pos_int(m, "vdim", where + ".mixer")
                decay = m.get("decay")
                if not isinstance(decay, (list, tuple)) or len(decay) != heads or \
                        any(isinstance(g, bool) or not isinstance(g, (int, float)) for g in decay):
                    raise ConfigError(f"config.json: {where}.mixer.decay must be one number for each of the {heads} heads")
            mlp = l.get("mlp")
            if mlp is None:
                continue
            if not isinstance(mlp, dict) or mlp.get("kind", "moe") != "moe":
                raise ConfigError(f"config.json: {where}.mlp.kind must be 'moe', found {mlp!r}")
            _pos_int(mlp.get("expert"), "ff", where + ".mlp.expert")
            n = _pos_int(mlp.get("router"), "experts", where + ".mlp.router")
            top = _pos_int(mlp.get("router"), "top", where + ".mlp.router")
            if top > n:
                raise ConfigError(f"config.json: {where}.mlp.router chooses {top} of {n} experts")

    def to_dict(self) -> Dict[str, Any]:
        d = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "max_positions": self.max_positions,
             "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
             "residual_mult": self.residual_mult, "layers": [copy.deepcopy(l) for l in self.layers]}
        if self.loop is not None:
            d["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        return d

    def run_order(self) -> List[Tuple[int, bool]]:
        """(layer, whether the embedding output is added right before it) for every layer run, in order."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        start, stop, times = self.loop
        order = [(i, False) for i in range(start)]
        for p in range(times):
            order += [(i, p > 0 and i == start) for i in range(start, stop)]
        return order + [(i, False) for i in range(stop, n)]


def _attention_spec(cfg: ZivovikConfig, m: Dict[str, Any], own_values: bool, gate: str, qk_norm: bool, out_scale: float) -> PartSpec:
    qt = m.get("q_temp")
    return PartSpec("pooled_window_attention", {
        "hidden_size": cfg.width, "num_heads": m["heads"], "num_kv_heads": m.get("kv_heads", m["heads"]),
        "key_dim": m["dim"], "value_dim": m.get("vdim", m["dim"]), "window": None, "pool": 0, "scale": float(m["scale"]),
        "sink": False, "bias": False, "qk_norm_eps": cfg.norm_eps if qk_norm else None, "qk_norm_weights": False,
        "position": None, "values_from_keys": not own_values,
        "q_temp": None if qt is None else (float(qt["coef"]), int(qt["every"])), "gate": gate, "out_scale": out_scale,
        "names": {"q": "q", "k": "k", "v": "v", "o": "o", "gate": "g"}})


def build_spec(cfg: ZivovikConfig) -> ModelSpec:
    """Zivovik as parts: `prenorm_residual` layers (`prenorm_side_by_side` for a parallel layer) of `rmsnorm` norms
    with their weights' offset, a `pooled_window_attention` without window, `gated_delta_rule` or
    `lightning_attention` mixer and `routed_experts`; `learned` positions on the embedding; one run-order entry per
    layer run, each with a cache unit and state of its own."""
    W, m_res = cfg.width, cfg.residual_mult

    def norm(offset=NORM_OFFSET, scale=1.0):
        return PartSpec("rmsnorm", {"size": W, "eps": cfg.norm_eps, "tensor": "", "offset": offset, "scale": scale})

    layers: List[LayerSpec] = []
    for i, l in enumerate(cfg.layers):
        m = l["mixer"]
        norms = {"mixer": norm()}
        names = {"norm.mixer": "norm1"}
        more: Dict[str, PartSpec] = {}
        block = "prenorm_residual"
        mlp, ffn = l.get("mlp"), None
        if mlp is not None:
            ffn = PartSpec("routed_experts", {"hidden_size": W, "intermediate_size": mlp["expert"]["ff"],
                                              "num_experts": mlp["router"]["experts"], "top": mlp["router"]["top"],
                                              "router_bias": False, "out_scale": m_res})
            norms["feed_forward"] = norm()
            names["norm.feed_forward"] = "norm2"
        if l["type"] == "attention":
            mixer = _attention_spec(cfg, m, own_values=False, gate="element", qk_norm=True, out_scale=m_res)
            names["mixer"] = "mix."
        elif l["type"] == "parallel":
            # each side's output is normed with a plain weight; the mean of the two and the residual multiplier ride on it
            block = "prenorm_side_by_side"
            mixer = _attention_spec(cfg, m["left"], own_values=True, gate="head", qk_norm=False, out_scale=1.0)
            r = m["right"]
            more["right"] = PartSpec("gated_delta_rule", {
                "hidden_size": W, "num_heads": r["heads"], "num_key_heads": r.get("kv_heads", r["heads"]), "key_dim": r["dim"],
                "value_dim": r["vdim"], "taps": r["conv"], "norm_eps": cfg.norm_eps})
            names["mixer"] = "mix.left."
            names["mixer.right"] = "mix.right."
            norms["mixer_out"] = norm(offset=0.0, scale=0.5 * m_res)
            norms["mixer_out.right"] = norm(offset=0.0, scale=0.5 * m_res)
            names["norm.mixer_out"] = "mix.left.out"
            names["norm.mixer_out.right"] = "mix.right.out"
        else:
            mixer = PartSpec("lightning_attention", {
                "hidden_size": W, "num_heads": m["heads"], "key_dim": m["dim"], "value_dim": m["vdim"],
                "decay": [float(g) for g in m["decay"]], "norm_eps": cfg.norm_eps, "out_scale": m_res})
            names["mixer"] = "mix."
        if ffn is not None:
            names["feed_forward"] = "mlp."
        layers.append(LayerSpec(prefix=f"l{i}.", mixer=mixer, feed_forward=ffn, norms=norms, block=block, names=names,
                                more_mixers=more))
    # every layer run has a cache unit of its own (a layer that is passed again shares weights, nothing else)
    schedule = [ScheduleEntry(layer=i, cache=n, adds_embedding=adds) for n, (i, adds) in enumerate(cfg.run_order())]
    return ModelSpec(
        architecture=ARCHITECTURE, hidden_size=W, vocab_size=cfg.vocab,
        embedding=PartSpec("embedding", {"vocab_size": cfg.vocab, "hidden_size": W, "scale": cfg.embedding_scale, "tensor": ""}),
        layers=layers, schedule=schedule, final_norm=norm(),
        lm_head=PartSpec("lm_head", {"vocab_size": cfg.vocab, "hidden_size": W, "tied_to": None, "scale": 1.0, "tensor": ""}),
        positions={"learned": PartSpec("learned", {"rows": cfg.max_positions, "hidden_size": W, "tensor": ""})},
        max_position_embeddings=cfg.max_positions,
        embedding_prefix="embed", final_norm_prefix="final.norm", lm_head_prefix="head",
        stop_token_ids=[], bos_token_id=None, position_prefixes={"learned": "pos"},
        optional_tensors=[f"l{i}.norm2" for i, l in enumerate(cfg.layers) if l.get("mlp") is None])


def _attention(heads, kv_heads, dim, coef=0.4, every=128):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
                                           "q_temp": {"coef": coef, "every": every}}}


def _parallel(heads, kv_heads, dim, vdim, r_heads, r_kv_heads, r_dim, r_vdim, conv=4, coef=0.4, every=128):
    return {"type": "parallel", "mixer": {
        "left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5,
                 "q_temp": {"coef": coef, "every": every}},
        "right": {"heads": r_heads, "kv_heads": r_kv_heads, "dim": r_dim, "vdim": r_vdim, "conv": conv}}}


def _lightning(heads, dim, vdim):
    # decays between a short and a long memory, head by head
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim,
                                           "decay": [1.0 - 2.0 ** (-3.0 - 5.0 * h / max(1, heads - 1)) for h in range(heads)]}}


def _moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def _with(layer, mlp):
    return dict(copy.deepcopy(layer), mlp=mlp)


# Shapes without a model folder: a tiny one for tests and tools, and two of the size of a real model's layers (eight
# layer runs each: a parallel and a lightning layer passed three times, then two attention layers; a token's share of
# the experts equals a dense layer's inner width of 5,632 / 14,336).
PRESETS: Dict[str, Dict[str, Any]] = {
    "zivovik-tiny": dict(vocab=320, width=96, max_positions=512, norm={"eps": 1e-5}, embedding={"scale": 2.0}, residual_mult=0.7,
                         loop={"start": 1, "stop": 3, "times": 2}, layers=[
        _with(_attention(4, 2, 24, every=16), _moe(48, 6, 2)),
        _with(_parallel(3, 1, 16, 24, 4, 2, 16, 24, conv=4, every=8), _moe(48, 6, 2)),
        _with(_lightning(3, 16, 24), None),
        _with(_attention(4, 2, 24, every=16), _moe(48, 6, 2))]),
    "zivovik-1b": dict(vocab=32768, width=2048, max_positions=16384, norm={"eps": 1e-6}, embedding={"scale": 1.0}, residual_mult=0.6,
                       loop={"start": 0, "stop": 2, "times": 3}, layers=[
        _with(_parallel(8, 4, 128, 128, 16, 8, 128, 128), _moe(1408, 16, 4)),
        _with(_lightning(16, 128, 128), _moe(1408, 16, 4)),
        _with(_attention(16, 4, 128), _moe(1408, 16, 4)),
        _with(_attention(16, 4, 128), _moe(1408, 16, 4))]),
    "zivovik-7b": dict(vocab=32768, width=4096, max_positions=16384, norm={"eps": 1e-6}, embedding={"scale": 1.0}, residual_mult=0.6,
                       loop={"start": 0, "stop": 2, "times": 3}, layers=[
        _with(_parallel(16, 8, 128, 128, 32, 16, 128, 128), _moe(1792, 32, 8)),
        _with(_lightning(32, 128, 128), _moe(1792, 32, 8)),
        _with(_attention(32, 8, 128), _moe(1792, 32, 8)),
        _with(_attention(32, 8, 128), _moe(1792, 32, 8))]),
}


def preset(name: str, **overrides) -> ZivovikConfig:
    if name not in PRESETS:
        raise ConfigError(f"unknown preset {name!r}; known: {sorted(PRESETS)}")
    d = dict(copy.deepcopy(PRESETS[name]), architecture=ARCHITECTURE)
    d.update(overrides)
    return ZivovikConfig.from_dict(d)
