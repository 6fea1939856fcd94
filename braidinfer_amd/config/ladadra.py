"""Typed configuration of the `Ladadra` design and its translation into parts.

A Ladadra model is a stack of layers whose halves read the residual rows themselves and are normed behind:
x += norm1(mixer(x)), then x += norm2(feed_forward(x)), with RMS norms of plain weights.  Mixers:

* `"attention"`: grouped-query attention with biased projections, one RMS norm over the whole query (key)
  projection, rotation of the first `rot.dims` elements of every head (pairs i, i + dims/2; frequencies stretched
  by wavelength as `rot.scaling` says), scores bounded by `softcap`, keys seen only within the query's own run of
  `mask.size` positions, a learnt sink per head in the softmax's denominator and a sigmoid gate per head.
* `"retention"`: linear attention with a fixed decay per head, S <- decay_h S + k v^T, o = S^T q, over rotated q and
  k (k times dim^-1/2), every head's o divided by its root mean square, times silu of a gate projection.
* `"attention_2"`: differential attention: two softmax maps a head (queries and keys normed per head and map with one
  shared weight, no rotation) over the same values inside a window of `mask.size` positions that also keeps the
  sequence's first `mask.keep_first` tokens; a2 is taken off a1 with a learnt factor, the head normed without weight
  and multiplied by 1 - diff.

The feed-forward is a dense gated unit, a set of routed experts (sigmoid scores, a correction on the choice, groups of
experts, a shared expert) or absent.  The embedding table is the output head.  The reference has no such model; its
configuration is one flat struct (crates/braidinfer-runtime/src/config.rs:75-115), this one keeps the nesting of the
design's config.json:

    {"architecture": "Ladadra", "vocab": V, "width": W, "norm": {"eps": e},
     "layers": [{"type": "attention",
                 "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "softcap", "mask": {"size"},
                           "rot": {"base", "dims", "scaling": {"factor", "low", "high", "original"}}},
                 "mlp": {"kind": "dense", "ff": F} | {"kind": "moe", "expert": {"ff": F}, "shared": {"ff": F},
                         "router": {"experts": E, "top": k, "groups": {"count", "keep"}}} | null},
                {"type": "retention", "mixer": {"heads", "dim", "vdim", "decay": [one per head], "rot": {"base", "dims"}}, ...},
                {"type": "attention_2", "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "diff",
                                                  "mask": {"size", "keep_first"}}, ...}]}

Keys a mixer may leave out: `kv_heads` (as many as heads), `vdim` (dim), `softcap`, `mask` (every earlier token),
`mask.keep_first`, `rot`, `rot.scaling`, `router.groups`, `shared`.  Tensor names: `embed`, `final.norm`, and under
`l<i>.`: `norm1`, `norm2`, `mix.*`, `mlp.gate|up|down`, `mlp.e<j>.gate|up|down`, `mlp.router`, `mlp.correction`,
`mlp.shared.gate|up|down`.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Dict, List, Tuple

from ..errors import ConfigError
from .kesitar import MAX_POSITIONS, _num, _pos_int
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

ARCHITECTURE = "Ladadra"
MIXERS = ("attention", "retention", "attention_2")


def _check_rot(m, where: str, scaling_allowed: bool) -> None:
    rot = m.get("rot")
    if rot is None:
        return
    if not isinstance(rot, dict):
        raise ConfigError(f"config.json: {where}.rot must be an object")
    dims = _pos_int(rot, "dims", where + ".rot")
    if dims % 2 or dims > m["dim"]:
        raise ConfigError(f"config.json: {where}.rot.dims must be even and at most dim ({m['dim']}), found {dims}")
    if float(_num(rot, "base", where + ".rot", kind=(int, float))) <= 0:
        raise ConfigError(f"config.json: {where}.rot.base must be positive")
    sc = rot.get("scaling")
    if sc is None:
        return
    if not scaling_allowed or not isinstance(sc, dict):
        raise ConfigError(f"config.json: {where}.rot.scaling is not part of this mixer")
    for key in ("factor", "low", "high", "original"):
        if float(_num(sc, key, where + ".rot.scaling", kind=(int, float))) <= 0:
            raise ConfigError(f"config.json: {where}.rot.scaling.{key} must be positive")
    if float(sc["low"]) == float(sc["high"]):
        raise ConfigError(f"config.json: {where}.rot.scaling.low and .high must differ")


def _check_heads(m, where: str) -> None:
    heads = _pos_int(m, "heads", where)
    kv = _pos_int(m, "kv_heads", where, required=False, default=heads)
    if heads % kv:
        raise ConfigError(f"config.json: {where}: {heads} heads are not a multiple of {kv} kv heads")
    _pos_int(m, "dim", where)
    _pos_int(m, "vdim", where, required=False)
    _num(m, "scale", where, kind=(int, float))
    mask = m.get("mask")
    if mask is not None:
        if not isinstance(mask, dict):
            raise ConfigError(f"config.json: {where}.mask must be an object")
        _pos_int(mask, "size", where + ".mask")


@dataclass(frozen=True)
class LadadraConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[Dict[str, Any], ...]        # as in config.json, checked

    architecture = ARCHITECTURE

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LadadraConfig":
        layers = d.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        cfg = cls(vocab=_pos_int(d, "vocab", "the model"), width=_pos_int(d, "width", "the model"),
                  norm_eps=float(_num(d.get("norm"), "eps", "norm", kind=(int, float))),
                  layers=tuple(copy.deepcopy(l) for l in layers))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.norm_eps < 0:
            raise ConfigError(f"config.json: norm.eps must not be negative, found {self.norm_eps}")
        for i, l in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(l, dict) or l.get("type") not in MIXERS:
                raise ConfigError(f"config.json: {where}.type must be one of {MIXERS}, found {l.get('type') if isinstance(l, dict) else l!r}")
            m = l.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"config.json: {where} has no 'mixer'")
            where += ".mixer"
            if l["type"] == "attention":
                _check_heads(m, where)
                _check_rot(m, where, scaling_allowed=True)
                cap = _num(m, "softcap", where, kind=(int, float), required=False)
                if cap is not None and not cap > 0:
                    raise ConfigError(f"config.json: {where}.softcap must be positive, found {cap}")
            elif l["type"] == "attention_2":
                _check_heads(m, where)
                _num(m, "diff", where, kind=(int, float))
                keep = _num(m.get("mask") or {}, "keep_first", where + ".mask", kind=int, required=False, default=0)
                if keep < 0:
                    raise ConfigError(f"config.json: {where}.mask.keep_first must not be negative, found {keep}")
            else:
                heads = _pos_int(m, "heads", where)
                _pos_int(m, "dim", where)
                _pos_int(m, "vdim", where, required=False)
                _check_rot(m, where, scaling_allowed=False)
                decay = m.get("decay")
                if not isinstance(decay, (list, tuple)) or len(decay) != heads or \
                        any(isinstance(g, bool) or not isinstance(g, (int, float)) for g in decay):
                    raise ConfigError(f"config.json: {where}.decay must be one number for each of the {heads} heads")
            mlp = l.get("mlp")
            if mlp is None:
                continue
            where = f"layers[{i}].mlp"
            if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
                raise ConfigError(f"config.json: {where}.kind must be 'dense' or 'moe', found {mlp!r}")
            if mlp["kind"] == "dense":
                _pos_int(mlp, "ff", where)
                continue
            _pos_int(mlp.get("expert"), "ff", where + ".expert")
            n = _pos_int(mlp.get("router"), "experts", where + ".router")
            top = _pos_int(mlp.get("router"), "top", where + ".router")
            if top > n:
                raise ConfigError(f"config.json: {where}.router chooses {top} of {n} experts")
            groups = mlp["router"].get("groups")
            if groups is not None:
                count = _pos_int(groups, "count", where + ".router.groups")
                keep = _pos_int(groups, "keep", where + ".router.groups")
                if n % count or keep > count or keep * (n // count) < top:
                    raise ConfigError(f"config.json: {where}.router: {count} groups of which {keep} are kept must divide "
                                      f"the {n} experts and leave {top} to choose")
            if mlp.get("shared") is not None:
                _pos_int(mlp["shared"], "ff", where + ".shared")

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
                "layers": [copy.deepcopy(l) for l in self.layers]}


def _rope(rot: Dict[str, Any], positions: Dict[str, PartSpec]) -> str:
    """The name of the rotary encoding of these numbers; one part per distinct (dims, base, scaling)."""
    sc = rot.get("scaling")
    tail = "" if sc is None else "/" + ",".join(repr(float(sc[k])) for k in ("factor", "low", "high", "original"))
    name = f"rope{rot['dims']}@{float(rot['base'])!r}{tail}"
    params = {"rotary_dim": rot["dims"], "theta": float(rot["base"]), "pairing": "half", "frequencies_from_float64": True}
    if sc is not None:
        params["scaling"] = {k: float(sc[k]) for k in ("factor", "low", "high", "original")}
        params["scaling_rule"] = "wavelength"
    positions[name] = PartSpec("rope", params)
    return name


def build_spec(cfg: LadadraConfig) -> ModelSpec:
    """Ladadra as parts: `sandwich_residual` layers whose norms in front are `rows` (the halves read the residual rows as
    they are) and whose norms behind are `rmsnorm`; `pooled_window_attention` with runs of positions, bounded scores, a
    learnt sink and a norm over the projection, or with two maps, a window and kept first tokens; `lightning_attention`
    in its retention form; `swiglu` or `routed_experts` with sigmoid scoring."""
    W = cfg.width

    def norm():
        return PartSpec("rmsnorm", {"size": W, "eps": cfg.norm_eps, "tensor": ""})

    rows = PartSpec("rows", {"size": W})
    layers: List[LayerSpec] = []
    positions: Dict[str, PartSpec] = {}
    for i, l in enumerate(cfg.layers):
        m = l["mixer"]
        rot = m.get("rot")
        position = _rope(rot, positions) if rot is not None else None
        if l["type"] == "attention":
            mask = m.get("mask") or {}
            mixer = PartSpec("pooled_window_attention", {
                "hidden_size": W, "num_heads": m["heads"], "num_kv_heads": m.get("kv_heads", m["heads"]), "key_dim": m["dim"],
                "value_dim": m.get("vdim", m["dim"]), "window": None, "pool": 0, "scale": float(m["scale"]), "sink": "learnt",
                "bias": True, "qk_norm_eps": cfg.norm_eps, "qk_norm_over": "projection", "position": position,
                "gate": "head", "chunk": mask.get("size"), "softcap": m.get("softcap"),
                "names": {"q": "q", "k": "k", "v": "v", "o": "o", "gate": "g", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
                          "q_norm": "q.norm", "k_norm": "k.norm", "sink": "sink"}})
        elif l["type"] == "attention_2":
            mask = m.get("mask") or {}
            mixer = PartSpec("pooled_window_attention", {
                "hidden_size": W, "num_heads": m["heads"], "num_kv_heads": m.get("kv_heads", m["heads"]), "key_dim": m["dim"],
                "value_dim": m.get("vdim", m["dim"]), "window": mask.get("size"), "pool": 0, "scale": float(m["scale"]),
                "sink": False, "bias": False, "qk_norm_eps": cfg.norm_eps, "position": None,
                "keep_first": int(mask.get("keep_first", 0) or 0) if mask.get("size") else 0, "maps": 2, "diff": float(m["diff"]),
                "head_norm_eps": cfg.norm_eps,
                "names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm"}})
        else:
            mixer = PartSpec("lightning_attention", {
                "hidden_size": W, "num_heads": m["heads"], "key_dim": m["dim"], "value_dim": m.get("vdim", m["dim"]),
                "decay": [float(g) for g in m["decay"]], "norm_eps": cfg.norm_eps, "activation": None, "position": position,
                "key_scale": float(m["dim"]) ** -0.5, "norm": "head", "norm_weight": False, "gate": "silu"})
        mlp, ffn = l.get("mlp"), None
        if mlp is not None and mlp["kind"] == "dense":
            ffn = PartSpec("swiglu", {"hidden_size": W, "intermediate_size": mlp["ff"],
                                      "names": {"gate": "gate", "up": "up", "down": "down"}})
        elif mlp is not None:
            groups = mlp["router"].get("groups") or {}
            ffn = PartSpec("routed_experts", {
                "hidden_size": W, "intermediate_size": mlp["expert"]["ff"], "num_experts": mlp["router"]["experts"],
                "top": mlp["router"]["top"], "router_bias": False, "scoring": "sigmoid",
                "groups": int(groups.get("count", 1)), "groups_keep": int(groups.get("keep", 1)),
                "shared_size": int((mlp.get("shared") or {}).get("ff", 0))})
        norms = {"mixer": rows, "mixer_out": norm()}
        names = {"norm.mixer": "", "norm.mixer_out": "norm1", "mixer": "mix."}
        if ffn is not None:
            norms.update({"feed_forward": rows, "feed_forward_out": norm()})
            names.update({"norm.feed_forward": "", "norm.feed_forward_out": "norm2", "feed_forward": "mlp."})
        layers.append(LayerSpec(prefix=f"l{i}.", mixer=mixer, feed_forward=ffn, norms=norms, block="sandwich_residual", names=names))
    return ModelSpec(
        architecture=ARCHITECTURE, hidden_size=W, vocab_size=cfg.vocab,
        embedding=PartSpec("embedding", {"vocab_size": cfg.vocab, "hidden_size": W, "scale": 1.0, "tensor": ""}),
        layers=layers, schedule=[ScheduleEntry(layer=i, cache=i) for i in range(len(layers))], final_norm=norm(),
        lm_head=PartSpec("lm_head", {"vocab_size": cfg.vocab, "hidden_size": W, "tied_to": "embed", "scale": 1.0}),
        positions=positions, max_position_embeddings=MAX_POSITIONS,
        embedding_prefix="embed", final_norm_prefix="final.norm", lm_head_prefix="head.",
        stop_token_ids=[], bos_token_id=None,
        optional_tensors=[f"l{i}.norm2" for i, l in enumerate(cfg.layers) if l.get("mlp") is None])


# ------------------------------------------------------------------ presets ---------
_STRETCH = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}


def _attention(heads, kv_heads, dim, chunk, base=500000.0, rot_dims=None, scaling=None, softcap=30.0):
    rot = {"base": base, "dims": rot_dims or dim}
    if scaling is not None:
        rot["scaling"] = dict(scaling)
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
                                           "softcap": softcap, "mask": {"size": chunk}, "rot": rot}}


def _retention(heads, dim, vdim, base=10000.0):
    # decays between a short and a long memory, head by head
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "rot": {"base": base, "dims": dim},
                                           "decay": [1.0 - 2.0 ** (-5.0 - 3.0 * h / max(1, heads - 1)) for h in range(heads)]}}


def _differential(heads, kv_heads, dim, vdim, window, keep_first, diff=0.2):
    return {"type": "attention_2", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5,
                                             "diff": diff, "mask": {"size": window, "keep_first": keep_first}}}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(ff, experts, top, groups, keep, shared):
    return {"kind": "moe", "expert": {"ff": ff}, "shared": {"ff": shared},
            "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}


def _with(layer, mlp):
    return dict(copy.deepcopy(layer), mlp=mlp)


# Shapes without a model folder: a tiny one for tests and tools, and two of the size of a real model's layers (eight
# layers: differential attention, attention within runs of positions and retention in turn; a dense feed-forward in
# three layers, routed experts in five, of which a token's experts with the shared one weigh what the dense unit does).
PRESETS: Dict[str, Dict[str, Any]] = {
    "ladadra-tiny": dict(vocab=320, width=96, norm={"eps": 1e-5}, layers=[
        _with(_differential(4, 2, 16, 24, window=40, keep_first=6), _dense(128)),
        _with(_attention(6, 2, 16, chunk=48, rot_dims=8, scaling={"factor": 2.0, "low": 1.0, "high": 3.0, "original": 64}),
              _moe(32, 8, 2, groups=4, keep=2, shared=48)),
        _with(_retention(3, 16, 24), _dense(128)),
        _with(_attention(6, 2, 16, chunk=48, rot_dims=8), None)]),
    "ladadra-1b": dict(vocab=32768, width=2048, norm={"eps": 1e-6}, layers=[
        _with(_differential(8, 4, 128, 256, window=2048, keep_first=64), _dense(5632)),
        _with(_attention(16, 4, 128, chunk=4096, rot_dims=64, scaling=_STRETCH), _moe(1408, 16, 3, groups=4, keep=2, shared=1408)),
        _with(_retention(8, 128, 256), _moe(1408, 16, 3, groups=4, keep=2, shared=1408)),
        _with(_attention(16, 4, 128, chunk=4096, rot_dims=64, scaling=_STRETCH), _dense(5632)),
        _with(_differential(8, 4, 128, 256, window=2048, keep_first=64), _moe(1408, 16, 3, groups=4, keep=2, shared=1408)),
        _with(_attention(16, 4, 128, chunk=4096, rot_dims=64, scaling=_STRETCH), _moe(1408, 16, 3, groups=4, keep=2, shared=1408)),
        _with(_retention(8, 128, 256), _dense(5632)),
        _with(_attention(16, 4, 128, chunk=4096, rot_dims=64, scaling=_STRETCH), _moe(1408, 16, 3, groups=4, keep=2, shared=1408))]),
    "ladadra-7b": dict(vocab=32768, width=4096, norm={"eps": 1e-6}, layers=[
        _with(_differential(16, 8, 128, 256, window=2048, keep_first=64), _dense(14336)),
        _with(_attention(32, 8, 128, chunk=4096, rot_dims=64, scaling=_STRETCH), _moe(1792, 32, 7, groups=8, keep=4, shared=1792)),
        _with(_retention(16, 128, 256), _moe(1792, 32, 7, groups=8, keep=4, shared=1792)),
        _with(_attention(32, 8, 128, chunk=4096, rot_dims=64, scaling=_STRETCH), _dense(14336)),
        _with(_differential(16, 8, 128, 256, window=2048, keep_first=64), _moe(1792, 32, 7, groups=8, keep=4, shared=1792)),
        _with(_attention(32, 8, 128, chunk=4096, rot_dims=64, scaling=_STRETCH), _moe(1792, 32, 7, groups=8, keep=4, shared=1792)),
        _with(_retention(16, 128, 256), _dense(14336)),
        _with(_attention(32, 8, 128, chunk=4096, rot_dims=64, scaling=_STRETCH), _moe(1792, 32, 7, groups=8, keep=4, shared=1792))]),
}


def preset(name: str, **overrides) -> LadadraConfig:
    if name not in PRESETS:
        raise ConfigError(f"unknown preset {name!r}; known: {sorted(PRESETS)}")
    d = dict(copy.deepcopy(PRESETS[name]), architecture=ARCHITECTURE)
    d.update(overrides)
    return LadadraConfig.from_dict(d)
