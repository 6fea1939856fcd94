"""Grouped-query attention over a sliding window and pooled blocks of what left it.

Per token: q, k, v = W n (+ bias); q and k are RMS-normed per head (one weight of the head's
width, shared by the heads) and rotated on the first `rotary_dim` elements by the position
encoding the mixer names; the values may be mixed with the values another layer made of the
same token, v <- (1 - m) v + m v_first with a learnt scalar m.  Keys (normed, rotated) and
values (mixed) are what the cache keeps.  A query at position i sees the tokens j with
0 <= i - j < window and, for every block b of `pool` tokens with b pool + pool - 1 <= i - window,
one pooled key and value: the means of the block's keys and of its values as the cache holds
them.  Tokens that left the window and whose block is not complete behind it are not seen.
Tokens and blocks share one softmax of the scores (q . k) * scale, which may carry a sink: a key
of score 0 without a value, i.e. one added to the denominator.  Key and value widths may differ.

Without a window (`window` None) every earlier token is seen: plain causal attention through the same kernels.
Further options, each a parameter: the values may be the keys as projected, before their norm (`values_from_keys`,
no value matrix); the query/key norm may go without weights (`qk_norm_weights` False); the query may be multiplied
by a temperature that grows with the logarithm of the position, 1 + c ln(floor((p + 1) / n) + 1) (`q_temp` = (c, n));
the heads' outputs may pass a sigmoid gate projected from the mixer's input, one number per output element or one
per head (`gate` "element" / "head"), before the output projection; `out_scale` multiplies what the mixer adds to the
residual rows (it rides on the gate, or on the output matrix where there is none).

Further rules of what a query sees, each a parameter: `chunk` C cuts the sequence into runs of C positions counted
from 0, and a query sees only keys of its own run (with or without a window beside it); `keep_first` F lets every query
also see the sequence's first F tokens, at their true positions, wherever its window begins (the cache then keeps the
pages that hold them).  `softcap` c bounds the scaled scores, s <- c tanh(s / c).  `sink` "learnt" adds exp(sink_h) of
a learnt number per head to the softmax's denominator (True: exp(0)).  `qk_norm_over` "projection" runs the
query/key norm over a token's whole query (key) projection at once, with a weight for every element of it, instead of
head by head.  `maps` 2 is differential attention: every query head and every key head is two vectors of `key_dim`
side by side (normed one by one), each pair gives a softmax map of its own over the same values, and with a1, a2 the
two maps' outputs the head's output is (a1 - f a2) / rms(a1 - f a2) * (1 - diff), f = exp(lq1 . lk1) - exp(lq2 . lk2) +
diff with four learnt vectors of `key_dim` and the constant `diff`.  In the cache a key row is then 2 key_dim wide,
and a map's query is laid out with zeros where the other map's key lies, so the kernels see 2 H query heads over
the G kv heads and read every key and value once for both maps.

Cache: the mixer's own unit keeps the tokens' rows as long as a later query or a block that is
not pooled yet needs them (`CacheNeed.live_from`); a further unit under the role "pooled" keeps
one row per block (`CacheNeed.tokens_per_row`).  Scores, softmax weights, norms and angles are
float in both precisions.  Nothing of this is in the reference, whose attention is full and
causal (kernels/megakernel_ops.hip:2150-2343).
"""
from __future__ import annotations

import functools
import math
from typing import Dict, List, Optional

import torch

from .. import kernels as K
from ..cache import CacheNeed
from ..errors import ConfigError, StepError
from ..weights import TensorSpec
from .base import Mixer, MixerContext, RotaryTables, Runtime, register_part
from .linear import fused_layout, linear, stream_layout

MAX_WIDTH = 512      # of a head's keys or values: the kernels' limit


@functools.lru_cache(maxsize=None)
def window_and_open_block(window: int, pool: int, chunk: int = 0):
    """`CacheNeed.live_from` of a window with pooled blocks: at length L the next query sees tokens
    from L - window + 1 on, and the block that is still open (from pool * floor(L / pool) on) has yet to be
    pooled.  With runs of `chunk` positions the next query (at position L) sees nothing before its run's first
    position, chunk * floor(L / chunk).  One function object per (window, pool, chunk), so that layers with equal
    sizes share a group."""
    def first_live(length: int) -> int:
        first = length - window + 1
        if pool > 0:
            first = min(first, (length // pool) * pool)
        first = max(0, first)
        if chunk > 0:
            first = max(first, (length // chunk) * chunk)
        return first
    return first_live


class PooledWindowAttention(Mixer):
    graph_safe = True
    through_linear_only = True

    NO_WINDOW = 1 << 30          # the kernels' window when every earlier token is seen: beyond any position
    NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight", "gate": "g_proj.weight",
             "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias",
             "q_norm": "q_norm.weight", "k_norm": "k_norm.weight", "value_mix": "value_mix", "sink": "sink",
             "lq1": "lq1", "lk1": "lk1", "lq2": "lq2", "lk2": "lk2"}

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int,
                 window: int, pool: int = 0, scale: Optional[float] = None, sink: bool = False, bias: bool = False,
                 qk_norm_eps: Optional[float] = None, position: Optional[str] = None,
                 value_mix: Optional[str] = None, value_mix_group: str = "v_first",
                 names: Optional[Dict[str, str]] = None, values_from_keys: bool = False, qk_norm_weights: bool = True,
                 q_temp=None, gate: Optional[str] = None, out_scale: float = 1.0, chunk: Optional[int] = None,
                 keep_first: int = 0, softcap: Optional[float] = None, qk_norm_over: str = "head", maps: int = 1,
                 diff: Optional[float] = None, head_norm_eps: Optional[float] = None):
        """`qk_norm_eps` None: no query/key norm.  `value_mix`: None, "source" (this layer's values are what
        later layers of the same `value_mix_group` mix with; its own scalar is loaded and unused) or "mix"."""
        if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
            raise ConfigError(f"attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if not 0 < key_dim <= MAX_WIDTH or not 0 < value_dim <= MAX_WIDTH:
            raise ConfigError(f"attention: head widths {key_dim} (keys) and {value_dim} (values) must lie in 1..{MAX_WIDTH}")
        if (window is not None and int(window) <= 0) or int(pool or 0) < 0 or (window is None and pool):
            raise ConfigError(f"attention: the window must be positive (or None: all earlier tokens, no pooled blocks) and the "
                              f"pooled block's size not negative, got {window}, {pool}")
        if gate not in (None, "element", "head"):
            raise ConfigError(f"attention: gate must be None, 'element' or 'head', got {gate!r}")
        if values_from_keys and (key_dim != value_dim or bias or value_mix is not None):
            raise ConfigError("attention: values taken from the keys have the keys' width, no bias and no mixing")
        if q_temp is not None and (len(q_temp) != 2 or int(q_temp[1]) <= 0):
            raise ConfigError(f"attention: q_temp is (coefficient, positions a step > 0), got {q_temp!r}")
        if value_mix not in (None, "source", "mix"):
            raise ConfigError(f"attention: value_mix must be None, 'source' or 'mix', got {value_mix!r}")
        if (chunk is not None and int(chunk) <= 0) or int(keep_first or 0) < 0 or (softcap is not None and not float(softcap) > 0):
            raise ConfigError(f"attention: runs of {chunk} positions, {keep_first} kept first tokens and a score bound of "
                              f"{softcap} must be positive where given")
        if qk_norm_over not in ("head", "projection") or (qk_norm_over == "projection" and (qk_norm_eps is None or not qk_norm_weights)):
            raise ConfigError("attention: qk_norm_over is 'head' or 'projection'; a norm over the projection has an eps and weights")
        if int(maps) not in (1, 2) or (int(maps) == 2) != (diff is not None) or (int(maps) == 2 and (values_from_keys or gate is not None or pool)):
            raise ConfigError("attention: one map, or two with the constant `diff` (then without keys as values, gate or pooled blocks)")
        if int(maps) * key_dim > MAX_WIDTH:
            raise ConfigError(f"attention: {maps} maps of {key_dim} make key rows wider than {MAX_WIDTH}")
        if sink not in (True, False, "learnt"):
            raise ConfigError(f"attention: sink is False, True (a score of 0) or 'learnt', got {sink!r}")
        self.H, self.nq, self.nkv = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dk, self.dv = int(key_dim), int(value_dim)
        self.full = window is None
        self.window, self.pool = (self.NO_WINDOW if window is None else int(window)), int(pool or 0)
        self.values_from_keys, self.qk_norm_weights = bool(values_from_keys), bool(qk_norm_weights)
        self.q_temp = None if q_temp is None else (float(q_temp[0]), int(q_temp[1]))
        self.gate, self.out_scale = gate, float(out_scale)
        self.n_gate = 0 if gate is None else (self.nq if gate == "head" else self.nq * self.dv)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.dk)
        self.sink, self.bias = bool(sink), bool(bias)
        self.learnt_sink = sink == "learnt"
        self.chunk, self.keep_first = int(chunk or 0), int(keep_first or 0)
        self.softcap = float(softcap or 0.0)
        self.norm_over_projection = qk_norm_over == "projection"
        self.maps, self.diff = int(maps), (None if diff is None else float(diff))
        self.head_norm_eps = None if head_norm_eps is None else float(head_norm_eps)
        self.kw = self.maps * self.dk          # a key row of the cache, and a query row the kernels see
        self.sinks = None
        self.pair_factor = 0.0
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.position = position
        self.value_mix, self.value_mix_group = value_mix, value_mix_group
        self.names = dict(self.NAMES, **(names or {}))
        self.w_qkv = self.w_o = self.b_qkv = self.q_norm = self.k_norm = self.mix = None
        self._expects_tables = False
        self.force_simple = False          # tests set it to run the one-wave-per-query kernel in bfloat16

    # ---- weights -----------------------------------------------------------------------
    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        n = self.names
        out = [TensorSpec(prefix + n["q"], (self.nq * self.kw, self.H))]
        if self.bias:
            out.append(TensorSpec(prefix + n["q_bias"], (self.nq * self.kw,), kind="vector", init="normal"))
        out.append(TensorSpec(prefix + n["k"], (self.nkv * self.kw, self.H)))
        if self.bias:
            out.append(TensorSpec(prefix + n["k_bias"], (self.nkv * self.kw,), kind="vector", init="normal"))
        if not self.values_from_keys:
            out.append(TensorSpec(prefix + n["v"], (self.nkv * self.dv, self.H)))
        if self.bias:
            out.append(TensorSpec(prefix + n["v_bias"], (self.nkv * self.dv,), kind="vector", init="normal"))
        if self.gate is not None:
            out.append(TensorSpec(prefix + n["gate"], (self.n_gate, self.H)))
        if self.qk_norm_eps is not None and self.qk_norm_weights:
            whole = self.norm_over_projection
            out += [TensorSpec(prefix + n["q_norm"], (self.nq * self.kw if whole else self.dk,), kind="vector", init="ones"),
                    TensorSpec(prefix + n["k_norm"], (self.nkv * self.kw if whole else self.dk,), kind="vector", init="ones")]
        if self.maps == 2:
            out += [TensorSpec(prefix + n[x], (self.dk,), kind="vector", init="normal") for x in ("lq1", "lk1", "lq2", "lk2")]
        if self.learnt_sink:
            out.append(TensorSpec(prefix + n["sink"], (self.nq,), kind="vector", init="normal"))
        if self.value_mix is not None:
            out.append(TensorSpec(prefix + n["value_mix"], (), kind="vector", init="normal"))
        out.append(TensorSpec(prefix + n["o"], (self.H, self.nq * self.dv)))
        return out

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        # one product for all projections of the mixer's input: q | k | v (unless the keys serve) | gate
        mats = ["q", "k"] + ([] if self.values_from_keys else ["v"]) + (["gate"] if self.gate is not None else [])
        self.w_qkv = fused_layout([tensors[prefix + n[x]] for x in mats], rt)
        self.gate_col0 = self.nq * self.kw + self.nkv * self.kw + (0 if self.values_from_keys else self.nkv * self.dv)
        w_o = tensors[prefix + n["o"]]
        if self.gate is None and self.out_scale != 1.0:          # no gate to carry the multiplier: the matrix does
            w_o = (w_o.to(torch.float32) * self.out_scale).to(w_o.dtype)
        self.w_o = stream_layout(w_o, rt)
        if self.bias:
            self.b_qkv = rt.own(torch.cat([tensors[prefix + n[x]].to(torch.float32).reshape(-1) for x in ("q_bias", "k_bias", "v_bias")]))
        if self.qk_norm_eps is not None and self.qk_norm_weights:
            self.q_norm = rt.own(tensors[prefix + n["q_norm"]].to(torch.float32))
            self.k_norm = rt.own(tensors[prefix + n["k_norm"]].to(torch.float32))
        elif self.qk_norm_eps is not None:
            ones = rt.empty((self.dk,), torch.float32)
            ones.fill_(1.0)
            self.q_norm = self.k_norm = ones
        if self.value_mix == "mix":
            self.mix = rt.own(tensors[prefix + n["value_mix"]].to(torch.float32).reshape(1))
        if self.learnt_sink:
            self.sinks = rt.own(tensors[prefix + n["sink"]].to(torch.float32).reshape(-1))
            if self.maps == 2:          # both maps of a head carry the head's sink
                self.sinks = rt.own(self.sinks.repeat_interleave(2))
        if self.maps == 2:
            # one number for the layer, from four learnt vectors, in float: exp(lq1 . lk1) - exp(lq2 . lk2) + diff
            lq1, lk1, lq2, lk2 = (tensors[prefix + n[x]].to(torch.float32).reshape(-1).cpu() for x in ("lq1", "lk1", "lq2", "lk2"))
            self.pair_factor = float(torch.exp(torch.sum(lq1 * lk1)) - torch.exp(torch.sum(lq2 * lk2)) + torch.tensor(self.diff, dtype=torch.float32))

    # ---- what it keeps -----------------------------------------------------------------
    def cache_need(self) -> CacheNeed:
        if self.full and not self.chunk:
            return CacheNeed(kv_heads=self.nkv, head_dim=self.kw, value_dim=self.dv)
        return CacheNeed(kv_heads=self.nkv, head_dim=self.kw, value_dim=self.dv,
                         live_from=window_and_open_block(self.window, self.pool, self.chunk), keep_first=self.keep_first)

    def more_cache_needs(self) -> Dict[str, CacheNeed]:
        if not self.pool:
            return {}
        return {"pooled": CacheNeed(kv_heads=self.nkv, head_dim=self.kw, value_dim=self.dv, tokens_per_row=self.pool)}

    def check_positions(self, encodings) -> None:
        if self.position is None:
            return
        enc = encodings.get(self.position)
        if enc is None:
            raise ConfigError(f"attention asks for the position encoding {self.position!r}, the model has {sorted(encodings)}")
        if getattr(enc, "gives", None) not in ("rotary", "embedding", "none"):
            raise ConfigError(f"attention cannot use the position encoding {self.position!r}: it gives {getattr(enc, 'gives', None)!r}")
        self._expects_tables = enc.gives == "rotary"
        if self._expects_tables and (enc.rotary_dim > self.dk or getattr(enc, "pairing", "half") != "half"):
            raise ConfigError(f"attention: the encoding {self.position!r} rotates {enc.rotary_dim} elements in "
                              f"{getattr(enc, 'pairing', None)!r} pairs; this mixer takes up to {self.dk} in 'half' pairs")

    # ---- one step ----------------------------------------------------------------------
    def forward(self, h, x, step, ctx: MixerContext) -> None:
        T = step.n_tokens
        nq, nkv, dk, dv = self.nq, self.nkv, self.dk, self.dv
        dt = self.rt.dtype
        tables = step.position_data.get(self.position) if self.position else None
        if (tables is None and self._expects_tables) or (tables is not None and not isinstance(tables, RotaryTables)):
            raise StepError(f"attention: the position encoding {self.position!r} gave {type(tables).__name__}, "
                            "rotary tables were expected")
        if ctx.storage is None or (self.pool and "pooled" not in ctx.others):
            raise StepError("attention: the run order gave this mixer no cache unit (or none for its pooled rows)")
        # the projections' float sums: norms and angles work on them before anything is rounded
        qkv = step.ws.get("pwa_qkv", (T, self.gate_col0 + self.n_gate), torch.float32)
        linear(h, self.w_qkv, qkv, step.ws)
        maps, kw = self.maps, self.kw
        # prompts and portions in bfloat16 go to the matrix cores; with two maps that kernel takes the maps itself (query
        # rows of key_dim), the others see every map as a query head over key rows that hold all maps (rows of maps * key_dim
        # with zeros outside the map's own elements)
        by_matrix_prefill = not step.is_decode and not self.force_simple and K.pwa_prefill_takes(dt, dk, dv, ctx.page_tokens)
        pad = not (by_matrix_prefill and maps > 1)
        q = step.ws.get("pwa_q", (T, nq * maps * (kw if pad else dk)), dt)
        row_ss = step.ws.get("pwa_row_ss", (T, 2), torch.float32) if self.norm_over_projection else None
        v_first, role = None, 0
        if self.value_mix is not None:
            key = ("value_mix", self.value_mix_group)
            if self.value_mix == "source":
                v_first = step.ws.get(f"pwa_{self.value_mix_group}", (T, nkv * dv), torch.float32)
                step.extras[key] = v_first
                role = 1
            else:
                v_first = step.extras.get(key)
                if v_first is None or v_first.shape != (T, nkv * dv):
                    raise StepError(f"attention: no layer before this one left values of width {nkv * dv} to mix with "
                                    f"(group {self.value_mix_group!r})")
                role = 2
        unit = ctx.storage
        K.pwa_prepare(qkv, self.b_qkv, self.q_norm, self.k_norm, self.qk_norm_eps or 0.0,
                      tables.cos if tables else None, tables.sin if tables else None, tables.rotary_dim if tables else 0,
                      step.positions, step.seq_of_token, step.slots, ctx.block_table, q, unit, v_first, self.mix, role,
                      nq, nkv, dk, dv, ctx.page_tokens, ctx.writes_cache, self.values_from_keys,
                      self.q_temp[0] if self.q_temp else 0.0, self.q_temp[1] if self.q_temp else 0, maps=maps, row_ss=row_ss,
                      pad_queries=pad)
        nq, dk = nq * maps, (kw if pad else dk)
        mask = dict(chunk=self.chunk, keep=self.keep_first, softcap=self.softcap)
        pooled = ctx.others.get("pooled")
        if pooled is not None and ctx.writes_cache:
            K.pwa_pool(unit, ctx.block_table, pooled.storage, pooled.block_table, step.cu_seqlens, step.ctx_lens, step.slots,
                       step.n_seqs, step.max_new, nkv, dk, dv, ctx.page_tokens, self.pool)
        o = step.ws.get("pwa_out" if maps == 1 else "pwa_out_maps", (T, nq * dv), dt)
        p_table = pooled.block_table if pooled is not None else None
        p_unit = pooled.storage if pooled is not None else None
        if by_matrix_prefill:
            K.pwa_prefill_bf16(q, o, step.cu_seqlens, step.slots, step.ctx_lens, ctx.block_table, unit, p_table, p_unit,
                               step.n_seqs, step.max_new, nq, nkv, dk, dv, ctx.page_tokens, self.window, self.pool,
                               self.scale, self.sink, self.sinks, maps=1 if pad else maps, **mask)
        elif step.is_decode and not self.force_simple and K.pwa_decode_takes(dt, nq, nkv, dk, dv, ctx.page_tokens):
            # single tokens in bfloat16: the matrix cores, a kv head's keys read once for its query heads
            K.pwa_decode_bf16(q, o, step.slots, step.ctx_lens, ctx.block_table, unit, p_table, p_unit, step.n_seqs,
                              nq, nkv, dk, dv, ctx.page_tokens, self.window, self.pool, self.scale, self.sink, self.sinks, **mask)
        else:
            # the 32-bit path and other sizes: four waves per (query, head) in float
            K.pwa_attend(q, o, step.positions, step.seq_of_token, step.slots, ctx.block_table, unit, p_table, p_unit,
                         nq, nkv, dk, dv, ctx.page_tokens, self.window, self.pool, self.scale, self.sink, self.sinks, **mask)
        if maps == 2:
            # the two maps of a head into its one output: a1 - f a2, normed over the head's values, times 1 - diff
            o2, nq = o, self.nq
            o = step.ws.get("pwa_out", (T, nq * dv), dt)
            K.pwa_pair_combine(o2, o, nq, dv, self.pair_factor, self.head_norm_eps, (1.0 - self.diff) * self.out_scale)
        if self.gate is not None:
            K.pwa_gate(o, qkv[:, self.gate_col0:], nq, dv, self.gate == "head", self.out_scale)
        linear(o, self.w_o, x, step.ws, accumulate=True)


register_part("mixer", "pooled_window_attention", PooledWindowAttention, replace=True)
