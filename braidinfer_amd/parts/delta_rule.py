"""Two recurrent mixers over an outer-product state with one decay number per head.

Gated delta rule.  With n the mixer's input: q = W_q n and k = W_k n (G heads of d channels), v = W_v n (H heads of
e channels; head h reads q/k head h // (H / G)).  Each of q, k, v passes a short causal convolution over time per
channel (`taps` numbers a channel, the last one the current token's, zeros before the sequence's start, no bias) and
silu; q and k are then made unit vectors per head, x / sqrt(sum(x^2) + 1e-6), and q is multiplied by d^-1/2.  With
beta = sigmoid(W_b n) and g = exp(-exp(A_log) * softplus(W_a n + dt_bias)), one number a head each,

    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

in this order (the read-out sees the token's own write).  Every head's o is divided by its root mean square over e,
multiplied by a weight [e] shared by the heads and by silu(W_g n) [H, e], and projected by W_o.

Lightning attention (linear attention with a fixed decay per head): q = silu(W_q n), k = silu(W_k n) (H heads of d),
v = silu(W_v n) (H of e); S <- decay_h S + k v^T, o = S^T q, no other scale.  The concatenated heads are RMS-normed
together with a weight [H e], multiplied by sigmoid(W_g n) and projected by W_o.  Parameters make the same mixer a
retention layer: `activation` None (q, k, v as projected), `position` (a rotary encoding that turns q and k by the
token's position before the sum), `key_scale` (k times a constant behind the rotation), `norm` "head" (every head's o
divided by its own root mean square) with or without weights, `gate` "silu".

What a sequence keeps is fixed in size and float in both precisions, in its slot of the cache's state area
(`StateNeed`): S per head (zero at first, laid out as the scan kernel's lanes hold it) and, for the convolution, the
last taps - 1 inputs of every channel behind it.  All projections of the input are one product that leaves float
sums, so convolution, activations, unit norms, decay, write strength, recurrence and head norm work on unrounded
numbers.  `out_scale` multiplies what the mixer adds to the residual rows (folded into the norm's weight at load).
The reference has no recurrent mixer.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from .. import kernels as K
from ..cache import StateNeed
from ..errors import ConfigError, StepError
from ..weights import TensorSpec
from .base import Mixer, MixerContext, RotaryTables, Runtime, register_part
from .gated_recurrence import HGRN2, pieces_for
from .linear import fused_layout, linear, stream_layout


def _floats(shape) -> int:
    n = 1
    for s in shape:
        n *= int(s)
    return n


class GatedDeltaRule(Mixer):
    graph_safe = True
    through_linear_only = True

    NAMES = {"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "b": "b", "a": "a",
             "A_log": "A_log", "dt_bias": "dt_bias", "norm": "norm", "g": "g", "o": "o"}

    def __init__(self, hidden_size: int, num_heads: int, num_key_heads: int, key_dim: int, value_dim: int, taps: int,
                 norm_eps: float, out_scale: float = 1.0, names: Optional[Dict[str, str]] = None):
        if num_heads <= 0 or num_key_heads <= 0 or num_heads % num_key_heads:
            raise ConfigError(f"delta rule: {num_heads} heads are not a multiple of {num_key_heads} key heads")
        if not 0 < key_dim <= 512 or not 0 < value_dim <= 512 or not 1 <= int(taps) <= 16:
            raise ConfigError(f"delta rule: heads of {key_dim} key and {value_dim} value channels with {taps} taps "
                              "(widths 1..512, 1..16 taps)")
        self.H, self.nh, self.ng, self.d, self.e = int(hidden_size), int(num_heads), int(num_key_heads), int(key_dim), int(value_dim)
        self.taps, self.eps, self.out_scale = int(taps), float(norm_eps), float(out_scale)
        self.names = dict(self.NAMES, **(names or {}))
        self.C = 2 * self.ng * self.d + self.nh * self.e          # convolved channels: q | k | v
        self.state_floats = _floats(K.glr_state_shape(self.nh, self.d, self.e))
        self.w_in = self.w_o = self.conv = self.conv_t = self.a_log = self.dt_bias = self.norm_w = None

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        n, gd, he = self.names, self.ng * self.d, self.nh * self.e
        return [TensorSpec(prefix + n["q"], (gd, self.H)),
                TensorSpec(prefix + n["q_conv"], (gd, self.taps), kind="vector", init="normal"),
                TensorSpec(prefix + n["k"], (gd, self.H)),
                TensorSpec(prefix + n["k_conv"], (gd, self.taps), kind="vector", init="normal"),
                TensorSpec(prefix + n["v"], (he, self.H)),
                TensorSpec(prefix + n["v_conv"], (he, self.taps), kind="vector", init="normal"),
                TensorSpec(prefix + n["b"], (self.nh, self.H)),
                TensorSpec(prefix + n["A_log"], (self.nh,), kind="vector", init="normal"),
                TensorSpec(prefix + n["norm"], (self.e,), kind="vector", init="ones"),
                TensorSpec(prefix + n["a"], (self.nh, self.H)),
                TensorSpec(prefix + n["dt_bias"], (self.nh,), kind="vector", init="normal"),
                TensorSpec(prefix + n["g"], (he, self.H)),
                TensorSpec(prefix + n["o"], (self.H, he))]

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        # one product: q | k | v | b | a | g
        self.w_in = fused_layout([tensors[prefix + n[x]] for x in ("q", "k", "v", "b", "a", "g")], rt)
        self.w_o = stream_layout(tensors[prefix + n["o"]], rt)
        self.conv = rt.own(torch.cat([tensors[prefix + n[x]].to(torch.float32).reshape(-1, self.taps)
                                      for x in ("q_conv", "k_conv", "v_conv")]))
        self.conv_t = rt.own(self.conv.t().contiguous())          # [taps, channels]: four channels a lane where the widths allow
        self.a_log = rt.own(tensors[prefix + n["A_log"]].to(torch.float32).reshape(-1))
        self.dt_bias = rt.own(tensors[prefix + n["dt_bias"]].to(torch.float32).reshape(-1))
        # the head norm's weight for every head, with the mixer's multiplier
        self.norm_w = rt.own((tensors[prefix + n["norm"]].to(torch.float32).reshape(-1) * self.out_scale).repeat(self.nh))

    def state_need(self) -> StateNeed:
        # the heads' states as the scan keeps them, then the convolution's last inputs [taps - 1][channels]
        return StateNeed((self.state_floats + (self.taps - 1) * self.C,), torch.float32)

    def forward(self, h, x, step, ctx: MixerContext) -> None:
        T, nh, ng, d, e, C = step.n_tokens, self.nh, self.ng, self.d, self.e, self.C
        if ctx.state is None:
            raise StepError("delta rule: the cache gave this mixer no state")
        rows = step.ws.get("dr_rows", (T, C + 2 * nh + nh * e), torch.float32)
        linear(h, self.w_in, rows, step.ws)
        q = step.ws.get("dr_q", (T, ng * d), torch.float32)
        k = step.ws.get("dr_k", (T, ng * d), torch.float32)
        v = step.ws.get("dr_v", (T, nh * e), torch.float32)
        gb = step.ws.get("dr_gb", (T, 2 * nh), torch.float32)
        kept = ctx.state[:, self.state_floats:] if self.taps > 1 else None
        K.dr_conv_prepare(rows, self.conv, kept, self.a_log, self.dt_bias, step.seq_of_token, step.cu_seqlens, step.slots,
                          q, k, v, gb, step.n_seqs, ng, nh, d, e, taps_t=self.conv_t)
        o = step.ws.get("dr_o", (T, nh * e), torch.float32)
        S = ctx.state[:, :self.state_floats].view((-1,) + tuple(K.glr_state_shape(nh, d, e)))
        K.dr_scan(q, k, v, gb, None, o, S, step.cu_seqlens, step.slots, step.n_seqs, nh, ng, d, e)
        y = step.ws.get("dr_y", (T, nh * e), self.rt.dtype)
        K.head_norm_gate(o, self.norm_w, rows[:, C + 2 * nh:], y, nh, e, self.eps)
        linear(y, self.w_o, x, step.ws, accumulate=True)


class LightningAttention(Mixer):
    graph_safe = True
    through_linear_only = True

    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "norm": "norm", "o": "o"}
    MIN_PIECE = 128          # tokens: shorter pieces do not pay for the second walk

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, decay: Sequence[float], norm_eps: float,
                 out_scale: float = 1.0, names: Optional[Dict[str, str]] = None, activation: Optional[str] = "silu",
                 position: Optional[str] = None, key_scale: float = 1.0, norm: str = "all", norm_weight: bool = True,
                 gate: str = "sigmoid"):
        if num_heads <= 0 or not 0 < key_dim <= 512 or not 0 < value_dim <= 512:
            raise ConfigError(f"lightning attention: {num_heads} heads of {key_dim} key and {value_dim} value channels "
                              "(all positive, widths at most 512)")
        if activation not in (None, "silu") or norm not in ("all", "head") or gate not in ("sigmoid", "silu"):
            raise ConfigError(f"lightning attention: activation None or 'silu', norm 'all' or 'head', gate 'sigmoid' or 'silu'; "
                              f"got {activation!r}, {norm!r}, {gate!r}")
        if len(decay) != num_heads:
            raise ConfigError(f"lightning attention: {len(decay)} decays for {num_heads} heads")
        self.H, self.nh, self.d, self.e = int(hidden_size), int(num_heads), int(key_dim), int(value_dim)
        self.decay_values = [float(g) for g in decay]
        self.eps, self.out_scale = float(norm_eps), float(out_scale)
        self.names = dict(self.NAMES, **(names or {}))
        self.silu, self.position, self.key_scale = activation == "silu", position, float(key_scale)
        self.norm_per_head, self.norm_weight, self.gate_sigmoid = norm == "head", bool(norm_weight), gate == "sigmoid"
        self._expects_tables = False
        self.w_in = self.w_o = self.decay = self.norm_w = None

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        n, hd, he = self.names, self.nh * self.d, self.nh * self.e
        out = [TensorSpec(prefix + n["q"], (hd, self.H)), TensorSpec(prefix + n["k"], (hd, self.H)),
               TensorSpec(prefix + n["v"], (he, self.H)), TensorSpec(prefix + n["g"], (he, self.H))]
        if self.norm_weight:
            out.append(TensorSpec(prefix + n["norm"], (he,), kind="vector", init="ones"))
        return out + [TensorSpec(prefix + n["o"], (self.H, he))]

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        self.w_in = fused_layout([tensors[prefix + n[x]] for x in ("q", "k", "v", "g")], rt)
        w_o = tensors[prefix + n["o"]]
        if not self.norm_weight and self.out_scale != 1.0:          # no norm weight to carry the multiplier: the matrix does
            w_o = (w_o.to(torch.float32) * self.out_scale).to(w_o.dtype)
        self.w_o = stream_layout(w_o, rt)
        decay = rt.empty((self.nh,), torch.float32)
        decay.copy_(torch.tensor(self.decay_values, dtype=torch.float32))
        self.decay = decay
        if self.norm_weight:
            self.norm_w = rt.own(tensors[prefix + n["norm"]].to(torch.float32).reshape(-1) * self.out_scale)

    def check_positions(self, encodings) -> None:
        if self.position is None:
            return
        enc = encodings.get(self.position)
        if enc is None or getattr(enc, "gives", None) != "rotary":
            raise ConfigError(f"lightning attention asks for the rotary encoding {self.position!r}, the model has {sorted(encodings)}")
        if enc.rotary_dim > self.d or getattr(enc, "pairing", "half") != "half":
            raise ConfigError(f"lightning attention: the encoding {self.position!r} rotates {enc.rotary_dim} elements in "
                              f"{getattr(enc, 'pairing', None)!r} pairs; this mixer takes up to {self.d} in 'half' pairs")
        self._expects_tables = True

    def state_need(self) -> StateNeed:
        return StateNeed(tuple(K.glr_state_shape(self.nh, self.d, self.e)), torch.float32)

    def forward(self, h, x, step, ctx: MixerContext) -> None:
        T, nh, d, e = step.n_tokens, self.nh, self.d, self.e
        if ctx.state is None:
            raise StepError("lightning attention: the cache gave this mixer no state")
        hd, he = nh * d, nh * e
        rows = step.ws.get("la_rows", (T, 2 * hd + 2 * he), torch.float32)
        linear(h, self.w_in, rows, step.ws)
        o = step.ws.get("la_o", (T, he), torch.float32)
        silu = self.silu
        if self._expects_tables or self.key_scale != 1.0:
            # q and k turned by the position and the key scaled, in place on the float sums (behind the activation)
            tables = step.position_data.get(self.position) if self.position else None
            if self._expects_tables and not isinstance(tables, RotaryTables):
                raise StepError(f"lightning attention: the position encoding {self.position!r} gave {type(tables).__name__}, "
                                "rotary tables were expected")
            if silu:
                K.silu_rows(rows[:, :2 * hd + he])
                silu = False
            K.dr_rotate_rows(rows[:, :hd], rows[:, hd:2 * hd], tables.cos if tables else None, tables.sin if tables else None,
                             tables.rotary_dim if tables else 0, nh, d, 1.0, self.key_scale)
        pieces = pieces_for(step, nh * -(-e // 16), self.MIN_PIECE)
        if pieces > 1:
            # long prompts: the recurrence is linear in the state, so every sequence is cut into pieces that are walked
            # side by side, twice
            cu, numbers = HGRN2._piece_arrays(step, pieces)
            piece_state = step.ws.get("la_piece_state", (step.n_seqs * pieces,) + tuple(K.glr_state_shape(nh, d, e)), torch.float32)
            # two walks by many workgroups a head: the activation once, ahead of them
            if silu:
                K.silu_rows(rows[:, :2 * hd + he])
            K.dr_scan_pieces(rows[:, :hd], rows[:, hd:2 * hd], rows[:, 2 * hd:2 * hd + he], self.decay, o, ctx.state, step.slots,
                             cu, numbers, piece_state, step.n_seqs, pieces, nh, d, e, silu=False)
        else:
            K.dr_scan(rows[:, :hd], rows[:, hd:2 * hd], rows[:, 2 * hd:2 * hd + he], None, self.decay, o, ctx.state,
                      step.cu_seqlens, step.slots, step.n_seqs, nh, nh, d, e, silu=silu)
        y = step.ws.get("la_y", (T, he), self.rt.dtype)
        if self.norm_per_head:
            K.head_norm_gate(o, self.norm_w, rows[:, 2 * hd + he:], y, nh, e, self.eps, gate_sigmoid=self.gate_sigmoid)
        else:
            # all heads normed together: one "head" of H e channels
            K.head_norm_gate(o, self.norm_w, rows[:, 2 * hd + he:], y, 1, he, self.eps, gate_sigmoid=self.gate_sigmoid)
        linear(y, self.w_o, x, step.ws, accumulate=True)


register_part("mixer", "gated_delta_rule", GatedDeltaRule, replace=True)
register_part("mixer", "lightning_attention", LightningAttention, replace=True)
