"""Rotary position encoding as a part: per step it turns the tokens' positions into
cos/sin tables that any mixer can rotate with.

inv_freq[p] = 1 / theta^(2p / rotary_dim) in float32 and theta = float(pos) * inv_freq[p]
(reference: compute_inv_freq, crates/braidinfer-runtime/src/weights.rs:743-751; op_mrope,
kernels/megakernel_ops.hip:2019-2024).  `pairing` says which elements form a pair:
"adjacent" (2p, 2p+1) as the reference's kernel does (:2025-2030), or "half"
(p, p + rotary_dim/2), the layout of MistralForCausalLM checkpoints.

`scaling` = {factor, original, fast, slow} stretches the encoding beyond the `original` positions a model was
made for: with i(t) = rotary_dim * ln(original / (2 pi t)) / (2 ln theta) the (real-valued) pair whose
wavelength makes t turns over `original` positions, lo = max(floor(i(fast)), 0), hi = min(ceil(i(slow)),
rotary_dim - 1) and ramp_p = clamp((p - lo) / max(hi - lo, 0.001), 0, 1), pair p turns with
inv_freq[p] / factor * ramp_p + inv_freq[p] * (1 - ramp_p) (fast pairs keep their frequency, slow ones are
slowed by `factor`), and cos and sin are multiplied by 0.1 ln(factor) + 1.  The reference has no such scaling.

`scaling` = {factor, original, low, high} (`scaling_rule` "wavelength") is the other common stretch: a pair whose
wavelength l = 2 pi / f is shorter than original / high keeps its frequency, one whose wavelength is longer than
original / low turns with f / factor, and between the two, with s = (original / l - low) / (high - low), with
(1 - s) f / factor + s f; cos and sin are not scaled.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from .. import kernels as K
from ..errors import ConfigError, StepError
from ..weights import TensorSpec
from .base import PositionEncoding, RotaryTables, Runtime, register_part


class RotaryEncoding(PositionEncoding):
    graph_safe = True
    gives = "rotary"

    def __init__(self, rotary_dim: int, theta: float, pairing: str = "half", scaling: Optional[Dict[str, float]] = None,
                 scaling_rule: str = "ramp", frequencies_from_float64: bool = False):
        """`frequencies_from_float64`: the frequencies are worked out in float64 on the host and rounded to float32 once
        (as with any `scaling`), instead of by float32 powers."""
        if rotary_dim <= 0 or rotary_dim % 2:
            raise ConfigError(f"rotary_dim must be positive and even, got {rotary_dim}")
        if pairing not in ("half", "adjacent"):
            raise ConfigError(f"rope pairing must be 'half' or 'adjacent', got {pairing!r}")
        self.rotary_dim, self.theta, self.pairing = int(rotary_dim), float(theta), pairing
        self.scaling = None
        self.magnitude = 1.0
        if scaling_rule not in ("ramp", "wavelength"):
            raise ConfigError(f"rope scaling rule must be 'ramp' or 'wavelength', got {scaling_rule!r}")
        self.scaling_rule = scaling_rule
        self.frequencies_from_float64 = bool(frequencies_from_float64)
        if scaling is not None and scaling_rule == "wavelength":
            try:
                self.scaling = {k: float(scaling[k]) for k in ("factor", "original", "low", "high")}
            except (KeyError, TypeError, ValueError):
                raise ConfigError(f"rope scaling by wavelength needs the numbers factor, original, low and high, got {scaling!r}") from None
            if min(self.scaling.values()) <= 0 or self.theta <= 0 or self.scaling["high"] == self.scaling["low"]:
                raise ConfigError(f"rope scaling by wavelength takes positive numbers with low and high apart, got {scaling!r}")
        elif scaling is not None:
            try:
                self.scaling = {k: float(scaling[k]) for k in ("factor", "original", "fast", "slow")}
            except (KeyError, TypeError, ValueError):
                raise ConfigError(f"rope scaling needs the numbers factor, original, fast and slow, got {scaling!r}") from None
            if min(self.scaling.values()) <= 0 or self.theta <= 1.0:
                raise ConfigError(f"rope scaling takes positive numbers and a base above 1, got {scaling!r} with base {theta}")
            self.magnitude = 0.1 * math.log(self.scaling["factor"]) + 1.0
        self.inv_freq = None

    def frequencies(self):
        """The pairs' frequencies as Python floats (float64 arithmetic; the device keeps their float32 roundings)."""
        n, half = self.rotary_dim, self.rotary_dim // 2
        f = [self.theta ** (-2.0 * p / n) for p in range(half)]
        sc = self.scaling
        if sc is None:
            return f
        if self.scaling_rule == "wavelength":
            out = []
            for fp in f:
                wavelength = 2.0 * math.pi / fp
                if wavelength < sc["original"] / sc["high"]:
                    out.append(fp)
                elif wavelength > sc["original"] / sc["low"]:
                    out.append(fp / sc["factor"])
                else:
                    s = (sc["original"] / wavelength - sc["low"]) / (sc["high"] - sc["low"])
                    out.append((1.0 - s) * fp / sc["factor"] + s * fp)
            return out

        def pair_of(turns):
            return n * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))
        lo = max(math.floor(pair_of(sc["fast"])), 0)
        hi = min(math.ceil(pair_of(sc["slow"])), n - 1)
        out = []
        for p in range(half):
            ramp = min(max((p - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            out.append(f[p] / sc["factor"] * ramp + f[p] * (1.0 - ramp))
        return out

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        if self.scaling is None and not self.frequencies_from_float64:
            expo = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / float(self.rotary_dim)
            inv = 1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float32), expo)
        else:
            inv = torch.tensor(self.frequencies(), dtype=torch.float64)
        self.inv_freq = inv.to(torch.float32).to(rt.device)

    def prepare(self, step) -> RotaryTables:
        if step.position_ids.dim() != 1:
            raise StepError(f"rotary encoding takes one position per token, the step brings {tuple(step.position_ids.shape)}")
        P = self.rotary_dim // 2
        cos = step.ws.get(f"rope_cos_{id(self)}", (step.n_tokens, P), torch.float32)
        sin = step.ws.get(f"rope_sin_{id(self)}", (step.n_tokens, P), torch.float32)
        K.rope_table(step.position_ids, self.inv_freq, cos, sin)
        if self.magnitude != 1.0:
            K.scale_(cos, self.magnitude)
            K.scale_(sin, self.magnitude)
        return RotaryTables(cos, sin, self.rotary_dim, self.pairing == "adjacent")


class NoPositionEncoding(PositionEncoding):
    """Mixers that ask for this encoding rotate nothing."""
    graph_safe = True


    def load(self, tensors, prefix, rt):
        self.rt = rt


class LearnedPositions(PositionEncoding):
    """A learnt vector per position, added to the embeddings (not scaled): x[t] += table[p_t].  The table has `rows`
    positions; a step that reaches beyond it is refused.  `tensor` is the piece of the table's name behind the part's
    prefix.  The mixers see nothing of it (`gives` "embedding")."""
    graph_safe = True
    gives = "embedding"

    def __init__(self, rows: int, hidden_size: int, tensor: str = "weight"):
        self.rows, self.H, self.tensor = int(rows), int(hidden_size), tensor
        self.table = None

    def weight_specs(self, prefix: str):
        return [TensorSpec(prefix + self.tensor, (self.rows, self.H))]

    def load(self, tensors, prefix, rt):
        self.rt = rt
        self.table = rt.own(tensors[prefix + self.tensor])

    def add_to_embedding(self, x, step) -> None:
        if step.position_ids.dim() != 1:
            raise StepError("learnt positions take one position number a token")
        if step.position_ids is step.positions:
            # a recorded single-token step carries no host lengths (its slots read -1): there the kernel adds
            # nothing for a position outside the table
            longest = max((s + n for s, n, slot in zip(step.host_start, step.host_new, step.host_slots) if slot >= 0), default=0)
            if longest > self.rows:
                raise StepError(f"a sequence of {longest} tokens is beyond the model's {self.rows} learnt positions")
        K.add_position_rows(x, self.table, step.position_ids)


register_part("position", "learned", LearnedPositions, replace=True)
register_part("position", "rope", RotaryEncoding, replace=True)
register_part("position", "none", NoPositionEncoding, replace=True)
