"""SwiGLU feed-forward: x += W_d (silu(W_g n) * (W_u n)), silu(g) = g / (1 + exp(-g))
(reference: op_ffn_gate_up_wx and op_ffn_down_res, kernels/megakernel_ops.hip:1474-1553,
:1559-1602; the activation is fixed to SiLU there, :1538-1544).

Clamped gated unit: with g = min(W_g n + b_g, limit) and u = clamp(W_u n + b_u, -limit, limit),
x += W_d (g sigmoid(alpha g) (u + 1)) + b_d; every projection has a bias, the clamps and the activation work on
the products' float sums.

Routed experts: router scores z = W_r n + b_r in float; a token takes the `top` experts with the largest scores
(ties to the lower number), weighted by the softmax over those scores only (which is also the softmax over all experts divided by the chosen
ones' sum), and x += sum_s share_s expert_s(n)
with an expert W_d (silu(W_g n) * (W_u n)) without biases.  `scoring` "sigmoid" routes otherwise: scores s = sigmoid(z);
the choice is made on s + a learnt correction per expert, among the experts of the best `groups_keep` of `groups`
equal runs of neighbouring experts (a run scores the sum of its two largest corrected scores); the shares are the
chosen experts' s over their sum.  `shared_size` adds a gated unit of that inner width that every token passes.  The
reference has neither."""
from __future__ import annotations

import os
from typing import Dict, List, Optional

import torch

from .. import kernels as K
from ..errors import ConfigError
from ..weights import TensorSpec
from .base import FeedForward, NormedInput, Runtime, register_part
from .linear import fused_layout, linear, stream_layout


class SwiGLU(FeedForward):
    graph_safe = True
    through_linear_only = True

    NAMES = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}

    def __init__(self, hidden_size: int, intermediate_size: int, names: Optional[Dict[str, str]] = None):
        """`names`: the pieces of the three matrices' names behind the part's prefix, for checkpoints
        that call them otherwise than "gate_proj.weight", "up_proj.weight", "down_proj.weight"."""
        self.H, self.I = int(hidden_size), int(intermediate_size)
        self.names = dict(self.NAMES, **(names or {}))
        self.w_gu = self.w_d = None

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        return [
            TensorSpec(prefix + self.names["gate"], (self.I, self.H)),
            TensorSpec(prefix + self.names["up"], (self.I, self.H)),
            TensorSpec(prefix + self.names["down"], (self.H, self.I)),
        ]

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        g, u = tensors[prefix + self.names["gate"]], tensors[prefix + self.names["up"]]
        # bf16: gate and up rows interleaved so that the product's epilogue applies silu * up
        # and the [T, 2 I] intermediate is never written
        self.fused = g.dtype == u.dtype == torch.bfloat16 and rt.is_bf16 and self.I % 8 == 0
        self.w_gu = fused_layout([g, u], rt, interleave=self.fused)
        self.w_d = stream_layout(tensors[prefix + self.names["down"]], rt)

    def forward(self, h, x, step) -> None:
        T = step.n_tokens
        dt = self.rt.dtype
        a = step.ws.get("ffn_act", (T, self.I), dt)
        if self.fused:
            if isinstance(h, NormedInput):
                if h.prepared is not None and h.norm.product_of_prepared(h.prepared, self.w_gu, a, swiglu=True):
                    h = None
                else:
                    h = h.tensor()
            if h is not None:
                scratch = step.ws.get("gemm_scratch", (K.GEMM_SCRATCH_FLOATS,), torch.float32) if 64 < T <= 1024 else None
                K.gemm_swiglu(h, self.w_gu, a, scratch=scratch)
        else:
            gu = step.ws.get("ffn_gu", (T, 2 * self.I), dt)
            linear(h, self.w_gu, gu, step.ws)
            K.silu_mul(gu, a)
        linear(a, self.w_d, x, step.ws, accumulate=True)


class ClampedGLU(FeedForward):
    graph_safe = True

    NAMES = {"gate": "gate", "gate_bias": "gate.b", "up": "up", "up_bias": "up.b", "down": "down", "down_bias": "down.b"}

    def __init__(self, hidden_size: int, intermediate_size: int, limit: float, alpha: float = 1.702,
                 names: Optional[Dict[str, str]] = None):
        self.H, self.I, self.limit, self.alpha = int(hidden_size), int(intermediate_size), float(limit), float(alpha)
        if self.I <= 0 or not self.limit > 0:
            raise ConfigError(f"clamped gated unit: an inner width of {intermediate_size} and a limit of {limit} must be positive")
        self.names = dict(self.NAMES, **(names or {}))
        self.w_gu = self.w_d = self.b_gu = self.b_d = None

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        n = self.names
        return [TensorSpec(prefix + n["gate"], (self.I, self.H)),
                TensorSpec(prefix + n["gate_bias"], (self.I,), kind="vector", init="normal"),
                TensorSpec(prefix + n["up"], (self.I, self.H)),
                TensorSpec(prefix + n["up_bias"], (self.I,), kind="vector", init="normal"),
                TensorSpec(prefix + n["down"], (self.H, self.I)),
                TensorSpec(prefix + n["down_bias"], (self.H,), kind="vector", init="normal")]

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        self.w_gu = fused_layout([tensors[prefix + n["gate"]], tensors[prefix + n["up"]]], rt)
        self.w_d = stream_layout(tensors[prefix + n["down"]], rt)
        self.b_gu = rt.own(torch.cat([tensors[prefix + n[x]].to(torch.float32).reshape(-1) for x in ("gate_bias", "up_bias")]))
        self.b_d = rt.own(tensors[prefix + n["down_bias"]].to(torch.float32).reshape(-1))

    def forward(self, h, x, step) -> None:
        T = step.n_tokens
        gu = step.ws.get("ffn_gu32", (T, 2 * self.I), torch.float32)
        linear(h, self.w_gu, gu, step.ws)
        a = step.ws.get("ffn_act", (T, self.I), self.rt.dtype)
        K.clamped_glu(gu, self.b_gu, a, self.limit, self.alpha)
        linear(a, self.w_d, x, step.ws, accumulate=True)
        K.add_bias_rows(x, self.b_d)


class RoutedExperts(FeedForward):
    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int, top: int, router_bias: bool = True,
                 names: Optional[Dict[str, str]] = None, out_scale: float = 1.0, scoring: str = "softmax",
                 groups: int = 1, groups_keep: int = 1, shared_size: int = 0):
        """`names`: "expert" with {e} for the expert's number (the prefix of its three matrices "gate", "up", "down"),
        "router", "router_bias".  `out_scale` multiplies what is added to the residual rows (it rides on the shares)."""
        self.out_scale = float(out_scale)
        self.H, self.I, self.E, self.top = int(hidden_size), int(intermediate_size), int(num_experts), int(top)
        if self.I <= 0 or not 0 < self.top <= self.E or self.E > 512 or self.top > 64:
            raise ConfigError(f"routed experts: {top} of {num_experts} experts of inner width {intermediate_size} "
                              "(at most 512 experts, 64 chosen)")
        if scoring not in ("softmax", "sigmoid"):
            raise ConfigError(f"routed experts: scoring is 'softmax' or 'sigmoid', got {scoring!r}")
        self.sigmoid = scoring == "sigmoid"
        self.groups, self.groups_keep, self.shared_size = int(groups), int(groups_keep), int(shared_size or 0)
        if self.groups < 1 or self.E % self.groups or (self.groups > 1 and not self.sigmoid) or self.shared_size < 0 or \
                (self.groups > 1 and not (1 <= self.groups_keep <= self.groups and self.groups_keep * (self.E // self.groups) >= self.top)):
            raise ConfigError(f"routed experts: {groups} runs of experts of which {groups_keep} are kept must divide the "
                              f"{num_experts} experts (sigmoid scoring) and leave {top} to choose")
        self.router_bias = bool(router_bias) and not self.sigmoid
        self.names = dict({"expert": "e{e}.", "gate": "gate", "up": "up", "down": "down", "router": "router",
                           "router_bias": "router.b", "correction": "correction", "shared": "shared."}, **(names or {}))
        self.shared = None
        if self.shared_size:
            sh = self.names["shared"]
            self.shared = SwiGLU(self.H, self.shared_size, names={k: sh + self.names[k] for k in ("gate", "up", "down")})
        self.correction = None
        self.w_gu = self.w_down = self.w_router = self.b_router = None

    def _expert(self, prefix: str, e: int, what: str) -> str:
        return prefix + self.names["expert"].format(e=e) + self.names[what]

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        out = []
        for e in range(self.E):
            out += [TensorSpec(self._expert(prefix, e, "gate"), (self.I, self.H)),
                    TensorSpec(self._expert(prefix, e, "up"), (self.I, self.H)),
                    TensorSpec(self._expert(prefix, e, "down"), (self.H, self.I))]
        out.append(TensorSpec(prefix + self.names["router"], (self.E, self.H)))
        if self.router_bias:
            out.append(TensorSpec(prefix + self.names["router_bias"], (self.E,), kind="vector", init="normal"))
        if self.sigmoid:
            out.append(TensorSpec(prefix + self.names["correction"], (self.E,), kind="vector", init="normal"))
        if self.shared is not None:
            out += self.shared.weight_specs(prefix)
        return out

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        first = tensors[self._expert(prefix, 0, "gate")]
        # the experts' matrices stacked, so that a kernel finds expert e's rows by its number: gate rows, then up rows
        self.w_gu = rt.empty((self.E, 2 * self.I, self.H), first.dtype)
        self.w_down = rt.empty((self.E, self.H, self.I), first.dtype)
        for e in range(self.E):
            self.w_gu[e, :self.I].copy_(first if e == 0 else tensors[self._expert(prefix, e, "gate")])
            self.w_gu[e, self.I:].copy_(tensors[self._expert(prefix, e, "up")])
            self.w_down[e].copy_(tensors[self._expert(prefix, e, "down")])
        self.w_router = rt.own(tensors[prefix + self.names["router"]])
        if self.router_bias:
            self.b_router = rt.own(tensors[prefix + self.names["router_bias"]].to(torch.float32).reshape(-1))
        if self.sigmoid:
            self.correction = rt.own(tensors[prefix + self.names["correction"]].to(torch.float32).reshape(-1))
        if self.shared is not None:
            self.shared.load(tensors, prefix, rt)

    # from this many tokens a step goes expert by expert through the matrix products (below it, every (token, slot)
    # pair reads its expert's rows itself, which is what a step of few tokens costs anyway)
    BY_EXPERT_FROM = 48
    ONE_BY_ONE_FROM = 1536          # pairs an expert from which the experts go one by one through the library's products

    def forward(self, h, x, step) -> None:
        T, dt = step.n_tokens, self.rt.dtype
        scores = step.ws.get("moe_scores", (T, self.E), torch.float32)
        linear(h, self.w_router, scores, step.ws)
        chosen = step.ws.get("moe_chosen", (T, self.top), torch.int32)
        share = step.ws.get("moe_share", (T, self.top), torch.float32)
        if self.sigmoid:
            K.route_sigmoid(scores, self.correction, chosen, share, self.top, self.groups, self.groups_keep, self.out_scale)
        else:
            K.route_topk(scores, self.b_router, chosen, share, self.top, self.out_scale)
        if self.shared is not None:
            self.shared.forward(h, x, step)          # every token's: added like the experts' outputs
        few = step.is_decode or T < int(os.environ.get("BRAIDINFER_BY_EXPERT_FROM", str(self.BY_EXPERT_FROM)))
        if few and not K.experts_grouped_takes(dt, self.H, self.I):
            # every pair reads its expert's rows itself: the 32-bit path, and widths the grouped kernels do not take
            y = step.ws.get("moe_y", (T, self.top, self.I), dt)
            K.experts_up(h, self.w_gu, chosen, y)
            K.experts_down(y, self.w_down, chosen, share, x)
            return
        # the pairs sorted by expert on the device
        n = T * self.top
        first = step.ws.get("moe_first", (self.E + 1,), torch.int32)
        order = step.ws.get("moe_order", (n,), torch.int32)
        place = step.ws.get("moe_place", (n,), torch.int32)
        K.experts_sort(chosen, first, order, place, self.E)
        if few:
            # few tokens: an expert's weights are read once for all its pairs, nothing goes back to the host
            y = step.ws.get("moe_y", (n, self.I), dt)
            K.experts_up_grouped(h, self.w_gu, first, order, y, self.top)
            out = step.ws.get("moe_out", (n, self.H), torch.float32)
            K.experts_down_grouped(y, self.w_down, first, out)
            K.experts_combine(out, place, share, x)
            return
        rows = step.ws.get("moe_rows", (n, self.H), dt)
        K.experts_gather(h, order, rows, self.top)
        gu = step.ws.get("moe_gu", (n, 2 * self.I), dt)
        act = step.ws.get("moe_act", (n, self.I), dt)
        out = step.ws.get("moe_out", (n, self.H), torch.float32)
        # Tiles of 128 pairs of one expert, all experts in one launch a product; from about 1,500 pairs an expert the
        # library's own products, expert by expert, make up for their launches (8 layers of width 4,096, 32 experts,
        # 8 chosen: 8,192 tokens 56.9 against 78.7 ms, 2,048 tokens 23.1 against 19.4; BRAIDINFER_EXPERTS_ONE_BY_ONE=0
        # or =1 forces one, for measurements)
        forced = os.environ.get("BRAIDINFER_EXPERTS_ONE_BY_ONE", "")
        one_by_one = forced == "1" or (forced != "0" and n // self.E >= self.ONE_BY_ONE_FROM)
        if K.experts_grouped_takes(dt, self.H, self.I) and not one_by_one:
            K.experts_gemm(rows, self.w_gu, first, gu)
            K.silu_mul(gu, act)
            K.experts_gemm(act, self.w_down, first, out)
        else:
            # the 32-bit path and other widths: expert by expert through the library's products, the experts' row
            # counts read by the host
            starts = first.tolist()
            scratch = step.ws.get("gemm_scratch", (K.GEMM_SCRATCH_FLOATS,), torch.float32) if dt == torch.bfloat16 else None
            for e in range(self.E):
                a, b = starts[e], starts[e + 1]
                if b > a:
                    sc = scratch if 16 < b - a <= 1024 else None          # products that may be cut along k
                    K.gemm(rows[a:b], self.w_gu[e], gu[a:b], scratch=sc)
                    K.silu_mul(gu[a:b], act[a:b])
                    K.gemm(act[a:b], self.w_down[e], out[a:b], scratch=sc)
        K.experts_combine(out, place, share, x)


register_part("feed_forward", "swiglu", SwiGLU, replace=True)
register_part("feed_forward", "clamped_glu", ClampedGLU, replace=True)
register_part("feed_forward", "routed_experts", RoutedExperts, replace=True)
