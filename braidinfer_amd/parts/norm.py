"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w, plain `w` (reference: op_rmsnorm_wx,
kernels/megakernel_ops.hip:862-904; eps default and key in config.rs:249-252).  A checkpoint that stores the weight
around zero names an `offset` (w = offset + stored), and a norm whose output is always multiplied by a constant
(a branch's share of a sum, a residual multiplier) names it as `scale`; both are folded into the kept float weight
at load.

LayerNorm: y = (x - mean) / sqrt(var + eps) * w, var the mean of the squared deviations, a weight
and no bias (absent in the reference, whose models norm without centering).

`tensor` is the piece of the weight's name behind the part's prefix ("weight" in the
checkpoints the reference loads; "" where the prefix is the whole name).

`rows`: no norm at all, y = x in the compute dtype, for a half of a layer that reads the residual rows themselves
(a design that norms a half's output only).  It has no weights; a norm that adds behind the half before can leave
these rows in the same kernel, as it would leave a following norm's."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels as K
from ..weights import TensorSpec
from .base import Norm, ProductRuns, Runtime, register_part


class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, size: int, eps: float, tensor: str = "weight", offset: float = 0.0, scale: float = 1.0):
        self.size, self.eps, self.tensor = int(size), float(eps), tensor
        self.offset, self.scale = float(offset), float(scale)
        self.weight: Optional[torch.Tensor] = None

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        return [TensorSpec(prefix + self.tensor, (self.size,), kind="vector", init="ones" if self.offset == 0.0 else "normal")]

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        w = tensors[prefix + self.tensor].to(torch.float32)
        if self.offset != 0.0:
            w = w + self.offset
        if self.scale != 1.0:
            w = w * self.scale
        self.weight = rt.own(w)

    def forward(self, x, out, rows=None):
        K.rmsnorm(x, self.weight, out, self.eps, rows)
        return out

    def then_args(self):
        return self.weight, self.eps, False

    def add_normed(self, y, x, then=None, then_out=None):
        nxt = then.then_args() if then is not None and then_out is not None else None
        K.layernorm(y, self.weight, x, self.eps, center=False, add=True,
                    then=(nxt[0], then_out, nxt[1], nxt[2]) if nxt else None)
        return nxt is not None

    def prepare_in_product(self, a, w, x, ws):
        M, N = x.shape
        if not (a.dtype == w.dtype == torch.bfloat16 and x.dtype == torch.float32 and N == self.size
                and N % (16 if M <= 16 else 256) == 0 and K.gemm_stream_takes(M, a.shape[1])
                and K.gemm_stream_takes(M, N) and a.is_contiguous() and x.is_contiguous()):
            return None
        # 17 to 64 rows: the preparation rides on the sum of a product cut along k
        if M > 16 and K.gemm_wide_parts(M, N, a.shape[1], K.GEMM_SCRATCH_FLOATS) < 2:
            return None
        xg = ws.get("norm_xg", (M, N), torch.bfloat16)
        ssq = ws.get("norm_ssq", ((N // 16) * K.SSQ_LD,), torch.float32)
        scratch = ws.get("gemm_scratch", (K.GEMM_SCRATCH_FLOATS,), torch.float32) if M > 16 else None
        tiles = K.gemm_norm_prepare(a, w, x, self.weight, xg, ssq, scratch)
        return xg, ssq, tiles, scratch

    def product_of_prepared(self, prepared, w, out, swiglu=False):
        xg, ssq, tiles, scratch = prepared
        if w.dtype != torch.bfloat16 or (not swiglu and out.dtype not in (torch.bfloat16, torch.float32)):
            return False
        K.gemm_norm_scaled(xg, ssq, tiles, self.eps, w, out, swiglu=swiglu, scratch=scratch)
        return True

    def runs_of_prepared(self, prepared, w, n_out, ws):
        xg, ssq, tiles, scratch = prepared
        if w.dtype != torch.bfloat16 or scratch is None:
            return None
        runs = K.gemm_wide_partial(xg, w, n_out, scratch, ssq, tiles, self.eps)
        return ProductRuns(scratch, runs, xg.shape[0], n_out) if runs else None


class LayerNorm(Norm):
    """Centered norm with a weight and no bias; statistics in float in both precisions."""

    graph_safe = True

    def __init__(self, size: int, eps: float, tensor: str = "weight"):
        self.size, self.eps, self.tensor = int(size), float(eps), tensor
        self.weight: Optional[torch.Tensor] = None

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        return [TensorSpec(prefix + self.tensor, (self.size,), kind="vector", init="ones")]

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        self.weight = rt.own(tensors[prefix + self.tensor].to(torch.float32))

    def forward(self, x, out, rows=None):
        K.layernorm(x, self.weight, out, self.eps, rows, center=True)
        return out

    def then_args(self):
        return self.weight, self.eps, True

    def add_normed(self, y, x, then=None, then_out=None):
        nxt = then.then_args() if then is not None and then_out is not None else None
        K.layernorm(y, self.weight, x, self.eps, center=True, add=True,
                    then=(nxt[0], then_out, nxt[1], nxt[2]) if nxt else None)
        return nxt is not None


class PlainRows(Norm):
    """The residual rows as they are, in the compute dtype: the "norm" in front of a half that reads the rows themselves."""

    graph_safe = True

    def __init__(self, size: int):
        self.size = int(size)

    def forward(self, x, out, rows=None):
        if rows is not None:
            if out.dtype != x.dtype:
                raise K.KernelError("rows: chosen rows are gathered in float32 only")
            K.gather_rows(x, rows, out)
        elif out.dtype == x.dtype:
            out.copy_(x)
        else:
            K.convert(x, out)
        return out

    def then_args(self):
        return None, 0.0, False          # no weight: the kernel behind another norm leaves the rows as they are


register_part("norm", "rows", PlainRows, replace=True)
register_part("norm", "rmsnorm", RMSNorm, replace=True)
register_part("norm", "layernorm", LayerNorm, replace=True)
