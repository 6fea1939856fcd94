"""Token embedding and output head.

x[t] = float(embed[token[t]]) * scale, scale 1 by default (reference: op_embedding,
kernels/megakernel_ops.hip:1757-1768, which has no scale); logits = W_lm n * scale in float, no
bias, no soft cap (op_lm_head, :1783-1835, no scale either); a tied head uses the embedding
tensor itself, without the embedding's scale (model_load.rs:388-398).  `tensor` is the piece of
the table's name behind the part's prefix."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels as K
from ..errors import WeightError
from ..weights import TensorSpec
from .base import Embedding, OutputHead, Runtime, register_part
from .linear import linear, stream_layout


class TokenEmbedding(Embedding):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0, tensor: str = "weight"):
        self.V, self.H, self.scale, self.tensor = int(vocab_size), int(hidden_size), float(scale), tensor
        self.weight = None

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        return [TensorSpec(prefix + self.tensor, (self.V, self.H))]

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        self.weight = rt.own(tensors[prefix + self.tensor])
        rt.published[prefix + self.tensor] = self.weight      # a tied output head reads the same table

    def forward(self, tokens, out) -> None:
        K.embedding(self.weight, tokens, out, self.scale)


class LMHead(OutputHead):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied_to: Optional[str] = None, scale: float = 1.0,
                 tensor: str = "weight"):
        self.V, self.H, self.tied_to, self.scale = int(vocab_size), int(hidden_size), tied_to, float(scale)
        self.tensor = tensor
        self.weight = None

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        return [] if self.tied_to else [TensorSpec(prefix + self.tensor, (self.V, self.H))]

    def optional_names(self, prefix: str) -> List[str]:
        # a tied checkpoint may still carry a copy of the head
        return [prefix + self.tensor] if self.tied_to else []

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        if self.tied_to:                           # a tied table is also read row by row by the embedding
            if self.tied_to in rt.published:
                self.weight = rt.published[self.tied_to]
            elif self.tied_to in tensors:
                self.weight = rt.own(tensors[self.tied_to])
            else:
                raise WeightError(f"output head: tensor {self.tied_to} is missing", missing=[self.tied_to])
            return
        name = prefix + self.tensor
        if name not in tensors:
            raise WeightError(f"output head: tensor {name} is missing", missing=[name])
        self.weight = stream_layout(tensors[name], rt)

    def forward(self, h, out, ws=None) -> None:
        linear(h, self.weight, out, ws)
        if self.scale != 1.0:
            K.scale_(out, self.scale)


register_part("embedding", "embedding", TokenEmbedding, replace=True)
register_part("lm_head", "lm_head", LMHead, replace=True)
