"""Token embedding and output head.

x[t] = float(embed[token[t]]), no scaling (reference: op_embedding,
kernels/megakernel_ops.hip:1757-1768); logits = W_lm n in float, no bias, no soft cap
(op_lm_head, :1783-1835); a tied head uses the embedding tensor itself
(model_load.rs:388-398)."""
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

    def __init__(self, vocab_size: int, hidden_size: int):
        self.V, self.H = int(vocab_size), int(hidden_size)
        self.weight = None

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        return [TensorSpec(prefix + "weight", (self.V, self.H))]

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        self.weight = rt.own(tensors[prefix + "weight"])
        rt.published[prefix + "weight"] = self.weight      # a tied output head reads the same table

    def forward(self, tokens, out) -> None:
        K.embedding(self.weight, tokens, out)


class LMHead(OutputHead):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied_to: Optional[str] = None):
        self.V, self.H, self.tied_to = int(vocab_size), int(hidden_size), tied_to
        self.weight = None

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        return [] if self.tied_to else [TensorSpec(prefix + "weight", (self.V, self.H))]

    def optional_names(self, prefix: str) -> List[str]:
        # a tied checkpoint may still carry a copy of the head
        return [prefix + "weight"] if self.tied_to else []

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
        name = prefix + "weight"
        if name not in tensors:
            raise WeightError(f"output head: tensor {name} is missing", missing=[name])
        self.weight = stream_layout(tensors[name], rt)

    def forward(self, h, out, ws=None) -> None:
        linear(h, self.weight, out, ws)


register_part("embedding", "embedding", TokenEmbedding, replace=True)
register_part("lm_head", "lm_head", LMHead, replace=True)
