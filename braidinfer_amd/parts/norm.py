"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w, plain `w` (reference: op_rmsnorm_wx,
kernels/megakernel_ops.hip:862-904; eps default and key in config.rs:249-252)."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels as K
from ..weights import TensorSpec
from .base import Norm, Runtime, register_part


class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, size: int, eps: float):
        self.size, self.eps = int(size), float(eps)
        self.weight: Optional[torch.Tensor] = None

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        return [TensorSpec(prefix + "weight", (self.size,), kind="vector", init="ones")]

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        self.weight = tensors[prefix + "weight"].to(torch.float32).contiguous()

    def forward(self, x, out, rows=None):
        K.rmsnorm(x, self.weight, out, self.eps, rows)
        return out


register_part("norm", "rmsnorm", RMSNorm, replace=True)
