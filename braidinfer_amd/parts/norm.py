"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w, plain `w` (reference: op_rmsnorm_wx,
kernels/megakernel_ops.hip:862-904; eps default and key in config.rs:249-252)."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels as K
from ..weights import TensorSpec
from .base import Norm, ProductRuns, Runtime, register_part


class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, size: int, eps: float):
        self.size, self.eps = int(size), float(eps)
        self.weight: Optional[torch.Tensor] = None

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        return [TensorSpec(prefix + "weight", (self.size,), kind="vector", init="ones")]

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        self.weight = rt.own(tensors[prefix + "weight"].to(torch.float32))

    def forward(self, x, out, rows=None):
        K.rmsnorm(x, self.weight, out, self.eps, rows)
        return out

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


register_part("norm", "rmsnorm", RMSNorm, replace=True)
