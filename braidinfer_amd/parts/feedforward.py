"""SwiGLU feed-forward: x += W_d (silu(W_g n) * (W_u n)), silu(g) = g / (1 + exp(-g))
(reference: op_ffn_gate_up_wx and op_ffn_down_res, kernels/megakernel_ops.hip:1474-1553,
:1559-1602; the activation is fixed to SiLU there, :1538-1544)."""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import kernels as K
from ..weights import TensorSpec
from .base import FeedForward, NormedInput, Runtime, register_part
from .linear import fused_layout, linear, stream_layout


class SwiGLU(FeedForward):
    graph_safe = True
    through_linear_only = True

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.H, self.I = int(hidden_size), int(intermediate_size)
        self.w_gu = self.w_d = None

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        return [
            TensorSpec(prefix + "gate_proj.weight", (self.I, self.H)),
            TensorSpec(prefix + "up_proj.weight", (self.I, self.H)),
            TensorSpec(prefix + "down_proj.weight", (self.H, self.I)),
        ]

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        g, u = tensors[prefix + "gate_proj.weight"], tensors[prefix + "up_proj.weight"]
        # bf16: gate and up rows interleaved so that the product's epilogue applies silu * up
        # and the [T, 2 I] intermediate is never written
        self.fused = g.dtype == u.dtype == torch.bfloat16 and rt.is_bf16 and self.I % 8 == 0
        self.w_gu = fused_layout([g, u], rt, interleave=self.fused)
        self.w_d = stream_layout(tensors[prefix + "down_proj.weight"], rt)

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


register_part("feed_forward", "swiglu", SwiGLU, replace=True)
