"""Rotary position encoding as a part: per step it turns the tokens' positions into
cos/sin tables that any mixer can rotate with.

inv_freq[p] = 1 / theta^(2p / rotary_dim) in float32 and theta = float(pos) * inv_freq[p]
(reference: compute_inv_freq, crates/braidinfer-runtime/src/weights.rs:743-751; op_mrope,
kernels/megakernel_ops.hip:2019-2024).  `pairing` says which elements form a pair:
"adjacent" (2p, 2p+1) as the reference's kernel does (:2025-2030), or "half"
(p, p + rotary_dim/2), the layout of MistralForCausalLM checkpoints.
"""
from __future__ import annotations

from typing import Dict

import torch

from .. import kernels as K
from ..errors import ConfigError, StepError
from .base import PositionEncoding, RotaryTables, Runtime, register_part


class RotaryEncoding(PositionEncoding):
    graph_safe = True
    gives = "rotary"

    def __init__(self, rotary_dim: int, theta: float, pairing: str = "half"):
        if rotary_dim <= 0 or rotary_dim % 2:
            raise ConfigError(f"rotary_dim must be positive and even, got {rotary_dim}")
        if pairing not in ("half", "adjacent"):
            raise ConfigError(f"rope pairing must be 'half' or 'adjacent', got {pairing!r}")
        self.rotary_dim, self.theta, self.pairing = int(rotary_dim), float(theta), pairing
        self.inv_freq = None

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        expo = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / float(self.rotary_dim)
        inv = 1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float32), expo)
        self.inv_freq = inv.to(torch.float32).to(rt.device)

    def prepare(self, step) -> RotaryTables:
        if step.position_ids.dim() != 1:
            raise StepError(f"rotary encoding takes one position per token, the step brings {tuple(step.position_ids.shape)}")
        P = self.rotary_dim // 2
        cos = step.ws.get(f"rope_cos_{id(self)}", (step.n_tokens, P), torch.float32)
        sin = step.ws.get(f"rope_sin_{id(self)}", (step.n_tokens, P), torch.float32)
        K.rope_table(step.position_ids, self.inv_freq, cos, sin)
        return RotaryTables(cos, sin, self.rotary_dim, self.pairing == "adjacent")


class NoPositionEncoding(PositionEncoding):
    """Mixers that ask for this encoding rotate nothing."""
    graph_safe = True


    def load(self, tensors, prefix, rt):
        self.rt = rt


register_part("position", "rope", RotaryEncoding, replace=True)
register_part("position", "none", NoPositionEncoding, replace=True)
