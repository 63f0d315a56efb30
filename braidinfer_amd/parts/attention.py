"""Grouped-query attention over the paged cache.

Per token: q, k, v = W n (no bias; reference compile_attention.rs:82-85 and
model_load.rs:635-670); q and k rotated by the position encoding; k (rotated) and v
stored in the token's page; scores (q . k_j) * scale over the keys the token may see,
softmax in float, weighted sum of v (reference: op_attn_paged,
kernels/megakernel_ops.hip:2150-2343: kv head = q head / (nq / nkv) :2192, scale
rsqrt(head_dim) :2194, causality by loop bound); x += W_o o (compile_attention.rs:333-376).
A window W limits a query at position i to keys i-W < j <= i (absent in the reference,
config.rs:416).
"""
from __future__ import annotations

import math
import warnings
from typing import Dict, List, Optional

import torch

from .. import kernels as K
from ..cache import CacheNeed
from ..errors import ConfigError, StepError
from ..weights import TensorSpec
from .base import Mixer, MixerContext, RotaryTables, Runtime, register_part
from .linear import fused_layout, linear, linear_runs, stream_layout


MAX_HEAD_DIM = 512      # attention_simple's limit; the matrix-core kernels take up to 256 in steps of 16


def decode_splits(batch: int, nkv: int, max_ctx: int, page: int, cus: int = 256) -> int:
    """Into how many runs a sequence's pages are cut for single-token steps: about one
    workgroup per compute unit (measured: more runs cost more in the combine than they gain)
    and at least two pages per run; beyond that, runs of at most 64 pages.  It depends on the
    step's shape only (batch and an upper bound of the context) and on the device's number
    of compute units, never on the tokens."""
    pages = max(1, -(-max_ctx // page))
    want = -(-max(1, cus) // max(1, batch * nkv))
    n = max(1, min(want, pages // 2 if pages >= 2 else 1, 64))
    while n < 64 and pages > 64 * n:
        n *= 2
    return n


class GQAAttention(Mixer):
    graph_safe = True
    through_linear_only = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 window: Optional[int] = None, position: Optional[str] = "rope", scale: Optional[float] = None):
        if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
            raise ConfigError(f"attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if head_dim <= 0 or head_dim % 2:
            raise ConfigError(f"attention: head_dim {head_dim} must be positive and even")
        if head_dim > MAX_HEAD_DIM:
            raise ConfigError(f"attention: head_dim {head_dim} is beyond what any attention kernel of this library "
                              f"takes ({MAX_HEAD_DIM})")
        self.H, self.nq, self.nkv, self.hd = int(hidden_size), int(num_heads), int(num_kv_heads), int(head_dim)
        self.window = None if window is None else int(window)
        self.position = position
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.hd)
        if not self.scale > 0:
            raise ConfigError(f"attention: the score scale must be positive, not {self.scale}")
        self.w_qkv = self.w_o = None
        self._expects_tables = False       # set by check_positions when the model is put together
        self.force_simple = False          # tests set it to run the one-wave-per-query kernel in bf16
        self._told_slow = False            # the notice below is given once per layer

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        return [
            TensorSpec(prefix + "q_proj.weight", (self.nq * self.hd, self.H)),
            TensorSpec(prefix + "k_proj.weight", (self.nkv * self.hd, self.H)),
            TensorSpec(prefix + "v_proj.weight", (self.nkv * self.hd, self.H)),
            TensorSpec(prefix + "o_proj.weight", (self.H, self.nq * self.hd)),
        ]

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        self.w_qkv = fused_layout([tensors[prefix + n + "_proj.weight"] for n in ("q", "k", "v")], rt)
        self.w_o = stream_layout(tensors[prefix + "o_proj.weight"], rt)

    def cache_need(self) -> CacheNeed:
        return CacheNeed(kv_heads=self.nkv, head_dim=self.hd, window=self.window)

    def check_positions(self, encodings) -> None:
        if self.position is None:
            return
        enc = encodings.get(self.position)
        if enc is None:
            raise ConfigError(f"attention asks for the position encoding {self.position!r}, the model has "
                              f"{sorted(encodings)}; name one of them, or None for attention without positions")
        if getattr(enc, "gives", None) not in ("rotary", "embedding", "none"):
            raise ConfigError(f"attention cannot use the position encoding {self.position!r}: it gives "
                              f"{getattr(enc, 'gives', None)!r}, attention rotates with 'rotary' tables or takes "
                              "'embedding' / 'none' encodings, which leave queries and keys alone")
        self._expects_tables = enc.gives == "rotary"

    def forward(self, h, x, step, ctx: MixerContext) -> None:
        T = step.n_tokens
        nq, nkv, hd = self.nq, self.nkv, self.hd
        dt = self.rt.dtype
        qkv = step.ws.get("attn_qkv", (T, (nq + 2 * nkv) * hd), dt)
        tables = step.position_data.get(self.position) if self.position else None
        if (tables is None and self._expects_tables) or (tables is not None and not isinstance(tables, RotaryTables)):
            raise StepError(f"attention: the position encoding {self.position!r} gave {type(tables).__name__}, "
                            "rotary tables were expected")
        if self._fused_decode(qkv, tables, step, ctx):
            # the kernel that rotates and writes the cache itself reads only its own heads of the
            # step's rows: where their product is cut into runs it adds the runs too
            runs = linear_runs(h, self.w_qkv, qkv.shape[1], step.ws)
            if runs is None:
                linear(h, self.w_qkv, qkv, step.ws)
            return self._finish(qkv, x, step, ctx, tables, True, runs)
        linear(h, self.w_qkv, qkv, step.ws)
        K.rope_kv_write(qkv, tables.cos if tables else None, tables.sin if tables else None,
                        step.positions, step.seq_of_token, step.slots, ctx.block_table, ctx.storage,
                        nq, nkv, hd, tables.rotary_dim if tables else 0, tables.adjacent if tables else False,
                        ctx.page_tokens, ctx.writes_cache)
        self._finish(qkv, x, step, ctx, None, False)

    def _fused_decode(self, qkv, tables, step, ctx: MixerContext) -> bool:
        """Single-token steps whose attention kernel also rotates and writes the cache:
        full-head rotation in (p, p + hd / 2) pairs, or none."""
        if not (step.is_decode and qkv.dtype == torch.bfloat16 and not self.force_simple and ctx.storage is not None):
            return False
        if tables is not None and (tables.adjacent or tables.rotary_dim != self.hd):
            return False
        nsplit = decode_splits(step.n_seqs, self.nkv, step.max_ctx_bound, ctx.page_tokens, K.device_cus())
        return K.attention_decode_fuses_rope(self.hd, self.nq, self.nkv, ctx.page_tokens, ctx.block_table.shape[1], nsplit)

    def _finish(self, qkv, x, step, ctx: MixerContext, fused_tables, fused: bool, runs=None) -> None:
        o = step.ws.get("attn_out", (step.n_tokens, self.nq * self.hd), self.rt.dtype)
        self.attend(qkv, o, step, ctx, fused_tables, fused, runs)
        linear(o, self.w_o, x, step.ws, accumulate=True)

    def attend(self, qkv, o, step, ctx: MixerContext, fused_tables=None, fused: bool = False, runs=None) -> None:
        """bf16 with a head size the matrix-core kernels take: split-context kernel when
        every sequence brings one token, flash kernel otherwise.  Else (32-bit path, head
        sizes beyond 256 or not in steps of 16) the one-wave-per-query kernel."""
        T = step.n_tokens
        nq, nkv, hd = self.nq, self.nkv, self.hd
        if qkv.dtype == torch.bfloat16 and hd % 16 == 0 and hd <= 256 and ctx.page_tokens == 64 and not self.force_simple:
            B = step.n_seqs
            if step.is_decode:
                nsplit = decode_splits(B, nkv, step.max_ctx_bound, ctx.page_tokens, K.device_cus())
                part_o = part_ml = None
                if nsplit > 1:
                    part_o = step.ws.get("attn_part_o", (B * nq * nsplit * hd,), torch.float32)
                    part_ml = step.ws.get("attn_part_ml", (B * nq * nsplit * 2,), torch.float32)
                K.attention_decode_bf16(qkv, qkv.stride(0), o, step.slots, step.ctx_lens, ctx.block_table,
                                        ctx.storage, B, nq, nkv, hd, ctx.page_tokens, self.window, self.scale,
                                        nsplit, part_o, part_ml, 0, fused,
                                        fused_tables.cos if fused_tables is not None else None,
                                        fused_tables.sin if fused_tables is not None else None, ctx.writes_cache,
                                        runs.sums if runs is not None else None, runs.runs if runs is not None else 0)
            else:
                K.attention_prefill_bf16(qkv, qkv.stride(0), o, step.cu_seqlens, step.slots, step.ctx_lens,
                                         ctx.block_table, ctx.storage, B, step.max_new, nq, nkv, hd,
                                         ctx.page_tokens, self.window, self.scale)
            return
        if qkv.dtype == torch.bfloat16 and not self.force_simple and not self._told_slow:
            # right, but an order of magnitude slower than the matrix-core kernels: said once, not silently
            self._told_slow = True
            warnings.warn(f"attention: head size {hd} with pages of {ctx.page_tokens} tokens is outside what the "
                          "matrix-core attention kernels take (head sizes in steps of 16 up to 256, pages of 64 "
                          "tokens); the one-wave-per-query kernel runs instead", RuntimeWarning, stacklevel=2)
        K.attention_simple(qkv, qkv.stride(0), o, step.positions, step.seq_of_token, step.slots,
                           ctx.block_table, ctx.storage, T, self.nq, self.nkv, self.hd, ctx.page_tokens,
                           self.window, self.scale)


register_part("mixer", "gqa_attention", GQAAttention, replace=True)
