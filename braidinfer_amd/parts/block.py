"""Arrangements of a layer's parts.  `prenorm_residual`: x += mixer(norm1(x)), then
x += ffn(norm2(x)) (reference: the per-layer emit order, megakernel/megakernel_compile.rs:115-236,
compile_attention.rs:78-376, compile_layers.rs:373-386).  The parts add into `x`
themselves, so the sum is part of their last projection."""
from __future__ import annotations

from .base import register_part


def prenorm_residual(layer, x, step, mixer_ctx) -> None:
    T, H = x.shape
    if layer.mixer is not None:
        h = step.ws.get("block_h", (T, H), layer.rt.dtype)
        if layer.mixer_norm is not None:
            layer.mixer_norm.forward(x, h)
        else:
            h = x
        layer.mixer.forward(h, x, step, mixer_ctx)
    if layer.feed_forward is not None:
        h = step.ws.get("block_h", (T, H), layer.rt.dtype)
        if layer.ffn_norm is not None:
            layer.ffn_norm.forward(x, h)
        else:
            h = x
        layer.feed_forward.forward(h, x, step)


register_part("block", "prenorm_residual", lambda: prenorm_residual, replace=True)
