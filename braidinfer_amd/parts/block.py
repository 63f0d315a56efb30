"""Arrangements of a layer's parts.  `prenorm_residual`: x += mixer(norm1(x)), then
x += ffn(norm2(x)) (reference: the per-layer emit order, megakernel/megakernel_compile.rs:115-236,
compile_attention.rs:78-376, compile_layers.rs:373-386).  The parts add into `x`
themselves, so the sum is part of their last projection."""
from __future__ import annotations

from .base import NormedInput, ResidualSink, register_part


def _run_part(part, norm, next_norm, x, step, dtype, *extra) -> None:
    """One residual branch: x += part(norm(x)).  A part that works through `linear` only gets
    the norm unrun (with what the product before prepared for it, if that was this norm and
    these rows) and the residual rows together with the norm that reads them next."""
    prepared, step.prepared_norm = step.prepared_norm, None
    if not part.through_linear_only:
        h = x
        if norm is not None:
            h = step.ws.get("block_h", tuple(x.shape), dtype)
            norm.forward(x, h)
        part.forward(h, x, step, *extra)
        return
    h = x
    if norm is not None:
        mine = prepared[2] if prepared is not None and prepared[0] is norm and prepared[1] is x else None
        h = NormedInput(x, norm, step.ws, dtype, mine)
    sink = ResidualSink(x, next_norm)
    part.forward(h, sink, step, *extra)
    if sink.prepared is not None:
        step.prepared_norm = (next_norm, x, sink.prepared)


def prenorm_residual(layer, x, step, mixer_ctx) -> None:
    after = step.norm_after_layer          # the norm that reads x after this layer, if known
    if layer.mixer is not None:
        nxt = layer.ffn_norm if layer.feed_forward is not None else after
        _run_part(layer.mixer, layer.mixer_norm, nxt, x, step, layer.rt.dtype, mixer_ctx)
    if layer.feed_forward is not None:
        _run_part(layer.feed_forward, layer.ffn_norm, after, x, step, layer.rt.dtype)


register_part("block", "prenorm_residual", lambda: prenorm_residual, replace=True)
