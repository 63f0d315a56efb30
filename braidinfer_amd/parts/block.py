"""Arrangements of a layer's parts.  `prenorm_residual`: x += mixer(norm(x)), then
x += feed_forward(norm(x)), with the layer's norms of the roles "mixer" and "feed_forward"
(reference: the per-layer emit order, megakernel/megakernel_compile.rs:115-236,
compile_attention.rs:78-376, compile_layers.rs:373-386).  The parts add into `x`
themselves, so the sum is part of their last projection.

An arrangement is an object with `run(layer, x, step, mixer_ctx)`; it reads whatever roles
of `layer.norms` it likes.  It may also have `first_norm(layer)`: the norm that reads the
residual rows first when the layer runs, which lets the layer before prepare that norm
inside its last product (see `parts.base.ResidualSink`); arrangements without it, and plain
functions `f(layer, x, step, mixer_ctx)`, work the same without that shortcut.  After the
mixer half and after the whole layer it calls `step.probe(name, x)` when the step carries
a probe (names as the reference's tracer, crates/braidinfer-runtime/src/tracer.rs:94-160).
"""
from __future__ import annotations

from .base import NormedInput, ResidualSink, register_part


def run_residual_branch(part, norm, next_norm, x, step, dtype, *extra) -> None:
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


class PrenormResidual:
    def first_norm(self, layer):
        return layer.norms.get("mixer") if layer.mixer is not None else layer.norms.get("feed_forward")

    def run(self, layer, x, step, mixer_ctx) -> None:
        after = step.norm_after_layer          # the norm that reads x after this layer, if known
        ffn_norm = layer.norms.get("feed_forward")
        if layer.mixer is not None:
            nxt = ffn_norm if layer.feed_forward is not None else after
            run_residual_branch(layer.mixer, layer.norms.get("mixer"), nxt, x, step, layer.rt.dtype, mixer_ctx)
        if step.probe is not None:
            step.probe(f"L{step.schedule_index}.post_mixer", x)
        if layer.feed_forward is not None:
            run_residual_branch(layer.feed_forward, ffn_norm, after, x, step, layer.rt.dtype)
        if step.probe is not None:
            step.probe(f"L{step.schedule_index}.post_ffn", x)


register_part("block", "prenorm_residual", PrenormResidual, replace=True)
