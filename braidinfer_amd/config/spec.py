"""The architecture-neutral description of a model: which parts, in which order.

A configuration class (one per architecture, read from that architecture's own
config.json keys) is turned into a `ModelSpec` by its architecture's builder.  The
spec is plain data: part kinds are strings looked up in the part registries, sizes
and constants are parameters, and the order in which layers run is a list.  Nothing
below the spec knows which architecture it came from.

The reference drives every architecture from one flat `ModelConfig` with a per-layer
`LayerConfig{layer_type, ffn_type}` list (crates/braidinfer-runtime/src/config.rs:75-115,
:9-37); the `(mixer kind, feed-forward kind)` pair per layer is kept, the flat struct
is not.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass(frozen=True)
class PartSpec:
    """A part by the name it is registered under, and its parameters."""

    kind: str
    params: Dict[str, Any] = field(default_factory=dict)

    def __hash__(self):
        return hash((self.kind, tuple(sorted((k, repr(v)) for k, v in self.params.items()))))


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a mixer, a feed-forward and any number of norms, arranged by `block`.

    `mixer` or `feed_forward` may be None (a layer with only the other half, as the
    reference's `LayerType::Ffn` / `FfnType::None`, config.rs:26-37).  `norms` maps a role
    to a norm; which roles exist is between the architecture's builder and the block
    arrangement it names (`prenorm_residual` reads "mixer" and "feed_forward", the norms in
    front of the two halves; an arrangement with norms behind the halves too would read two
    more roles).  `prefix` is the tensor-name prefix of the layer's weights, e.g.
    ``model.layers.3.``; `names` gives the piece under it for "mixer", "feed_forward" and
    every role of `norms` as "norm.<role>" (the names of the architecture's checkpoints: the
    builder supplies them, nothing here knows any).
    """

    prefix: str
    mixer: Optional[PartSpec] = None
    feed_forward: Optional[PartSpec] = None
    norms: Dict[str, PartSpec] = field(default_factory=dict)
    block: str = "prenorm_residual"
    names: Dict[str, str] = field(default_factory=dict)
    # further mixers of the layer by a role of the architecture's choosing (mixers side by side, say attention
    # and a recurrent one over the same input): built, loaded and given a cache unit and state like `mixer`;
    # the block arrangement the layer names is what runs them (`mixer_ctx.others[role]`).  Their tensor-name
    # pieces are `names["mixer.<role>"]`, their cache units `ScheduleEntry.more_caches[role]`.
    more_mixers: Dict[str, PartSpec] = field(default_factory=dict)

    def name_of(self, what: str) -> str:
        if what not in self.names:
            raise KeyError(f"layer {self.prefix!r}: no tensor-name piece for {what!r} (names: {sorted(self.names)})")
        return self.prefix + self.names[what]


def prenorm_layer(prefix: str, mixer: Optional[PartSpec], feed_forward: Optional[PartSpec],
                  mixer_norm: Optional[PartSpec], ffn_norm: Optional[PartSpec], mixer_name: str,
                  feed_forward_name: str, mixer_norm_name: str, ffn_norm_name: str) -> LayerSpec:
    """The common layer: x += mixer(norm(x)); x += feed_forward(norm(x)), with the four
    tensor-name pieces of the architecture's checkpoints."""
    norms, names = {}, {}
    if mixer is not None:
        if mixer_norm is not None:
            norms["mixer"], names["norm.mixer"] = mixer_norm, mixer_norm_name
        names["mixer"] = mixer_name
    if feed_forward is not None:
        if ffn_norm is not None:
            norms["feed_forward"], names["norm.feed_forward"] = ffn_norm, ffn_norm_name
        names["feed_forward"] = feed_forward_name
    return LayerSpec(prefix=prefix, mixer=mixer, feed_forward=feed_forward, norms=norms, block="prenorm_residual",
                     names=names)


@dataclass(frozen=True)
class ScheduleEntry:
    """One position of the run order.

    `layer` indexes `ModelSpec.layers`; a layer may appear more than once (its weights
    are then shared).  `cache` names the cache unit the mixer works on: entries with
    the same `cache` see the same keys and values.  An entry with `writes_cache=False`
    only reads what another entry wrote earlier in the same step.
    """

    layer: int
    cache: Optional[int] = None
    writes_cache: bool = True
    # cache units of the layer's further mixers, by their role in `LayerSpec.more_mixers`
    more_caches: Dict[str, int] = field(default_factory=dict)


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    layers: List[LayerSpec]
    schedule: List[ScheduleEntry]
    final_norm: PartSpec
    lm_head: PartSpec
    # position encodings by name; mixers refer to them by that name
    positions: Dict[str, PartSpec]
    max_position_embeddings: int
    # tensor-name prefixes of the parts outside the layers, as the architecture's checkpoints name them
    embedding_prefix: str
    final_norm_prefix: str
    lm_head_prefix: str
    stop_token_ids: List[int] = field(default_factory=list)
    bos_token_id: Optional[int] = None


def default_schedule(n_layers: int) -> List[ScheduleEntry]:
    """Every layer once, in order, each with a cache unit of its own."""
    return [ScheduleEntry(layer=i, cache=i) for i in range(n_layers)]
