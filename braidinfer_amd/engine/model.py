"""A decoder built from a `ModelSpec`: parts by kind, layers by list, run order by list.

The model is the same code for every architecture; what differs is the spec its
architecture's builder returns.  reference: `Model` owns weights, activations, cache
and the compiled program (crates/braidinfer-runtime/src/model/mod.rs:23-119); the
per-layer order is megakernel/megakernel_compile.rs:115-236, the tail (last-row gather,
final norm, lm_head) :238-262 and :521-551.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import torch

from .. import kernels as K
from ..cache import CacheNeed, SequenceCache, StateNeed
from ..config import ModelSpec, spec_of
from ..errors import ConfigError, StepError
from ..parts import MixerContext, Runtime, block_arrangement, build_part
from ..weights import TensorSpec
from .step import StepBatch


class Layer:
    """The parts of one layer; built from a `LayerSpec`."""

    def __init__(self, spec):
        self.spec = spec
        self.mixer = build_part("mixer", spec.mixer) if spec.mixer else None
        # further mixers by role (run by the layer's arrangement, each with a context of its own)
        self.more_mixers: Dict[str, object] = {role: build_part("mixer", ms) for role, ms in spec.more_mixers.items()}
        self.feed_forward = build_part("feed_forward", spec.feed_forward) if spec.feed_forward else None
        self.norms: Dict[str, object] = {role: build_part("norm", ns) for role, ns in spec.norms.items()}
        arrangement = block_arrangement(spec.block)
        # an arrangement is an object with `run` (and optionally `first_norm`), or a plain function
        self.run = getattr(arrangement, "run", arrangement)
        self._first_norm = getattr(arrangement, "first_norm", None)
        self.rt: Optional[Runtime] = None

    # the two norms of the common arrangement, by their roles
    @property
    def mixer_norm(self):
        return self.norms.get("mixer")

    @property
    def ffn_norm(self):
        return self.norms.get("feed_forward")

    def first_norm(self):
        """The norm that reads the residual rows first when this layer runs, if its
        arrangement says."""
        return self._first_norm(self) if self._first_norm is not None else None

    def named_parts(self):
        """(part, tensor-name prefix) in the order of the spec's `names`, which is the order
        of the layer's tensors in the model's name table."""
        s = self.spec
        for what in s.names:
            if what == "mixer":
                part = self.mixer
            elif what == "feed_forward":
                part = self.feed_forward
            elif what.startswith("norm."):
                part = self.norms.get(what[5:])
            elif what.startswith("mixer."):
                part = self.more_mixers.get(what[6:])
            else:
                raise ConfigError(f"layer {s.prefix!r}: names has {what!r}; known: mixer, mixer.<role>, feed_forward, "
                                  "norm.<role>")
            if part is not None:
                yield part, s.name_of(what)
        named = set(s.names)
        missing = [w for w, p in [("mixer", self.mixer), ("feed_forward", self.feed_forward)]
                   + [("norm." + r, n) for r, n in self.norms.items()]
                   + [("mixer." + r, m) for r, m in self.more_mixers.items()] if p is not None and w not in named]
        if missing:
            raise ConfigError(f"layer {s.prefix!r}: no tensor-name piece for {missing}")


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.embedding = build_part("embedding", spec.embedding)
        self.layers: List[Layer] = [Layer(ls) for ls in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm)
        self.lm_head = build_part("lm_head", spec.lm_head)
        self.positions = {name: build_part("position", ps) for name, ps in spec.positions.items()}
        self.schedule = list(spec.schedule)
        for e in self.schedule:
            if not 0 <= e.layer < len(self.layers):
                raise ConfigError(f"schedule names layer {e.layer}, the model has {len(self.layers)}")
        written = set()
        for e in self.schedule:
            if e.cache is not None and self.layers[e.layer].mixer is not None:
                if e.writes_cache:
                    written.add(e.cache)
                elif e.cache not in written:
                    raise ConfigError(f"schedule entry reads cache {e.cache} before any entry writes it")
        for e in self.schedule:
            unknown = sorted(set(e.more_caches) - set(self.layers[e.layer].more_mixers))
            if unknown:
                raise ConfigError(f"schedule entry of layer {e.layer} names cache units for mixers the layer has not: {unknown}")
        for layer in self.layers:
            for m in self._mixers_of(layer).values():
                m.check_positions(self.positions)
        self.rt: Optional[Runtime] = None

    @staticmethod
    def _mixers_of(layer: Layer) -> Dict[Optional[str], object]:
        """The layer's mixers by role; the role of `Layer.mixer` is None."""
        out: Dict[Optional[str], object] = {}
        if layer.mixer is not None:
            out[None] = layer.mixer
        out.update(layer.more_mixers)
        return out

    @staticmethod
    def _unit_of(e, role: Optional[str]) -> Optional[int]:
        return e.cache if role is None else e.more_caches.get(role)

    @staticmethod
    def _state_key(i: int, role: Optional[str]):
        return ("entry", i) if role is None else ("entry", i, role)

    # ---- weights -------------------------------------------------------------------
    def _named_parts(self):
        s = self.spec
        yield self.embedding, s.embedding_prefix
        for layer in self.layers:
            yield from layer.named_parts()
        yield self.final_norm, s.final_norm_prefix
        yield self.lm_head, s.lm_head_prefix
        for name, p in self.positions.items():
            yield p, f"position.{name}."

    def weight_specs(self) -> List[TensorSpec]:
        out: List[TensorSpec] = []
        for part, prefix in self._named_parts():
            out.extend(part.weight_specs(prefix))
        names = [s.name for s in out]
        if len(set(names)) != len(names):
            dup = sorted({n for n in names if names.count(n) > 1})
            raise ConfigError(f"two parts declare the same tensor: {dup}")
        return out

    def optional_names(self) -> List[str]:
        out: List[str] = []
        for part, prefix in self._named_parts():
            f = getattr(part, "optional_names", None)
            if f:
                out.extend(f(prefix))
        return out

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        for part, prefix in self._named_parts():
            part.load(tensors, prefix, rt)
        for layer in self.layers:
            layer.rt = rt

    def graph_safe(self) -> bool:
        """True when every part may run under HIP graph capture (see `Part.graph_safe`)."""
        return all(getattr(part, "graph_safe", False) for part, _ in self._named_parts())

    # ---- what the cache must hold ----------------------------------------------------
    def cache_needs(self) -> Dict[int, CacheNeed]:
        needs: Dict[int, CacheNeed] = {}
        for e in self.schedule:
            for role, m in self._mixers_of(self.layers[e.layer]).items():
                unit = self._unit_of(e, role)
                if unit is None:
                    continue
                n = m.cache_need()
                if n is None:
                    continue
                if unit in needs and needs[unit] != n:
                    raise ConfigError(f"cache unit {unit} is shared by mixers with different needs: "
                                      f"{needs[unit]} and {n}")
                needs[unit] = n
        return needs

    def state_needs(self) -> Dict[object, StateNeed]:
        out: Dict[object, StateNeed] = {}
        for i, e in enumerate(self.schedule):
            for role, m in self._mixers_of(self.layers[e.layer]).items():
                n = m.state_need()
                if n is not None:
                    out[self._state_key(i, role)] = n
        return out

    def _mixer_context(self, cache: SequenceCache, e, i: int, role: Optional[str]) -> MixerContext:
        """What entry i of the run order hands one of its layer's mixers: its cache unit's storage and
        table, and its slice of the state area."""
        unit = self._unit_of(e, role)
        ctx = MixerContext(unit=unit, writes_cache=e.writes_cache)
        if unit is not None and unit in cache.group_of_unit:
            g = cache.unit_group(unit)
            ctx.storage, ctx.block_table, ctx.page_tokens = g.storage_view(unit), g.table_dev, g.page_tokens
            ctx.keys, ctx.values = g.keys(unit), g.values(unit)
        ctx.state = cache.state(self._state_key(i, role))
        return ctx

    # ---- one step ----------------------------------------------------------------------
    def forward(self, step: StepBatch, cache: SequenceCache, want_rows: torch.Tensor, n_want: int,
                logits_out: Optional[torch.Tensor] = None, probe=None) -> torch.Tensor:
        """Run the step's tokens through every scheduled layer; return float32 logits
        `[n_want, vocab]` of the rows `want_rows` (indices into the packed tokens), in
        `logits_out` when given, else in a tensor of their own.

        `probe(name, tensor)`, when given, is called with the residual rows after the
        embedding ("embed"), after each scheduled layer's mixer and feed-forward
        ("L{i}.post_mixer", "L{i}.post_ffn", i the place in the run order), and with the
        normed wanted rows ("final_norm") and the logits ("logits"): the reference's probe
        names (crates/braidinfer-runtime/src/tracer.rs:94-160).  The tensors are the
        step's own buffers: a probe that keeps one copies it."""
        rt = self.rt
        T, H = step.n_tokens, self.spec.hidden_size
        ws = step.ws
        step.probe = probe
        x = ws.get("residual", (T, H), torch.float32)
        self.embedding.forward(step.tokens, x)
        step.position_data = {}
        for name, enc in self.positions.items():
            step.position_data[name] = enc.prepare(step)
            enc.add_to_embedding(x, step)
        if probe is not None:
            probe("embed", x)
        step.prepared_norm = None
        for i, e in enumerate(self.schedule):
            layer = self.layers[e.layer]
            step.schedule_index = i
            # the norm that reads the residual rows after this layer: the next scheduled layer's first
            # (the final norm reads chosen rows only and is left alone)
            step.norm_after_layer = None
            if i + 1 < len(self.schedule):
                step.norm_after_layer = self.layers[self.schedule[i + 1].layer].first_norm()
            ctx = (self._mixer_context(cache, e, i, None) if layer.mixer is not None
                   else MixerContext(unit=e.cache, writes_cache=e.writes_cache))
            for role in layer.more_mixers:
                ctx.others[role] = self._mixer_context(cache, e, i, role)
            layer.run(layer, x, step, ctx)
        if logits_out is None:
            logits = torch.empty((n_want, self.spec.vocab_size), dtype=torch.float32, device=rt.device)
        else:
            logits = logits_out[:n_want]
        if n_want == 0:
            return logits
        hn = ws.get("final_h", (n_want, H), rt.dtype)
        self.final_norm.forward(x, hn, rows=want_rows)
        if probe is not None:
            probe("final_norm", hn)
        self.lm_head.forward(hn, logits, ws)
        if probe is not None:
            probe("logits", logits)
        return logits
