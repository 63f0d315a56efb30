"""Interfaces of the parts a model is put together from, and their registries.

A part is built from the parameters of its `PartSpec` alone; it never sees the model's
configuration or name.  Kinds:

* `Norm`             x[T, H] float32 -> activations [T, H] in the compute dtype
* `PositionEncoding` per step: `prepare(step)`; offers rotary tables and/or an addition
                     to the embeddings
* `Mixer`            adds its output to the residual stream; declares what it keeps per
                     sequence: a `CacheNeed` (growing keys/values) and/or a `StateNeed`
                     (fixed size)
* `FeedForward`      adds its output to the residual stream
* block arrangements functions that run one layer's parts in order

Tensors: the residual stream `x` is float32 `[T, hidden]` in both precisions; `h` is the
normed input in the compute dtype (`runtime.dtype`).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional

import torch

from ..cache import CacheNeed, StateNeed
from ..errors import ConfigError
from ..weights import TensorSpec


@dataclass
class Runtime:
    """Where and in which precision a model runs, and where its parts keep their weights.

    `arena`: when set (anything with `empty(shape, dtype)` and `holds(tensor)`, e.g.
    `weights.WeightArena`), `empty` and `own` place what a part keeps inside it, so a
    loaded model is one device allocation.  `published`: tensors a part offers to parts
    loaded after it, by tensor name (a tied output head finds the embedding table there)."""

    device: torch.device
    dtype: torch.dtype            # torch.float32 (true 32-bit path) or torch.bfloat16
    arena: Any = None
    published: Dict[str, torch.Tensor] = field(default_factory=dict)

    @property
    def is_bf16(self) -> bool:
        return self.dtype == torch.bfloat16

    def empty(self, shape, dtype: torch.dtype) -> torch.Tensor:
        """Uninitialised memory for a tensor the part keeps."""
        if self.arena is not None:
            return self.arena.empty(shape, dtype)
        return torch.empty(tuple(shape), dtype=dtype, device=self.device)

    def own(self, t: torch.Tensor) -> torch.Tensor:
        """`t` as the part keeps it: dense, on the device, inside the arena when there is one
        (a copy unless it already is all that)."""
        if t.device == self.device and t.is_contiguous() and (self.arena is None or self.arena.holds(t)):
            return t
        out = self.empty(t.shape, t.dtype)
        out.copy_(t)
        return out


class Part:
    """Base of every part: declares tensors by name, receives them once loaded.

    `graph_safe`: the part's forward launches the same kernels with the same arguments
    for every step of one shape and reads everything that varies from device arrays of
    the step, so a single-token step may be captured in a HIP graph and replayed.  Parts
    that decide anything on the host from the step's contents leave it False."""

    graph_safe = False
    # A mixer or feed-forward that reads its input and adds to the residual stream only
    # through `parts.linear.linear` sets this.  It may then be handed a `NormedInput`
    # instead of the normed rows and a `ResidualSink` instead of the residual tensor, which
    # lets the product that adds into the stream prepare the norm that reads it next.
    through_linear_only = False

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        return []

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt


class Norm(Part):
    def forward(self, x: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError

    def prepare_in_product(self, a: torch.Tensor, w: torch.Tensor, x: torch.Tensor, ws) -> Any:
        """x += a @ w^T with this norm of the new x prepared in the same kernel, if the norm
        has such a kernel for these sizes and types: returns what `product_of_prepared`
        takes, or None with nothing done."""
        return None

    def product_of_prepared(self, prepared: Any, w: torch.Tensor, out: torch.Tensor, swiglu: bool = False) -> bool:
        """out = norm(x) @ w^T from what `prepare_in_product` left; False with nothing done
        if there is no kernel for these sizes."""
        return False


    def runs_of_prepared(self, prepared: Any, w: torch.Tensor, n_out: int, ws) -> Optional["ProductRuns"]:
        """norm(x) @ w^T from what `prepare_in_product` left, as the float sums of its runs
        along k (see `ProductRuns`); None with nothing done if the product is not cut so."""
        return None


@dataclass
class ProductRuns:
    """A product [rows, width] left as the float sums of `runs` runs along k, matrix after
    matrix in `sums`; its bfloat16 value is the rounded sum of the runs in run order.  A kernel
    that needs only a few of the product's elements adds them itself and saves the launch
    that would."""

    sums: torch.Tensor
    runs: int
    rows: int
    width: int


class ResidualSink:
    """The residual rows as a part that adds to them sees them, with the norm that reads them
    next.  `linear(a, w, sink, ws, accumulate=True)` adds the product and, where the norm
    can, leaves its preparation in `prepared`."""

    def __init__(self, x: torch.Tensor, next_norm: Optional["Norm"]):
        self.x, self.next_norm, self.prepared = x, next_norm, None


class NormedInput:
    """The input of a mixer or feed-forward before its norm has run: the residual rows, the
    norm, and what the product before may have prepared for it.  `linear(h, w, out, ws)`
    multiplies the normed rows with a matrix, from the preparation where there is one;
    `tensor` norms into a buffer (once) for everything else."""

    def __init__(self, x: torch.Tensor, norm: "Norm", ws, dtype: torch.dtype, prepared: Any = None):
        self.x, self.norm, self.ws, self.dtype, self.prepared = x, norm, ws, dtype, prepared
        self._tensor: Optional[torch.Tensor] = None

    def tensor(self) -> torch.Tensor:
        if self._tensor is None:
            self._tensor = self.ws.get("block_h", tuple(self.x.shape), self.dtype)
            self.norm.forward(self.x, self._tensor)
        return self._tensor


class PositionEncoding(Part):
    # what the encoding gives the mixers that name it: "rotary" (`prepare` returns
    # `RotaryTables`), "embedding" (it acts on the embeddings only) or "none"
    gives = "none"

    def prepare(self, step) -> Any:
        """Called once per step before the layers, with the step's `position_ids` (int32 [T],
        or [T, k] when the caller gives k numbers per token); the result is kept in
        `step.position_data[name]` for the mixers."""
        return None

    def add_to_embedding(self, x: torch.Tensor, step) -> None:
        """Encodings that act on the embeddings override this."""


@dataclass
class RotaryTables:
    """cos/sin [T, rotary_dim/2] float32 for the step's tokens."""

    cos: torch.Tensor
    sin: torch.Tensor
    rotary_dim: int
    adjacent: bool


class Mixer(Part):
    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def check_positions(self, encodings: Dict[str, "PositionEncoding"]) -> None:
        """Called once when the model is put together, with its position encodings by name:
        a mixer that asks for one raises `ConfigError` here if it is absent or of a kind the
        mixer cannot use, instead of running without positions later."""

    def state_need(self) -> Optional[StateNeed]:
        return None

    def forward(self, h: torch.Tensor, x: torch.Tensor, step, ctx: "MixerContext") -> None:
        """Add the mixer's output for the step's tokens to `x` in place."""
        raise NotImplementedError


@dataclass
class MixerContext:
    """What one schedule entry hands its mixer: its cache unit and state, if it asked."""

    unit: Optional[int] = None
    storage: Optional[torch.Tensor] = None        # [pages, 2, kv_heads, page_tokens, head_dim] (equal key and value widths)
    keys: Optional[torch.Tensor] = None           # [pages, kv_heads, page_tokens * key width], a view of the same memory
    values: Optional[torch.Tensor] = None         # [pages, kv_heads, page_tokens * value width]
    block_table: Optional[torch.Tensor] = None    # int32 [slots, pages per sequence], device
    page_tokens: int = 0
    writes_cache: bool = True
    state: Optional[torch.Tensor] = None          # [slots, *StateNeed.shape]
    # the contexts of the layer's further mixers (`LayerSpec.more_mixers`), by role
    others: Dict[str, "MixerContext"] = field(default_factory=dict)


class FeedForward(Part):
    def forward(self, h: torch.Tensor, x: torch.Tensor, step) -> None:
        """Add the feed-forward's output for the step's tokens to `x` in place."""
        raise NotImplementedError


class Embedding(Part):
    def forward(self, tokens: torch.Tensor, out: torch.Tensor) -> None:
        raise NotImplementedError


class OutputHead(Part):
    def forward(self, h: torch.Tensor, out: torch.Tensor) -> None:
        raise NotImplementedError


# ------------------------------------------------------------------ registries ------
_REGISTRIES: Dict[str, Dict[str, Callable[..., Any]]] = {
    "norm": {}, "position": {}, "mixer": {}, "feed_forward": {}, "embedding": {}, "lm_head": {}, "block": {},
}


def register_part(category: str, kind: str, factory: Callable[..., Any], replace: bool = False) -> None:
    """`factory(**params)` builds the part (for "block": the arrangement function)."""
    if category not in _REGISTRIES:
        raise ConfigError(f"unknown part category {category!r}; known: {sorted(_REGISTRIES)}")
    if kind in _REGISTRIES[category] and not replace:
        raise ConfigError(f"{category} {kind!r} is already registered")
    _REGISTRIES[category][kind] = factory


def unregister_part(category: str, kind: str) -> None:
    _REGISTRIES[category].pop(kind, None)


def build_part(category: str, spec) -> Any:
    reg = _REGISTRIES[category]
    if spec.kind not in reg:
        raise ConfigError(f"unknown {category} {spec.kind!r}; registered: {sorted(reg)}")
    return reg[spec.kind](**spec.params)


def block_arrangement(kind: str):
    reg = _REGISTRIES["block"]
    if kind not in reg:
        raise ConfigError(f"unknown block arrangement {kind!r}; registered: {sorted(reg)}")
    return reg[kind]()


def registered_parts(category: str) -> List[str]:
    return sorted(_REGISTRIES[category])
