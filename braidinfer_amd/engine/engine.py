"""The engine: a loaded model, its cache, and the one step function.

reference: `Model::prefill(&[u32]) -> logits of the last token` and
`Model::decode_step(token, position) -> logits` for the one sequence a `Model` holds
(crates/braidinfer-runtime/src/model/state.rs:39-206, model/mod.rs:279-286).  Here one
`step` serves a batch: every entry brings the next tokens of its sequence, and logits
come back for the places asked for.
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Union

import numpy as np
import torch

from .. import kernels as K
from ..cache import SequenceCache
from ..config import config_from_folder, generation_stop_tokens, spec_of
from ..errors import BraidError, CacheError, ConfigError, KernelError, StepError
from ..parts import Runtime
from ..weights import FolderTensors, RandomTensors, write_model_folder
from .model import DecoderModel
from .step import StepBatch, Workspace, pack_step

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def parse_dtype(dtype) -> torch.dtype:
    if dtype not in _DTYPES:
        raise ConfigError(f"dtype {dtype!r} is not supported; use 'bfloat16' or 'float32'")
    return _DTYPES[dtype]


@dataclass
class StepEntry:
    """The next tokens of one sequence, and the places among them whose logits are wanted."""

    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = ()
    # position numbers for the position encodings, one integer or k integers per token; None: the
    # tokens' places in the sequence.  All entries of a step give them, or none does.
    position_ids: Optional[Sequence] = None


def _require_gpu(device: torch.device) -> None:
    if device.type != "cuda":
        raise KernelError(f"the engine runs on a GPU only (asked for {device}); there is no CPU path")
    if not torch.cuda.is_available():
        raise KernelError("no GPU is visible to this process; the engine has no CPU path")


class Engine:
    def __init__(self, config, model: DecoderModel, rt: Runtime, max_tokens: int,
                 max_seq_len: Optional[int] = None, n_slots: Optional[int] = None, use_graphs: bool = True):
        self.config = config
        self.model = model
        self.spec = model.spec
        self.rt = rt
        self.device = rt.device
        self.ws = Workspace(rt.device)
        if max_seq_len is None:
            # the block tables are [slots, pages of the longest sequence]: the longest sequence is
            # what the cache holds, but no longer than the positions the model was made for
            # (a caller who wants more says so with max_seq_len)
            max_seq_len = min(max(int(max_tokens), 64), int(model.spec.max_position_embeddings))
        self.cache = SequenceCache(model.cache_needs(), model.state_needs(), max_tokens=max_tokens,
                                   max_seq_len=max_seq_len, n_slots=n_slots, dtype=rt.dtype, device=rt.device)
        self.vocab_size = self.spec.vocab_size
        # single-token steps are replayed from HIP graphs when every part allows it
        self.use_graphs = bool(use_graphs) and model.graph_safe()
        self._graphs = None
        self.load_profile = None
        # tokens that end a sequence: the configuration's, and for a folder also its generation_config.json's
        self.stop_token_ids: List[int] = list(self.spec.stop_token_ids)

    # ---- construction ------------------------------------------------------------------
    @classmethod
    def _from_source(cls, config, make_source, dtype, device, max_tokens, max_seq_len, n_slots, use_graphs) -> "Engine":
        """Build the model of `config`, size one arena for what its parts keep, and let the
        parts pull their tensors from the source `make_source(specs, allowed, device, dtype)` makes."""
        from ..weights import WeightArena
        device = torch.device(device)
        _require_gpu(device)
        model = DecoderModel(spec_of(config))
        rt = Runtime(device=device, dtype=parse_dtype(dtype))
        source = make_source(model.weight_specs(), model.optional_names(), device, rt.dtype)
        rt.arena = WeightArena(device, source.resident_bytes())
        model.load(source, rt)
        profile = source.finish(rt.arena)
        eng = cls(config, model, rt, max_tokens, max_seq_len, n_slots, use_graphs)
        eng.load_profile = profile
        return eng

    @classmethod
    def from_folder(cls, folder: str, dtype="bfloat16", device="cuda:0", max_tokens: int = 8192,
                    max_seq_len: Optional[int] = None, n_slots: Optional[int] = None,
                    use_graphs: bool = True) -> "Engine":
        """A model folder (config.json and model.safetensors, or shards with their index).
        `engine.load_profile.line()` says how the load went (the reference prints a
        `LOAD PROFILE` line, bin/generate.rs:62-68)."""
        config = config_from_folder(folder)
        more_stops = generation_stop_tokens(folder)
        eng = cls._from_source(config, lambda specs, allowed, dev, dt: FolderTensors(folder, specs, dev, dt, allowed),
                               dtype, device, max_tokens, max_seq_len, n_slots, use_graphs)
        eng.stop_token_ids += [t for t in more_stops if t not in eng.stop_token_ids]
        return eng

    @classmethod
    def random(cls, config, seed: int = 0, dtype="bfloat16", device="cuda:0", max_tokens: int = 8192,
               max_seq_len: Optional[int] = None, n_slots: Optional[int] = None, std: float = 0.02,
               use_graphs: bool = True, vector_jitter: float = 0.0) -> "Engine":
        """Seeded random weights made on the device (no folder): the same bits a
        random-weights folder of that configuration, seed and std holds (bfloat16 N(0, std)
        matrices, norm weights 1), widened for the 32-bit path."""
        return cls._from_source(config, lambda specs, allowed, dev, dt: RandomTensors(specs, seed, dev, dt, std, vector_jitter),
                                dtype, device, max_tokens, max_seq_len, n_slots, use_graphs)

    @staticmethod
    def write_random_folder(folder: str, config, seed: int = 0, std: float = 0.02,
                            vector_jitter: float = 0.0, device="cpu", shard_bytes: Optional[int] = None) -> str:
        """Random-weights mode: a model folder (config.json, model.safetensors; with
        `shard_bytes` several files and their index).  `device` is where the values are
        made: the bits are the same everywhere, a GPU is faster for large shapes."""
        model = DecoderModel(spec_of(config))
        return write_model_folder(folder, config, model.weight_specs(), seed, std, vector_jitter, device=device,
                                  shard_bytes=shard_bytes)

    # ---- slots -----------------------------------------------------------------------
    def alloc_slot(self) -> int:
        return self.cache.alloc_slot()

    def free_slot(self, slot: int) -> None:
        self.cache.free_slot(slot)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    # ---- the step function -------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry], probe=None) -> torch.Tensor:
        """Run the given tokens of each entry's sequence as one batch, from the cache
        earlier steps left; return float32 logits `[number of wanted places, vocab]` on the
        device, in the order of the entries and of each entry's `want`, in a tensor of
        their own (later steps do not touch it).

        `probe(name, tensor)` is handed to the model (see `DecoderModel.forward`); a probed
        step runs its kernels one by one, never from a recorded graph.

        Nothing is changed if the step cannot be run (bad entry, no room in the cache, a size
        no kernel takes): the sequences keep their lengths and pages taken for the step go back."""
        if not entries:
            raise StepError("a step needs at least one entry")
        slots = [e.slot for e in entries]
        token_lists = [list(e.tokens) for e in entries]
        V = self.vocab_size
        rows: List[int] = []
        base = 0
        for e, tl in zip(entries, token_lists):
            if not tl:
                raise StepError(f"slot {e.slot}: an entry brings no tokens")
            try:
                arr = np.asarray(tl)
            except (ValueError, TypeError):
                arr = np.asarray([], dtype=object)
            if arr.ndim != 1 or arr.dtype.kind not in "iu" or int(arr.min()) < 0 or int(arr.max()) >= V:
                bad = next((t for t in tl if not isinstance(t, (int, np.integer)) or isinstance(t, bool)
                            or not 0 <= t < V), None)
                raise StepError(f"slot {e.slot}: token {bad!r} is outside the vocabulary of {V}")
            for w in e.want:
                if not isinstance(w, (int, np.integer)) or isinstance(w, bool) or not 0 <= w < len(tl):
                    raise StepError(f"slot {e.slot}: wanted place {w!r} is outside its {len(tl)} tokens")
                rows.append(base + int(w))
            base += len(tl)
        with_ids = [e.position_ids is not None for e in entries]
        if any(with_ids) and not all(with_ids):
            raise StepError("position_ids: given for some entries of the step and not for others")
        position_ids = None
        if all(with_ids):
            position_ids = [e.position_ids for e in entries]
            for e, tl in zip(entries, token_lists):
                if len(e.position_ids) != len(tl):
                    raise StepError(f"slot {e.slot}: {len(e.position_ids)} position numbers for {len(tl)} tokens")
        new = [len(tl) for tl in token_lists]
        held = self.cache.pages_held(slots)
        self.cache.reserve(slots, new)          # all or nothing
        try:
            starts = [self.cache.lengths[s] for s in slots]
            n_want = len(rows)
            if self.use_graphs and probe is None and all(n == 1 for n in new) and len(slots) <= 256:
                if self._graphs is None:
                    from .graph import DecodeGraphs
                    self._graphs = DecodeGraphs(self.model, self.cache, self.device)
                pid = None
                if position_ids is not None:
                    # the caller's position numbers, k per token: a recorded step of their own per k
                    try:
                        pid = np.asarray([p[0] for p in position_ids], dtype=np.int64).reshape(len(slots), -1)
                    except (ValueError, TypeError):
                        pid = np.zeros((len(slots), 0), dtype=np.int64)
                    if pid.shape[1] == 0 or np.abs(pid).max() >= 2 ** 31:
                        raise StepError("position_ids: every token needs the same number of position numbers, each a 32-bit integer")
                g = self._graphs.of(len(slots), 0 if pid is None else pid.shape[1])
                all_logits = g.run(slots, [tl[0] for tl in token_lists], starts, pid)
                # the graph's buffer is overwritten by the next step: the wanted rows go into a tensor
                # of the caller's own (one copy kernel; nothing wanted: nothing copied)
                logits = torch.empty((n_want, V), dtype=torch.float32, device=self.device)
                if n_want:
                    which = (g.want_rows[:n_want] if rows == list(range(n_want))
                             else torch.tensor(rows, dtype=torch.int32).to(self.device))
                    K.gather_rows(all_logits, which, logits)
            else:
                try:
                    step = pack_step(slots, token_lists, starts, self.device, self.ws, position_ids=position_ids)
                except ValueError as e:
                    raise StepError(str(e)) from None
                want_rows = (torch.tensor(rows, dtype=torch.int32).to(self.device) if n_want
                             else torch.empty(0, dtype=torch.int32, device=self.device))
                logits = self.model.forward(step, self.cache, want_rows, n_want, probe=probe)
        except BaseException:
            self.cache.release_reserved(slots, held)
            raise
        self.cache.commit(slots, new)
        return logits

    def chain(self, slots: Sequence[int], tokens: Sequence[int], sampler_state=None):
        """A `DecodeChain` over these sequences, each with the token it takes next, or None when
        single-token steps of this engine are not replayed from graphs (then `step` and the
        sampler do the same work one step at a time).  Without `sampler_state` the chain is greedy;
        with one (`Sampler.state` of these rows, in this order) it draws through that state."""
        if not self.use_graphs or len(slots) > 256:
            return None
        V = self.vocab_size
        for t in tokens:
            if not isinstance(t, (int, np.integer)) or isinstance(t, bool) or not 0 <= t < V:
                raise StepError(f"token {t!r} is outside the vocabulary of {V}")
        if self._graphs is None:
            from .graph import DecodeGraphs
            self._graphs = DecodeGraphs(self.model, self.cache, self.device)
        from .graph import DecodeChain
        return DecodeChain(self._graphs, self.cache, slots, tokens, sampler_state)

    # ---- generation (the Python entry point) -----------------------------------------------
    def generate(self, prompts, max_new_tokens: int = 64, temperature: float = 0.0, seed=None,
                 stop_token_ids=None, top_k: int = 0, top_p: float = 1.0, min_p: float = 0.0,
                 repetition_penalty: float = 1.0, logit_bias=None, include_stop: bool = False,
                 max_batch=None, return_stats: bool = False):
        """Token ids in, generated token ids out: `prompts` is one list of ids or a list of
        such lists.  Sampling options carry the reference's names (sampling.rs:7-19);
        temperature 0 is greedy.  Returns the new tokens of each prompt (and the
        throughput statistics with `return_stats`)."""
        from ..sampling import SamplingParams
        from .generate import generate as _generate
        single = bool(prompts) and isinstance(prompts[0], int)
        plist = [list(prompts)] if single else [list(p) for p in prompts]
        params = SamplingParams(temperature=temperature, top_k=top_k, top_p=top_p,
                                repetition_penalty=repetition_penalty, seed=seed, min_p=min_p,
                                logit_bias=logit_bias)
        results, stats = _generate(self, plist, params, max_new_tokens, stop_token_ids, include_stop, max_batch)
        toks = [r.tokens for r in results]
        out = toks[0] if single else toks
        return (out, stats) if return_stats else out
