"""The sampler: rows of float logits on the device in, one token per row out, through
the HIP kernels in csrc/sampling.hip.  Order of operations as the reference's `sample`
(crates/braidinfer-runtime/src/sampling.rs:49-171).

`SamplerState` is the sampler of one fixed set of rows over many steps: the rows' options,
their bias lists and their histories (a table of occurrences per token, for the repetition
penalty) live on the device; a step brings only its uniform numbers, and the kernel that draws
a token also adds it to the row's history.  With `random` (each row's seed, request number and
next draw) the uniform numbers are made by that kernel too (`sampling.uniform`, bit for bit), and a
step brings nothing.  `Sampler.sample` is the same for a single call.
"""
from __future__ import annotations

from collections import Counter
from typing import List, Optional, Sequence

import numpy as np
import torch

from .. import kernels as K
from .params import SamplingParams, uniform_key


class SamplerState:
    def __init__(self, device, vocab_size: int, params: Sequence[SamplingParams],
                 histories: Optional[Sequence[Sequence[int]]] = None, random: Optional[Sequence[tuple]] = None):
        """`random[b]` = (seed, request number, next draw) of row b: `launch` without numbers then
        draws with `uniform(seed, request number, draw)` for draw = next draw, next draw + 1, ..."""
        self.device, self.V, self.params = torch.device(device), int(vocab_size), list(params)
        B, V = len(self.params), self.V
        self.B = B
        self.greedy = all(p.is_plain_greedy for p in self.params)
        self.out = torch.empty(B, dtype=torch.int32, device=self.device)
        self.rng_key = self.rng_draw = None
        if self.greedy:
            return
        if random is not None:
            if len(random) != B:
                raise ValueError(f"{len(random)} random states for {B} rows")
            keys = np.array([uniform_key(int(s), int(q)) for s, q, _ in random], dtype=np.uint64)
            self.rng_key = torch.from_numpy(keys.view(np.int64)).to(self.device)
            self.rng_draw = self._i32([int(d) for _, _, d in random])
        # the per-row numbers go over in one copy: four float rows and one int row
        host = np.empty((5, B), dtype=np.float32)
        host[0] = [p.temperature for p in self.params]
        host[1] = [p.repetition_penalty for p in self.params]
        host[2] = [p.min_p for p in self.params]
        host[3] = [p.top_p for p in self.params]
        host[4].view(np.int32)[:] = [p.top_k for p in self.params]
        dev = torch.from_numpy(host).to(self.device)
        self.temperature, self.penalty, self.min_p, self.top_p = dev[0], dev[1], dev[2], dev[3]
        self.top_k = dev[4].view(torch.int32)
        self.bias_off = self.bias_tok = self.bias_val = None
        if any(p.logit_bias for p in self.params):
            off, tok, val = [0], [], []
            for p in self.params:
                for t, d in (p.logit_bias or []):
                    tok.append(int(t))
                    val.append(float(d))
                off.append(len(tok))
            self.bias_off, self.bias_tok = self._i32(off), self._i32(tok or [0])
            self.bias_val = torch.tensor(val or [0.0], dtype=torch.float32).to(self.device)
        self.counts = None
        if any(p.repetition_penalty != 1.0 for p in self.params):
            self.counts = torch.zeros((B, V), dtype=torch.int32, device=self.device)
            rows, toks, cnts = [], [], []
            for b, (p, h) in enumerate(zip(self.params, histories or [[]] * B)):
                if p.repetition_penalty != 1.0:
                    for t, c in Counter(int(t) for t in h).items():
                        rows.append(b)
                        toks.append(t)
                        cnts.append(c)
            if rows:
                K.sample_count_add(self.counts, self._i32(rows), self._i32(toks), self._i32(cnts))
        self.filtered = any(p.temperature != 0.0 and ((0 < p.top_k < V) or p.min_p > 0.0 or p.top_p < 1.0)
                            for p in self.params)
        self.work = torch.empty((B, V), dtype=torch.float32, device=self.device)
        self._make_u()

    def _make_u(self):
        # the step's uniform numbers: two pinned buffers used in turn, so that a step can be
        # launched while the copy of the step before may still be waiting in the stream
        self.u = torch.zeros(self.B, dtype=torch.float32, device=self.device)
        pinned = self.device.type == "cuda"
        self.u_host = [torch.zeros(self.B, dtype=torch.float32, pin_memory=pinned) for _ in range(2)]
        self.u_copied = [None, None]
        self.u_turn = 0

    def _i32(self, v):
        return torch.tensor(v, dtype=torch.int32).to(self.device)

    @property
    def device_random(self) -> bool:
        """Whether `launch` needs no uniform numbers from its caller."""
        return self.greedy or self.rng_key is not None

    def launch(self, logits: torch.Tensor, us: Optional[Sequence[float]] = None) -> torch.Tensor:
        """Enqueue the sampling of one step; returns the device tensor the tokens will stand in
        (int32 [B], overwritten by the next launch).  `us[b]` is row b's uniform number in [0, 1);
        without `us` a state made with `random` draws its own (one draw per row and call)."""
        B, V = logits.shape
        assert V == self.V and B == self.B
        if self.greedy:
            K.argmax(logits, self.out)
            return self.out
        if us is not None:
            k = self.u_turn
            self.u_turn ^= 1
            if self.u_copied[k] is not None:
                self.u_copied[k].synchronize()
            self.u_host[k].numpy()[:] = us
            self.u.copy_(self.u_host[k], non_blocking=True)
            if self.device.type == "cuda":
                if self.u_copied[k] is None:
                    self.u_copied[k] = torch.cuda.Event()
                self.u_copied[k].record()
        K.sample_prepare(logits, self.work, self.bias_off, self.bias_tok, self.bias_val, self.counts, self.penalty,
                         self.temperature)
        if self.filtered:
            K.sample_filter(self.work, self.top_k, self.min_p, self.top_p, self.temperature)
        if us is None and self.rng_key is not None:
            K.sample_draw(self.work, self.out, self.temperature, None, self.counts, self.rng_key, self.rng_draw)
        else:
            K.sample_draw(self.work, self.out, self.temperature, self.u, self.counts)
        return self.out

    def sample(self, logits: torch.Tensor, us: Optional[Sequence[float]] = None) -> List[int]:
        return self.launch(logits, us).tolist()

    def keep(self, rows: Sequence[int]) -> "SamplerState":
        """The state of a subset of the rows (those that go on), in the given order; histories
        stay on the device."""
        st = SamplerState.__new__(SamplerState)
        st.device, st.V, st.params = self.device, self.V, [self.params[r] for r in rows]
        st.B, st.greedy = len(rows), self.greedy
        st.out = torch.empty(st.B, dtype=torch.int32, device=self.device)
        st.rng_key = st.rng_draw = None
        if self.greedy:
            return st
        idx = torch.tensor(list(rows), dtype=torch.long, device=self.device)
        pick = lambda t: t.index_select(0, idx)
        if self.rng_key is not None:
            st.rng_key, st.rng_draw = pick(self.rng_key), pick(self.rng_draw)
        st.temperature, st.penalty, st.min_p, st.top_p, st.top_k = (pick(t) for t in (
            self.temperature, self.penalty, self.min_p, self.top_p, self.top_k))
        st.bias_off = st.bias_tok = st.bias_val = None
        if self.bias_off is not None:
            off = self.bias_off.tolist()
            tok, val = self.bias_tok.tolist(), self.bias_val.tolist()
            noff, ntok, nval = [0], [], []
            for r in rows:
                ntok += tok[off[r]:off[r + 1]]
                nval += val[off[r]:off[r + 1]]
                noff.append(len(ntok))
            st.bias_off, st.bias_tok = st._i32(noff), st._i32(ntok or [0])
            st.bias_val = torch.tensor(nval or [0.0], dtype=torch.float32).to(self.device)
        st.counts = pick(self.counts) if self.counts is not None else None
        V = self.V
        flt = lambda p: p.temperature != 0.0 and ((0 < p.top_k < V) or p.min_p > 0.0 or p.top_p < 1.0)
        st.filtered = any(flt(p) for p in st.params)
        st.work = self.work[:st.B]
        st._make_u()
        return st


class Sampler:
    takes_random = True        # `state` accepts `random`: the generation loop then sends no numbers per step

    def __init__(self, device, vocab_size: int):
        self.device = torch.device(device)
        self.V = int(vocab_size)

    def argmax(self, logits: torch.Tensor) -> torch.Tensor:
        out = torch.empty(logits.shape[0], dtype=torch.int32, device=self.device)
        K.argmax(logits, out)
        return out

    def state(self, params: Sequence[SamplingParams], histories: Optional[Sequence[Sequence[int]]] = None,
              random: Optional[Sequence[tuple]] = None) -> SamplerState:
        """The resident sampler of these rows: `state.sample(logits, us)` step after step, or with
        `random` (see `SamplerState`) `state.sample(logits)`."""
        return SamplerState(self.device, self.V, params, histories, random)

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams],
               histories: Optional[Sequence[Sequence[int]]] = None,
               us: Optional[Sequence[float]] = None) -> List[int]:
        """One token per row.  `histories[b]` is the sequence so far (for the repetition
        penalty), `us[b]` the row's uniform number in [0, 1)."""
        B, V = logits.shape
        assert V == self.V and len(params) == B
        return self.state(params, histories).sample(logits, us if us is not None else [0.0] * B)
