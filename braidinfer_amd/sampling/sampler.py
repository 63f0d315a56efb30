"""The sampler: rows of float logits on the device in, one token per row out, through
the HIP kernels in csrc/sampling.hip.  Order of operations as the reference's `sample`
(crates/braidinfer-runtime/src/sampling.rs:49-171)."""
from __future__ import annotations

from collections import Counter
from typing import List, Optional, Sequence

import numpy as np
import torch

from .. import kernels as K
from .params import SamplingParams


class Sampler:
    def __init__(self, device, vocab_size: int):
        self.device = torch.device(device)
        self.V = int(vocab_size)
        self._keys = None          # scratch for whole-row sorts, made when first needed

    def _i32(self, v):
        return torch.tensor(v, dtype=torch.int32).to(self.device)

    def _f32(self, v):
        return torch.tensor(v, dtype=torch.float32).to(self.device)

    def argmax(self, logits: torch.Tensor) -> torch.Tensor:
        out = torch.empty(logits.shape[0], dtype=torch.int32, device=self.device)
        K.argmax(logits, out)
        return out

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams],
               histories: Optional[Sequence[Sequence[int]]] = None,
               us: Optional[Sequence[float]] = None) -> List[int]:
        """One token per row.  `histories[b]` is the sequence so far (for the repetition
        penalty), `us[b]` the row's uniform number in [0, 1)."""
        B, V = logits.shape
        assert V == self.V and len(params) == B
        if all(p.is_plain_greedy for p in params):
            return self.argmax(logits).tolist()
        histories = histories if histories is not None else [[] for _ in range(B)]
        us = us if us is not None else [0.0] * B
        work = torch.empty_like(logits)
        bias_off = bias_tok = bias_val = None
        if any(p.logit_bias for p in params):
            off, tok, val = [0], [], []
            for p in params:
                for t, d in (p.logit_bias or []):
                    tok.append(int(t))
                    val.append(float(d))
                off.append(len(tok))
            bias_off, bias_tok, bias_val = self._i32(off), self._i32(tok or [0]), self._f32(val or [0.0])
        hist_off = hist_tok = hist_cnt = None
        if any(p.repetition_penalty != 1.0 for p in params):
            off, tok, cnt = [0], [], []
            for p, h in zip(params, histories):
                if p.repetition_penalty != 1.0:
                    for t, c in Counter(int(t) for t in h).items():
                        tok.append(t)
                        cnt.append(c)
                off.append(len(tok))
            hist_off, hist_tok, hist_cnt = self._i32(off), self._i32(tok or [0]), self._i32(cnt or [0])
        # the per-row numbers go over in one copy: five float rows and one int row
        host = np.empty((6, B), dtype=np.float32)
        host[0] = [p.temperature for p in params]
        host[1] = [p.repetition_penalty for p in params]
        host[2] = [p.min_p for p in params]
        host[3] = [p.top_p for p in params]
        host[4] = list(us)
        host[5].view(np.int32)[:] = [p.top_k for p in params]
        dev = torch.from_numpy(host).to(self.device)
        temperature, penalty, min_p, top_p, u = dev[0], dev[1], dev[2], dev[3], dev[4]
        top_k = dev[5].view(torch.int32)
        K.sample_prepare(logits, work, bias_off, bias_tok, bias_val, hist_off, hist_tok, hist_cnt, penalty, temperature)
        filtered = [p for p in params if p.temperature != 0.0 and ((0 < p.top_k < V) or p.min_p > 0.0 or p.top_p < 1.0)]
        if filtered:
            # rows that the short-list kernel may hand on need room for a sort of the whole row
            keys = None
            if any(p.top_k > K.FILTER_CANDIDATES or (not 0 < p.top_k < V and p.top_p < 1.0) for p in filtered):
                n2 = 1 << (V - 1).bit_length()
                if self._keys is None or self._keys.shape[0] < B:
                    self._keys = torch.empty((B, n2), dtype=torch.int64, device=self.device)
                keys = self._keys
            slow = torch.empty(B, dtype=torch.int32, device=self.device)
            K.sample_filter(work, top_k, min_p, top_p, temperature, slow, keys)
        out = torch.empty(B, dtype=torch.int32, device=self.device)
        K.sample_draw(work, out, temperature, u)
        return out.tolist()
