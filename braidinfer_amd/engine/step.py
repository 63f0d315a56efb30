"""What one step hands to the parts: the packed tokens of a batch and where they sit.

A step runs the tokens it is given, as one batch: `n_i >= 1` new tokens for each of B
sequences, packed one after another.  All arrays are int32 on the device; the same
numbers are kept as Python lists for host-side decisions.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch


class Workspace:
    """Named scratch buffers that grow and are reused from step to step."""

    def __init__(self, device):
        self.device = torch.device(device)
        self._bufs: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}

    def get(self, name: str, shape, dtype: torch.dtype) -> torch.Tensor:
        n = 1
        for s in shape:
            n *= int(s)
        key = (name, dtype)
        buf = self._bufs.get(key)
        if buf is None or buf.numel() < n:
            buf = torch.empty(max(n, 1), dtype=dtype, device=self.device)
            self._bufs[key] = buf
        return buf[:n].view(tuple(int(s) for s in shape))

    def clear(self) -> None:
        self._bufs.clear()


@dataclass
class StepBatch:
    n_tokens: int                    # T: tokens in this step (padding included)
    n_seqs: int                      # B: sequences (padding included)
    tokens: torch.Tensor             # [T] token ids
    positions: torch.Tensor          # [T] place of each token in its sequence (its index in the cache)
    seq_of_token: torch.Tensor       # [T] index into the batch
    cu_seqlens: torch.Tensor         # [B + 1] offsets of the sequences' tokens
    slots: torch.Tensor              # [B] cache slot of each sequence, -1 = padding
    ctx_lens: torch.Tensor           # [B] length of each sequence after this step
    # the same on the host
    host_slots: List[int] = field(default_factory=list)
    host_new: List[int] = field(default_factory=list)       # n_i
    host_start: List[int] = field(default_factory=list)     # length before the step
    is_decode: bool = False          # every sequence brings exactly one token
    max_new: int = 0
    max_ctx: int = 0
    max_ctx_bound: int = 0           # an upper bound of max_ctx that kernels may size their grids by
    ws: Optional[Workspace] = None
    position_data: Dict[str, Any] = field(default_factory=dict)
    # between the parts of a step: the norm that reads the residual rows after the running layer, and
    # what the last product into the rows prepared for a norm, as (norm, rows, preparation)
    norm_after_layer: Any = None
    prepared_norm: Any = None
    extras: Dict[str, Any] = field(default_factory=dict)     # per-step scratch of parts (keyed by them)
    # what the position encodings read: [T], the same tensor as `positions` unless the caller gave
    # position numbers of its own, which may be k per token: [T, k]
    position_ids: Optional[torch.Tensor] = None
    probe: Any = None                # probe(name, tensor) of the running step, or None
    schedule_index: int = 0          # place in the run order of the layer that is running

    def __post_init__(self):
        if self.position_ids is None:
            self.position_ids = self.positions


def pack_step(slots: Sequence[int], token_lists: Sequence[Sequence[int]], starts: Sequence[int],
              device, ws: Workspace, pad_seqs: int = 0, position_ids: Optional[Sequence] = None) -> StepBatch:
    """Build the device arrays of a step in one host-to-device copy.  `pad_seqs` extra
    sequences of one dummy token (slot -1, position 0) may follow the real ones.
    `position_ids`: per sequence the position numbers of its tokens for the position
    encodings, one integer or k integers per token (the same k for all); None: each token's
    place in its sequence."""
    B = len(slots) + pad_seqs
    new = [len(t) for t in token_lists] + [1] * pad_seqs
    T = sum(new)
    all_slots = list(slots) + [-1] * pad_seqs
    all_starts = list(starts) + [0] * pad_seqs
    new_a = np.asarray(new, dtype=np.int64)
    starts_a = np.asarray(all_starts, dtype=np.int64)
    cu = np.zeros(B + 1, dtype=np.int64)
    np.cumsum(new_a, out=cu[1:])
    sot = np.repeat(np.arange(B, dtype=np.int64), new_a)
    pos = np.arange(T, dtype=np.int64) - cu[sot] + starts_a[sot]
    toks = np.concatenate([np.asarray(t, dtype=np.int64) for t in token_lists] + [np.zeros(pad_seqs, dtype=np.int64)])
    ctx = np.where(np.asarray(all_slots) >= 0, starts_a + new_a, 0)
    pid = np.zeros(0, dtype=np.int64)
    k = 0
    if position_ids is not None:
        rows = [np.asarray(p, dtype=np.int64).reshape(len(t), -1) for p, t in zip(position_ids, token_lists)]
        k = rows[0].shape[1]
        if any(r.shape[1] != k for r in rows) or k == 0:
            raise ValueError("position_ids: every token needs the same number of position numbers")
        pid = np.concatenate(rows + [np.zeros((pad_seqs, k), dtype=np.int64)]).reshape(-1)
    # layout of the one int32 staging array: tokens | positions | seq_of_token | cu | slots | ctx | position ids
    flat = np.concatenate([toks, pos, sot, cu, np.asarray(all_slots, dtype=np.int64), ctx, pid]).astype(np.int32)
    dev = torch.from_numpy(flat).to(device)
    o = 0

    def take(n):
        nonlocal o
        v = dev[o:o + n]
        o += n
        return v
    tokens, positions, seq_of_token = take(T), take(T), take(T)
    cu_seqlens, slots_d, ctx_d = take(B + 1), take(B), take(B)
    pid_d = None
    if k:
        pid_d = take(T * k)
        pid_d = pid_d if k == 1 else pid_d.view(T, k)
    max_ctx = int(ctx.max()) if B else 0
    return StepBatch(
        n_tokens=T, n_seqs=B, tokens=tokens, positions=positions, seq_of_token=seq_of_token,
        cu_seqlens=cu_seqlens, slots=slots_d, ctx_lens=ctx_d, host_slots=all_slots, host_new=new,
        host_start=all_starts, is_decode=all(n == 1 for n in new), max_new=max(new) if new else 0,
        max_ctx=max_ctx, max_ctx_bound=max_ctx, ws=ws, position_ids=pid_d)
