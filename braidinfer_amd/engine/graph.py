"""Single-token steps as HIP graphs: the launches of a decode step are the same for
every step of one batch size, so they are recorded once per size and replayed, which
takes the per-launch host work out of the inner loop.

Everything that varies from step to step (tokens, positions, slots, lengths, block
tables) lives in device arrays that are refreshed before a replay; kernels take their
grids from the batch size and from the cache's longest sequence, never from a step's
contents.  Batch sizes are rounded up to a power of two with padding sequences (slot -1),
which store nothing and whose rows are dropped.  No hipMemset is recorded: nothing in a
step clears memory.
"""
from __future__ import annotations

import gc
from typing import Dict, List, Sequence

import torch

from .step import StepBatch, Workspace


def bucket_of(n: int) -> int:
    b = 1
    while b < n:
        b <<= 1
    return b


class DecodeGraph:
    """One recorded step of `batch` sequences.  It refers to the model and the cache, not
    to the engine that owns it: an engine dropped by its user is then freed at once by
    reference counting, never by the cycle collector at an arbitrary later moment (which
    may be another graph's capture, where destroying a graph or freeing device memory is
    not permitted)."""

    def __init__(self, model, cache, device, batch: int):
        self.B = B = batch
        dev = device
        self.ws = Workspace(dev)            # its buffers belong to the recorded graph for good
        # one int32 array: tokens | positions | slots | ctx   (refreshed per step)
        self.ints = torch.zeros(4 * B, dtype=torch.int32, device=dev)
        self.ints[2 * B:3 * B] = -1
        ar = torch.arange(B + 1, dtype=torch.int32, device=dev)
        self.want_rows = ar[:B].contiguous()
        self.step = StepBatch(
            n_tokens=B, n_seqs=B, tokens=self.ints[0:B], positions=self.ints[B:2 * B],
            seq_of_token=self.want_rows, cu_seqlens=ar, slots=self.ints[2 * B:3 * B],
            ctx_lens=self.ints[3 * B:4 * B], host_slots=[-1] * B, host_new=[1] * B, host_start=[0] * B,
            is_decode=True, max_new=1, max_ctx=cache.max_seq_len,
            max_ctx_bound=cache.max_seq_len, ws=self.ws)
        # once eagerly with padding only: loads the kernels, sizes the workspace, stores nothing
        self.logits = torch.empty((B, model.spec.vocab_size), dtype=torch.float32, device=dev)
        model.forward(self.step, cache, self.want_rows, B, self.logits)
        torch.cuda.synchronize(dev)
        self.graph = torch.cuda.CUDAGraph()
        # no garbage collection while the stream is capturing: a collected tensor or graph
        # would call into the runtime in the middle of the capture
        gc_was_on = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(self.graph):
                model.forward(self.step, cache, self.want_rows, B, self.logits)
        finally:
            if gc_was_on:
                gc.enable()
        torch.cuda.synchronize(dev)

    def run(self, slots: Sequence[int], tokens: Sequence[int], starts: Sequence[int]) -> torch.Tensor:
        B, n = self.B, len(slots)
        pad = B - n
        host = (list(tokens) + [0] * pad + list(starts) + [0] * pad + list(slots) + [-1] * pad
                + [s + 1 for s in starts] + [0] * pad)
        self.ints.copy_(torch.tensor(host, dtype=torch.int32))
        self.graph.replay()
        return self.logits[:n]


class DecodeGraphs:
    """The graphs of one engine, by batch size bucket."""

    def __init__(self, model, cache, device, max_batch: int = 256):
        self.model, self.cache, self.device = model, cache, device
        self.max_batch = max_batch
        self.graphs: Dict[int, DecodeGraph] = {}

    def run(self, slots, tokens, starts) -> torch.Tensor:
        b = bucket_of(len(slots))
        g = self.graphs.get(b)
        if g is None:
            g = self.graphs[b] = DecodeGraph(self.model, self.cache, self.device, b)
        return g.run(slots, tokens, starts)
