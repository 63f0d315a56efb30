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

from collections import deque

from .. import kernels as K
from ..errors import StepError
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

    def __init__(self, model, cache, device, batch: int, position_numbers: int = 0):
        """`position_numbers` k > 0: the step's position encodings read k numbers per token that the
        caller brings with every step (`StepEntry.position_ids`), kept in the same refreshed array;
        0: they read the tokens' places in their sequences."""
        self.B = B = batch
        self.k = k = int(position_numbers)
        dev = device
        self.ws = Workspace(dev)            # its buffers belong to the recorded graph for good
        # one int32 array: tokens | positions | slots | ctx | the caller's position numbers   (refreshed per step)
        self.ints = torch.zeros((4 + k) * B, dtype=torch.int32, device=dev)
        self.ints[2 * B:3 * B] = -1
        ar = torch.arange(B + 1, dtype=torch.int32, device=dev)
        self.want_rows = ar[:B].contiguous()
        pid = None
        if k:
            pid = self.ints[4 * B:(4 + k) * B]
            pid = pid if k == 1 else pid.view(B, k)
        self.step = StepBatch(
            n_tokens=B, n_seqs=B, tokens=self.ints[0:B], positions=self.ints[B:2 * B],
            seq_of_token=self.want_rows, cu_seqlens=ar, slots=self.ints[2 * B:3 * B],
            ctx_lens=self.ints[3 * B:4 * B], host_slots=[-1] * B, host_new=[1] * B, host_start=[0] * B,
            is_decode=True, max_new=1, max_ctx=cache.max_seq_len,
            max_ctx_bound=cache.max_seq_len, ws=self.ws, position_ids=pid)
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
        self.model, self.cache, self.device = model, cache, dev
        # the step's arrays on the host, pinned, so that the copy to the device does not wait
        # (two, used in turn: a buffer is written again only when its last copy has been made)
        self.host_ints = [torch.zeros((4 + k) * B, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self.host_copied = [None, None]
        self.host_turn = 0
        self.greedy_graph = None
        self.next_tokens = torch.zeros(B, dtype=torch.int32, device=dev)
        self.owner = None                # the chain whose sequences the device arrays describe, if any

    def load(self, slots: Sequence[int], tokens: Sequence[int], starts: Sequence[int], position_ids=None) -> None:
        """Write the step's arrays: tokens, positions, slots and lengths of the n live rows,
        padding rows behind them; `position_ids` [n, k] for a graph recorded with k position numbers."""
        B, n = self.B, len(slots)
        turn = self.host_turn
        self.host_turn ^= 1
        if self.host_copied[turn] is not None:
            self.host_copied[turn].synchronize()
        h = self.host_ints[turn].numpy()
        h[0:n] = tokens
        h[B:B + n] = starts
        h[2 * B:2 * B + n] = slots
        h[3 * B:3 * B + n] = starts
        h[3 * B:3 * B + n] += 1
        if n < B:
            h[n:B] = 0
            h[B + n:2 * B] = 0
            h[2 * B + n:3 * B] = -1
            h[3 * B + n:4 * B] = 0
        if self.k:
            pid = h[4 * B:].reshape(B, self.k)
            pid[:n] = position_ids
            pid[n:] = 0
        self.ints.copy_(self.host_ints[turn], non_blocking=True)
        if self.host_copied[turn] is None:
            self.host_copied[turn] = torch.cuda.Event()
        self.host_copied[turn].record()

    def run(self, slots: Sequence[int], tokens: Sequence[int], starts: Sequence[int], position_ids=None) -> torch.Tensor:
        self.owner = None
        self.load(slots, tokens, starts, position_ids)
        self.graph.replay()
        return self.logits[:len(slots)]

    def run_greedy(self) -> None:
        """One more step of the rows the arrays describe: the recorded step, the argmax of
        every row into `next_tokens`, and the arrays moved on by that token, all on the
        device (recorded as a second graph over the same buffers when first asked for)."""
        if self.greedy_graph is None:
            torch.cuda.synchronize(self.device)
            saved = self.ints.clone()
            # once eagerly, so that the kernel is loaded before the capture begins (nothing may be
            # loaded under capture); the arrays it moves on are put back below
            K.argmax_advance(self.logits, self.next_tokens, self.step.tokens, self.step.positions,
                             self.step.slots, self.step.ctx_lens)
            torch.cuda.synchronize(self.device)
            self.ints.copy_(saved)
            g = torch.cuda.CUDAGraph()
            gc_was_on = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(g):
                    self.model.forward(self.step, self.cache, self.want_rows, self.B, self.logits)
                    K.argmax_advance(self.logits, self.next_tokens, self.step.tokens, self.step.positions,
                                     self.step.slots, self.step.ctx_lens)
            finally:
                if gc_was_on:
                    gc.enable()
            torch.cuda.synchronize(self.device)
            self.ints.copy_(saved)       # recording runs nothing, but keep the arrays as they were in any case
            self.greedy_graph = g
        self.greedy_graph.replay()


class DecodeGraphs:
    """The graphs of one engine, by batch size bucket."""

    def __init__(self, model, cache, device, max_batch: int = 256):
        self.model, self.cache, self.device = model, cache, device
        self.max_batch = max_batch
        self.graphs: Dict[int, DecodeGraph] = {}          # plain steps, by bucket
        self.with_ids: Dict[tuple, DecodeGraph] = {}      # steps that bring k position numbers, by (bucket, k)

    def of(self, n: int, position_numbers: int = 0) -> DecodeGraph:
        b = bucket_of(n)
        if position_numbers:
            g = self.with_ids.get((b, position_numbers))
            if g is None:
                g = self.with_ids[(b, position_numbers)] = DecodeGraph(self.model, self.cache, self.device, b, position_numbers)
            return g
        g = self.graphs.get(b)
        if g is None:
            g = self.graphs[b] = DecodeGraph(self.model, self.cache, self.device, b)
        return g

    def run(self, slots, tokens, starts) -> torch.Tensor:
        return self.of(len(slots)).run(slots, tokens, starts)


class DecodeChain:
    """Single-token steps of one fixed set of sequences with the host out of the way: a
    step's tokens go into the next step's input on the device, so a step can be launched
    before the tokens of the one before have been read.  `launch` runs one step for every
    sequence (reserving cache pages first, as `Engine.step` does); `read` returns the tokens of
    the oldest launched step that has not been read.  At most two steps may be unread.

    Without a sampler state the tokens are the argmax of each row, taken inside the recorded
    step.  With one (`sampling.SamplerState` of these rows, in the order of `slots`) the recorded
    step is followed by the state's kernels and by one that moves the step's arrays on by the
    drawn tokens; `launch(us)` then brings the step's uniform numbers.

    The chain owns the recorded step of its batch size until it is closed or any other
    single-token step of that size runs, after which `launch` refuses."""

    def __init__(self, graphs: DecodeGraphs, cache, slots: Sequence[int], tokens: Sequence[int], sampler_state=None):
        if not slots or len(slots) != len(tokens) or len(set(slots)) != len(slots):
            raise StepError("a chain needs one token for each of its distinct slots")
        if sampler_state is not None and sampler_state.B != len(slots):
            raise StepError(f"a sampler state of {sampler_state.B} rows for a chain of {len(slots)} sequences")
        self.state = sampler_state
        self.cache, self.slots, self.n = cache, list(slots), len(slots)
        for s in self.slots:
            cache.slots.check_live(s)
        self.g = graphs.of(self.n)
        self.g.load(self.slots, list(tokens), [cache.lengths[s] for s in self.slots])
        self.g.owner = self
        self.ones = [1] * self.n
        self.host = [torch.zeros(self.g.B, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self.turn = 0
        self.pending = deque()

    def _run(self, us) -> torch.Tensor:
        g, n = self.g, self.n
        if self.state is None:
            g.run_greedy()
            return g.next_tokens[:n]
        g.graph.replay()
        drawn = self.state.launch(g.logits[:n], us)
        K.step_advance(drawn, g.step.tokens, g.step.positions, g.step.slots, g.step.ctx_lens, n)
        return drawn

    def launch(self, us: Sequence[float] = None) -> None:
        if self.g.owner is not self:
            raise StepError("this chain's recorded step has been used by another step since; open a new chain")
        if len(self.pending) >= 2:
            raise StepError("two launched steps are unread; read one first")
        held = self.cache.pages_held(self.slots)
        self.cache.reserve(self.slots, self.ones)
        try:
            drawn = self._run(us)
        except BaseException:
            self.cache.release_reserved(self.slots, held)
            raise
        self.cache.commit(self.slots, self.ones)
        buf = self.host[self.turn]
        self.turn ^= 1
        buf[:self.n].copy_(drawn, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self.pending.append((ev, buf))

    def read(self) -> List[int]:
        if not self.pending:
            raise StepError("no launched step is unread")
        ev, buf = self.pending.popleft()
        ev.synchronize()
        return buf[:self.n].tolist()

    def close(self) -> None:
        """Wait for what was launched and give the recorded step back."""
        while self.pending:
            self.pending.popleft()[0].synchronize()
        if self.g.owner is self:
            self.g.owner = None

