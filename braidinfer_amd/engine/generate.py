"""The generation loop above the step function: batches of unequal prompts, stop tokens,
sequences that end earlier, and as many batches one after another as there are requests.

reference: `generate_from_ids` (crates/braidinfer-runtime/src/generate.rs:314-439) for
one sequence: first token from the prompt's last logits (:399), a stop token ends the
sequence before it is emitted (:405-407), at most `max_tokens` new tokens (:404), and
the `PPTG pp=... tg=...` throughput line (:423-433); `sampling::generate`
(sampling.rs:181-220) for the sampled variant, whose history is prompt + generated.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Union

from ..errors import CacheError, StepError
from ..sampling import Sampler, SamplingParams, resolve_seed, uniform
from .engine import Engine, StepEntry


@dataclass
class GenerationResult:
    tokens: List[int]
    finish_reason: str            # "stop" | "length" | "context" | "empty"
    prompt_tokens: int


@dataclass
class GenerationStats:
    prefill_tokens: int = 0
    prefill_seconds: float = 0.0
    decode_tokens: int = 0
    decode_seconds: float = 0.0
    batches: int = 0

    def pptg_line(self) -> str:
        """The reference's throughput line (generate.rs:427-433)."""
        pp = self.prefill_tokens / self.prefill_seconds if self.prefill_seconds > 0 else 0.0
        tg = self.decode_tokens / self.decode_seconds if self.decode_seconds > 0 else 0.0
        return (f"PPTG pp={pp:.1f} tok/s ({self.prefill_tokens} prompt tok / {self.prefill_seconds:.3f}s) "
                f"tg={tg:.1f} tok/s ({self.decode_tokens} tok / {self.decode_seconds:.3f}s)")


def plan_batches(prompt_lens: Sequence[int], max_new_tokens: int, capacity_tokens: int,
                 max_seq_len: int, max_batch: Optional[int] = None, page_tokens: int = 64,
                 n_slots: Optional[int] = None) -> List[List[int]]:
    """Which requests run together: in request order, as many as the cache can hold when
    each grows to its prompt plus `max_new_tokens` (capped by the longest sequence the
    cache takes), each rounded up to whole pages.  Empty prompts take no room.  A request
    that cannot fit alone is an error."""
    def room(n):
        full = min(n + max_new_tokens, max_seq_len)
        return -(-full // page_tokens) * page_tokens
    cap = (capacity_tokens // page_tokens) * page_tokens
    limit = min(x for x in (max_batch, n_slots) if x is not None) if (max_batch or n_slots) else None
    batches: List[List[int]] = []
    cur: List[int] = []
    used = 0
    for i, n in enumerate(prompt_lens):
        if n == 0:
            cur.append(i)
            continue
        if n > max_seq_len:
            raise CacheError(f"request {i}: a prompt of {n} tokens exceeds the longest sequence {max_seq_len}")
        need = room(n)
        if need > cap:
            raise CacheError(f"request {i}: {need} tokens of cache needed, the cache holds {cap}")
        live = sum(1 for j in cur if prompt_lens[j] > 0)
        if cur and (used + need > cap or (limit is not None and live >= limit)):
            batches.append(cur)
            cur, used = [], 0
        cur.append(i)
        used += need
    if cur:
        batches.append(cur)
    return batches


def generate(engine: Engine, prompts: Sequence[Sequence[int]],
             params: Union[None, SamplingParams, Sequence[SamplingParams]] = None,
             max_new_tokens: int = 64, stop_token_ids: Optional[Sequence[int]] = None,
             include_stop: bool = False, max_batch: Optional[int] = None, sampler=None):
    """Generate for every prompt; returns (results in request order, stats).

    `params`: one `SamplingParams` for all or one per request; None is greedy.
    `stop_token_ids`: None takes the engine's (`eos_token_id` of config.json and of
    generation_config.json)."""
    n = len(prompts)
    if params is None:
        plist = [SamplingParams.greedy() for _ in range(n)]
    elif isinstance(params, SamplingParams):
        plist = [params] * n
    else:
        plist = list(params)
        if len(plist) != n:
            raise StepError(f"{len(plist)} sampling parameter sets for {n} prompts")
    for p in plist:
        p.validate()
    if max_new_tokens < 0:
        raise StepError(f"max_new_tokens must be >= 0, got {max_new_tokens}")
    stops = set(engine.stop_token_ids if stop_token_ids is None else stop_token_ids)
    seeds = [resolve_seed(p.seed) for p in plist]
    if sampler is None:
        sampler = Sampler(engine.device, engine.vocab_size)
    cache = engine.cache
    results: List[Optional[GenerationResult]] = [None] * n
    stats = GenerationStats()
    batches = plan_batches([len(p) for p in prompts], max_new_tokens, cache.n_pages * cache.page_tokens,
                           cache.max_seq_len, max_batch, cache.page_tokens, cache.n_slots)
    for batch in batches:
        stats.batches += 1
        live = []
        for i in batch:
            if len(prompts[i]) == 0 or max_new_tokens == 0:
                results[i] = GenerationResult([], "empty" if len(prompts[i]) == 0 else "length", len(prompts[i]))
            else:
                live.append(i)
        if not live:
            continue
        slot = {i: engine.alloc_slot() for i in live}
        out = {i: [] for i in live}
        hist = {i: list(prompts[i]) for i in live}
        try:
            t0 = time.perf_counter()
            logits = engine.step([StepEntry(slot[i], list(prompts[i]), [len(prompts[i]) - 1]) for i in live])
            first = True
            while True:
                toks = sampler.sample(logits, [plist[i] for i in live], [hist[i] for i in live],
                                      [uniform(seeds[i], i, len(out[i])) for i in live])
                dt = time.perf_counter() - t0       # sampling returned the tokens: the step is done
                if first:
                    stats.prefill_tokens += sum(len(prompts[i]) for i in live)
                    stats.prefill_seconds += dt
                    first = False
                else:
                    stats.decode_tokens += len(live)
                    stats.decode_seconds += dt
                still = []
                for i, t in zip(live, toks):
                    reason = None
                    if t in stops:
                        reason = "stop"
                        if include_stop:
                            out[i].append(t)
                    else:
                        out[i].append(t)
                        hist[i].append(t)
                        if len(out[i]) >= max_new_tokens:
                            reason = "length"
                        elif engine.length(slot[i]) + 1 > cache.max_seq_len:
                            reason = "context"
                    if reason is None:
                        still.append(i)
                    else:
                        results[i] = GenerationResult(out[i], reason, len(prompts[i]))
                        engine.free_slot(slot.pop(i))      # an ended sequence leaves the batch at once
                live = still
                if not live:
                    break
                t0 = time.perf_counter()
                logits = engine.step([StepEntry(slot[i], [out[i][-1]], [0]) for i in live])
        finally:
            for s in slot.values():
                engine.free_slot(s)
    return results, stats
