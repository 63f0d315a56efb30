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


def _run_chain(chain, live, out, slot, take, finish, max_new_tokens, engine, cache, stats, t0, us_of=None):
    """Steps of the requests `live` through a chain until one of them ends; returns those
    that go on.  A second step is launched before the first one's tokens are read whenever
    no request can end for a reason known beforehand (its budget, the longest sequence the
    cache takes); a request that meets a stop token has then been given one token too many,
    which is dropped with its slot.  `us_of(ahead)`: the uniform numbers of a step launched
    while `ahead` steps are unread (a sampled chain), None for a greedy one."""
    def launch(ahead):
        if us_of is None:
            chain.launch()
        else:
            chain.launch(us_of(ahead))
    try:
        launch(0)
        launched, read = 1, 0
        while True:
            ahead = launched - read              # steps whose tokens are still to come
            if ahead < 2 and all(len(out[i]) + ahead + 1 <= max_new_tokens
                                 and engine.length(slot[i]) + 1 <= cache.max_seq_len for i in live):
                launch(ahead)
                launched += 1
            toks = chain.read()
            read += 1
            now = time.perf_counter()
            stats.decode_tokens += len(live)
            stats.decode_seconds += now - t0
            t0 = now
            ended = {}
            for i, t in zip(live, toks):
                reason = take(i, t, launched - read)
                if reason is not None:
                    ended[i] = reason
            if not ended and launched == read:
                launch(0)
                launched += 1
                continue
            if not ended:
                continue
            # someone ended: the tokens of a step launched ahead still belong to the others
            going = [i for i in live if i not in ended]
            while launched > read:
                toks = chain.read()
                read += 1
                now = time.perf_counter()
                stats.decode_tokens += len(going)
                stats.decode_seconds += now - t0
                t0 = now
                for i, t in zip(live, toks):
                    if i in going:
                        reason = take(i, t, launched - read)
                        if reason is not None:
                            ended[i] = reason
                going = [i for i in going if i not in ended]
            for i, reason in ended.items():
                finish(i, reason)
            return going
    finally:
        chain.close()


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
        # Longest prompts first: the single-token attention starts its workgroups in row order, and where
        # they are more than the chip holds at once, long sequences that start first do not end last
        # (128 sequences of 128 to 2,048 tokens: 99 against 107 us a layer).
        live.sort(key=lambda i: -len(prompts[i]))
        slot = {i: engine.alloc_slot() for i in live}
        out = {i: [] for i in live}
        hist = {i: list(prompts[i]) for i in live}

        def take(i, t, ahead=0):
            """Book the token request i was given; the reason it ends with, or None.  `ahead`:
            steps already launched beyond the one this token comes from."""
            if t in stops:
                if include_stop:
                    out[i].append(t)
                return "stop"
            out[i].append(t)
            hist[i].append(t)
            if len(out[i]) >= max_new_tokens:
                return "length"
            if engine.length(slot[i]) - ahead + 1 > cache.max_seq_len:
                return "context"
            return None

        def finish(i, reason):
            results[i] = GenerationResult(out[i], reason, len(prompts[i]))
            engine.free_slot(slot.pop(i))      # an ended sequence leaves the batch at once

        # the sampler of the live rows stays on the device from step to step (options, bias lists,
        # histories); it is cut down to the rows that go on when some end
        resident = {"rows": None, "state": None}

        make_state = getattr(sampler, "state", None)

        def state_of(live):
            if resident["rows"] != live:
                old = resident["rows"]
                if old is not None and set(live) <= set(old):
                    resident["state"] = resident["state"].keep([old.index(i) for i in live])
                elif getattr(sampler, "takes_random", False):
                    # the state draws its own numbers: uniform(seed, request, draw) from each request's next draw on
                    resident["state"] = make_state([plist[i] for i in live], [hist[i] for i in live],
                                                   random=[(seeds[i], i, len(out[i])) for i in live])
                else:
                    resident["state"] = make_state([plist[i] for i in live], [hist[i] for i in live])
                resident["rows"] = list(live)
            return resident["state"]

        def draw(logits, live):
            us = lambda: [uniform(seeds[i], i, len(out[i])) for i in live]
            if make_state is None:
                return sampler.sample(logits, [plist[i] for i in live], [hist[i] for i in live], us())
            state = state_of(live)
            return state.sample(logits) if getattr(state, "device_random", False) else state.sample(logits, us())

        def sample_and_book(logits, live, prefill):
            toks = draw(logits, live)
            dt = time.perf_counter() - t0       # sampling returned the tokens: the step is done
            if prefill:
                stats.prefill_tokens += sum(len(prompts[i]) for i in live)
                stats.prefill_seconds += dt
            else:
                stats.decode_tokens += len(live)
                stats.decode_seconds += dt
            still = []
            for i, t in zip(live, toks):
                reason = take(i, t)
                if reason is None:
                    still.append(i)
                else:
                    finish(i, reason)
            return still

        try:
            t0 = time.perf_counter()
            logits = engine.step([StepEntry(slot[i], list(prompts[i]), [len(prompts[i]) - 1]) for i in live])
            live = sample_and_book(logits, live, True)
            # requests decode through a chain when the engine has one: a step's tokens feed the next
            # step on the device, and the host reads them one step behind.  Plain greedy requests
            # take the argmax inside the recorded step; others draw through the resident sampler
            open_chain = getattr(engine, "chain", None)
            while live:
                t0 = time.perf_counter()
                chain = us_of = None
                if open_chain is not None:
                    rows = list(live)
                    if all(plist[i].is_plain_greedy for i in rows):
                        chain = open_chain([slot[i] for i in rows], [out[i][-1] for i in rows])
                    elif make_state is not None:
                        state = state_of(rows)
                        chain = open_chain([slot[i] for i in rows], [out[i][-1] for i in rows], state)
                        if not getattr(state, "device_random", False):
                            us_of = lambda ahead: [uniform(seeds[i], i, len(out[i]) + ahead) for i in rows]
                if chain is not None:
                    live = _run_chain(chain, live, out, slot, take, finish, max_new_tokens, engine, cache, stats, t0, us_of)
                else:
                    logits = engine.step([StepEntry(slot[i], [out[i][-1]], [0]) for i in live])
                    live = sample_and_book(logits, live, False)
        finally:
            for s in slot.values():
                engine.free_slot(s)
    return results, stats
