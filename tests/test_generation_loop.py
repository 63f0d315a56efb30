"""The generation loop's decisions, with a stand-in engine that needs no GPU: batches,
stop tokens, budgets, sequences that end earlier, slots given back."""
import pytest
import torch

from braidinfer_amd.engine import generate, plan_batches
from braidinfer_amd.errors import CacheError, StepError
from braidinfer_amd.sampling import SamplingParams, uniform


class FakeCache:
    def __init__(self, n_pages, page_tokens=64, max_seq_len=None, n_slots=None):
        self.n_pages, self.page_tokens = n_pages, page_tokens
        self.max_seq_len = max_seq_len or n_pages * page_tokens
        self.n_slots = n_slots or n_pages


class FakeSpec:
    stop_token_ids = [0]
    vocab_size = 50


class FakeEngine:
    """Next token = (last token + 1) % V: every sequence counts upwards."""

    def __init__(self, n_pages=32, **kw):
        self.cache = FakeCache(n_pages, **kw)
        self.spec = FakeSpec()
        self.stop_token_ids = list(self.spec.stop_token_ids)
        self.vocab_size = 50
        self.device = "cpu"
        self.live = {}
        self.next_slot = 0
        self.steps = []            # (slots, number of tokens each) per step
        self.max_live = 0

    def alloc_slot(self):
        s = self.next_slot
        self.next_slot += 1
        self.live[s] = 0
        self.max_live = max(self.max_live, len(self.live))
        return s

    def free_slot(self, s):
        assert s in self.live, "slot freed twice"
        del self.live[s]

    def length(self, s):
        return self.live[s]

    def step(self, entries):
        self.steps.append(([e.slot for e in entries], [len(e.tokens) for e in entries]))
        rows = []
        for e in entries:
            assert e.slot in self.live
            self.live[e.slot] += len(e.tokens)
            for w in e.want:
                row = torch.zeros(50)
                row[(e.tokens[w] + 1) % 50] = 1.0
                rows.append(row)
        return torch.stack(rows)


class ArgmaxSampler:
    def sample(self, logits, params, histories, us):
        return [int(r.argmax()) for r in logits]


def run(engine, prompts, **kw):
    return generate(engine, prompts, sampler=ArgmaxSampler(), **kw)


def test_counts_upwards_until_the_budget():
    e = FakeEngine()
    res, stats = run(e, [[5, 6, 7]], max_new_tokens=4, stop_token_ids=[])
    assert res[0].tokens == [8, 9, 10, 11] and res[0].finish_reason == "length" and res[0].prompt_tokens == 3
    assert e.steps[0] == ([0], [3]) and all(s == ([0], [1]) for s in e.steps[1:])
    assert len(e.steps) == 4            # the prompt step gives the first token; no step after the last
    assert stats.prefill_tokens == 3 and stats.decode_tokens == 3 and not e.live


def test_stop_token_ends_without_being_emitted():
    e = FakeEngine()
    res, _ = run(e, [[46]], max_new_tokens=10)             # model's stop token is 0
    assert res[0].tokens == [47, 48, 49] and res[0].finish_reason == "stop"
    res, _ = run(e, [[46]], max_new_tokens=10, include_stop=True)
    assert res[0].tokens == [47, 48, 49, 0]
    res, _ = run(e, [[49]], max_new_tokens=10)             # the very first token stops
    assert res[0].tokens == [] and res[0].finish_reason == "stop"


def test_shorter_sequences_leave_the_batch_and_give_their_slot_back():
    e = FakeEngine()
    res, _ = run(e, [[40], [47], [10, 11]], max_new_tokens=5, stop_token_ids=[0])
    assert res[0].tokens == [41, 42, 43, 44, 45] and res[1].tokens == [48, 49] and res[2].tokens == [12, 13, 14, 15, 16]
    sizes = [len(s[0]) for s in e.steps]
    assert sizes == [3, 3, 3, 2, 2]     # request 1 stops on its third token and leaves before the fourth step
    assert e.steps[0][1] == [2, 1, 1] and not e.live         # a batch's longest prompts come first


def test_batches_run_one_after_another_when_the_cache_is_small():
    e = FakeEngine(n_pages=2)            # two pages: two short requests at a time
    res, stats = run(e, [[1], [2], [3], [4], [5]], max_new_tokens=3, stop_token_ids=[])
    assert [r.tokens for r in res] == [[2, 3, 4], [3, 4, 5], [4, 5, 6], [5, 6, 7], [6, 7, 8]]
    assert stats.batches == 3 and e.max_live == 2 and not e.live


def test_empty_prompt_and_zero_budget():
    e = FakeEngine()
    res, _ = run(e, [[], [3]], max_new_tokens=2, stop_token_ids=[])
    assert res[0].tokens == [] and res[0].finish_reason == "empty" and res[1].tokens == [4, 5]
    res, _ = run(e, [[3]], max_new_tokens=0)
    assert res[0].tokens == [] and e.live == {}


def test_context_limit_is_a_reason():
    e = FakeEngine(n_pages=4, max_seq_len=6)
    res, _ = run(e, [[1, 2, 3, 4]], max_new_tokens=10, stop_token_ids=[])
    # the cache takes 6 tokens: prompt 4, then tokens 5 and 6 are fed; the third new token is the last
    assert res[0].finish_reason == "context" and res[0].tokens == [5, 6, 7]


def test_slots_are_returned_when_a_step_fails():
    e = FakeEngine()
    def boom(entries):
        raise StepError("no")
    e.step = boom
    with pytest.raises(StepError):
        run(e, [[1], [2]], max_new_tokens=2)
    assert not e.live


def test_plan_batches():
    assert plan_batches([5, 9, 12], 8, 64 * 3, 4096) == [[0, 1, 2]]
    assert plan_batches([5, 9, 12], 8, 64 * 2, 4096) == [[0, 1], [2]]
    assert plan_batches([60, 60], 8, 64 * 3, 4096) == [[0], [1]]          # 68 tokens need two pages each
    assert plan_batches([1, 1, 1, 1], 1, 64 * 8, 4096, max_batch=3) == [[0, 1, 2], [3]]
    assert plan_batches([1, 1, 1], 1, 64 * 8, 4096, n_slots=2) == [[0, 1], [2]]
    assert plan_batches([100], 1000, 64 * 2, 128) == [[0]]                # growth is capped by the longest sequence
    with pytest.raises(CacheError, match="longest"):
        plan_batches([200], 8, 64 * 8, 128)
    with pytest.raises(CacheError, match="cache holds"):
        plan_batches([200], 8, 64 * 2, 4096)


def test_one_parameter_set_per_request_or_one_for_all():
    e = FakeEngine()
    with pytest.raises(StepError):
        run(e, [[1], [2]], params=[SamplingParams.greedy()])
    with pytest.raises(ValueError):
        run(e, [[1]], params=SamplingParams(top_p=0.0))


def test_sampling_defaults_are_the_references():
    d, g = SamplingParams(), SamplingParams.greedy()
    assert (d.temperature, d.top_k, d.top_p, d.repetition_penalty, d.seed, d.min_p, d.logit_bias) == (1.0, 50, 1.0, 1.0, None, 0.0, None)
    assert (g.temperature, g.top_k) == (0.0, 0) and g.is_plain_greedy


def test_uniform_numbers_depend_only_on_seed_sequence_and_draw():
    a = [uniform(7, 3, i) for i in range(1000)]
    assert a == [uniform(7, 3, i) for i in range(1000)] and all(0.0 <= x < 1.0 for x in a)
    assert abs(sum(a) / 1000 - 0.5) < 0.05
    assert uniform(7, 3, 0) != uniform(7, 4, 0) != uniform(8, 3, 0)


# ---- greedy requests through a chain: the host reads a step behind -------------------------
class FakeChain:
    """What `Engine.chain` hands out, with the stand-in model: every launch feeds each
    row the token the launch before gave it, whether or not the host has read it yet."""

    def __init__(self, engine, slots, tokens, state=None):
        self.e, self.slots, self.tokens, self.unread, self.closed = engine, list(slots), list(tokens), [], False
        self.state, self.us = state, []
        engine.chains.append(self)

    def launch(self, us=None):
        assert not self.closed and len(self.unread) < 2
        assert (us is None) == (self.state is None)
        self.us.append(us)
        for s in self.slots:
            assert s in self.e.live, "a step for a slot that was given back"
            self.e.live[s] += 1
            assert self.e.live[s] <= self.e.cache.max_seq_len, "a step beyond the longest sequence"
        self.tokens = [(t + 1) % 50 for t in self.tokens]
        self.unread.append(list(self.tokens))
        self.e.steps.append((list(self.slots), [1] * len(self.slots)))
        self.e.launched_ahead += len(self.unread) == 2

    def read(self):
        return self.unread.pop(0)

    def close(self):
        self.closed = True


class ChainEngine(FakeEngine):
    def __init__(self, *a, **k):
        super().__init__(*a, **k)
        self.chains, self.launched_ahead = [], 0

    def chain(self, slots, tokens, state=None):
        return FakeChain(self, slots, tokens, state)


def test_a_chain_gives_the_tokens_of_single_steps_for_every_way_of_ending():
    import random
    rnd = random.Random(3)
    for trial in range(60):
        n = rnd.randint(1, 5)
        prompts = [[rnd.randint(1, 49) for _ in range(rnd.randint(1, 4))] for _ in range(n)]
        kw = dict(max_new_tokens=rnd.randint(1, 9), stop_token_ids=rnd.choice([[], [0], [rnd.randint(1, 49)]]),
                  include_stop=rnd.random() < 0.3)
        limit = rnd.choice([None, 6, 9])
        plain, chained = FakeEngine(max_seq_len=limit), ChainEngine(max_seq_len=limit)
        a, sa = run(plain, prompts, **kw)
        b, sb = run(chained, prompts, **kw)
        assert [(r.tokens, r.finish_reason) for r in a] == [(r.tokens, r.finish_reason) for r in b], (trial, prompts, kw, limit)
        assert not chained.live and all(c.closed and not c.unread for c in chained.chains)
        assert sa.decode_tokens <= sb.decode_tokens <= sa.decode_tokens + n       # at most one token too many per request


def test_a_chain_runs_a_step_ahead_only_when_nobody_can_end_for_a_known_reason():
    e = ChainEngine()
    res, _ = run(e, [[5], [20]], max_new_tokens=6, stop_token_ids=[])
    assert [r.tokens for r in res] == [[6, 7, 8, 9, 10, 11], [21, 22, 23, 24, 25, 26]]
    assert len(e.chains) == 1 and e.launched_ahead == 4       # of 5 chain steps, the last is never launched ahead
    assert len(e.steps) == 6                                  # and none beyond the budget
    e = ChainEngine()
    res, _ = run(e, [[46], [10]], max_new_tokens=8)           # request 0 meets the stop token 0 on its fourth token
    assert res[0].tokens == [47, 48, 49] and res[0].finish_reason == "stop" and res[1].tokens == list(range(11, 19))
    assert len(e.chains) == 2 and e.chains[0].slots == [0, 1] and e.chains[1].slots == [1]
    # sampled requests do not use the chain when the sampler keeps no state on the device
    e = ChainEngine()
    run(e, [[5]], max_new_tokens=3, stop_token_ids=[], params=SamplingParams(temperature=0.5, seed=1))
    assert not e.chains


class FakeState:
    def __init__(self, rows):
        self.rows = list(rows)

    def sample(self, logits, us):
        return [int(r.argmax()) for r in logits]

    def keep(self, rows):
        return FakeState([self.rows[r] for r in rows])


class StateSampler:
    def state(self, params, histories):
        return FakeState(range(len(params)))


def test_a_sampled_chain_brings_each_step_the_uniform_numbers_of_its_draws():
    """Draw k of request i uses uniform(seed, i, k) whether it is launched ahead or not, and the
    state handed to a chain is that of the rows that go on."""
    p = SamplingParams(temperature=0.5, seed=11)
    e = ChainEngine()
    res, _ = generate(e, [[46], [10]], params=p, max_new_tokens=6, sampler=StateSampler())
    assert res[0].tokens == [47, 48, 49] and res[0].finish_reason == "stop" and res[1].tokens == list(range(11, 17))
    first, second = e.chains
    assert first.state.rows == [0, 1] and second.state.rows == [1]
    # the first token comes from the prompt step (draw 0); the chain's launches draw 1, 2, ...
    assert first.us[:3] == [[uniform(11, 0, k), uniform(11, 1, k)] for k in (1, 2, 3)]
    drawn_for_1 = [u[1] for u in first.us] + [u[0] for u in second.us]
    assert drawn_for_1 == [uniform(11, 1, k) for k in range(1, 6)]
    assert not e.live and all(c.closed for c in e.chains)
