"""The GPU sampler against the plain sampler (tests/plain_mistral.py: sample), which is
the reference's order of operations with the uniform draw given."""
import numpy as np
import pytest
import torch

import plain_mistral as P
from braidinfer_amd.sampling import Sampler, SamplingParams

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def run(logits, params, histories=None, us=None):
    l = torch.tensor(np.asarray(logits, np.float32)).to(DEV)
    if l.dim() == 1:
        l = l[None]
    if isinstance(params, SamplingParams):
        params = [params] * l.shape[0]
    return Sampler(DEV, l.shape[1]).sample(l, params, histories, us)


def test_reference_vectors():
    # sampling.rs:232-241, :268-278, :322-339, :342-357, :360-378
    assert run([0.1, 0.5, 0.2, 0.8, 0.3], SamplingParams.greedy()) == [3]
    assert run([1, 2, 3, 4, 5], SamplingParams(temperature=0.01, top_k=0), us=[0.5]) == [4]
    for u in (0.0, 0.3, 0.999):
        assert run([10, 0, 0, 0], SamplingParams(temperature=1.0, top_k=0, min_p=0.5), us=[u]) == [0]
    g = SamplingParams.greedy(); g.logit_bias = [(1, 100.0)]
    assert run([1.0, 1.0, 1.0], g) == [1]
    g = SamplingParams.greedy(); g.repetition_penalty = 2.0
    assert run([0.1, 0.2, 0.3, 1.1, 1.0], g, histories=[[3]]) == [4]


@pytest.mark.parametrize("V", [301, 4096, 5000])
def test_rows_match_the_plain_sampler(V):
    rng = np.random.default_rng(V)
    B = 12
    logits = rng.normal(size=(B, V)).astype(np.float32) * 3
    params, hists, us = [], [], []
    for b in range(B):
        p = SamplingParams(temperature=[0.0, 0.7, 1.0, 1.3][b % 4], top_k=[0, 5, 50, 0][(b // 2) % 4],
                           top_p=[1.0, 0.9, 0.5][b % 3], min_p=[0.0, 0.05][b % 2],
                           repetition_penalty=[1.0, 1.3][(b // 3) % 2],
                           logit_bias=[(3, 2.5), (7, -1.0), (3, 0.5)] if b % 5 == 0 else None)
        params.append(p)
        hists.append([int(t) for t in rng.integers(0, V, 30)] + [5, 5, 5])
        us.append(float(rng.random()))
    got = run(logits, params, hists, us)
    for b in range(B):
        p = params[b]
        want = P.sample(logits[b], us[b], p.temperature, p.top_k, p.top_p, p.min_p, p.repetition_penalty,
                        hists[b], p.logit_bias)
        if got[b] != want:
            # float sums in another order may move a boundary by rounding: then the draw must sit
            # within rounding of the boundary between the two tokens
            near = [P.sample(logits[b], min(max(us[b] + d, 0.0), 0.999999), p.temperature, p.top_k, p.top_p, p.min_p,
                             p.repetition_penalty, hists[b], p.logit_bias) for d in (-2e-6, 2e-6)]
            assert got[b] in near, f"row {b}: {got[b]} vs {want}"


def test_a_row_samples_the_same_alone_or_in_a_batch():
    rng = np.random.default_rng(1)
    logits = rng.normal(size=(6, 1000)).astype(np.float32) * 2
    p = SamplingParams(temperature=0.8, top_k=40, top_p=0.95)
    us = [float(u) for u in rng.random(6)]
    together = run(logits, p, us=us)
    alone = [run(logits[b], p, us=[us[b]])[0] for b in range(6)]
    assert together == alone


def test_distribution_follows_the_probabilities():
    logits = np.array([2.0, 1.0, 0.0, -1.0, -30.0], np.float32)
    want = np.exp(logits) / np.exp(logits).sum()
    n = 4000
    us = [(i + 0.5) / n for i in range(n)]
    got = run(np.tile(logits, (n, 1)), SamplingParams(temperature=1.0, top_k=0), us=us)
    freq = np.bincount(got, minlength=5) / n
    assert np.abs(freq - want).max() < 2e-3


# ---- the filter kernels alone -------------------------------------------------------------
def _filter_gpu(rows, top_k, min_p, top_p, general):
    """The masks of `sample_filter`, or with `general` of the kernel that sorts every row whole."""
    from braidinfer_amd import kernels as K
    B, V = rows.shape
    work = torch.tensor(rows).to(DEV)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32).to(DEV)
    f32 = lambda v: torch.tensor(v, dtype=torch.float32).to(DEV)
    temp = f32([1.0] * B)
    if general:
        keys = torch.empty((B, 1 << (V - 1).bit_length()), dtype=torch.int64, device=DEV)
        K.sample_filter_sort(work, keys, i32(top_k), f32(min_p), f32(top_p), temp)
    else:
        K.sample_filter(work, i32(top_k), f32(min_p), f32(top_p), temp)
    return work.cpu().numpy()


def _check_row(row, got, k, mp, tp, label):
    """`got` keeps a prefix of the (value descending, index ascending) order whose length is
    the plain filter's, or, where a float sum in another order moves the top-p cut by
    rounding, the plain filter's at a top_p within that rounding."""
    V = row.shape[0]
    order = sorted(range(V), key=lambda i: (-row[i], i))
    kept = [i for i in range(V) if got[i] > -np.inf]
    assert all(got[i] == row[i] for i in kept), label
    assert sorted(kept) == sorted(order[:len(kept)]), f"{label}: kept entries are not the first of the order"
    count = lambda t: int((P.filter_logits(row, k, min(max(t, 0.0), 1.0), mp) > -np.inf).sum())
    counts = {count(tp)}
    if tp < 1.0:
        # a running float32 sum of n probabilities is off by at most n * 2^-24
        eps = max(counts) * 2.0 ** -24
        counts |= {count(tp - eps), count(tp + eps)}
    assert min(counts) <= len(kept) <= max(counts), f"{label}: kept {len(kept)}, plain {sorted(counts)}"


@pytest.mark.parametrize("V", [257, 3000, 20000, 32768, 32768 + 5, 131072])
def test_the_filter_agrees_with_the_plain_filter_and_with_a_sort_of_the_whole_row(V):
    """`sample_filter` sorts nothing (a radix descent over exact weights); the kernel beside it sorts
    the whole row and adds float probabilities in that order.  Both against the plain filter: rows
    with peaks, ties, all entries equal, entries already masked; cuts that fall inside runs of
    equal values; top_k below, at and above any size the kernel treats specially."""
    rng = np.random.default_rng(V)
    smooth = (rng.normal(size=V) * 3).astype(np.float32)
    peaked = smooth.copy(); peaked[rng.integers(0, V, 5)] += 12.0
    tied = np.round(rng.normal(size=V) * 2).astype(np.float32)           # many equal values
    flat = np.zeros(V, np.float32)                                        # all equal
    holes = smooth.copy(); holes[rng.integers(0, V, V // 3)] = -np.inf    # already masked entries
    cases = []
    for name, row in (("smooth", smooth), ("peaked", peaked), ("tied", tied), ("flat", flat), ("holes", holes)):
        for k, mp, tp in ((1, 0.0, 1.0), (5, 0.0, 1.0), (50, 0.0, 1.0), (50, 0.05, 0.9), (200, 0.0, 0.5),
                          (1024, 0.0, 1.0), (1025, 0.0, 0.95), (0, 0.1, 1.0), (0, 0.0, 0.9), (0, 0.02, 0.999),
                          (0, 0.0, 0.3), (V, 0.0, 0.7), (V - 1, 0.0, 1.0), (V // 2, 0.0, 0.99)):
            cases.append((f"{name} k={k} min_p={mp} top_p={tp}", row, k, mp, tp))
    rows = np.stack([c[1] for c in cases])
    ks, mps, tps = [c[2] for c in cases], [c[3] for c in cases], [c[4] for c in cases]
    fast = _filter_gpu(rows, ks, mps, tps, general=False)
    whole = _filter_gpu(rows, ks, mps, tps, general=True) if V <= 40000 else None
    for b, (label, row, k, mp, tp) in enumerate(cases):
        _check_row(row, fast[b], k, mp, tp, "radix descent, " + label)
        if whole is not None:
            _check_row(row, whole[b], k, mp, tp, "whole row sorted, " + label)
    # where no rounding is in play (no top-p) the two kernels keep the same entries
    if whole is not None:
        for b, c in enumerate(cases):
            if c[4] == 1.0:
                assert np.array_equal(fast[b], whole[b]), c[0]


def test_zeros_of_either_sign_are_equal_in_the_filters_order():
    """-0.0 and +0.0 are one value to the reference's sort, so a cut inside a row's zeros keeps
    those with the lowest indices whatever their signs, in every form of the filter."""
    rng = np.random.default_rng(9)
    for V in (300, 5000):
        row = np.where(rng.random(V) < 0.5, np.float32(0.0), np.float32(-0.0)).astype(np.float32)
        big = rng.choice(V, 20, replace=False)
        row[big] = 3.0
        row[rng.choice(np.setdiff1d(np.arange(V), big), V // 3, replace=False)] = -2.0
        cases = [(60, 0.0, 1.0), (0, 0.0, 0.9), (1025, 0.0, 0.97), (100, 0.0, 0.95)]
        rows = np.stack([row] * len(cases))
        ks, mps, tps = [c[0] for c in cases], [c[1] for c in cases], [c[2] for c in cases]
        forms = [_filter_gpu(rows, ks, mps, tps, general=False), _filter_gpu(rows, ks, mps, tps, general=True)]
        for b, (k, mp, tp) in enumerate(cases):
            for name, got in zip(("radix descent", "whole row sorted"), forms):
                _check_row(row, got[b], k, mp, tp, f"{name}, V={V} k={k} top_p={tp}")
                kept = np.nonzero(got[b] > -np.inf)[0]
                zeros = [i for i in kept if row[i] == 0.0]
                assert zeros and len(zeros) < int((row == 0.0).sum()), "the cut was meant to fall among the zeros"
                assert zeros == [i for i in range(V) if row[i] == 0.0][:len(zeros)]


def test_a_resident_state_keeps_its_rows_histories_on_the_device():
    """Step after step with only the uniform numbers coming from the host: every drawn token
    joins its row's history (what the repetition penalty sees), rows that end are dropped with
    `keep`, and each step equals the plain sampler given the history so far."""
    V, B = 500, 6
    rng = np.random.default_rng(3)
    params = [SamplingParams(temperature=[0.8, 1.0, 0.0][b % 3], top_k=[0, 20][b % 2], top_p=1.0, min_p=0.0,
                             repetition_penalty=[1.5, 1.0, 1.2][b % 3],
                             logit_bias=[(b, 1.0), (b + 1, -2.0)] if b in (1, 4) else None) for b in range(B)]
    hists = [[int(t) for t in rng.integers(0, V, 12)] + [7, 7] for _ in range(B)]
    state = Sampler(DEV, V).state(params, hists)
    rows = list(range(B))
    for step in range(8):
        logits = rng.normal(size=(len(rows), V)).astype(np.float32) * 2
        logits[:, 7] += 3.0                                  # a token that is in every history and would win unpenalised
        us = [float(rng.random()) for _ in rows]
        got = state.sample(torch.tensor(logits).to(DEV), us)
        for r, b in enumerate(rows):
            p = params[b]
            want = P.sample(logits[r], us[r], p.temperature, p.top_k, p.top_p, p.min_p, p.repetition_penalty, hists[b],
                            p.logit_bias)
            near = [P.sample(logits[r], min(max(us[r] + d, 0.0), 0.999999), p.temperature, p.top_k, p.top_p, p.min_p,
                             p.repetition_penalty, hists[b], p.logit_bias) for d in (-2e-6, 2e-6)]
            assert got[r] == want or got[r] in near, f"step {step}, row {b}"
            hists[b].append(got[r])
        if step == 2:
            rows = [0, 2, 3, 5]
            state = state.keep([0, 2, 3, 5])
        if step == 5:
            rows = [5, 0]                                    # another order, too
            state = state.keep([3, 0])


def test_a_state_that_draws_its_own_numbers_draws_the_hosts():
    """With `random` the draw kernel makes each row's uniform number itself from the request's
    seed, number and draw count: the tokens of a state that is handed `uniform(seed, request, draw)`
    step by step, through `keep` and for rows of temperature 0, whose count goes on too."""
    from braidinfer_amd.sampling import uniform
    V, B = 700, 5
    rng = np.random.default_rng(4)
    params = [SamplingParams(temperature=[1.0, 0.7, 0.0][b % 3], top_k=[0, 30][b % 2], repetition_penalty=[1.0, 1.3][b % 2])
              for b in range(B)]
    hists = [[int(t) for t in rng.integers(0, V, 5)] for _ in range(B)]
    random = [(2 ** 63 + 11 * b, 3 * b + 1, 4 + b) for b in range(B)]        # seeds beyond 63 bits too
    own = Sampler(DEV, V).state(params, hists, random=random)
    told = Sampler(DEV, V).state(params, hists)
    assert own.device_random and not told.device_random
    rows, draws = list(range(B)), [d for _, _, d in random]
    seen = set()
    for step in range(9):
        logits = torch.tensor(rng.normal(size=(len(rows), V)).astype(np.float32)).to(DEV)
        a = own.sample(logits)
        b = told.sample(logits, [uniform(random[r][0], random[r][1], draws[r]) for r in rows])
        assert a == b, step
        seen.update(a)
        for r in rows:
            draws[r] += 1
        if step == 3:
            rows = [4, 1, 2]
            own, told = own.keep([4, 1, 2]), told.keep([4, 1, 2])
    assert len(seen) > 10
    assert own.rng_draw.tolist() == [draws[r] for r in rows]
    with pytest.raises(ValueError):
        Sampler(DEV, V).state(params, hists, random=random[:2])
