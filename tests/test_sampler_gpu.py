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
