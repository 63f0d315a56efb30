"""Pins of the plain implementation (tests/plain_mistral.py) beside the reference's text:
vectors the reference's own tests hold, special cases that reduce to a library routine,
and invariants, each chosen so that a plausible mistake fails it.  No GPU."""
import math

import numpy as np
import pytest
import torch

import plain_mistral as P

F = np.float32


# ------------------------------------------------------------------------ RMSNorm ----
def test_rmsnorm_reference_vector():
    # inputs of tests/op_rmsnorm_test.rs:51-66 (H=1024, 4 rows, eps 1e-6, x = sin(0.01 i),
    # w = bf16(1 + 0.001 i)), expected from a float64 evaluation of the formula, tol 1e-4 (:109)
    H, rows, eps = 1024, 4, 1e-6
    x = np.sin(0.01 * np.arange(rows * H, dtype=np.float64)).reshape(rows, H)
    w = (1.0 + 0.001 * np.arange(H)).astype(np.float32)
    w = torch.tensor(w).bfloat16().float().numpy()
    want = x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * w.astype(np.float64)
    got = P.rms_norm(x.astype(F), w, eps)
    assert np.abs(got - want).max() < 1e-4


def test_rmsnorm_unit_weight_gives_unit_mean_square_and_eps_sits_inside_the_root():
    x = np.random.default_rng(0).normal(size=(3, 50)).astype(F) * 7
    y = P.rms_norm(x, np.ones(50, F), 0.0)
    assert np.allclose((y * y).mean(-1), 1.0, atol=1e-5)
    # scale invariance without eps; with a large eps the output shrinks as 1/sqrt(ms + eps)
    assert np.allclose(P.rms_norm(3 * x, np.ones(50, F), 0.0), y, atol=1e-5)
    big = P.rms_norm(x, np.ones(50, F), 100.0)
    ms = (x.astype(np.float64) ** 2).mean(-1, keepdims=True)
    assert np.allclose(big, x / np.sqrt(ms + 100.0), atol=1e-5)
    # a (1 + w) norm, which the reference uses for another family, would fail this
    assert np.allclose(P.rms_norm(x, np.zeros(50, F), 1e-5), 0.0)


# --------------------------------------------------------------------------- RoPE ----
def test_rope_reference_vector_adjacent_pairs():
    # tests/mrope_test.rs:5-23,61-72: hd 256, rotary 64, theta 1e7, q = sin(0.017 i); with
    # one position for all sections it is plain rotary.  Expected by complex multiplication.
    nh, hd, rd, theta, pos = 8, 256, 64, 1e7, 42
    q = np.sin(0.017 * np.arange(nh * hd)).astype(F).reshape(1, nh, hd)
    inv = P.rope_inv_freq(rd, theta)
    assert inv.shape == (32,) and abs(inv[0] - 1.0) < 1e-7
    assert abs(inv[5] - 1.0 / theta ** (10 / 64)) < 1e-7
    got = P.rope(q, [pos], inv, "adjacent")
    z = (q[0, :, 0:rd:2].astype(np.float64) + 1j * q[0, :, 1:rd:2]) * np.exp(1j * pos * inv.astype(np.float64))
    assert np.abs(got[0, :, 0:rd:2] - z.real).max() < 1e-4 and np.abs(got[0, :, 1:rd:2] - z.imag).max() < 1e-4
    assert np.array_equal(got[0, :, rd:], q[0, :, rd:])          # the rest of the head is untouched


def test_rope_half_pairs_and_sign():
    inv = P.rope_inv_freq(4, 10000.0)
    x = np.zeros((1, 1, 4), F); x[0, 0, 0] = 1.0               # pair (0, 2) holds (1, 0)
    y = P.rope(x, [3], inv, "half")
    assert np.allclose(y[0, 0], [math.cos(3.0), 0.0, math.sin(3.0), 0.0], atol=1e-6)   # rotates counter-clockwise
    x2 = np.zeros((1, 1, 4), F); x2[0, 0, 0] = 1.0
    y2 = P.rope(x2, [3], inv, "adjacent")
    assert np.allclose(y2[0, 0], [math.cos(3.0), math.sin(3.0), 0.0, 0.0], atol=1e-6)


def test_rope_identity_norm_composition_and_relative_scores():
    rng = np.random.default_rng(1)
    inv = P.rope_inv_freq(16, 10000.0)
    q, k = rng.normal(size=(1, 2, 16)).astype(F), rng.normal(size=(1, 2, 16)).astype(F)
    for pairing in ("half", "adjacent"):
        assert np.allclose(P.rope(q, [0], inv, pairing), q)
        assert np.allclose(np.linalg.norm(P.rope(q, [77], inv, pairing), axis=-1), np.linalg.norm(q, axis=-1), atol=1e-5)
        twice = P.rope(P.rope(q, [5], inv, pairing), [9], inv, pairing)
        assert np.allclose(twice, P.rope(q, [14], inv, pairing), atol=1e-5)       # rotating twice adds the angles
        s1 = (P.rope(q, [10], inv, pairing) * P.rope(k, [3], inv, pairing)).sum(-1)
        s2 = (P.rope(q, [110], inv, pairing) * P.rope(k, [103], inv, pairing)).sum(-1)
        assert np.allclose(s1, s2, atol=1e-4)                                     # only the distance counts


# ---------------------------------------------------------------------- attention ----
def _sdpa(q, k, v, mask):
    t = lambda a: torch.tensor(a).permute(1, 0, 2)[None].double()
    o = torch.nn.functional.scaled_dot_product_attention(t(q), t(k), t(v), attn_mask=torch.tensor(mask)[None, None])
    return o[0].permute(1, 0, 2).numpy()


def test_attention_reduces_to_the_library_routine():
    rng = np.random.default_rng(2)
    T, nq, hd = 9, 3, 8
    q, k, v = (rng.normal(size=(T, nq, hd)).astype(F) for _ in range(3))
    causal = np.tril(np.ones((T, T), bool))
    assert np.abs(P.attention(q, k, v, nq, nq) - _sdpa(q, k, v, causal)).max() < 1e-5
    # one head
    assert np.abs(P.attention(q[:, :1], k[:, :1], v[:, :1], 1, 1) - _sdpa(q[:, :1], k[:, :1], v[:, :1], causal)).max() < 1e-5


def test_attention_groups_equal_repeated_heads_and_window_convention():
    rng = np.random.default_rng(3)
    T, nq, nkv, hd = 12, 6, 2, 4
    q = rng.normal(size=(T, nq, hd)).astype(F)
    k, v = rng.normal(size=(T, nkv, hd)).astype(F), rng.normal(size=(T, nkv, hd)).astype(F)
    rep = lambda a: np.repeat(a, nq // nkv, axis=1)         # q head h uses kv head h // (nq / nkv)
    causal = np.tril(np.ones((T, T), bool))
    assert np.abs(P.attention(q, k, v, nq, nkv) - _sdpa(q, rep(k), rep(v), causal)).max() < 1e-5
    W = 5
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    band = (j <= i) & (j > i - W)                            # query i sees the W keys i-W+1 .. i
    assert band[7].sum() == W
    assert np.abs(P.attention(q, k, v, nq, nkv, window=W) - _sdpa(q, rep(k), rep(v), band)).max() < 1e-5
    assert np.array_equal(P.attention(q, k, v, nq, nkv, window=T), P.attention(q, k, v, nq, nkv))
    # the first position sees only itself: its output is its value
    assert np.allclose(P.attention(q, k, v, nq, nkv)[0], rep(v)[0], atol=1e-6)


def test_attention_scale_is_rsqrt_head_dim():
    q = np.zeros((2, 1, 16), F); k = np.zeros((2, 1, 16), F); v = np.zeros((2, 1, 16), F)
    q[1, 0, 0] = 4.0; k[1, 0, 0] = 4.0; v[0, 0, 0] = 1.0
    # scores of query 1: key 0 -> 0, key 1 -> 16 / sqrt(16) = 4: weight of key 0 is 1 / (1 + e^4)
    o = P.attention(q, k, v, 1, 1)
    assert abs(o[1, 0, 0] - 1.0 / (1.0 + math.exp(4.0))) < 1e-6


# --------------------------------------------------------------------- feed-forward ----
def test_silu_reference_vector_and_swiglu_chain():
    # tests/op_silu_mul_test.rs:37-81: g = 3 sin(0.011 i), u = cos(0.009 i), tol 1e-3
    i = np.arange(1024)
    g, u = (3 * np.sin(0.011 * i)).astype(F), np.cos(0.009 * i).astype(F)
    want = torch.nn.functional.silu(torch.tensor(g).double()).numpy() * u
    assert np.abs(P.silu(g) * u - want).max() < 1e-6
    assert P.silu(np.zeros(1, F))[0] == 0.0
    rng = np.random.default_rng(4)
    n = rng.normal(size=(3, 8)).astype(F)
    Wg, Wu, Wd = rng.normal(size=(12, 8)).astype(F), rng.normal(size=(12, 8)).astype(F), rng.normal(size=(8, 12)).astype(F)
    want = (torch.nn.functional.silu(torch.tensor(n @ Wg.T)) * torch.tensor(n @ Wu.T)).numpy() @ Wd.T
    assert np.abs(P.swiglu(n, Wg, Wu, Wd) - want).max() < 1e-4
    # gate and up are not interchangeable
    assert np.abs(P.swiglu(n, Wu, Wg, Wd) - want).max() > 1e-2


def test_linear_and_embedding_vectors():
    # tests/wmma_gemm_test.rs:27-69: A = 0.5 sin, B = 0.3 cos ramps, 32x32x64, tol 1e-3
    M, N, K = 32, 32, 64
    A = (0.5 * np.sin(0.01 * np.arange(M * K))).astype(F).reshape(M, K)
    W = (0.3 * np.cos(0.01 * np.arange(N * K))).astype(F).reshape(N, K)
    assert np.abs(P.linear(A, W) - A.astype(np.float64) @ W.astype(np.float64).T).max() < 1e-3
    table = np.arange(256 * 8, dtype=F).reshape(256, 8)          # tests/embedding_test.rs: token 42
    assert np.array_equal(P.embedding(table, [42])[0], table[42])


# -------------------------------------------------------------------- whole model ----
def test_shifting_all_positions_changes_nothing(tiny_folders):
    # rotary scores depend on distances only, so a whole sequence moved by 100 positions
    # has the same logits; a position encoding added in the wrong place breaks this
    for name in ("a", "c"):
        _, cfg, w = tiny_folders[name]
        toks = list(np.random.default_rng(5).integers(0, cfg["vocab_size"], 20))
        a = P.forward(cfg, w, toks)
        b = P.forward(cfg, w, toks, positions=np.arange(20) + 100)
        assert np.abs(a - b).max() < 2e-4 * np.abs(a).max()


def test_window_matters_and_prefix_is_causal(tiny_folders):
    _, cfg, w = tiny_folders["b"]                      # window 8
    toks = list(np.random.default_rng(6).integers(0, cfg["vocab_size"], 30))
    full = P.forward(dict(cfg, sliding_window=None), w, toks)
    win = P.forward(cfg, w, toks)
    assert np.abs(full[:8] - win[:8]).max() < 1e-5      # the first 8 positions see everything either way
    assert np.abs(full[20:] - win[20:]).max() > 1e-3
    assert np.abs(P.forward(cfg, w, toks[:11]) - win[:11]).max() < 1e-5


# ----------------------------------------------------------------------- sampling ----
def test_sampler_vectors_of_the_reference():
    # sampling.rs:232-241, :268-278, :322-339, :342-357, :360-378
    assert P.sample([0.1, 0.5, 0.2, 0.8, 0.3], u=0.5, temperature=0.0) == 3
    assert P.sample([1, 2, 3, 4, 5], u=0.5, temperature=0.01, top_k=0) == 4
    for u in (0.0, 0.3, 0.999):
        assert P.sample([10, 0, 0, 0], u=u, temperature=1.0, min_p=0.5) == 0
    assert P.sample([1.0, 1.0, 1.0], u=0.5, temperature=0.0, logit_bias=[(1, 100.0)]) == 1
    assert P.sample([0.1, 0.2, 0.3, 1.1, 1.0], u=0.5, temperature=0.0, repetition_penalty=2.0, history=[3]) == 4


def test_sampler_filters():
    logits = [2.0, 1.0, 0.0, -1.0]
    p = np.exp(logits) / np.exp(logits).sum()
    assert [P.sample(logits, u, top_k=1) for u in (0.0, 0.5, 0.99)] == [0, 0, 0]
    assert P.sample(logits, u=0.999, top_k=2) == 1
    # top_p just above p0 keeps two tokens, just below keeps one
    assert P.sample(logits, u=0.999, top_p=float(p[0]) + 0.01) == 1
    assert P.sample(logits, u=0.999, top_p=float(p[0]) - 0.01) == 0
    # the draw is the inverse CDF in index order
    cum = np.cumsum(p)
    assert P.sample(logits, u=float(cum[0]) - 1e-3) == 0 and P.sample(logits, u=float(cum[0]) + 1e-3) == 1
    # a repeated token is penalised once per occurrence
    assert P.sample([4.0, 3.9], u=0.0, temperature=0.0, repetition_penalty=1.01, history=[0, 0, 0]) == 1


def test_uniform_numbers_and_the_sampled_loop():
    us = [P.uniform(7, s, d) for s in range(3) for d in range(200)]
    assert all(0.0 <= u < 1.0 for u in us) and len(set(us)) > 590           # 24 bits: hardly a repeat in 600
    assert abs(np.mean(us) - 0.5) < 0.05
    assert P.uniform(7, 1, 5) == P.uniform(7, 1, 5) != P.uniform(8, 1, 5)
    cfg = dict(num_hidden_layers=1, hidden_size=16, num_attention_heads=2, num_key_value_heads=1, head_dim=8,
               intermediate_size=24, vocab_size=20)
    w = P.random_weights(cfg, 3, std=0.5)
    # temperature 0 through the sampled loop is the greedy loop; a request's tokens depend on its number
    assert P.sampled_generate(cfg, w, [1, 2, 3], 5, seed=1, temperature=0.0) == P.greedy_generate(cfg, w, [1, 2, 3], 5)
    a = P.sampled_generate(cfg, w, [1, 2, 3], 12, seed=1, sequence=0, temperature=1.5)
    assert a == P.sampled_generate(cfg, w, [1, 2, 3], 12, seed=1, sequence=0, temperature=1.5)
    assert a != P.sampled_generate(cfg, w, [1, 2, 3], 12, seed=1, sequence=1, temperature=1.5)


def test_rounding_to_bfloat16():
    import torch
    x = np.random.default_rng(0).standard_normal(5000).astype(np.float32) * np.float32(3.0)
    x[:4] = [1.0, 1.00390625, 1.01171875, -0.0]          # a tie that goes down to even, one that goes up
    assert np.array_equal(P.bf16_round(x), torch.from_numpy(x).bfloat16().float().numpy())
    cfg = dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
               intermediate_size=96, vocab_size=50)
    w = P.random_weights(cfg, 1, std=0.1)
    toks = list(range(1, 30))
    a, b = P.forward(cfg, w, toks), P.forward(cfg, w, toks, act_dtype="bfloat16")
    assert np.array_equal(a, P.forward(cfg, w, toks, act_dtype="float32"))
    d = np.abs(a - b).max() / np.abs(a).max()
    assert 1e-5 < d < 2e-2                                 # rounding moves the logits, by about 2^-8 of them
