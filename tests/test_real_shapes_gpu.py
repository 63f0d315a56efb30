"""The sizes and schedules the benchmark runs, against fp64 expressions and the plain
implementation: the products of a 2,048- to 32,768-token prompt with the tile the library itself
chooses, the widths of the 24B shape, a 2,048-token prompt through one layer of the 7B shape,
eight windowed sequences of thousands of tokens decoding together from a graph, and the sampled
run of the benchmark description's second configuration."""
import numpy as np
import pytest
import torch

import braidinfer_amd as B
import plain_mistral as P
from braidinfer_amd import StepEntry
from braidinfer_amd import kernels as K

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rnd(*shape, seed=0, scale=1.0, dtype=torch.bfloat16):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return (torch.randn(*shape, generator=g, device=DEV) * scale).to(dtype)


def sample_of(n, k, seed):
    """k of range(n): both ends, the edges of tiles of 128 and 256, and random places."""
    fixed = [i for i in (0, 1, 127, 128, 255, 256, 257, n // 2, n - 257, n - 2, n - 1) if 0 <= i < n]
    more = np.random.default_rng(seed).integers(0, n, max(0, k - len(fixed)))
    return torch.tensor(sorted(set(fixed) | {int(i) for i in more}), device=DEV)


# ------------------------------------------------------- prompt products, the chooser's tiles ----
@pytest.mark.parametrize("M,N,Kd,mode", [(2048, 6144, 4096, "bf16"), (2048, 4096, 4096, "accumulate"),
                                         (2048, 4096, 14336, "accumulate"), (32768, 4096, 4096, "accumulate"),
                                         (8192, 6144, 4096, "bf16"), (32768, 6144, 4096, "bf16")])
def test_prompt_products_with_the_chosen_tile(M, N, Kd, mode):
    """The products of a prompt at the 7B shape as `parts.linear` asks for them (kernel 0: the
    library's own choice of tile and cut), sampled rows against fp64."""
    a, w = rnd(M, Kd, seed=1, scale=0.5), rnd(N, Kd, seed=2, scale=0.05)
    rows = sample_of(M, 24, M + N)
    want = a[rows].double() @ w.double().T
    scratch = torch.full((K.GEMM_SCRATCH_FLOATS,), float("nan"), device=DEV) if 16 < M <= 1024 else None
    if mode == "bf16":
        out = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
        K.gemm(a, w, out, scratch=scratch)
        tol = 1e-2
    else:
        base = rnd(M, N, seed=3, dtype=torch.float32)
        out = base.clone()
        K.gemm(a, w, out, accumulate=True, scratch=scratch)
        want = want + base[rows].double()
        tol = 1e-4
    assert torch.isfinite(out.float()).all()
    assert (out[rows].double() - want).abs().max() < tol * want.abs().max()


@pytest.mark.parametrize("M", [2048, 4096, 8192])
def test_prompt_gate_up_product_with_the_chosen_tile(M):
    """Gate and up of the 7B shape (28,672 interleaved rows in the blocked layout the engine keeps
    them in) with the SwiGLU epilogue: 256x256 tiles over whole rounds, 128x256 over the rest."""
    I, Kd = 14336, 4096
    a = rnd(M, Kd, seed=1, scale=0.5)
    wg, wu = rnd(I, Kd, seed=2, scale=0.03), rnd(I, Kd, seed=3, scale=0.03)
    w = K.block_weight(K.interleave_gate_up(wg, wu))
    out = torch.full((M, I), float("nan"), device=DEV, dtype=torch.bfloat16)
    K.gemm_swiglu(a, w, out)
    rows = sample_of(M, 16, M)
    g, u = a[rows].double() @ wg.double().T, a[rows].double() @ wu.double().T
    want = g / (1 + torch.exp(-g)) * u
    assert torch.isfinite(out.float()).all()
    assert (out[rows].double() - want).abs().max() < 1e-2 * want.abs().max()


# --------------------------------------------------------------------- the 24B shape's widths ----
@pytest.mark.parametrize("M", [1, 8, 16, 40, 300])
def test_head_product_of_the_24b_shape(M):
    """131,072 rows of 5,120 in the blocked layout, for the rows a step wants logits of."""
    N, Kd = 131072, 5120
    a, w = rnd(M, Kd, seed=1, scale=0.5), rnd(N, Kd, seed=2, scale=0.05)
    wb = K.block_weight(w)
    out = torch.full((M, N), float("nan"), device=DEV)
    scratch = torch.full((K.GEMM_SCRATCH_FLOATS,), float("nan"), device=DEV) if 16 < M <= 1024 else None
    K.gemm(a, wb, out, scratch=scratch)
    assert torch.isfinite(out).all()
    cols = sample_of(N, 4096, M)
    want = a.double() @ w[cols].double().T
    assert (out[:, cols].double() - want).abs().max() < 1e-4 * want.abs().max()


@pytest.mark.parametrize("M", [1, 16, 48, 2048])
def test_gate_up_and_down_products_of_the_24b_shape(M):
    """2 x 32,768 interleaved rows of 5,120 with the SwiGLU epilogue, then 5,120 rows of 32,768 added
    into float rows, sampled columns and rows against fp64."""
    I, H = 32768, 5120
    a = rnd(M, H, seed=1, scale=0.5)
    wg, wu = rnd(I, H, seed=2, scale=0.03), rnd(I, H, seed=3, scale=0.03)
    w = K.block_weight(K.interleave_gate_up(wg, wu))
    act = torch.full((M, I), float("nan"), device=DEV, dtype=torch.bfloat16)
    scratch = torch.full((K.GEMM_SCRATCH_FLOATS,), float("nan"), device=DEV) if 16 < M <= 1024 else None
    K.gemm_swiglu(a, w, act, scratch=scratch)
    rows = sample_of(M, 12, M)
    cols = sample_of(I, 3000, M + 1)
    g, u = a[rows].double() @ wg[cols].double().T, a[rows].double() @ wu[cols].double().T
    want = g / (1 + torch.exp(-g)) * u
    assert torch.isfinite(act.float()).all()
    assert (act[rows][:, cols].double() - want).abs().max() < 1e-2 * want.abs().max()
    wd = rnd(H, I, seed=4, scale=0.02)
    base = rnd(M, H, seed=5, dtype=torch.float32)
    x = base.clone()
    K.gemm(act, wd, x, accumulate=True, scratch=scratch)
    want = base[rows].double() + act[rows].double() @ wd.double().T
    assert (x[rows].double() - want).abs().max() < 1e-4 * want.abs().max()


# ------------------------------------------------------- one layer, rows of a long sequence ----
def plain_rows(pc, pw, toks, rows, act_dtype=None):
    """The plain implementation's logits at `rows` of a long sequence through a one-layer model:
    only the attention needs every position (keys and values of all of them); the rest is done
    on the asked rows with the plain functions."""
    rnd_ = P.rounding(act_dtype)
    sz = P.sizes(pc)
    assert sz["L"] == 1
    T = len(toks)
    p = "model.layers.0."
    x = P.embedding(pw["model.embed_tokens.weight"], toks)
    n = rnd_(P.rms_norm(x, pw[p + "input_layernorm.weight"], sz["eps"]))
    inv = P.rope_inv_freq(sz["hd"], sz["theta"])
    k = rnd_(P.rope(rnd_(P.linear(n, pw[p + "self_attn.k_proj.weight"])).reshape(T, sz["nkv"], sz["hd"]),
                    np.arange(T), inv, sz["pairing"]))
    v = rnd_(P.linear(n, pw[p + "self_attn.v_proj.weight"])).reshape(T, sz["nkv"], sz["hd"])
    rows = np.asarray(rows)
    q = rnd_(P.rope(rnd_(P.linear(n[rows], pw[p + "self_attn.q_proj.weight"])).reshape(len(rows), sz["nq"], sz["hd"]),
                    rows, inv, sz["pairing"]))
    out = np.zeros((len(rows), sz["nq"], sz["hd"]), np.float32)
    W = P.layer_window(sz, 0)
    g = sz["nq"] // sz["nkv"]
    for r, i in enumerate(rows):                 # the keys of query i are lo..i
        lo = 0 if W is None else max(0, i - W + 1)
        out[r] = _one_query(q[r], k[lo:i + 1], v[lo:i + 1], g, sz["hd"], rnd_)
    o = rnd_(out).reshape(len(rows), -1)
    xl = x[rows] + P.linear(o, pw[p + "self_attn.o_proj.weight"])
    xl = P.ffn_block(xl, pw, p, sz, rnd_)
    head = pw["model.embed_tokens.weight"] if sz["tied"] else pw["lm_head.weight"]
    return P.linear(rnd_(P.rms_norm(xl, pw["model.norm.weight"], sz["eps"])), head)


def _one_query(q, k, v, g, hd, rnd_):
    """P.attention's formula for one query that sees every given key (a 1 x n problem per head)."""
    out = np.zeros((q.shape[0], hd), np.float32)
    for h in range(q.shape[0]):
        s = (k[:, h // g] @ q[h]) * np.float32(1.0 / np.sqrt(hd))
        e = np.exp(s - s.max(), dtype=np.float32)
        out[h] = (e / e.sum(dtype=np.float32)) @ v[:, h // g] if rnd_ is P._same else (rnd_(e) @ v[:, h // g]) / e.sum(dtype=np.float32)
    return out


TOL = {"float32": 1e-4, "bfloat16": 3e-2}
COS = {"float32": 0.999999, "bfloat16": 0.999}


def close(got, want, dtype, what):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape and np.isfinite(got).all(), what
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err <= TOL[dtype], f"{what}: error {err:.3e}"
    cos = (got * want).sum(-1) / (np.linalg.norm(got, axis=-1) * np.linalg.norm(want, axis=-1))
    assert cos.min() >= COS[dtype], f"{what}: cosine {cos.min():.6f} at row {int(cos.argmin())}"


def test_plain_rows_is_the_plain_forward():
    cfg = dict(num_hidden_layers=1, hidden_size=32, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
               intermediate_size=48, vocab_size=60, sliding_window=70)
    w = P.random_weights(cfg, 2, std=0.2)
    toks = [int(t) for t in np.random.default_rng(0).integers(0, 60, 150)]
    rows = [0, 1, 63, 64, 69, 70, 71, 149]
    for act in (None, "bfloat16"):
        full = P.forward(cfg, w, toks, act_dtype=act)
        assert np.abs(plain_rows(cfg, w, toks, rows, act) - full[rows]).max() < 2e-5 * np.abs(full).max()


@pytest.fixture(scope="module")
def one_layer_7b(tmp_path_factory):
    folder = str(tmp_path_factory.mktemp("one_layer_7b"))
    cfg = B.preset("mistral-7b-v0.3", num_hidden_layers=1, vocab_size=2000)
    B.Engine.write_random_folder(folder, cfg, seed=23, std=0.02, vector_jitter=0.3, device=DEV)
    pc, pw = P.read_folder(folder)
    return folder, pc, pw


def test_a_prompt_of_2048_tokens_at_the_7b_layer_sizes(one_layer_7b):
    """What the benchmark's prefill runs (256x192, 256x256 and 128x256 tiles at 2,048 rows, flash
    attention over 32 pages), whole and as two steps of 1,024, against the plain implementation at
    rows spread over the prompt."""
    folder, pc, pw = one_layer_7b
    eng = B.Engine.from_folder(folder, dtype="bfloat16", max_tokens=4096)
    toks = [int(t) for t in np.random.default_rng(3).integers(0, pc["vocab_size"], 2048)]
    rows = [0, 1, 63, 64, 255, 256, 1000, 1023, 1024, 1025, 1500, 2046, 2047]
    ref = plain_rows(pc, pw, toks, rows)
    s = eng.alloc_slot()
    got = eng.step([StepEntry(s, toks, rows)]).cpu().numpy()
    eng.free_slot(s)
    close(got, ref, "bfloat16", "2,048 tokens whole")
    s = eng.alloc_slot()
    a = eng.step([StepEntry(s, toks[:1024], [r for r in rows if r < 1024])]).cpu().numpy()
    b = eng.step([StepEntry(s, toks[1024:], [r - 1024 for r in rows if r >= 1024])]).cpu().numpy()
    eng.free_slot(s)
    cut = np.concatenate([a, b])
    close(cut, ref, "bfloat16", "2,048 tokens as 2 x 1,024")
    assert np.abs(cut - got).max() <= 2e-2 * np.abs(ref).max()


def test_one_layer_of_the_24b_widths(tmp_path):
    """Hidden 5,120, 32 heads of 128 over 8 kv heads (q width 4,096), intermediate 32,768, a small
    vocabulary: a prompt of 300 tokens whole, its last tokens one by one, 20 requests together."""
    cfg = B.preset("mistral-small-24b", num_hidden_layers=1, vocab_size=1500)
    folder = str(tmp_path / "m")
    B.Engine.write_random_folder(folder, cfg, seed=29, std=0.02, vector_jitter=0.3, device=DEV)
    pc, pw = P.read_folder(folder)
    eng = B.Engine.from_folder(folder, dtype="bfloat16", max_tokens=8192)
    toks = [int(t) for t in np.random.default_rng(4).integers(0, 1500, 300)]
    ref = P.forward(pc, pw, toks)
    s = eng.alloc_slot()
    close(eng.step([StepEntry(s, toks, list(range(300)))]).cpu().numpy(), ref, "bfloat16", "24B widths, whole")
    eng.free_slot(s)
    s = eng.alloc_slot()
    parts = [eng.step([StepEntry(s, toks[:294], [293])]).cpu().numpy()]
    for t in toks[294:]:
        parts.append(eng.step([StepEntry(s, [t], [0])]).cpu().numpy())
    eng.free_slot(s)
    close(np.concatenate(parts), ref[293:], "bfloat16", "24B widths, last tokens one by one")
    lens = [2 + 7 * i for i in range(20)]
    slots = [eng.alloc_slot() for _ in lens]
    first = eng.step([StepEntry(sl, toks[:n], [n - 1]) for sl, n in zip(slots, lens)]).cpu().numpy()
    then = eng.step([StepEntry(sl, [toks[n]], [0]) for sl, n in zip(slots, lens)]).cpu().numpy()
    for sl in slots:
        eng.free_slot(sl)
    close(first, ref[[n - 1 for n in lens]], "bfloat16", "24B widths, 20 prompts in one step")
    close(then, ref[lens], "bfloat16", "24B widths, one token each after them")


# -------------------------------------------- windowed sequences decoding together from a graph ----
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_eight_windowed_sequences_of_thousands_of_tokens_decode_together(tmp_path, dtype):
    """The marker model at head size 128 with a window of 4,096: eight sequences of 4,100 to 7,200
    tokens decode 70 tokens together from a graph, every decoded token the asker.  Each sequence's
    marker sits where it leaves the window at a step of its own (seen at distance 4,095, not at
    4,096); sequences cross page edges at different steps, returning the page behind the window
    while others return none.  Every step's logits against the plain implementation."""
    from test_engine_gpu import _marker_model
    folder, pc, pw = _marker_model(tmp_path, sliding_window=4096, head_dim=128, rope_theta=1e8, max_positions=16384)
    steps = 70
    rng = np.random.default_rng(6)
    lens = [4100, 4159, 4160, 5000, 5695, 6400, 7001, 7200]
    leaves_at = [0, 3, 69, 17, 64, 40, 1, 1000]          # the decode step at which the marker is first out of sight (1000: never within the run)
    seqs = []
    for n, s_out in zip(lens, leaves_at):
        toks = [int(x) for x in rng.integers(3, 40, n)] + [2] * steps
        toks[n + s_out - 4096] = 1                          # the query at n + s_out is the first not to see it
        seqs.append(toks)
    eng = B.Engine.from_folder(folder, dtype=dtype, max_tokens=8 * 7360, max_seq_len=7360)
    assert eng.use_graphs
    slots = [eng.alloc_slot() for _ in seqs]
    for sl, toks, n in zip(slots, seqs, lens):
        eng.step([StepEntry(sl, toks[:n], [])])
    got = []
    for t in range(steps):
        got.append(eng.step([StepEntry(sl, [toks[n + t]], [0]) for sl, toks, n in zip(slots, seqs, lens)]).cpu().numpy())
        assert eng.cache.groups[0].pool.held_count <= 8 * (4096 // 64 + 1)       # pages behind the window went back
    assert 8 in eng._graphs.graphs
    got = np.stack(got, 1)                                   # [sequence, step, vocab]
    for b, (toks, n, s_out) in enumerate(zip(seqs, lens, leaves_at)):
        ref = plain_rows(pc, pw, toks, list(range(n, n + steps)))
        sees = [int(r.argmax()) == 1 for r in ref]
        assert sees == [t < s_out for t in range(steps)], "the plain implementation must see the marker exactly inside the window"
        assert [int(r.argmax()) == 1 for r in got[b]] == sees, f"sequence {b}: the window's edge is off"
        close(got[b], ref, dtype, f"sequence {b} of {n} tokens")
    for sl in slots:
        eng.free_slot(sl)
    assert eng.cache.groups[0].pool.held_count == 0


# --------------------------------------------------------------- the sampled configuration ----
def test_sampled_generation_equals_the_plain_sampled_loop(engines, tiny_folders):
    """The benchmark description's second configuration: prompts of 3, 11, 17 and 20 tokens, 12 tokens
    each at temperature 0.7 from a seed, in 32-bit: the tokens of the plain loop (history = prompt and
    everything generated, one uniform number a token, a request's numbers its own), also with the other
    options of the sampler on and with requests served in two batches."""
    _, cfg, w = tiny_folders["b"]
    eng = engines("b", "float32")
    rng = np.random.default_rng(1)
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for n in (3, 11, 17, 20)]
    for opts in (dict(temperature=0.7, top_k=0), dict(temperature=0.9, top_k=12, top_p=0.9, repetition_penalty=1.3),
                 dict(temperature=1.2, top_k=0, min_p=0.02, logit_bias=[(5, 1.5), (7, -2.0)])):
        want = [P.sampled_generate(cfg, w, p, 12, seed=1234, sequence=i, **opts) for i, p in enumerate(prompts)]
        assert eng.generate(prompts, max_new_tokens=12, seed=1234, stop_token_ids=[], **opts) == want
        assert eng.generate(prompts, max_new_tokens=12, seed=1234, stop_token_ids=[], max_batch=2, **opts) == want
    assert len({tuple(x) for x in want}) == 4
