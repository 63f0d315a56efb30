"""The engine against the plain implementation on the GPU, in 32-bit and in bfloat16,
under every way of cutting the work: each request alone and whole; with the last 32
tokens one by one; in batches of unequal lengths whose shorter requests end earlier, one
batch after another so that slots are used again; long decoding; the first tokens."""
import numpy as np
import pytest
import torch

import braidinfer_amd as B
import plain_mistral as P
from braidinfer_amd import StepEntry

pytestmark = pytest.mark.gpu

# Bounds, fixed up front.  32-bit: the engine and the plain implementation differ only in
# the order of float additions: 1e-4 of the largest logit.  bfloat16: activations, keys and
# values carry 8 significant bits (relative 2^-9 per rounding), a few dozen roundings deep:
# 3e-2 of the largest logit, and every position's logits point the same way (cosine).
TOL = {"float32": 1e-4, "bfloat16": 3e-2}
COS = {"float32": 0.999999, "bfloat16": 0.999}
# the same position through different cuts, both from the engine: equal in 32-bit (the
# 32-bit kernels add in an order that does not depend on the cut), rounding apart in bf16
CUT_TOL = {"float32": 0.0, "bfloat16": 2e-2}


def tokens(cfg, n, seed):
    return [int(t) for t in np.random.default_rng(seed).integers(0, cfg["vocab_size"], n)]


def close(got, want, dtype, what=""):
    got, want = np.asarray(got, np.float32), np.asarray(want, np.float32)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite logits"
    scale = np.abs(want).max()
    err = np.abs(got - want).max()
    assert err <= TOL[dtype] * scale, f"{what}: max error {err:.3e} against {scale:.3e} ({dtype})"
    cos = (got * want).sum(-1) / (np.linalg.norm(got, axis=-1) * np.linalg.norm(want, axis=-1))
    assert cos.min() >= COS[dtype], f"{what}: cosine {cos.min():.6f} at position {int(cos.argmin())}"


def close_or_rounding(got, want, rounded, what=""):
    """bfloat16 at widths where the usual bound has no footing (a norm over one or three elements
    turns a rounding of the residual row into a change of sign or direction; a cosine over two
    logits is an angle of noise): the engine may differ from the float result by no more than the
    usual bound or three times what the plain implementation itself moves by when it rounds its
    activations to bfloat16 where a bfloat16 engine does (`rounded`)."""
    got, want, rounded = (np.asarray(a, np.float64) for a in (got, want, rounded))
    assert got.shape == want.shape and np.isfinite(got).all(), what
    scale = np.abs(want).max()

    def dist(a):
        cos = (a * want).sum(-1) / (np.linalg.norm(a, axis=-1) * np.linalg.norm(want, axis=-1) + 1e-300)
        return np.abs(a - want).max() / scale, 1.0 - cos.min()
    (err, ang), (err_r, ang_r) = dist(got), dist(rounded)
    assert err <= max(TOL["bfloat16"], 3 * err_r), f"{what}: error {err:.3e}, rounding alone gives {err_r:.3e}"
    assert ang <= max(1 - COS["bfloat16"], 3 * ang_r), f"{what}: 1 - cosine {ang:.3e}, rounding alone gives {ang_r:.3e}"


def whole(engine, toks):
    s = engine.alloc_slot()
    try:
        return engine.step([StepEntry(s, toks, list(range(len(toks))))]).cpu().numpy()
    finally:
        engine.free_slot(s)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_each_request_alone_and_whole(engines, tiny_folders, name, dtype):
    _, cfg, w = tiny_folders[name]
    eng = engines(name, dtype)
    for n, seed in ((1, 0), (7, 1), (64, 2), (65, 3), (200, 4)):
        toks = tokens(cfg, n, seed)
        close(whole(eng, toks), P.forward(cfg, w, toks), dtype, f"{name} whole n={n}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_last_32_tokens_one_by_one(engines, tiny_folders, name, dtype):
    _, cfg, w = tiny_folders[name]
    eng = engines(name, dtype)
    toks = tokens(cfg, 150, 10)
    ref = P.forward(cfg, w, toks)
    one = whole(eng, toks)
    s = eng.alloc_slot()
    n0 = len(toks) - 32
    parts = [eng.step([StepEntry(s, toks[:n0], list(range(n0)))]).cpu().numpy()]
    for t in toks[n0:]:
        parts.append(eng.step([StepEntry(s, [t], [0])]).cpu().numpy())
    assert eng.length(s) == len(toks)
    eng.free_slot(s)
    cut = np.concatenate(parts)
    close(cut, ref, dtype, f"{name} last 32 one by one")
    assert np.abs(cut - one).max() <= CUT_TOL[dtype] * np.abs(ref).max()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_unequal_batches_one_after_another(engines, tiny_folders, name, dtype):
    """Prompts of unequal lengths in one step, then one token each; shorter requests end
    earlier; three batches on one engine so that slots and pages are used again."""
    _, cfg, w = tiny_folders[name]
    eng = engines(name, dtype)
    free_before = [g.pool.free_count for g in eng.cache.groups]
    for round_, lens in enumerate(([3, 11, 17, 20], [70, 5, 129, 64, 1], [40, 41])):
        total = [n + 6 + 3 * i for i, n in enumerate(lens)]        # requests end at different steps
        seqs = [tokens(cfg, t, 100 * round_ + i) for i, t in enumerate(total)]
        refs = [P.forward(cfg, w, s) for s in seqs]
        slots = [eng.alloc_slot() for _ in seqs]
        got = [[] for _ in seqs]
        out = eng.step([StepEntry(sl, s[:n], list(range(n))) for sl, s, n in zip(slots, seqs, lens)]).cpu().numpy()
        o = 0
        for i, n in enumerate(lens):
            got[i].append(out[o:o + n]); o += n
        pos = list(lens)
        live = list(range(len(seqs)))
        while live:
            out = eng.step([StepEntry(slots[i], [seqs[i][pos[i]]], [0]) for i in live]).cpu().numpy()
            for r, i in enumerate(live):
                got[i].append(out[r:r + 1]); pos[i] += 1
            for i in [i for i in live if pos[i] == total[i]]:
                eng.free_slot(slots[i]); live.remove(i)
        for i in range(len(seqs)):
            close(np.concatenate(got[i]), refs[i], dtype, f"{name} batch {round_} request {i}")
    assert [g.pool.free_count for g in eng.cache.groups] == free_before     # every page came back


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_crosses_pages_and_the_window(engines, tiny_folders, dtype):
    name = "c"                                     # window 70 on layers 0 and 2, full on 1 and 3
    _, cfg, w = tiny_folders[name]
    eng = engines(name, dtype)
    toks = tokens(cfg, 5 + 300, 20)
    ref = P.forward(cfg, w, toks)
    s = eng.alloc_slot()
    got = [eng.step([StepEntry(s, toks[:5], [4])]).cpu().numpy()]
    for t in toks[5:]:
        got.append(eng.step([StepEntry(s, [t], [0])]).cpu().numpy())
    gw = eng.cache.groups[0]
    assert gw.need.window == 70 and gw.pool.held_count <= 3       # pages behind the window went back
    eng.free_slot(s)
    close(np.concatenate(got), ref[4:], dtype, "long decoding")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(engines, tiny_folders, dtype):
    """Positions 0, 1, 2: a one-token prompt, then single tokens (the reference sends a
    one-token prompt through its decode path, generate.rs:328-329)."""
    for name in ("a", "b"):
        _, cfg, w = tiny_folders[name]
        eng = engines(name, dtype)
        toks = tokens(cfg, 4, 30)
        ref = P.forward(cfg, w, toks)
        s = eng.alloc_slot()
        got = [eng.step([StepEntry(s, [t], [0])]).cpu().numpy() for t in toks]
        eng.free_slot(s)
        close(np.concatenate(got), ref, dtype, f"{name} first tokens")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_wanted_places_and_chunked_prompts(engines, tiny_folders, dtype):
    _, cfg, w = tiny_folders["b"]
    eng = engines("b", dtype)
    toks = tokens(cfg, 90, 40)
    ref = P.forward(cfg, w, toks)
    a, b = eng.alloc_slot(), eng.alloc_slot()
    # nothing wanted in the first step; prompts cut at different places in the second
    out = eng.step([StepEntry(a, toks[:50], []), StepEntry(b, toks[:13], [12, 0])]).cpu().numpy()
    close(out, ref[[12, 0]], dtype, "wanted places")
    out = eng.step([StepEntry(a, toks[50:], [39]), StepEntry(b, toks[13:70], [0, 56])]).cpu().numpy()
    close(out, ref[[89, 13, 69]], dtype, "chunked prompt")
    eng.free_slot(a); eng.free_slot(b)


def _marker_model(tmp_path, sliding_window=None, head_dim=16, rope_theta=10000.0, max_positions=4096):
    """A one-layer model in which token 2 (the asker) attends almost only to token 1 (the
    marker), wherever it sits, and copies its content into the logits."""
    hd = head_dim
    cfg = B.MistralConfig.from_dict(dict(num_hidden_layers=1, hidden_size=32, num_attention_heads=2,
                                         num_key_value_heads=1, head_dim=hd, intermediate_size=16,
                                         vocab_size=40, rope_theta=rope_theta, rms_norm_eps=1e-5,
                                         max_position_embeddings=max_positions, sliding_window=sliding_window))
    folder = B.Engine.write_random_folder(str(tmp_path / f"m{hd}"), cfg, seed=1, std=0.02)
    from braidinfer_amd.weights import SafetensorsFolder, write_safetensors
    st = SafetensorsFolder(folder)
    t = {n: st.tensor(n).clone() for n in st.names()}
    H = 32
    emb = torch.zeros(40, H)
    content = torch.randn(40, 8, generator=torch.Generator().manual_seed(0))
    emb[:, :8] = content / content.norm(dim=-1, keepdim=True) * 8 ** 0.5              # content, equal norms
    emb[1, 8] = 8.0          # token 1 is the marker: it alone has a large key direction
    emb[2, 9] = 8.0          # token 2 is the asker: it alone has the matching query direction
    t["model.embed_tokens.weight"] = emb.bfloat16()
    q = torch.zeros(2 * hd, H); k = torch.zeros(hd, H); v = torch.zeros(hd, H); o = torch.zeros(H, 2 * hd)
    # rotary leaves the last pair of each half almost unrotated at these positions (lowest
    # frequency): put the matching direction there (elements hd/2 - 1 and hd - 1 pair up in "half")
    q[hd // 2 - 1, 9] = 6.0; k[hd // 2 - 1, 8] = 6.0
    v[:8, :8] = torch.eye(8) * 4
    o[10:18, :8] = torch.eye(8)
    for n_, m in (("q", q), ("k", k), ("v", v), ("o", o)):
        t[f"model.layers.0.self_attn.{n_}_proj.weight"] = m.bfloat16()
    for n_ in ("gate", "up", "down"):
        t[f"model.layers.0.mlp.{n_}_proj.weight"] = torch.zeros_like(t[f"model.layers.0.mlp.{n_}_proj.weight"])
    head = torch.zeros(40, H); head[:, 10:18] = emb[:, :8]
    t["lm_head.weight"] = head.bfloat16()
    write_safetensors(f"{folder}/model.safetensors", t.items())
    pc, pw = P.read_folder(folder)
    return folder, pc, pw


def test_a_far_key_among_hundreds_is_found(tmp_path):
    """Random weights give near-uniform attention, which would hide a lost key.  Here the
    weights are made so that the last token's query matches one early key far more than
    any other: one head copies that token's value, and its identity shows in the logits."""
    folder, pc, pw = _marker_model(tmp_path)
    rng = np.random.default_rng(0)
    for dtype in ("float32", "bfloat16"):
        eng = B.Engine.from_folder(folder, dtype=dtype, max_tokens=1024)
        for far in (0, 63, 64, 300):
            toks = [int(x) for x in rng.integers(3, 40, 500)]
            toks[far] = 1                     # the marker sits `far`; its value is its own content...
            toks[-1] = 2
            ref = P.forward(pc, pw, toks)[-1]
            s = eng.alloc_slot()
            eng.step([StepEntry(s, toks[:-1], [])])
            got = eng.step([StepEntry(s, [toks[-1]], [0])]).cpu().numpy()[0]
            eng.free_slot(s)
            assert int(ref.argmax()) == 1, "the test's weights must make the marker win in the plain implementation"
            assert int(got.argmax()) == 1, f"{dtype}: the key at position {far} was lost"
            close(got[None], ref[None], dtype, f"far key at {far}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_equal_eager_steps(tiny_folders, dtype):
    """Single-token steps are replayed from HIP graphs.  Every replay is checked against
    the same step run eagerly on a second engine, with eager work (prompts of other
    requests, slots freed and used again, batch sizes that change) between the replays."""
    folder, cfg, w = tiny_folders["b"]
    g = B.Engine.from_folder(folder, dtype=dtype, max_tokens=2048)
    e = B.Engine.from_folder(folder, dtype=dtype, max_tokens=2048, use_graphs=False)
    assert g.use_graphs and not e.use_graphs
    rng = np.random.default_rng(0)
    seqs = [tokens(cfg, 90, 50 + i) for i in range(5)]
    slots_g, slots_e, pos = {}, {}, {}

    def start(i, n):
        slots_g[i], slots_e[i], pos[i] = g.alloc_slot(), e.alloc_slot(), n
        a = g.step([StepEntry(slots_g[i], seqs[i][:n], [n - 1])]).cpu().numpy()
        b_ = e.step([StepEntry(slots_e[i], seqs[i][:n], [n - 1])]).cpu().numpy()
        assert np.array_equal(a, b_)

    def stop(i):
        g.free_slot(slots_g.pop(i)); e.free_slot(slots_e.pop(i)); pos.pop(i)

    start(0, 10); start(1, 3)
    for it in range(60):
        live = sorted(pos)
        a = g.step([StepEntry(slots_g[i], [seqs[i][pos[i]]], [0]) for i in live]).cpu().numpy()
        b_ = e.step([StepEntry(slots_e[i], [seqs[i][pos[i]]], [0]) for i in live]).cpu().numpy()
        ref = np.stack([P.forward(cfg, w, seqs[i][:pos[i] + 1])[-1] for i in live])
        close(a, ref, dtype, f"replay {it}")
        # the split count of the graph follows the cache's longest sequence, the eager step's its
        # own: the same numbers added in another order
        assert np.abs(a - b_).max() <= CUT_TOL[dtype] * np.abs(ref).max() + 1e-5 * np.abs(ref).max()
        for i in live:
            pos[i] += 1
        if it == 5: start(2, 40)
        if it == 9: stop(1)
        if it == 12: start(3, 64); start(1, 7)
        if it == 30: stop(0); start(4, 5)
        for i in [i for i in pos if pos[i] >= 89]:
            stop(i)
        if not pos:
            break


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_with_the_callers_position_numbers_replay_from_graphs_too(tiny_folders, dtype):
    """Single-token steps whose entries bring position numbers of their own (here each token's place plus
    1,000: rotary attention sees distances only, so the plain forward at shifted positions is the reference
    and equals the unshifted one) run from recorded steps of their own, next to the plain ones, with the
    results of eager steps."""
    folder, cfg, w = tiny_folders["a"]
    g = B.Engine.from_folder(folder, dtype=dtype, max_tokens=2048)
    e = B.Engine.from_folder(folder, dtype=dtype, max_tokens=2048, use_graphs=False)
    seqs = [tokens(cfg, 40, 70 + i) for i in range(3)]
    refs = [P.forward(cfg, w, q, positions=np.arange(len(q)) + 1000) for q in seqs]
    assert all(np.abs(r - P.forward(cfg, w, q)).max() < 1e-4 * np.abs(r).max() for r, q in zip(refs, seqs))
    got = {}
    for eng in (g, e):
        slots = [eng.alloc_slot() for _ in seqs]
        n0 = [5, 17, 30]
        eng.step([StepEntry(sl, q[:n], [], position_ids=[1000 + t for t in range(n)]) for sl, q, n in zip(slots, seqs, n0)])
        rows = [[] for _ in seqs]
        for k in range(10):
            live = [i for i in range(3) if n0[i] + k < 40]
            out = eng.step([StepEntry(slots[i], [seqs[i][n0[i] + k]], [0], position_ids=[1000 + n0[i] + k]) for i in live])
            # a plain step of another request in between: its recorded step is another one
            other = eng.alloc_slot()
            eng.step([StepEntry(other, [3], [0])])
            eng.free_slot(other)
            for r, i in enumerate(live):
                rows[i].append(out[r:r + 1].cpu().numpy())
        for sl in slots:
            eng.free_slot(sl)
        got[eng.use_graphs] = [np.concatenate(r) for r in rows]
    assert g._graphs is not None and (4, 1) in g._graphs.with_ids and 1 in g._graphs.graphs and e._graphs is None
    for i in range(3):
        ref = refs[i][[5, 17, 30][i]:[5, 17, 30][i] + 10]
        close(got[True][i], ref, dtype, f"request {i} with shifted positions, from a graph")
        assert np.abs(got[True][i] - got[False][i]).max() <= CUT_TOL[dtype] * np.abs(ref).max()


@pytest.mark.parametrize("which", ["all", "some"])
def test_tensors_stored_in_32_bit_stay_so_in_the_bfloat16_engine(tmp_path, which):
    """A matrix stored as F32 is multiplied in 32-bit even when the engine runs in bfloat16
    (its activations are widened for it); bf16 and F32 matrices may meet in one model."""
    import torch
    from braidinfer_amd.weights import SafetensorsFolder, write_safetensors
    cfg = B.MistralConfig.from_dict(dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=4,
                                         num_key_value_heads=2, head_dim=16, intermediate_size=96, vocab_size=120,
                                         max_position_embeddings=512))
    folder = B.Engine.write_random_folder(str(tmp_path / "m"), cfg, seed=3, std=0.1, vector_jitter=0.2)
    st = SafetensorsFolder(folder)
    wide = (lambda n: True) if which == "all" else (lambda n: n in ("lm_head.weight", "model.layers.0.self_attn.q_proj.weight",
                                                                    "model.layers.1.mlp.up_proj.weight", "model.norm.weight"))
    write_safetensors(f"{folder}/model.safetensors",
                      [(n, st.tensor(n).float() if wide(n) else st.tensor(n).clone()) for n in st.names()])
    pc, pw = P.read_folder(folder)
    eng = B.Engine.from_folder(folder, dtype="bfloat16", max_tokens=512)
    assert eng.model.lm_head.weight.dtype == torch.float32
    assert eng.model.layers[1].feed_forward.w_d.dtype == (torch.float32 if which == "all" else torch.bfloat16)
    toks = tokens(pc, 70, 3)
    ref = P.forward(pc, pw, toks)
    s = eng.alloc_slot()
    got = [eng.step([StepEntry(s, toks[:50], list(range(50)))]).cpu().numpy()]
    for t in toks[50:]:
        got.append(eng.step([StepEntry(s, [t], [0])]).cpu().numpy())
    eng.free_slot(s)
    close(np.concatenate(got), ref, "bfloat16", f"32-bit tensors ({which})")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_windows_edge_is_exact(tmp_path, dtype):
    """With a window of 100 the asker at position 499 sees position 400 and not 399.  The
    marker on either side of that edge decides the logits, for the asker decoded alone, as
    the end of a whole prompt, and as the end of a chunk."""
    folder, pc, pw = _marker_model(tmp_path, sliding_window=100)
    eng = B.Engine.from_folder(folder, dtype=dtype, max_tokens=1024)
    rng = np.random.default_rng(1)
    for at, seen in ((400, True), (399, False), (499 - 63, True), (401, True)):
        toks = [int(x) for x in rng.integers(3, 40, 500)]
        toks[at] = 1
        toks[-1] = 2
        ref = P.forward(pc, pw, toks)[-1]
        assert (int(ref.argmax()) == 1) == seen, "the plain implementation must see the marker exactly inside the window"
        for cut in (499, 0, 450):                    # asker alone; whole prompt; a last chunk of 50
            s = eng.alloc_slot()
            if cut:
                eng.step([StepEntry(s, toks[:cut], [])])
            got = eng.step([StepEntry(s, toks[cut:], [len(toks) - cut - 1])]).cpu().numpy()[0]
            eng.free_slot(s)
            assert (int(got.argmax()) == 1) == seen, f"marker at {at}, cut {cut}: window edge is off"
            close(got[None], ref[None], dtype, f"window edge, marker at {at}, cut {cut}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["b", "c"])
def test_random_schedules_of_cuts_and_batches(engines, tiny_folders, name, dtype):
    """Requests arrive at random steps, bring chunks of random sizes (1, a few, a page and
    more), leave when they are done; every position's logits are compared with the plain
    implementation, whatever the step it fell into."""
    _, cfg, w = tiny_folders[name]
    eng = engines(name, dtype)
    rng = np.random.default_rng(7 if name == "b" else 8)
    free_before = [g.pool.free_count for g in eng.cache.groups]
    seqs = [tokens(cfg, int(n), 200 + i) for i, n in enumerate(rng.integers(1, 260, 9))]
    refs = [P.forward(cfg, w, s) for s in seqs]
    waiting = list(range(len(seqs)))
    live, pos, got = {}, {}, {i: [] for i in range(len(seqs))}
    while waiting or live:
        for i in list(waiting):
            if len(live) < 4 and rng.random() < 0.5:
                waiting.remove(i); live[i] = eng.alloc_slot(); pos[i] = 0
        if not live:
            continue
        chosen = [i for i in live if rng.random() < 0.8] or list(live)[:1]
        entries, takes = [], []
        for i in chosen:
            n = min(int(rng.choice([1, 1, 2, 7, 64, 65, 130])), len(seqs[i]) - pos[i])
            entries.append(StepEntry(live[i], seqs[i][pos[i]:pos[i] + n], list(range(n))))
            takes.append(n)
        out = eng.step(entries).cpu().numpy()
        o = 0
        for i, n in zip(chosen, takes):
            got[i].append(out[o:o + n]); o += n; pos[i] += n
            if pos[i] == len(seqs[i]):
                eng.free_slot(live.pop(i))
    for i in range(len(seqs)):
        close(np.concatenate(got[i]), refs[i], dtype, f"{name} request {i} of {len(seqs[i])} tokens")
    assert [g.pool.free_count for g in eng.cache.groups] == free_before


# ---- sizes that take the kernels of serving shapes -------------------------------------
# The tiny configurations run through the kernels for any shape.  This one is wide enough
# for the others: head size 128 (attention through LDS rings, for prompts and for single
# tokens), widths of 1024 and 1536 (products by direct-to-LDS tiles for prompts, by the
# streaming kernels for 1 to 16 and 17 to 64 rows), a vocabulary that is no multiple of 16,
# a window on one of the two layers.
SERVING = dict(num_hidden_layers=2, hidden_size=1024, num_attention_heads=8, num_key_value_heads=2, head_dim=128,
               intermediate_size=1536, vocab_size=1000, rope_theta=1e6, rms_norm_eps=1e-5, sliding_window=100,
               max_position_embeddings=4096, tie_word_embeddings=False,
               layer_types=["full_attention", "sliding_attention"])


@pytest.fixture(scope="module")
def serving(tmp_path_factory):
    folder = str(tmp_path_factory.mktemp("serving_sizes"))
    B.Engine.write_random_folder(folder, B.MistralConfig.from_dict(SERVING), seed=3, std=0.03, vector_jitter=0.3)
    cfg, w = P.read_folder(folder)
    return folder, cfg, w


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_serving_sizes_whole_then_one_by_one_then_batched(serving, dtype):
    folder, cfg, w = serving
    eng = B.Engine.from_folder(folder, dtype=dtype, max_tokens=8192)
    toks = tokens(cfg, 340, 7)
    ref = P.forward(cfg, w, toks)
    one = whole(eng, toks)
    close(one, ref, dtype, "serving sizes, whole")
    s = eng.alloc_slot()
    n0 = 300
    parts = [eng.step([StepEntry(s, toks[:n0], list(range(n0)))]).cpu().numpy()]
    for t in toks[n0:]:
        parts.append(eng.step([StepEntry(s, [t], [0])]).cpu().numpy())
    eng.free_slot(s)
    cut = np.concatenate(parts)
    close(cut, ref, dtype, "serving sizes, last 40 one by one")
    assert np.abs(cut - one).max() <= CUT_TOL[dtype] * np.abs(ref).max()
    # 20 requests of unequal lengths: prompts in one step, then 6 tokens each in steps of 20 rows
    lens = [5 + 13 * i for i in range(20)]
    seqs = [tokens(cfg, n + 6, 50 + i) for i, n in enumerate(lens)]
    slots = [eng.alloc_slot() for _ in seqs]
    got = [[] for _ in seqs]
    out = eng.step([StepEntry(sl, q[:n], [n - 1]) for sl, q, n in zip(slots, seqs, lens)]).cpu().numpy()
    for i in range(20):
        got[i].append(out[i:i + 1])
    for k in range(6):
        out = eng.step([StepEntry(sl, [q[n + k]], [0]) for sl, q, n in zip(slots, seqs, lens)]).cpu().numpy()
        for i in range(20):
            got[i].append(out[i:i + 1])
    for sl in slots:
        eng.free_slot(sl)
    for i in (0, 7, 19):
        close(np.concatenate(got[i]), P.forward(cfg, w, seqs[i])[lens[i] - 1:], dtype, f"serving sizes, request {i} of 20")


def test_single_token_steps_launch_few_norm_kernels(serving, monkeypatch):
    """bfloat16, steps of up to 64 rows, sizes the streaming products take: only the first
    layer's first norm and the final norm run as kernels of their own; the others are prepared
    by the product before them.  A longer prompt runs all five."""
    from braidinfer_amd import kernels as K
    folder, cfg, w = serving
    eng = B.Engine.from_folder(folder, dtype="bfloat16", max_tokens=1024, use_graphs=False)
    calls = []
    real = K.rmsnorm
    monkeypatch.setattr(K, "rmsnorm", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    s = eng.alloc_slot()
    eng.step([StepEntry(s, tokens(cfg, 100, 1), [99])])
    assert len(calls) == 2 * cfg["num_hidden_layers"] + 1
    calls.clear()
    eng.step([StepEntry(s, [5], [0])])
    assert len(calls) == 2
    calls.clear()
    eng.step([StepEntry(s, tokens(cfg, 40, 2), [39])])
    assert len(calls) == 2
    eng.free_slot(s)


@pytest.mark.parametrize("live", [17, 24, 48, 64])
def test_single_token_steps_of_17_to_64_rows_add_the_runs_of_q_k_v_inside_attention(serving, live, monkeypatch):
    """At 17 to 64 rows the product that makes queries, keys and values is cut along k; its
    runs are added by the attention kernel for the heads it reads, not by a launch of their own.
    The step must give the bits it gives with that launch, and the cache the same keys and values
    (the next step reads them)."""
    from braidinfer_amd.parts import attention as A
    folder, cfg, w = serving
    rng = np.random.default_rng(live)
    lens = [int(x) for x in rng.integers(1, 150, live)]
    seqs = [tokens(cfg, n + 2, 300 + i) for i, n in enumerate(lens)]
    outs = []
    for fold in (True, False):
        eng = B.Engine.from_folder(folder, dtype="bfloat16", max_tokens=16384, use_graphs=False)
        used = []
        real = A.linear_runs
        if fold:
            monkeypatch.setattr(A, "linear_runs", lambda *a: (lambda r: (used.append(r is not None), r)[1])(real(*a)))
        else:
            monkeypatch.setattr(A, "linear_runs", lambda *a: None)
        slots = [eng.alloc_slot() for _ in range(live)]
        eng.step([StepEntry(sl, sq[:n], []) for sl, sq, n in zip(slots, seqs, lens)])
        a = eng.step([StepEntry(sl, [sq[n]], [0]) for sl, sq, n in zip(slots, seqs, lens)])
        b = eng.step([StepEntry(sl, [sq[n + 1]], [0]) for sl, sq, n in zip(slots, seqs, lens)])
        outs.append((a.clone(), b.clone()))
        if fold:
            assert used and all(used), "the product of q, k and v was not left in runs"
        monkeypatch.setattr(A, "linear_runs", real)
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    for i in (0, live // 2, live - 1):
        close(np.stack([outs[0][0][i].cpu().numpy(), outs[0][1][i].cpu().numpy()]),
              P.forward(cfg, w, seqs[i])[lens[i]:], "bfloat16", f"request {i} of {live}")


@pytest.mark.parametrize("dtype,layout", [("float32", ""), ("bfloat16", ""), ("bfloat16", "blocks")])
def test_serving_sizes_random_schedule(serving, dtype, layout, monkeypatch):
    """The random schedule at the sizes that take the serving kernels: up to 30 requests live,
    so steps bring 1 to 16, 17 to 64 and more rows; chunks of 1 (mostly), a few, and more than
    a page.  Once more with every matrix in the blocked layout that only wide matrices get
    by themselves (none of this configuration is wide enough)."""
    folder, cfg, w = serving
    if layout:
        monkeypatch.setenv("BRAIDINFER_WEIGHT_LAYOUT", layout)
    eng = B.Engine.from_folder(folder, dtype=dtype, max_tokens=16384)
    assert eng.model.layers[0].feed_forward.w_gu.dim() == (4 if layout == "blocks" else 2)
    assert eng.model.lm_head.weight.dim() == (4 if layout == "blocks" else 2)
    rng = np.random.default_rng(11)
    free_before = [g.pool.free_count for g in eng.cache.groups]
    seqs = [tokens(cfg, int(n), 300 + i) for i, n in enumerate(rng.integers(1, 230, 36))]
    waiting = list(range(len(seqs)))
    live, pos, got = {}, {}, {i: [] for i in range(len(seqs))}
    while waiting or live:
        for i in list(waiting):
            if len(live) < 30 and rng.random() < 0.6:
                waiting.remove(i); live[i] = eng.alloc_slot(); pos[i] = 0
        if not live:
            continue
        chosen = [i for i in live if rng.random() < 0.85] or list(live)[:1]
        single = rng.random() < 0.7                     # mostly steps of one token each, as in generation
        entries, takes = [], []
        for i in chosen:
            n = 1 if single else min(int(rng.choice([1, 3, 17, 64, 70])), len(seqs[i]) - pos[i])
            entries.append(StepEntry(live[i], seqs[i][pos[i]:pos[i] + n], list(range(n))))
            takes.append(n)
        out = eng.step(entries).cpu().numpy()
        o = 0
        for i, n in zip(chosen, takes):
            got[i].append(out[o:o + n]); o += n; pos[i] += n
            if pos[i] == len(seqs[i]):
                eng.free_slot(live.pop(i))
    for i in range(0, len(seqs), 3):                     # every third request against the plain implementation
        close(np.concatenate(got[i]), P.forward(cfg, w, seqs[i]), dtype, f"request {i} of {len(seqs[i])} tokens")
    assert [g.pool.free_count for g in eng.cache.groups] == free_before


def test_wide_matrices_take_the_blocked_layout_by_themselves(tmp_path):
    """Matrices of 8,192 rows and more (here gate/up and the head) are laid out in blocks at load
    without being asked; the others keep their rows.  Whole, the last tokens one by one, and a batch."""
    cfg_d = dict(SERVING, num_hidden_layers=1, intermediate_size=4096, vocab_size=8200, layer_types=["full_attention"])
    folder = str(tmp_path / "wide")
    B.Engine.write_random_folder(folder, B.MistralConfig.from_dict(cfg_d), seed=4, std=0.03, vector_jitter=0.3)
    cfg, w = P.read_folder(folder)
    eng = B.Engine.from_folder(folder, dtype="bfloat16", max_tokens=8192)
    layer = eng.model.layers[0]
    assert layer.feed_forward.w_gu.dim() == 4 and eng.model.lm_head.weight.dim() == 4
    assert layer.feed_forward.w_d.dim() == 2 and layer.mixer.w_qkv.dim() == 2 and layer.mixer.w_o.dim() == 2
    toks = tokens(cfg, 150, 3)
    ref = P.forward(cfg, w, toks)
    close(whole(eng, toks), ref, "bfloat16", "wide matrices, whole")
    s = eng.alloc_slot()
    parts = [eng.step([StepEntry(s, toks[:140], list(range(140)))]).cpu().numpy()]
    for t in toks[140:]:
        parts.append(eng.step([StepEntry(s, [t], [0])]).cpu().numpy())
    eng.free_slot(s)
    close(np.concatenate(parts), ref, "bfloat16", "wide matrices, last 10 one by one")
    seqs = [tokens(cfg, 20 + 3 * i, 80 + i) for i in range(24)]               # 24 rows: the wide streaming product
    slots = [eng.alloc_slot() for _ in seqs]
    out = eng.step([StepEntry(sl, q[:-1], [len(q) - 2]) for sl, q in zip(slots, seqs)]).cpu().numpy()
    out2 = eng.step([StepEntry(sl, [q[-1]], [0]) for sl, q in zip(slots, seqs)]).cpu().numpy()
    for sl in slots:
        eng.free_slot(sl)
    for i in (0, 11, 23):
        r = P.forward(cfg, w, seqs[i])
        close(np.stack([out[i], out2[i]]), r[-2:], "bfloat16", f"wide matrices, request {i} of 24")


def test_a_head_size_outside_the_matrix_core_kernels_is_said_and_right(tmp_path):
    """A head size that is no multiple of 16 is allowed; in bfloat16 its attention runs by the one-wave-per-query
    kernel, which the engine says once per layer instead of slowing down silently; the logits are right."""
    from conftest import TINY
    cfg_d = dict(TINY["a"], head_dim=24)
    folder = str(tmp_path / "m")
    B.Engine.write_random_folder(folder, B.MistralConfig.from_dict(cfg_d), seed=4, std=0.08, vector_jitter=0.2)
    cfg, w = P.read_folder(folder)
    toks = tokens(cfg, 40, 3)
    ref = P.forward(cfg, w, toks)
    eng = B.Engine.from_folder(folder, dtype="bfloat16", max_tokens=512)
    s = eng.alloc_slot()
    with pytest.warns(RuntimeWarning, match="head size 24") as seen:
        first = eng.step([StepEntry(s, toks[:30], list(range(30)))]).cpu().numpy()
        rest = [eng.step([StepEntry(s, [t], [0])]).cpu().numpy() for t in toks[30:]]
    eng.free_slot(s)
    assert len([x for x in seen if "head size 24" in str(x.message)]) == cfg_d["num_hidden_layers"]
    close(np.concatenate([first] + rest), ref, "bfloat16", "head size 24")
    eng32 = B.Engine.from_folder(folder, dtype="float32", max_tokens=512)
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("error")                        # the 32-bit path is that kernel by design: nothing to say
        close(whole(eng32, toks), ref, "float32", "head size 24")


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12])
def test_configurations_drawn_at_random(seed, tmp_path):
    """Sizes drawn at random (head sizes in steps of 16, groups of 1 to 6 heads, widths and vocabularies
    that are no powers of two, down to a width of one element and a vocabulary of two, windows, tied
    heads, 1 to 3 layers): a prompt whole, its last 8 tokens one by one, and 20 requests of unequal
    lengths in one step and one token each, in both precisions.  32-bit is held to its bound at every
    size; bfloat16 to its bound or to what rounding alone does to the plain implementation."""
    rng = np.random.default_rng(1000 + seed)
    hd = int(rng.choice([16, 32, 48, 64, 80, 96, 128]))
    nkv = int(rng.choice([1, 2, 3, 4]))
    nq = nkv * int(rng.choice([1, 2, 3, 4, 6]))
    window = None if rng.random() < 0.4 else int(rng.choice([4, 17, 64, 100]))
    L = int(rng.integers(1, 4))
    cfg_d = dict(num_hidden_layers=L, hidden_size=int(rng.choice([1, 3, 9, 64, 96, 127, 200, 264, 520, 1024, 1152, 2047])),
                 num_attention_heads=nq, num_key_value_heads=nkv, head_dim=hd,
                 intermediate_size=int(rng.choice([96, 192, 328, 520, 1024, 1536, 2048])),
                 vocab_size=int(rng.choice([2, 3, 17, 100, 257, 1000, 4100, 9000])), rope_theta=float(rng.choice([1e4, 1e6])),
                 rms_norm_eps=float(rng.choice([1e-5, 1e-6])), sliding_window=window, max_position_embeddings=4096,
                 tie_word_embeddings=bool(rng.random() < 0.3),
                 layer_types=[str(rng.choice(["full_attention", "sliding_attention"])) if window else "full_attention"
                              for _ in range(L)])
    folder = str(tmp_path / "drawn")
    B.Engine.write_random_folder(folder, B.MistralConfig.from_dict(cfg_d), seed=seed, std=0.03, vector_jitter=0.3)
    cfg, w = P.read_folder(folder)
    n = int(rng.choice([30, 90, 150, 300]))
    toks = tokens(cfg, n, seed)
    ref = P.forward(cfg, w, toks)
    rounded = P.forward(cfg, w, toks, act_dtype="bfloat16")

    def check(got, rows, dtype, what):
        if dtype == "float32":
            close(got, ref[rows], dtype, what)
        else:
            close_or_rounding(got, ref[rows], rounded[rows], what)
    for dtype in ("float32", "bfloat16"):
        eng = B.Engine.from_folder(folder, dtype=dtype, max_tokens=2048)
        s = eng.alloc_slot()
        parts = [eng.step([StepEntry(s, toks[:n - 8], list(range(n - 8)))]).cpu().numpy()]
        for t in toks[n - 8:]:
            parts.append(eng.step([StepEntry(s, [t], [0])]).cpu().numpy())
        eng.free_slot(s)
        check(np.concatenate(parts), slice(None), dtype, f"{cfg_d}: whole, then 8 one by one")
        slots = [eng.alloc_slot() for _ in range(20)]
        first = eng.step([StepEntry(sl, toks[:10 + i], [9 + i]) for i, sl in enumerate(slots)]).cpu().numpy()
        then = eng.step([StepEntry(sl, [toks[10 + i]], [0]) for i, sl in enumerate(slots)]).cpu().numpy()
        for sl in slots:
            eng.free_slot(sl)
        check(first, slice(9, 29), dtype, f"{cfg_d}: 20 prompts of 10 to 29 tokens in one step")
        check(then, slice(10, 30), dtype, f"{cfg_d}: one token each after them")


DEGENERATE = {
    # four of the configurations at which a wide search of sizes found bfloat16 beyond its usual bound
    # (32-bit was within its bound at every one): a width of 1 or 3 elements, or a vocabulary of 2
    "width 1": dict(num_hidden_layers=3, hidden_size=1, num_attention_heads=9, num_key_value_heads=3, head_dim=128,
                    intermediate_size=2049, vocab_size=4099, rope_theta=500.0, rms_norm_eps=1e-6, sliding_window=None,
                    tie_word_embeddings=True, n=130),
    "vocabulary 2": dict(num_hidden_layers=1, hidden_size=2047, num_attention_heads=8, num_key_value_heads=4, head_dim=256,
                         intermediate_size=1023, vocab_size=2, rope_theta=500.0, rms_norm_eps=1e-5, sliding_window=63,
                         tie_word_embeddings=False, n=330),
    "width 3, vocabulary 2": dict(num_hidden_layers=2, hidden_size=3, num_attention_heads=3, num_key_value_heads=1,
                                  head_dim=160, intermediate_size=2049, vocab_size=2, rope_theta=1e6, rms_norm_eps=1e-5,
                                  sliding_window=None, tie_word_embeddings=False, n=330),
    "width 3": dict(num_hidden_layers=2, hidden_size=3, num_attention_heads=24, num_key_value_heads=8, head_dim=160,
                    intermediate_size=1023, vocab_size=255, rope_theta=1e4, rms_norm_eps=1e-5, sliding_window=5,
                    tie_word_embeddings=False, layer_types=["full_attention", "sliding_attention"], n=40),
}


@pytest.mark.parametrize("which", sorted(DEGENERATE))
def test_degenerate_widths_differ_by_rounding_only(which, tmp_path):
    """At a width of one element the norm of a row is its sign times the weight: a rounding that moves
    a residual value across zero flips every logit of that row (cosine -1), in the engine and in the
    plain implementation alike once the latter rounds where the engine does.  The engine in 32-bit stays
    within 1e-4 at these sizes, in bfloat16 within three times the plain implementation's own move."""
    d = dict(DEGENERATE[which])
    n = d.pop("n")
    folder = str(tmp_path / "m")
    B.Engine.write_random_folder(folder, B.MistralConfig.from_dict(dict(d, max_position_embeddings=4096)),
                                 seed=5, std=0.03, vector_jitter=0.3)
    cfg, w = P.read_folder(folder)
    toks = tokens(cfg, n, 9)
    ref = P.forward(cfg, w, toks)
    rounded = P.forward(cfg, w, toks, act_dtype="bfloat16")
    for dtype in ("float32", "bfloat16"):
        eng = B.Engine.from_folder(folder, dtype=dtype, max_tokens=4096)
        s = eng.alloc_slot()
        parts = [eng.step([StepEntry(s, toks[:n - 8], list(range(n - 8)))]).cpu().numpy()]
        for t in toks[n - 8:]:
            parts.append(eng.step([StepEntry(s, [t], [0])]).cpu().numpy())
        eng.free_slot(s)
        got = np.concatenate(parts)
        if dtype == "float32":
            close(got, ref, dtype, which)
        else:
            close_or_rounding(got, ref, rounded, which)


# ----------------------------------------------------------------- probes, failed steps ----
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_probes_see_the_residual_rows_where_the_plain_implementation_has_them(engines, tiny_folders, dtype):
    """`step(..., probe=)` hands out the residual rows under the reference's probe names
    (tracer.rs:94-160), for a whole prompt and for single-token steps (which then run eagerly
    instead of from a graph), and leaves the logits as they are without a probe."""
    _, cfg, w = tiny_folders["b"]
    eng = engines("b", dtype)
    sz = P.sizes(cfg)
    toks = tokens(cfg, 21, 50)
    x = P.embedding(w["model.embed_tokens.weight"], toks)
    want = {"embed": x}
    for i in range(sz["L"]):
        p = f"model.layers.{i}."
        x = P.attention_block(x, np.arange(len(toks)), w, p, sz, P.layer_window(sz, i))
        want[f"L{i}.post_mixer"] = x
        x = P.ffn_block(x, w, p, sz)
        want[f"L{i}.post_ffn"] = x
    want["final_norm"] = P.rms_norm(x, w["model.norm.weight"], sz["eps"])
    want["logits"] = P.forward(cfg, w, toks)
    seen = {}
    s = eng.alloc_slot()
    first = eng.step([StepEntry(s, toks[:20], list(range(20)))], probe=lambda n, t: seen.setdefault(n, t.float().cpu().numpy().copy()))
    assert list(seen) == list(want)
    for n in want:
        close(seen[n], want[n][:20], dtype, n)
    assert np.array_equal(seen["logits"], first.cpu().numpy())
    one = {}
    last = eng.step([StepEntry(s, toks[20:], [0])], probe=lambda n, t: one.setdefault(n, t.float().cpu().numpy().copy()))
    eng.free_slot(s)
    for n in want:
        close(one[n], want[n][20:], dtype, n + " of a single-token step")
    s = eng.alloc_slot()
    eng.step([StepEntry(s, toks[:20], [])])
    plain_last = eng.step([StepEntry(s, toks[20:], [0])])           # no probe: the recorded graph
    eng.free_slot(s)
    assert np.abs(plain_last.cpu().numpy() - last.cpu().numpy()).max() <= CUT_TOL[dtype] * np.abs(want["logits"]).max()


def test_a_step_that_fails_inside_the_model_leaves_nothing_behind(tiny_folders):
    folder, cfg, w = tiny_folders["a"]
    eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=512)
    s1, s2 = eng.alloc_slot(), eng.alloc_slot()
    toks = tokens(cfg, 130, 3)
    eng.step([StepEntry(s1, toks[:70], [])])
    free = [g.pool.free_count for g in eng.cache.groups]
    real = eng.model.forward

    def broken(*a, **k):
        raise B.KernelError("a size no kernel takes")
    eng.model.forward = broken
    with pytest.raises(B.KernelError):
        eng.step([StepEntry(s1, toks[70:], [0]), StepEntry(s2, toks[:100], [0])])     # needs three new pages
    eng.model.forward = real
    assert [g.pool.free_count for g in eng.cache.groups] == free and eng.length(s1) == 70 and eng.length(s2) == 0
    got = eng.step([StepEntry(s1, toks[70:], list(range(60)))]).cpu().numpy()         # and the sequence goes on as if nothing happened
    close(got, P.forward(cfg, w, toks)[70:], "float32", "after a failed step")
    eng.free_slot(s1); eng.free_slot(s2)
    assert all(g.pool.held_count == 0 for g in eng.cache.groups)


def test_the_longest_sequence_is_the_models_unless_the_caller_says_more(tiny_folders):
    folder, cfg, _ = tiny_folders["c"]                     # max_position_embeddings 2048
    eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=8192)
    assert eng.cache.max_seq_len == 2048
    assert B.Engine.from_folder(folder, dtype="float32", max_tokens=8192, max_seq_len=4096).cache.max_seq_len == 4096
    assert B.Engine.from_folder(folder, dtype="float32", max_tokens=640).cache.max_seq_len == 640


# ----------------------------------------------- thousands of tokens at the serving head size ----
def _plain_last_rows(pc, pw, toks, n_last):
    """The plain implementation's logits of the last rows of a long sequence.  One layer, so
    only the attention needs the whole sequence: everything row-wise is done on the last rows,
    the attention with the plain functions on keys and values of all positions."""
    sz = P.sizes(pc)
    T = len(toks)
    p = "model.layers.0."
    x = P.embedding(pw["model.embed_tokens.weight"], toks)
    n = P.rms_norm(x, pw[p + "input_layernorm.weight"], sz["eps"])
    inv = P.rope_inv_freq(sz["hd"], sz["theta"])
    k = P.rope(P.linear(n, pw[p + "self_attn.k_proj.weight"]).reshape(T, sz["nkv"], sz["hd"]), np.arange(T), inv, sz["pairing"])
    v = P.linear(n, pw[p + "self_attn.v_proj.weight"]).reshape(T, sz["nkv"], sz["hd"])
    rows = np.arange(T - n_last, T)
    q = P.rope(P.linear(n[rows], pw[p + "self_attn.q_proj.weight"]).reshape(n_last, sz["nq"], sz["hd"]), rows, inv, sz["pairing"])
    out = np.zeros((n_last, sz["nq"], sz["hd"]), np.float32)
    W = P.layer_window(sz, 0)
    for r, i in enumerate(rows):                               # P.attention of one query: a 1 x T problem each
        lo = 0 if W is None else max(0, i - W + 1)
        for h in range(sz["nq"]):
            kh = h // (sz["nq"] // sz["nkv"])
            sc = (k[lo:i + 1, kh] @ q[r, h]) * np.float32(1.0 / np.sqrt(sz["hd"]))
            e = np.exp(sc - sc.max())
            out[r, h] = (e / e.sum()) @ v[lo:i + 1, kh]
    xl = x[rows] + P.linear(out.reshape(n_last, -1), pw[p + "self_attn.o_proj.weight"])
    xl = P.ffn_block(xl, pw, p, sz)
    return P.linear(P.rms_norm(xl, pw["model.norm.weight"], sz["eps"]), pw["lm_head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [None, 4096])
def test_a_key_thousands_of_tokens_back_at_head_size_128(tmp_path, dtype, window):
    """The marker model at the head size of the serving shapes (in bfloat16: the attention kernels that bring
    pages through LDS rings, the doubling of the decode runs beyond 4,096 tokens) with 9,000
    tokens: the marker at the start, at the window's edge (seen at distance 4,095, not at
    4,096), in the last page; the asker as the end of the whole prompt, of a last chunk of 64,
    and decoded alone, from a graph and eagerly."""
    folder, pc, pw = _marker_model(tmp_path, sliding_window=window, head_dim=128, rope_theta=1e8, max_positions=16384)
    small = _plain_last_rows(pc, pw, [5, 1, 7, 2], 1)            # the helper against the whole plain forward
    assert np.abs(small - P.forward(pc, pw, [5, 1, 7, 2])[-1:]).max() < 1e-5 * np.abs(small).max()
    T = 9000
    rng = np.random.default_rng(2)
    engines_ = [B.Engine.from_folder(folder, dtype=dtype, max_tokens=9216, max_seq_len=9216, use_graphs=g) for g in (True, False)]
    places = [(0, window is None), (T - 1 - 4095, True), (T - 1 - 4096, window is None), (T - 30, True), (4095, window is None)]
    for at, seen in places:
        toks = [int(x) for x in rng.integers(3, 40, T)]
        toks[at], toks[-1] = 1, 2
        ref = _plain_last_rows(pc, pw, toks, 1)[0]
        assert (int(ref.argmax()) == 1) == seen, "the plain implementation must see the marker exactly where the window allows"
        for eng in engines_:
            for cut in ((T - 1, 0, T - 64) if eng.use_graphs else (T - 1,)):
                s = eng.alloc_slot()
                if cut:
                    eng.step([StepEntry(s, toks[:cut], [])])
                got = eng.step([StepEntry(s, toks[cut:], [T - cut - 1])]).cpu().numpy()[0]
                if window:
                    assert eng.cache.groups[0].pool.held_count <= 4096 // 64 + 1
                eng.free_slot(s)
                assert (int(got.argmax()) == 1) == seen, f"marker at {at}, cut {cut}, graphs {eng.use_graphs}"
                close(got[None], ref[None], dtype, f"marker at {at}, cut {cut}, graphs {eng.use_graphs}")


@pytest.mark.parametrize("live", [65, 100, 130, 200])
def test_single_token_steps_of_many_requests(serving, live):
    """65 to 200 requests decode together (graph buckets of 128 and 256 rows with padding
    sequences, products by tiles cut along k, attention over 128 or 256 rows): every request
    against the plain forward, graphs against eager steps, requests ending on the way."""
    folder, cfg, w = serving
    g = B.Engine.from_folder(folder, dtype="bfloat16", max_tokens=live * 128)
    e = B.Engine.from_folder(folder, dtype="bfloat16", max_tokens=live * 128, use_graphs=False)
    rng = np.random.default_rng(live)
    lens = [int(n) for n in rng.integers(1, 100, live)]
    more = [int(n) for n in rng.integers(2, 7, live)]            # tokens decoded after the prompt
    seqs = [tokens(cfg, n + m, 900 + i) for i, (n, m) in enumerate(zip(lens, more))]
    got = {}
    for eng in (g, e):
        slots = [eng.alloc_slot() for _ in seqs]
        out = eng.step([StepEntry(sl, q[:n], [n - 1]) for sl, q, n in zip(slots, seqs, lens)]).cpu().numpy()
        rows = [[out[i:i + 1]] for i in range(live)]
        alive = list(range(live))
        k = 0
        while alive:
            out = eng.step([StepEntry(slots[i], [seqs[i][lens[i] + k]], [0]) for i in alive]).cpu().numpy()
            for r, i in enumerate(alive):
                rows[i].append(out[r:r + 1])
            k += 1
            for i in [i for i in alive if lens[i] + k == len(seqs[i])]:
                eng.free_slot(slots[i]); alive.remove(i)
        got[eng.use_graphs] = [np.concatenate(r) for r in rows]
        assert all(gr.pool.held_count == 0 for gr in eng.cache.groups)
    assert g.use_graphs and (128 if live <= 128 else 256) in g._graphs.graphs and e._graphs is None
    for i in range(live):
        ref = P.forward(cfg, w, seqs[i])[lens[i] - 1:]
        close(got[True][i], ref, "bfloat16", f"request {i} of {live}, graphs")
        assert np.abs(got[True][i] - got[False][i]).max() <= CUT_TOL["bfloat16"] * np.abs(ref).max()


# ------------------------------------------------- the layer sizes of the benchmark's shape ----
@pytest.fixture(scope="module")
def real_sizes(tmp_path_factory):
    """Two layers of the Mistral-7B-v0.3 shape (hidden 4096, 32 heads over 8 kv heads of 128,
    intermediate 14336, vocabulary 32768): the matrices that the benchmark's kernels multiply."""
    folder = str(tmp_path_factory.mktemp("real_sizes"))
    cfg = B.preset("mistral-7b-v0.3", num_hidden_layers=2)
    B.Engine.write_random_folder(folder, cfg, seed=17, std=0.02, vector_jitter=0.3, device="cuda:0")
    pc, w = P.read_folder(folder)
    return folder, pc, w


def test_real_layer_sizes_prompt_single_steps_and_a_batch(real_sizes):
    """bfloat16 at the sizes the benchmark runs (tiles of 256x256, 256x192 and 128x256 for the
    prompt, the streaming products over rows and over blocks of 16 rows for 1 to 16 and 17 to
    64 sequences, attention through the LDS rings): a prompt of 300 tokens whole, its last
    tokens one by one, and 20 requests of unequal lengths decoding together, all against the
    plain implementation."""
    folder, cfg, w = real_sizes
    eng = B.Engine.from_folder(folder, dtype="bfloat16", max_tokens=8192)
    assert eng.model.layers[0].feed_forward.w_gu.dim() == 4 and eng.model.lm_head.weight.dim() == 4      # blocked layout
    toks = tokens(cfg, 300, 21)
    ref = P.forward(cfg, w, toks)
    close(whole(eng, toks), ref, "bfloat16", "7B sizes, whole prompt")
    s = eng.alloc_slot()
    parts = [eng.step([StepEntry(s, toks[:292], [291])]).cpu().numpy()]
    for t in toks[292:]:
        parts.append(eng.step([StepEntry(s, [t], [0])]).cpu().numpy())
    eng.free_slot(s)
    close(np.concatenate(parts), ref[291:], "bfloat16", "7B sizes, last tokens one by one")
    lens = [3 + 9 * i for i in range(20)]
    seqs = [tokens(cfg, n + 3, 400 + i) for i, n in enumerate(lens)]
    slots = [eng.alloc_slot() for _ in seqs]
    got = [[] for _ in seqs]
    out = eng.step([StepEntry(sl, q[:n], [n - 1]) for sl, q, n in zip(slots, seqs, lens)]).cpu().numpy()
    for i in range(20):
        got[i].append(out[i:i + 1])
    for k in range(3):
        out = eng.step([StepEntry(sl, [q[n + k]], [0]) for sl, q, n in zip(slots, seqs, lens)]).cpu().numpy()
        for i in range(20):
            got[i].append(out[i:i + 1])
    for sl in slots:
        eng.free_slot(sl)
    for i in (0, 11, 19):
        close(np.concatenate(got[i]), P.forward(cfg, w, seqs[i])[lens[i] - 1:], "bfloat16", f"7B sizes, request {i} of 20")


def test_real_layer_sizes_in_32_bit(real_sizes):
    folder, cfg, w = real_sizes
    eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=1024)
    toks = tokens(cfg, 70, 22)
    ref = P.forward(cfg, w, toks)
    s = eng.alloc_slot()
    parts = [eng.step([StepEntry(s, toks[:66], list(range(66)))]).cpu().numpy()]
    for t in toks[66:]:
        parts.append(eng.step([StepEntry(s, [t], [0])]).cpu().numpy())
    eng.free_slot(s)
    close(np.concatenate(parts), ref, "float32", "7B sizes in 32-bit")
