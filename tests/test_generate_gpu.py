"""Generation through the entry points against the plain implementation's greedy loop."""
import os
import subprocess
import sys

import numpy as np
import pytest

import braidinfer_amd as B
import plain_mistral as P
from braidinfer_amd import SamplingParams

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def prompts_of(cfg, lens, seed):
    rng = np.random.default_rng(seed)
    return [[int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for n in lens]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_matches_the_plain_loop(engines, tiny_folders, dtype):
    # the first configuration of the benchmark description: prompts of 5, 9 and 12, 8 tokens, greedy
    _, cfg, w = tiny_folders["a"]
    eng = engines("a", dtype)
    prompts = prompts_of(cfg, [5, 9, 12], 0)
    got = eng.generate(prompts, max_new_tokens=8, temperature=0.0, stop_token_ids=[])
    want = [P.greedy_generate(cfg, w, p, 8) for p in prompts]
    if dtype == "float32":
        assert got == want
    else:
        # bf16 may pick the runner-up where two logits are within rounding: the sequences agree
        # up to the first such place, and there the plain logits are nearly tied
        for g, wnt, p in zip(got, want, prompts):
            for i, (a, b) in enumerate(zip(g, wnt)):
                if a != b:
                    l = P.forward(cfg, w, p + wnt[:i])[-1]
                    assert abs(l[a] - l[b]) < 3e-2 * np.abs(l).max()
                    break


def test_stop_tokens_and_unequal_ends(engines, tiny_folders):
    _, cfg, w = tiny_folders["b"]
    eng = engines("b", "float32")
    prompts = prompts_of(cfg, [3, 11, 17, 20], 1)
    free = [g.pool.free_count for g in eng.cache.groups]
    plain = [P.greedy_generate(cfg, w, p, 12) for p in prompts]
    stop = plain[1][4]                                  # a token request 1 meets at its fifth step
    want = [P.greedy_generate(cfg, w, p, 12, stop_ids=[stop]) for p in prompts]
    assert len(want[1]) <= 4
    got, stats = eng.generate(prompts, max_new_tokens=12, stop_token_ids=[stop], return_stats=True)
    assert got == want
    assert [g.pool.free_count for g in eng.cache.groups] == free and eng.cache.slots.free_count == eng.cache.n_slots
    assert stats.prefill_tokens == 51 and "PPTG pp=" in stats.pptg_line()


def test_alone_or_in_a_batch_gives_the_same_tokens(engines, tiny_folders):
    _, cfg, _ = tiny_folders["b"]
    eng = engines("b", "float32")
    prompts = prompts_of(cfg, [3, 11, 17, 20], 2)
    # the second configuration of the benchmark description: 12 tokens at temperature 0.7, seeded
    kw = dict(max_new_tokens=12, temperature=0.7, seed=1234, top_k=0, stop_token_ids=[])
    together = eng.generate(prompts, **kw)
    assert together == eng.generate(prompts, **kw)                       # seeded: the same again
    assert together != eng.generate(prompts, **{**kw, "seed": 99})
    assert eng.generate(prompts[0], **kw) == together[0]                 # request 0 alone
    by_two = eng.generate(prompts, max_batch=2, **kw)                    # two batches, slots used again
    assert by_two == together


def test_greedy_through_the_chain_equals_greedy_step_by_step(tiny_folders):
    """Plain greedy requests decode through a chain (a step's tokens feed the next on the
    device, one step is launched ahead).  In 32-bit that must give the tokens and reasons of
    single steps, with stop tokens, unequal budgets of context, and page edges on the way."""
    folder, cfg, w = tiny_folders["b"]
    with_chain = B.Engine.from_folder(folder, dtype="float32", max_tokens=4096, max_seq_len=160)
    without = B.Engine.from_folder(folder, dtype="float32", max_tokens=4096, max_seq_len=160, use_graphs=False)
    assert without.chain([0], [1]) is None
    prompts = prompts_of(cfg, [3, 60, 17, 120, 1, 63, 150], 5)
    free_run = without.generate(prompts, max_new_tokens=70, stop_token_ids=[])
    stop = free_run[2][9]
    for kw in (dict(max_new_tokens=70, stop_token_ids=[]), dict(max_new_tokens=70, stop_token_ids=[stop]),
               dict(max_new_tokens=5, stop_token_ids=[stop], include_stop=True), dict(max_new_tokens=1, stop_token_ids=[])):
        a, sa = without.generate(prompts, return_stats=True, **kw)
        b, sb = with_chain.generate(prompts, return_stats=True, **kw)
        assert a == b, kw
        assert sb.decode_tokens >= sa.decode_tokens
        for eng in (with_chain, without):
            assert all(g.pool.held_count == 0 for g in eng.cache.groups) and eng.cache.slots.free_count == eng.cache.n_slots
    # the cache's longest sequence is 192 (whole pages): 150 + 42 tokens are fed, the 43rd new token is the last
    assert with_chain.cache.max_seq_len == 192 and len(free_run[6]) == 43
    assert free_run[6] == P.greedy_generate(cfg, w, prompts[6], 43)
    assert free_run[0] == P.greedy_generate(cfg, w, prompts[0], 70)


def test_sampled_through_the_chain_equals_sampled_step_by_step(tiny_folders):
    """Sampled requests decode through a chain too: the recorded step, the resident sampler's
    kernels and the move to the next step's arrays, one step launched ahead.  Every option of
    the sampler, mixed in one batch with greedy rows, stop tokens and the context's end: the
    tokens and reasons of single steps."""
    from braidinfer_amd.engine import generate
    from braidinfer_amd.sampling import SamplingParams
    folder, cfg, w = tiny_folders["b"]
    with_chain = B.Engine.from_folder(folder, dtype="float32", max_tokens=4096, max_seq_len=160)
    without = B.Engine.from_folder(folder, dtype="float32", max_tokens=4096, max_seq_len=160, use_graphs=False)
    prompts = prompts_of(cfg, [3, 60, 17, 120, 1, 63, 150, 9], 6)
    V = cfg["vocab_size"]
    params = [SamplingParams(temperature=0.8, top_k=0, seed=5),
              SamplingParams(temperature=1.0, top_k=7, seed=5),
              SamplingParams(temperature=0.9, top_k=0, top_p=0.8, seed=6),
              SamplingParams(temperature=0.0, top_k=0, repetition_penalty=1.3),
              SamplingParams.greedy(),
              SamplingParams(temperature=1.1, top_k=0, min_p=0.05, repetition_penalty=1.2, seed=7),
              SamplingParams(temperature=0.7, top_k=40, top_p=0.9, seed=8, logit_bias=[(3, 4.0), (V - 1, -2.0)]),
              SamplingParams(temperature=1.0, top_k=V + 5, seed=9)]
    free_run, _ = generate(without, prompts, params, max_new_tokens=50, stop_token_ids=[])
    stop = free_run[2].tokens[7]
    for kw in (dict(max_new_tokens=50, stop_token_ids=[]), dict(max_new_tokens=50, stop_token_ids=[stop]),
               dict(max_new_tokens=6, stop_token_ids=[stop], include_stop=True), dict(max_new_tokens=2, stop_token_ids=[])):
        a, sa = generate(without, prompts, params, **kw)
        b, sb = generate(with_chain, prompts, params, **kw)
        assert [(r.tokens, r.finish_reason) for r in a] == [(r.tokens, r.finish_reason) for r in b], kw
        assert sb.decode_tokens >= sa.decode_tokens
        for eng in (with_chain, without):
            assert all(g.pool.held_count == 0 for g in eng.cache.groups) and eng.cache.slots.free_count == eng.cache.n_slots
    assert free_run[6].finish_reason == "context" and len(free_run[6].tokens) == 43
    assert len({tuple(r.tokens) for r in free_run}) == len(prompts)
    # a chain of these rows by hand: two launches ahead of the first read, uniform numbers per launch
    eng = with_chain
    slots = [eng.alloc_slot() for _ in range(2)]
    eng.step([B.StepEntry(s, p, []) for s, p in zip(slots, prompts[:2])])
    from braidinfer_amd.sampling import Sampler
    state = Sampler(eng.device, V).state(params[:2], [list(p) for p in prompts[:2]])
    with pytest.raises(B.StepError, match="rows"):
        eng.chain(slots[:1], [1], state)
    chain = eng.chain(slots, [1, 2], state)
    chain.launch([0.25, 0.5])
    chain.launch([0.75, 0.125])
    t1, t2 = chain.read(), chain.read()
    chain.close()
    for s in slots:
        eng.free_slot(s)
    # the same two steps one at a time through the step function and a fresh state
    slots = [eng.alloc_slot() for _ in range(2)]
    eng.step([B.StepEntry(s, p, []) for s, p in zip(slots, prompts[:2])])
    state = Sampler(eng.device, V).state(params[:2], [list(p) for p in prompts[:2]])
    s1 = state.sample(eng.step([B.StepEntry(s, [t], [0]) for s, t in zip(slots, [1, 2])]), [0.25, 0.5])
    s2 = state.sample(eng.step([B.StepEntry(s, [t], [0]) for s, t in zip(slots, s1)]), [0.75, 0.125])
    assert (t1, t2) == (s1, s2)
    for s in slots:
        eng.free_slot(s)


def test_the_chain_by_hand(tiny_folders):
    folder, cfg, w = tiny_folders["a"]
    eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=1024)
    prompts = prompts_of(cfg, [5, 70], 8)
    want = [P.greedy_generate(cfg, w, p, 4) for p in prompts]
    slots = [eng.alloc_slot() for _ in prompts]
    logits = eng.step([B.StepEntry(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)])
    first = logits.argmax(-1).tolist()
    chain = eng.chain(slots, first)
    chain.launch()
    chain.launch()
    with pytest.raises(B.StepError, match="unread"):
        chain.launch()
    got = [first, chain.read(), chain.read()]
    chain.launch()
    got.append(chain.read())
    assert [list(t) for t in zip(*got)] == want and [eng.length(s) for s in slots] == [8, 73]
    with pytest.raises(B.StepError, match="unread"):
        chain.read()
    # any other single-token step of that size takes the recorded step away from the chain
    other = [eng.alloc_slot(), eng.alloc_slot()]
    eng.step([B.StepEntry(other[0], [1, 2], []), B.StepEntry(other[1], [3], [])])
    eng.step([B.StepEntry(other[0], [4], [0]), B.StepEntry(other[1], [5], [0])])
    with pytest.raises(B.StepError, match="another step"):
        chain.launch()
    chain.close()
    with pytest.raises(B.StepError, match="vocabulary"):
        eng.chain(slots, [0, cfg["vocab_size"]])
    again = eng.chain(slots, got[-1])       # a new chain goes on where the old one stopped
    again.launch()
    more = again.read()
    again.close()
    assert more == [P.greedy_generate(cfg, w, p, 5)[-1] for p in prompts]
    for s in slots + other:
        eng.free_slot(s)


def test_a_chain_keeps_two_steps_unread_while_sequences_take_new_pages(tiny_folders):
    """64 sequences whose lengths straddle a page edge: in each of the next steps some of them take a
    new page (a changed piece of the block table goes to the device).  Launching must not wait for the
    device: with torch's check for synchronizing calls set to raise, two steps are launched and left
    unread across such steps; the tokens are those of single steps on an engine without graphs."""
    import torch
    folder, cfg, w = tiny_folders["b"]
    eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=64 * 192)
    plain = B.Engine.from_folder(folder, dtype="float32", max_tokens=64 * 192, use_graphs=False)
    lens = [58 + i % 8 for i in range(64)]                      # 58..65: pages are taken at steps 0 to 6
    prompts = prompts_of(cfg, lens, 12)
    outs = []
    for e in (eng, plain):
        slots = [e.alloc_slot() for _ in prompts]
        first = e.step([B.StepEntry(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)]).argmax(-1).tolist()
        got = [first]
        if e is plain:
            for _ in range(9):
                got.append(e.step([B.StepEntry(s, [t], [0]) for s, t in zip(slots, got[-1])]).argmax(-1).tolist())
        else:
            chain = e.chain(slots, first)
            chain.launch()                                      # records the chain's graph: that may wait
            got.append(chain.read())
            pages = [g.pool.held_count for g in e.cache.groups]
            torch.cuda.set_sync_debug_mode("error")
            try:
                with pytest.raises(RuntimeError):               # the check itself: a blocking copy raises
                    torch.zeros(4, device=e.device).copy_(torch.ones(4))
                for _ in range(4):
                    chain.launch()
                    chain.launch()
                    torch.cuda.set_sync_debug_mode("default")
                    got += [chain.read(), chain.read()]          # reading waits, by design
                    torch.cuda.set_sync_debug_mode("error")
            finally:
                torch.cuda.set_sync_debug_mode("default")
            chain.close()
            assert [g.pool.held_count for g in e.cache.groups] != pages     # pages were taken on the way
        outs.append(got)
        for s in slots:
            e.free_slot(s)
    assert outs[0] == outs[1]


def test_command_line(tiny_folders):
    folder, cfg, w = tiny_folders["a"]
    p = [7, 3, 200, 5]
    want = P.greedy_generate(cfg, w, p, 6)
    env = dict(os.environ, MODEL=folder, MAX_TOKENS="6")
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "generate"), "--dtype", "float32",
                        "--prompt-ids", ",".join(map(str, p))], env=env, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    assert [int(t) for t in r.stdout.split()] == want
    assert "PPTG pp=" in r.stderr and "tokens in" in r.stderr and "stop tokens:" in r.stderr
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "generate"), folder, "--dtype", "fp32",
                        "--prompt-ids", "1,2", "--prompt-ids", "3,4,5"],
                       env={k: v for k, v in env.items() if k != "MODEL"}, capture_output=True, text=True)
    assert r.returncode == 0 and len(r.stdout.strip().splitlines()) == 2
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "generate"), "some words"], env=env,
                       capture_output=True, text=True)
    assert r.returncode == 2 and "tokenizer" in r.stderr


def _word_tokenizer(folder, vocab_size, bos):
    """A tokenizer.json made here with the `tokenizers` package: one token per word."""
    tk = pytest.importorskip("tokenizers")
    words = {f"w{i}": i for i in range(vocab_size)}
    words["<s>"] = bos
    del words[f"w{bos}"]
    tok = tk.Tokenizer(tk.models.WordLevel(vocab=words, unk_token="w0"))
    tok.pre_tokenizer = tk.pre_tokenizers.WhitespaceSplit()
    tok.decoder = tk.decoders.Fuse()
    tok.save(os.path.join(folder, "tokenizer.json"))
    return tok


def test_command_line_with_text_a_tokenizer_and_the_folders_stop_tokens(tmp_path):
    """The text path: the prompt is tokenized with the folder's tokenizer.json, the BOS of
    config.json goes in front unless tokenizer_config.json says no (generate.rs:479-489), the
    stop tokens come from config.json and generation_config.json, the answer is text."""
    import json
    import shutil
    cfg = B.preset("tiny-a", bos_token_id=1, eos_token_id=250)
    folder = B.Engine.write_random_folder(str(tmp_path / "m"), cfg, seed=31, std=0.08)
    _word_tokenizer(folder, 256, bos=1)
    pc, w = P.read_folder(folder)
    ids = [7, 3, 200, 5]
    text = " ".join(f"w{i}" for i in ids)
    free_run = P.greedy_generate(pc, w, [1] + ids, 8)
    stop = free_run[3]
    with open(os.path.join(folder, "generation_config.json"), "w") as f:
        json.dump({"eos_token_id": [stop, 251]}, f)
    gen = [sys.executable, os.path.join(ROOT, "bin", "generate"), "--dtype", "float32"]
    env = dict(os.environ, MODEL=folder, MAX_TOKENS="8")
    r = subprocess.run(gen + [text], env=env, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    want = P.greedy_generate(pc, w, [1] + ids, 8, stop_ids=[250, stop, 251])
    assert 0 < len(want) <= 3 and r.stdout.strip() == "".join(f"w{t}" for t in want)
    assert f"stop tokens: [250, {stop}, 251]" in r.stderr and "LOAD PROFILE:" in r.stderr and "GB/s" in r.stderr
    # no BOS when the tokenizer's configuration says so
    with open(os.path.join(folder, "tokenizer_config.json"), "w") as f:
        json.dump({"add_bos_token": False}, f)
    os.remove(os.path.join(folder, "generation_config.json"))
    r = subprocess.run(gen + [text], env=env, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    assert r.stdout.strip() == "".join(f"w{t}" for t in P.greedy_generate(pc, w, ids, 8, stop_ids=[250]))
    shutil.rmtree(folder)


def test_command_line_writes_a_random_folder_in_shards_and_reads_it_again(tmp_path):
    keep = str(tmp_path / "kept")
    gen = [sys.executable, os.path.join(ROOT, "bin", "generate"), "--dtype", "float32", "--prompt-ids", "9,8,7"]
    env = {k: v for k, v in os.environ.items() if k != "MODEL"}
    env["MAX_TOKENS"] = "5"
    r1 = subprocess.run(gen + ["--random-weights", "3", "--preset", "tiny-b", "--save-folder", keep, "--shard-bytes", "40000"],
                        env=env, capture_output=True, text=True)
    assert r1.returncode == 0, r1.stderr
    assert os.path.isfile(os.path.join(keep, "model.safetensors.index.json")) and "written to" in r1.stderr
    r2 = subprocess.run(gen, env=dict(env, MODEL=keep), capture_output=True, text=True)
    assert r2.returncode == 0 and r2.stdout == r1.stdout
    pc, w = P.read_folder(keep)
    assert [int(t) for t in r1.stdout.split()] == P.greedy_generate(pc, w, [9, 8, 7], 5)


def test_smoke_entry():
    import __graft_entry__
    __graft_entry__.smoke()
