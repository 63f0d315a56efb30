"""bin/trace_run as a user runs it: a child process fed steps on standard input, logits
read back from files, compared with the plain implementation; the same requests whole,
with the last 32 tokens one by one, and in batches of unequal lengths."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import plain_mistral as P

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {"float32": 1e-4, "bfloat16": 3e-2}


class Trace:
    def __init__(self, folder, dtype, out, max_tokens):
        self.out = out
        self.p = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder,
                                   "--dtype", dtype, "--out", out, "--max-tokens", str(max_tokens)],
                                  stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
        self.n = 0

    def step(self, entries, end=()):
        self.p.stdin.write(json.dumps({"step": self.n, "entries": entries, "end": list(end)}) + "\n")
        self.p.stdin.flush()
        line = self.p.stdout.readline().strip()
        assert line == f"done {self.n}", f"trace_run said {line!r} (exit {self.p.poll()})"
        path = os.path.join(self.out, f"{self.n}.f32")
        self.n += 1
        return np.fromfile(path, dtype="<f4") if os.path.exists(path) else None

    def close(self):
        self.p.stdin.close()
        assert self.p.wait(timeout=60) == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["b", "c"])
def test_replay_under_every_cut(tiny_folders, tmp_path, name, dtype):
    folder, cfg, w = tiny_folders[name]
    V = cfg["vocab_size"]
    rng = np.random.default_rng(7)
    lens = [100, 37, 64, 5]
    seqs = [[int(t) for t in rng.integers(0, V, n)] for n in lens]
    refs = [P.forward(cfg, w, s) for s in seqs]
    tr = Trace(folder, dtype, str(tmp_path / "out"), max_tokens=512)

    def check(got, want, what):
        got = got.reshape(-1, V)
        assert got.shape == want.shape, what
        assert np.abs(got - want).max() <= TOL[dtype] * np.abs(want).max(), what

    # whole, alone
    for i, s in enumerate(seqs):
        got = tr.step([{"id": f"w{i}", "tokens": s, "want": list(range(len(s)))}], end=[f"w{i}"])
        check(got, refs[i], f"whole {i}")
    # the last 32 tokens one by one (requests longer than 32)
    for i in (0, 1):
        s, n0 = seqs[i], lens[i] - 32
        assert tr.step([{"id": f"d{i}", "tokens": s[:n0], "want": []}]) is None
        for t in range(n0, lens[i]):
            got = tr.step([{"id": f"d{i}", "tokens": [s[t]], "want": [0]}], end=[f"d{i}"] if t == lens[i] - 1 else [])
            check(got, refs[i][t:t + 1], f"one by one {i}@{t}")
    # two batches of unequal lengths; prompts then one token each; shorter requests end earlier
    for batch in ([0, 1, 2, 3], [3, 1]):
        cut = {i: max(1, lens[i] - 3 - 2 * k) for k, i in enumerate(batch)}
        got = tr.step([{"id": f"b{i}", "tokens": seqs[i][:cut[i]], "want": [cut[i] - 1]} for i in batch])
        check(got, np.stack([refs[i][cut[i] - 1] for i in batch]), "batch prompts")
        pos, live = dict(cut), list(batch)
        while live:
            ending = [i for i in live if pos[i] + 1 == lens[i]]
            got = tr.step([{"id": f"b{i}", "tokens": [seqs[i][pos[i]]], "want": [0]} for i in live],
                          end=[f"b{i}" for i in ending])
            check(got, np.stack([refs[i][pos[i]] for i in live]), "batch decode")
            for i in live:
                pos[i] += 1
            live = [i for i in live if i not in ending]
    tr.close()


def test_bad_input_is_an_error_not_a_crash(tiny_folders, tmp_path):
    folder, cfg, _ = tiny_folders["a"]
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "fp32",
                        "--out", str(tmp_path / "o"), "--max-tokens", "64"],
                       input=json.dumps({"step": 0, "entries": [{"id": "a", "tokens": [99999], "want": [0]}], "end": []}) + "\n",
                       capture_output=True, text=True)
    assert p.returncode == 1 and "vocabulary" in p.stderr
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                        "--out", str(tmp_path / "o"), "--max-tokens", "64"],
                       input=json.dumps({"step": 0, "entries": [{"id": "a", "tokens": [1] * 65, "want": []}], "end": []}) + "\n",
                       capture_output=True, text=True)
    assert p.returncode == 1 and "cache" in p.stderr


def test_probes_switched_on_leave_statistics_beside_the_logits(tiny_folders, tmp_path):
    folder, cfg, w = tiny_folders["a"]
    out = str(tmp_path / "o")
    toks = [3, 9, 200, 41, 7]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:4], "want": [3]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[4:], "want": [0]}], "end": ["a"]}]
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                        "--out", out, "--max-tokens", "64", "--probes"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True)
    assert p.returncode == 0 and p.stdout.split() == ["done", "0", "done", "1"], p.stderr
    ref = P.forward(cfg, w, toks)
    for n, row in ((0, 3), (1, 4)):
        stats = json.load(open(os.path.join(out, f"{n}.probes.json")))
        assert list(stats) == ["embed", "L0.post_mixer", "L0.post_ffn", "L1.post_mixer", "L1.post_ffn", "final_norm", "logits"]
        assert stats["logits"]["shape"] == [1, cfg["vocab_size"]]
        assert abs(stats["logits"]["absmax"] - np.abs(ref[row]).max()) < 1e-4 * np.abs(ref[row]).max()
        got = np.fromfile(os.path.join(out, f"{n}.f32"), dtype="<f4")
        assert np.abs(got - ref[row]).max() < 1e-4 * np.abs(ref[row]).max()
    emb = P.embedding(w["model.embed_tokens.weight"], toks[:4])
    first = json.load(open(os.path.join(out, "0.probes.json")))["embed"]
    assert first["shape"] == [4, cfg["hidden_size"]] and np.allclose(first["head"], emb.reshape(-1)[:8], atol=1e-6)
    assert abs(first["rms"] - np.sqrt((emb ** 2).mean())) < 1e-5


def test_a_replay_is_not_bound_by_the_configurations_positions(tmp_path):
    """config.json without max_position_embeddings means 2,048 to the engine's own entry
    points; a replay sized for a longer request still takes it."""
    import json as _json
    import braidinfer_amd as B
    cfg = B.preset("tiny-a")
    folder = B.Engine.write_random_folder(str(tmp_path / "m"), cfg, seed=3, std=0.08)
    d = _json.load(open(os.path.join(folder, "config.json")))
    del d["max_position_embeddings"]
    _json.dump(d, open(os.path.join(folder, "config.json"), "w"))
    pc, w = P.read_folder(folder)
    toks = [int(t) for t in np.random.default_rng(0).integers(0, 256, 2100)]
    tr = Trace(folder, "float32", str(tmp_path / "o"), max_tokens=2112)
    assert tr.step([{"id": "a", "tokens": toks[:2090], "want": []}]) is None
    got = tr.step([{"id": "a", "tokens": toks[2090:], "want": [9]}], end=["a"])
    tr.close()
    ref = P.forward(pc, w, toks)[-1]
    assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max()
