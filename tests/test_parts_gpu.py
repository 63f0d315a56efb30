"""Each part alone on the GPU against the plain implementation's function for it, and
the generality of the arrangement: a toy mixer with state of its own that is registered,
built and stepped without a change to the library; a layer run twice; a layer that reads
another layer's cache."""
from dataclasses import dataclass

import numpy as np
import pytest
import torch

import braidinfer_amd as B
import plain_mistral as P
from braidinfer_amd import StepEntry
from braidinfer_amd.cache import SequenceCache, StateNeed
from braidinfer_amd.config import (LayerSpec, ModelSpec, PartSpec, ScheduleEntry, prenorm_layer, register_architecture,
                                   unregister_architecture)
from braidinfer_amd.engine import Workspace, pack_step
from braidinfer_amd.parts import (Mixer, MixerContext, RotaryTables, Runtime, build_part, register_part, unregister_part)
from braidinfer_amd.weights import TensorSpec

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
# the tensor-name pieces the toy models below use for the common layer
NAMES = dict(mixer_name="self_attn.", feed_forward_name="mlp.", mixer_norm_name="input_layernorm.",
             ffn_norm_name="post_attention_layernorm.")


def rt(dtype):
    return Runtime(DEV, dtype)


def bf(a):
    """Values as the bf16 path stores them."""
    return torch.tensor(a).bfloat16().float().numpy()


def dev(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a, np.float32)).to(dtype).to(DEV)


def make_step(lens, starts=None, slots=None):
    starts = starts or [0] * len(lens)
    slots = slots if slots is not None else list(range(len(lens)))
    toks = [[1] * n for n in lens]
    return pack_step(slots, toks, starts, DEV, Workspace(DEV))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    part = build_part("norm", PartSpec("rmsnorm", {"size": 100, "eps": 3e-6}))
    assert [(s.name, s.shape, s.kind) for s in part.weight_specs("n.")] == [("n.weight", (100,), "vector")]
    rng = np.random.default_rng(0)
    w, x = (1 + 0.3 * rng.normal(size=100)).astype(np.float32), rng.normal(size=(6, 100)).astype(np.float32) * 4
    part.load({"n.weight": dev(w)}, "n.", rt(dtype))
    out = torch.empty(6, 100, device=DEV, dtype=dtype)
    part.forward(dev(x), out)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert np.abs(out.float().cpu().numpy() - P.rms_norm(x, w, 3e-6)).max() < tol * 8


@pytest.mark.parametrize("pairing", ["half", "adjacent"])
def test_position_part_gives_the_plain_angles(pairing):
    part = build_part("position", PartSpec("rope", {"rotary_dim": 48, "theta": 5e5, "pairing": pairing}))
    part.load({}, "", rt(torch.float32))
    assert np.abs(part.inv_freq.cpu().numpy() - P.rope_inv_freq(48, 5e5)).max() < 1e-9
    step = make_step([5, 3], starts=[100, 4000])
    tabs = part.prepare(step)
    pos = np.array([100, 101, 102, 103, 104, 4000, 4001, 4002], np.float32)
    th = pos[:, None] * P.rope_inv_freq(48, 5e5)[None, :]
    assert np.abs(tabs.cos.cpu().numpy() - np.cos(th)).max() < 1e-5
    assert np.abs(tabs.sin.cpu().numpy() - np.sin(th)).max() < 1e-5
    assert tabs.adjacent == (pairing == "adjacent") and tabs.rotary_dim == 48


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_part(dtype):
    part = build_part("feed_forward", PartSpec("swiglu", {"hidden_size": 100, "intermediate_size": 172}))
    rng = np.random.default_rng(1)
    g, u, d = (bf(rng.normal(size=s).astype(np.float32) * 0.1) for s in ((172, 100), (172, 100), (100, 172)))
    wdt = dtype
    part.load({"f.gate_proj.weight": dev(g, wdt), "f.up_proj.weight": dev(u, wdt), "f.down_proj.weight": dev(d, wdt)},
              "f.", rt(dtype))
    h = bf(rng.normal(size=(9, 100)).astype(np.float32))
    x0 = rng.normal(size=(9, 100)).astype(np.float32)
    x = dev(x0)
    part.forward(dev(h, dtype), x, make_step([9]))
    want = x0 + P.swiglu(h, g, u, d)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert np.abs(x.cpu().numpy() - want).max() < tol * np.abs(want).max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [None, 5])
def test_attention_part_with_its_cache(dtype, window):
    nq, nkv, hd, H = 6, 3, 32, 96
    part = build_part("mixer", PartSpec("gqa_attention", {"hidden_size": H, "num_heads": nq, "num_kv_heads": nkv,
                                                          "head_dim": hd, "window": window, "position": "rope"}))
    assert part.cache_need() == B.cache.CacheNeed(nkv, hd, window) if hasattr(B, "cache") else True
    rope = build_part("position", PartSpec("rope", {"rotary_dim": hd, "theta": 1e4, "pairing": "half"}))
    rng = np.random.default_rng(2)
    w = {n: bf(rng.normal(size=s).astype(np.float32) * 0.15) for n, s in
         (("q", (nq * hd, H)), ("k", (nkv * hd, H)), ("v", (nkv * hd, H)), ("o", (H, nq * hd)))}
    part.load({f"a.{n}_proj.weight": dev(m, dtype) for n, m in w.items()}, "a.", rt(dtype))
    rope.load({}, "", rt(dtype))
    cache = SequenceCache({0: part.cache_need()}, {}, max_tokens=256, dtype=dtype, device=DEV)
    T = 20
    h = bf(rng.normal(size=(T, H)).astype(np.float32))
    x0 = rng.normal(size=(T, H)).astype(np.float32)
    # plain: the attention half of a block without its norm
    q = P.rope(P.linear(h, w["q"]).reshape(T, nq, hd), np.arange(T), P.rope_inv_freq(hd, 1e4), "half")
    k = P.rope(P.linear(h, w["k"]).reshape(T, nkv, hd), np.arange(T), P.rope_inv_freq(hd, 1e4), "half")
    v = P.linear(h, w["v"]).reshape(T, nkv, hd)
    want = x0 + P.linear(P.attention(q, k, v, nq, nkv, window).reshape(T, nq * hd), w["o"])
    slot = cache.alloc_slot()
    got = []
    for lo, hi in ((0, 13), (13, 14), (14, 20)):          # a prompt, one token, a further chunk
        cache.reserve([slot], [hi - lo])
        step = pack_step([slot], [[1] * (hi - lo)], [lo], DEV, Workspace(DEV))
        step.position_data = {"rope": rope.prepare(step)}
        g = cache.unit_group(0)
        ctx = MixerContext(unit=0, storage=g.storage_view(0), block_table=g.table_dev, page_tokens=g.page_tokens)
        x = dev(x0[lo:hi])
        part.forward(dev(h[lo:hi], dtype), x, step, ctx)
        cache.commit([slot], [hi - lo])
        got.append(x.cpu().numpy())
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert np.abs(np.concatenate(got) - want).max() < tol * np.abs(want).max()


def test_embedding_and_head_parts():
    emb = build_part("embedding", PartSpec("embedding", {"vocab_size": 301, "hidden_size": 100}))
    head = build_part("lm_head", PartSpec("lm_head", {"vocab_size": 301, "hidden_size": 100,
                                                      "tied_to": "e.weight"}))
    assert head.weight_specs("lm_head.") == [] and head.optional_names("lm_head.") == ["lm_head.weight"]
    table = bf(np.random.default_rng(3).normal(size=(301, 100)).astype(np.float32))
    tensors = {"e.weight": dev(table, torch.bfloat16)}
    emb.load(tensors, "e.", rt(torch.bfloat16))
    head.load(tensors, "lm_head.", rt(torch.bfloat16))
    x = torch.empty(4, 100, device=DEV)
    emb.forward(torch.tensor([300, 0, 17, 17], dtype=torch.int32, device=DEV), x)
    assert np.array_equal(x.cpu().numpy(), table[[300, 0, 17, 17]])
    logits = torch.empty(4, 301, device=DEV)
    head.forward(x.bfloat16(), logits, Workspace(DEV))
    assert np.abs(logits.cpu().numpy() - table[[300, 0, 17, 17]] @ table.T).max() < 1e-3 * 100


# ------------------------------------------------------------- a toy mixer with state ----
class RunningSumMixer(Mixer):
    """out[t] = W (sum of the sequence's inputs up to and including t).  Its per-sequence
    state is the running sum: fixed size, kept in the cache's state area.  It uses torch
    operations: it is a test's toy, not a part of the library."""

    def __init__(self, hidden_size):
        self.H = hidden_size

    def weight_specs(self, prefix):
        return [TensorSpec(prefix + "mix.weight", (self.H, self.H))]

    def load(self, tensors, prefix, rt):
        self.rt = rt
        self.w = tensors[prefix + "mix.weight"].float()

    def state_need(self):
        return StateNeed((self.H,), torch.float32)

    def forward(self, h, x, step, ctx):
        o = 0
        for b, n in enumerate(step.host_new):
            slot = step.host_slots[b]
            if slot >= 0:
                c = torch.cumsum(h[o:o + n].float(), 0) + ctx.state[slot]
                ctx.state[slot] = c[-1]
                x[o:o + n] += c @ self.w.T
            o += n


@dataclass(frozen=True)
class ToyConfig:
    hidden_size: int = 40
    vocab_size: int = 90
    architecture = "ToyRunningSumForCausalLM"

    @classmethod
    def from_dict(cls, d):
        return cls(d["hidden_size"], d["vocab_size"])

    def to_dict(self):
        return {"architectures": [self.architecture], "hidden_size": self.hidden_size, "vocab_size": self.vocab_size}


def toy_spec(cfg):
    H = cfg.hidden_size
    norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-5})
    attn = PartSpec("gqa_attention", {"hidden_size": H, "num_heads": 2, "num_kv_heads": 1, "head_dim": 16,
                                      "window": None, "position": "rope"})
    layers = [
        prenorm_layer("toy.layers.0.", PartSpec("running_sum", {"hidden_size": H}), None, norm, None, **NAMES),
        prenorm_layer("toy.layers.1.", attn, PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 56}), norm, norm, **NAMES),
    ]
    return ModelSpec(architecture=cfg.architecture, hidden_size=H, vocab_size=cfg.vocab_size,
                     embedding=PartSpec("embedding", {"vocab_size": cfg.vocab_size, "hidden_size": H}),
                     layers=layers, schedule=[ScheduleEntry(0, None), ScheduleEntry(1, 0)], final_norm=norm,
                     lm_head=PartSpec("lm_head", {"vocab_size": cfg.vocab_size, "hidden_size": H, "tied_to": None}),
                     positions={"rope": PartSpec("rope", {"rotary_dim": 16, "theta": 1e4, "pairing": "half"})},
                     max_position_embeddings=512, embedding_prefix="toy.embed.", final_norm_prefix="toy.norm.",
                     lm_head_prefix="toy.head.")


@pytest.fixture
def toy_registered():
    register_part("mixer", "running_sum", RunningSumMixer)
    register_architecture("ToyRunningSumForCausalLM", ToyConfig, toy_spec)
    yield
    unregister_architecture("ToyRunningSumForCausalLM")
    unregister_part("mixer", "running_sum")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_mixer_with_state_is_registered_built_and_stepped(toy_registered, tmp_path, dtype):
    cfg = ToyConfig()
    folder = B.Engine.write_random_folder(str(tmp_path / "toy"), cfg, seed=4, std=0.1)
    eng = B.Engine.from_folder(folder, dtype=dtype, max_tokens=512)      # the registry finds the toy by config.json
    assert eng.cache.state_bytes_per_slot == 40 * 4 and len(eng.cache.groups) == 1
    _, w = P.read_folder(folder)

    def plain(toks):
        x = P.embedding(w["toy.embed.weight"], toks)
        n = P.rms_norm(x, w["toy.layers.0.input_layernorm.weight"], 1e-5)
        x = x + np.cumsum(n, axis=0) @ w["toy.layers.0.self_attn.mix.weight"].T
        sz = dict(nq=2, nkv=1, hd=16, theta=1e4, eps=1e-5, pairing="half")
        x = P.attention_block(x, np.arange(len(toks)), w, "toy.layers.1.", sz, None)
        x = P.ffn_block(x, w, "toy.layers.1.", sz)
        return P.linear(P.rms_norm(x, w["toy.norm.weight"], 1e-5), w["toy.head.weight"])

    rng = np.random.default_rng(0)
    seqs = [[int(t) for t in rng.integers(0, 90, n)] for n in (30, 9, 17)]
    refs = [plain(s) for s in seqs]
    tol = 1e-4 if dtype == "float32" else 4e-2
    for round_ in range(2):                                   # twice: the state of a reused slot starts at zero
        slots = [eng.alloc_slot() for _ in seqs]
        cut = [12, 4, 16]
        out = eng.step([StepEntry(sl, s[:c], list(range(c))) for sl, s, c in zip(slots, seqs, cut)]).cpu().numpy()
        got = [[out[sum(cut[:i]):sum(cut[:i + 1])]] for i in range(3)]
        pos = list(cut)
        live = [0, 1, 2]
        while live:
            out = eng.step([StepEntry(slots[i], [seqs[i][pos[i]]], [0]) for i in live]).cpu().numpy()
            for r, i in enumerate(live):
                got[i].append(out[r:r + 1]); pos[i] += 1
            for i in [i for i in live if pos[i] == len(seqs[i])]:
                eng.free_slot(slots[i]); live.remove(i)
        for i in range(3):
            g = np.concatenate(got[i])
            assert np.abs(g - refs[i]).max() < tol * np.abs(refs[i]).max(), (round_, i)


# ------------------------------------------------------------- mixers side by side ----
@dataclass(frozen=True)
class SideConfig:
    architecture = "ToySideBySideForCausalLM"

    @classmethod
    def from_dict(cls, d):
        return cls()

    def to_dict(self):
        return {"architectures": [self.architecture]}


def side_by_side(layer, x, step, mixer_ctx):
    """x += mixer(n) + every further mixer(n), n = norm(x): all read the same normed rows; then the
    feed-forward half as usual."""
    h = step.ws.get("side_h", tuple(x.shape), layer.rt.dtype)
    layer.norms["mixer"].forward(x, h)
    layer.mixer.forward(h, x, step, mixer_ctx)
    for role, m in layer.more_mixers.items():
        m.forward(h, x, step, mixer_ctx.others[role])
    h2 = step.ws.get("side_h2", tuple(x.shape), layer.rt.dtype)
    layer.norms["feed_forward"].forward(x, h2)
    layer.feed_forward.forward(h2, x, step)


def side_spec(cfg):
    H = 48
    norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-5})
    attn = lambda window: PartSpec("gqa_attention", {"hidden_size": H, "num_heads": 3, "num_kv_heads": 1, "head_dim": 16,
                                                     "window": window, "position": "rope"})
    ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 56})
    names = {"mixer": "self_attn.", "feed_forward": "mlp.", "norm.mixer": "input_layernorm.",
             "norm.feed_forward": "post_attention_layernorm."}
    layers = [
        # attention beside a mixer with state of its own
        LayerSpec("s.layers.0.", attn(None), ffn, {"mixer": norm, "feed_forward": norm}, "side_by_side",
                  dict(names, **{"mixer.recurrent": "rec."}), more_mixers={"recurrent": PartSpec("running_sum", {"hidden_size": H})}),
        # attention over everything beside attention over the last 5 tokens, each with a cache unit of its own
        LayerSpec("s.layers.1.", attn(None), ffn, {"mixer": norm, "feed_forward": norm}, "side_by_side",
                  dict(names, **{"mixer.local": "local_attn."}), more_mixers={"local": attn(5)}),
    ]
    return ModelSpec(architecture=cfg.architecture, hidden_size=H, vocab_size=70,
                     embedding=PartSpec("embedding", {"vocab_size": 70, "hidden_size": H}), layers=layers,
                     schedule=[ScheduleEntry(0, 0), ScheduleEntry(1, 1, more_caches={"local": 2})], final_norm=norm,
                     lm_head=PartSpec("lm_head", {"vocab_size": 70, "hidden_size": H, "tied_to": None}),
                     positions={"rope": PartSpec("rope", {"rotary_dim": 16, "theta": 1e4, "pairing": "half"})},
                     max_position_embeddings=512, embedding_prefix="s.embed.", final_norm_prefix="s.norm.",
                     lm_head_prefix="s.head.")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_with_mixers_side_by_side(tmp_path, dtype):
    """A layer may hold further mixers by role (`LayerSpec.more_mixers`), each with a cache unit
    (`ScheduleEntry.more_caches`) and state of its own; an arrangement registered here runs them beside the
    layer's mixer.  Whole prompts, single tokens and a batch, twice over so that slots and state are used again."""
    register_part("mixer", "running_sum", RunningSumMixer)
    register_part("block", "side_by_side", lambda: side_by_side)
    register_architecture("ToySideBySideForCausalLM", SideConfig, side_spec)
    try:
        folder = B.Engine.write_random_folder(str(tmp_path / "s"), SideConfig(), seed=6, std=0.12)
        eng = B.Engine.from_folder(folder, dtype=dtype, max_tokens=512)
        assert len(eng.cache.groups) == 2 and sorted(len(g.unit_ids) for g in eng.cache.groups) == [1, 2]
        assert eng.cache.state_bytes_per_slot == 48 * 4 and not eng.use_graphs        # the toy mixer is not graph safe
        _, w = P.read_folder(folder)
        assert "s.layers.0.rec.mix.weight" in w and "s.layers.1.local_attn.q_proj.weight" in w
        sz = dict(nq=3, nkv=1, hd=16, theta=1e4, eps=1e-5, pairing="half")

        def plain(toks):
            pos = np.arange(len(toks))
            x = P.embedding(w["s.embed.weight"], toks)
            n = P.rms_norm(x, w["s.layers.0.input_layernorm.weight"], 1e-5)
            x = P.attention_block(x, pos, w, "s.layers.0.", sz, None) + np.cumsum(n, axis=0) @ w["s.layers.0.rec.mix.weight"].T
            x = P.ffn_block(x, w, "s.layers.0.", sz)
            local = {k.replace("local_attn.", "self_attn."): v for k, v in w.items()
                     if k.startswith("s.layers.1.local_attn.") or k == "s.layers.1.input_layernorm.weight"}
            x = P.attention_block(x, pos, w, "s.layers.1.", sz, None) + (P.attention_block(x, pos, local, "s.layers.1.", sz, 5) - x)
            x = P.ffn_block(x, w, "s.layers.1.", sz)
            return P.linear(P.rms_norm(x, w["s.norm.weight"], 1e-5), w["s.head.weight"])

        rng = np.random.default_rng(3)
        seqs = [[int(t) for t in rng.integers(0, 70, n)] for n in (40, 11, 23)]
        refs = [plain(q) for q in seqs]
        tol = 1e-4 if dtype == "float32" else 4e-2
        for round_ in range(2):
            slots = [eng.alloc_slot() for _ in seqs]
            cut = [30, 3, 22]
            out = eng.step([StepEntry(sl, q[:c], list(range(c))) for sl, q, c in zip(slots, seqs, cut)]).cpu().numpy()
            got = [[out[sum(cut[:i]):sum(cut[:i + 1])]] for i in range(3)]
            pos, live = list(cut), [0, 1, 2]
            while live:
                out = eng.step([StepEntry(slots[i], [seqs[i][pos[i]]], [0]) for i in live]).cpu().numpy()
                for r, i in enumerate(live):
                    got[i].append(out[r:r + 1]); pos[i] += 1
                for i in [i for i in live if pos[i] == len(seqs[i])]:
                    eng.free_slot(slots[i]); live.remove(i)
            assert all(g.pool.held_count == 0 for g in eng.cache.groups)
            for i in range(3):
                g = np.concatenate(got[i])
                assert np.abs(g - refs[i]).max() < tol * np.abs(refs[i]).max(), (round_, i)
    finally:
        unregister_architecture("ToySideBySideForCausalLM")
        unregister_part("block", "side_by_side")
        unregister_part("mixer", "running_sum")


# ------------------------------------------------------- the run order is data too ----
@dataclass(frozen=True)
class LoopConfig:
    mode: str = "twice"
    architecture = "ToyLoopForCausalLM"

    @classmethod
    def from_dict(cls, d):
        return cls(d["mode"])

    def to_dict(self):
        return {"architectures": [self.architecture], "mode": self.mode}


def loop_spec(cfg):
    H = 48
    norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-5})
    attn = PartSpec("gqa_attention", {"hidden_size": H, "num_heads": 3, "num_kv_heads": 1, "head_dim": 16,
                                      "window": None, "position": "rope"})
    layers = [prenorm_layer(f"m.layers.{i}.", attn, None, norm, None, **NAMES) for i in range(2)]
    if cfg.mode == "twice":       # layer 0, layer 1, layer 0 again with a cache of its own
        schedule = [ScheduleEntry(0, 0), ScheduleEntry(1, 1), ScheduleEntry(0, 2)]
    else:                         # layer 1 reads the keys and values layer 0 stored, and stores none
        schedule = [ScheduleEntry(0, 0), ScheduleEntry(1, 0, writes_cache=False)]
    return ModelSpec(architecture=cfg.architecture, hidden_size=H, vocab_size=70,
                     embedding=PartSpec("embedding", {"vocab_size": 70, "hidden_size": H}), layers=layers,
                     schedule=schedule, final_norm=norm,
                     lm_head=PartSpec("lm_head", {"vocab_size": 70, "hidden_size": H, "tied_to": "m.embed.weight"}),
                     positions={"rope": PartSpec("rope", {"rotary_dim": 16, "theta": 1e4, "pairing": "half"})},
                     max_position_embeddings=512, embedding_prefix="m.embed.", final_norm_prefix="m.norm.",
                     lm_head_prefix="m.head.")


@pytest.mark.parametrize("mode", ["twice", "shared"])
def test_schedule_names_a_layer_twice_or_shares_a_cache(tmp_path, mode):
    register_architecture("ToyLoopForCausalLM", LoopConfig, loop_spec)
    try:
        folder = B.Engine.write_random_folder(str(tmp_path / mode), LoopConfig(mode), seed=2, std=0.15)
        eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=256)
        _, w = P.read_folder(folder)
        sz = dict(nq=3, nkv=1, hd=16, theta=1e4, eps=1e-5, pairing="half")
        toks = [int(t) for t in np.random.default_rng(1).integers(0, 70, 40)]
        T = len(toks)
        x = P.embedding(w["m.embed.weight"], toks)
        if mode == "twice":
            assert sorted(eng.cache.group_of_unit) == [0, 1, 2]
            for p in ("m.layers.0.", "m.layers.1.", "m.layers.0."):
                x = P.attention_block(x, np.arange(T), w, p, sz, None)
        else:
            assert sorted(eng.cache.group_of_unit) == [0]
            inv = P.rope_inv_freq(16, 1e4)
            n0 = P.rms_norm(x, w["m.layers.0.input_layernorm.weight"], 1e-5)
            k0 = P.rope(P.linear(n0, w["m.layers.0.self_attn.k_proj.weight"]).reshape(T, 1, 16), np.arange(T), inv, "half")
            v0 = P.linear(n0, w["m.layers.0.self_attn.v_proj.weight"]).reshape(T, 1, 16)
            x = P.attention_block(x, np.arange(T), w, "m.layers.0.", sz, None)
            n1 = P.rms_norm(x, w["m.layers.1.input_layernorm.weight"], 1e-5)
            q1 = P.rope(P.linear(n1, w["m.layers.1.self_attn.q_proj.weight"]).reshape(T, 3, 16), np.arange(T), inv, "half")
            x = x + P.linear(P.attention(q1, k0, v0, 3, 1).reshape(T, 48), w["m.layers.1.self_attn.o_proj.weight"])
        ref = P.linear(P.rms_norm(x, w["m.norm.weight"], 1e-5), w["m.embed.weight"])
        s = eng.alloc_slot()
        got = [eng.step([StepEntry(s, toks[:25], list(range(25)))]).cpu().numpy()]
        for t in toks[25:]:
            got.append(eng.step([StepEntry(s, [t], [0])]).cpu().numpy())
        eng.free_slot(s)
        assert np.abs(np.concatenate(got) - ref).max() < 1e-4 * np.abs(ref).max()
    finally:
        unregister_architecture("ToyLoopForCausalLM")


def test_a_schedule_that_reads_an_unwritten_cache_is_refused():
    register_architecture("ToyLoopForCausalLM", LoopConfig, loop_spec)
    try:
        spec = loop_spec(LoopConfig("shared"))
        bad = ModelSpec(**{**spec.__dict__, "schedule": [ScheduleEntry(1, 0, writes_cache=False), ScheduleEntry(0, 0)]})
        with pytest.raises(B.ConfigError, match="before"):
            B.DecoderModel(bad)
    finally:
        unregister_architecture("ToyLoopForCausalLM")


# ---------------------------------- a toy routed feed-forward and a toy position encoding ----
from braidinfer_amd.parts import FeedForward, PositionEncoding   # noqa: E402


class Top1Experts(FeedForward):
    """Two small experts and a router; each token goes to the expert with the larger router
    logit (computed in float), weighted by the softmax of the two.  torch operations: a
    test's toy."""

    def __init__(self, hidden_size, expert_size, num_experts=2):
        self.H, self.E, self.n = hidden_size, expert_size, num_experts

    def weight_specs(self, prefix):
        specs = [TensorSpec(prefix + "router.weight", (self.n, self.H))]
        for e in range(self.n):
            specs += [TensorSpec(prefix + f"experts.{e}.up.weight", (self.E, self.H)),
                      TensorSpec(prefix + f"experts.{e}.down.weight", (self.H, self.E))]
        return specs

    def load(self, tensors, prefix, rt):
        self.rt = rt
        self.router = tensors[prefix + "router.weight"].float()
        self.up = [tensors[prefix + f"experts.{e}.up.weight"].float() for e in range(self.n)]
        self.down = [tensors[prefix + f"experts.{e}.down.weight"].float() for e in range(self.n)]

    def forward(self, h, x, step):
        hf = h.float()
        logits = hf @ self.router.T
        gate = torch.softmax(logits, -1)
        pick = logits.argmax(-1)
        for e in range(self.n):
            m = pick == e
            if m.any():
                y = torch.relu(hf[m] @ self.up[e].T) @ self.down[e].T
                x[m] += y * gate[m, e:e + 1]


class LearnedPositions(PositionEncoding):
    """A table of position vectors added to the embeddings (no rotation anywhere)."""
    gives = "embedding"

    def __init__(self, max_positions, hidden_size):
        self.P, self.H = max_positions, hidden_size

    def weight_specs(self, prefix):
        return [TensorSpec(prefix + "weight", (self.P, self.H))]

    def load(self, tensors, prefix, rt):
        self.rt = rt
        self.table = tensors[prefix + "weight"].float()

    def add_to_embedding(self, x, step):
        x += self.table[step.positions.long()]


@dataclass(frozen=True)
class RoutedConfig:
    architecture = "ToyRoutedForCausalLM"

    @classmethod
    def from_dict(cls, d):
        return cls()

    def to_dict(self):
        return {"architectures": [self.architecture]}


def routed_spec(cfg):
    H = 48
    norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-5})
    attn = PartSpec("gqa_attention", {"hidden_size": H, "num_heads": 3, "num_kv_heads": 3, "head_dim": 16,
                                      "window": None, "position": None})          # attention without rotation
    layers = [prenorm_layer("r.layers.0.", attn, PartSpec("top1_experts", {"hidden_size": H, "expert_size": 24}), norm, norm, **NAMES),
              prenorm_layer("r.layers.1.", attn, PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 64}), norm, norm, **NAMES)]
    return ModelSpec(architecture=cfg.architecture, hidden_size=H, vocab_size=60,
                     embedding=PartSpec("embedding", {"vocab_size": 60, "hidden_size": H}), layers=layers,
                     schedule=[ScheduleEntry(0, 0), ScheduleEntry(1, 1)], final_norm=norm,
                     lm_head=PartSpec("lm_head", {"vocab_size": 60, "hidden_size": H, "tied_to": None}),
                     positions={"learned": PartSpec("learned_positions", {"max_positions": 128, "hidden_size": H})},
                     max_position_embeddings=128, embedding_prefix="r.embed.", final_norm_prefix="r.norm.",
                     lm_head_prefix="r.head.")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_routed_feed_forward_and_learned_positions(tmp_path, dtype):
    """Different feed-forwards in different layers, a position encoding that acts on the
    embeddings, attention that rotates nothing: registered, built and stepped from outside."""
    register_part("feed_forward", "top1_experts", Top1Experts)
    register_part("position", "learned_positions", LearnedPositions)
    register_architecture("ToyRoutedForCausalLM", RoutedConfig, routed_spec)
    try:
        folder = B.Engine.write_random_folder(str(tmp_path / "routed"), RoutedConfig(), seed=6, std=0.15)
        eng = B.Engine.from_folder(folder, dtype=dtype, max_tokens=256)
        assert not eng.use_graphs                          # the toys decide on the host: no graph capture
        _, w = P.read_folder(folder)

        gaps = []

        def plain(toks):
            T = len(toks)
            x = P.embedding(w["r.embed.weight"], toks) + w["position.learned.weight"][:T]
            for l, ffn in ((0, "experts"), (1, "swiglu")):
                p = f"r.layers.{l}."
                n = P.rms_norm(x, w[p + "input_layernorm.weight"], 1e-5)
                q, k, v = (P.linear(n, w[p + f"self_attn.{m}_proj.weight"]).reshape(T, 3, 16) for m in "qkv")
                x = x + P.linear(P.attention(q, k, v, 3, 3).reshape(T, 48), w[p + "self_attn.o_proj.weight"])
                n = P.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-5)
                if ffn == "swiglu":
                    x = x + P.swiglu(n, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
                else:
                    logits = n @ w[p + "mlp.router.weight"].T
                    gaps.append(np.abs(logits[:, 0] - logits[:, 1]).min())
                    gate = np.exp(logits - logits.max(-1, keepdims=True)); gate /= gate.sum(-1, keepdims=True)
                    for t in range(T):
                        e = int(logits[t].argmax())
                        y = np.maximum(n[t] @ w[p + f"mlp.experts.{e}.up.weight"].T, 0) @ w[p + f"mlp.experts.{e}.down.weight"].T
                        x[t] = x[t] + y * gate[t, e]
            return P.linear(P.rms_norm(x, w["r.norm.weight"], 1e-5), w["r.head.weight"])

        # tokens for which every routing decision is clear: the least difference of the two router logits is
        # 0.12 (of logits up to 2.3), ten times what bfloat16 rounding moves them by, so both precisions send
        # every token to the same expert and every position can be held to the usual bounds
        toks = [int(t) for t in np.random.default_rng(7).integers(0, 60, 50)]
        ref = plain(toks)
        assert min(gaps) > 0.1
        s = eng.alloc_slot()
        got = [eng.step([StepEntry(s, toks[:30], list(range(30)))]).cpu().numpy()]
        for t in toks[30:]:
            got.append(eng.step([StepEntry(s, [t], [0])]).cpu().numpy())
        eng.free_slot(s)
        got = np.concatenate(got)
        if dtype == "float32":
            assert np.abs(got - ref).max() < 1e-4 * np.abs(ref).max()
        else:
            cos = (got * ref).sum(-1) / (np.linalg.norm(got, axis=-1) * np.linalg.norm(ref, axis=-1))
            assert np.abs(got - ref).max() < 3e-2 * np.abs(ref).max() and cos.min() > 0.999
    finally:
        unregister_architecture("ToyRoutedForCausalLM")
        unregister_part("feed_forward", "top1_experts")
        unregister_part("position", "learned_positions")


# ------------------------------ four norms a layer, arranged by a function from outside ----
@dataclass(frozen=True)
class SandwichConfig:
    architecture = "ToySandwichForCausalLM"

    @classmethod
    def from_dict(cls, d):
        return cls()

    def to_dict(self):
        return {"architectures": [self.architecture]}


def sandwich(layer, x, step, ctx):
    """x += post_norm(part(pre_norm(x))) for the mixer, then for the feed-forward: the parts add
    into a zeroed buffer instead of the residual rows, and a second norm stands behind each."""
    for part, pre, post, extra in ((layer.mixer, "mixer", "post_mixer", (ctx,)),
                                   (layer.feed_forward, "feed_forward", "post_feed_forward", ())):
        h = torch.empty(x.shape, dtype=layer.rt.dtype, device=x.device)
        layer.norms[pre].forward(x, h)
        y = torch.zeros_like(x)
        part.forward(h, y, step, *extra)
        yn = torch.empty_like(x)
        layer.norms[post].forward(y, yn)
        x += yn


SANDWICH_NAMES = {"norm.mixer": "ln1.", "mixer": "attn.", "norm.post_mixer": "ln2.", "norm.feed_forward": "ln3.",
                  "feed_forward": "ffn.", "norm.post_feed_forward": "ln4."}


def sandwich_spec(cfg):
    H = 64
    norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-5})
    attn = PartSpec("gqa_attention", {"hidden_size": H, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16,
                                      "window": None, "position": "rope"})
    ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 96})
    roles = {r: norm for r in ("mixer", "post_mixer", "feed_forward", "post_feed_forward")}
    layers = [LayerSpec(f"s.layers.{i}.", attn, ffn, norms=roles, block="sandwich", names=SANDWICH_NAMES) for i in range(2)]
    return ModelSpec(architecture=cfg.architecture, hidden_size=H, vocab_size=80,
                     embedding=PartSpec("embedding", {"vocab_size": 80, "hidden_size": H}), layers=layers,
                     schedule=[ScheduleEntry(0, 0), ScheduleEntry(1, 1)], final_norm=norm,
                     lm_head=PartSpec("lm_head", {"vocab_size": 80, "hidden_size": H, "tied_to": None}),
                     positions={"rope": PartSpec("rope", {"rotary_dim": 16, "theta": 1e4, "pairing": "half"})},
                     max_position_embeddings=256, embedding_prefix="s.embed.", final_norm_prefix="s.norm.",
                     lm_head_prefix="s.head.")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_with_four_norms_arranged_from_outside(tmp_path, dtype):
    register_part("block", "sandwich", lambda: sandwich)
    register_architecture("ToySandwichForCausalLM", SandwichConfig, sandwich_spec)
    try:
        folder = B.Engine.write_random_folder(str(tmp_path / "s"), SandwichConfig(), seed=3, std=0.2, vector_jitter=0.3)
        eng = B.Engine.from_folder(folder, dtype=dtype, max_tokens=256)
        _, w = P.read_folder(folder)
        assert all(f"s.layers.1.ln{i}.weight" in w for i in (1, 2, 3, 4)) and "s.layers.0.attn.q_proj.weight" in w
        sz = dict(nq=4, nkv=2, hd=16)

        def plain(toks):
            T = len(toks)
            x = P.embedding(w["s.embed.weight"], toks)
            inv = P.rope_inv_freq(16, 1e4)
            for l in range(2):
                p = f"s.layers.{l}."
                n = P.rms_norm(x, w[p + "ln1.weight"], 1e-5)
                q, k, v = (P.linear(n, w[p + f"attn.{m}_proj.weight"]).reshape(T, -1, 16) for m in "qkv")
                q, k = P.rope(q, np.arange(T), inv, "half"), P.rope(k, np.arange(T), inv, "half")
                a = P.linear(P.attention(q, k, v, 4, 2).reshape(T, 64), w[p + "attn.o_proj.weight"])
                x = x + P.rms_norm(a, w[p + "ln2.weight"], 1e-5)
                n = P.rms_norm(x, w[p + "ln3.weight"], 1e-5)
                f = P.swiglu(n, w[p + "ffn.gate_proj.weight"], w[p + "ffn.up_proj.weight"], w[p + "ffn.down_proj.weight"])
                x = x + P.rms_norm(f, w[p + "ln4.weight"], 1e-5)
            return P.linear(P.rms_norm(x, w["s.norm.weight"], 1e-5), w["s.head.weight"])

        toks = [int(t) for t in np.random.default_rng(5).integers(0, 80, 70)]
        ref = plain(toks)
        s = eng.alloc_slot()
        got = [eng.step([StepEntry(s, toks[:66], list(range(66)))]).cpu().numpy()]
        for t in toks[66:]:
            got.append(eng.step([StepEntry(s, [t], [0])]).cpu().numpy())
        eng.free_slot(s)
        got = np.concatenate(got)
        assert np.abs(got - ref).max() < (1e-4 if dtype == "float32" else 4e-2) * np.abs(ref).max()
    finally:
        unregister_architecture("ToySandwichForCausalLM")
        unregister_part("block", "sandwich")


# ------------------------------------- a rotary encoding with two position numbers a token ----
class TwoSectionRotary(B.parts.PositionEncoding):
    """The lower half of the frequencies turns with a token's first position number, the upper
    half with its second (as encodings with sectioned positions do)."""
    gives = "rotary"

    def __init__(self, rotary_dim, theta):
        self.rd, self.theta = rotary_dim, theta

    def load(self, tensors, prefix, rt):
        self.rt = rt
        self.inv = torch.tensor(P.rope_inv_freq(self.rd, self.theta), device=rt.device)

    def prepare(self, step):
        ids = step.position_ids
        assert ids.dim() == 2 and ids.shape[1] == 2, "two position numbers per token"
        half = self.rd // 4
        which = torch.cat([ids[:, :1].expand(-1, half), ids[:, 1:].expand(-1, self.rd // 2 - half)], 1).float()
        th = which * self.inv[None, :]
        return RotaryTables(torch.cos(th).contiguous(), torch.sin(th).contiguous(), self.rd, False)


@dataclass(frozen=True)
class SectionConfig:
    architecture = "ToySectionForCausalLM"

    @classmethod
    def from_dict(cls, d):
        return cls()

    def to_dict(self):
        return {"architectures": [self.architecture]}


def section_spec(cfg):
    H = 48
    norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-5})
    attn = PartSpec("gqa_attention", {"hidden_size": H, "num_heads": 3, "num_kv_heads": 1, "head_dim": 16,
                                      "window": None, "position": "sections"})
    layers = [prenorm_layer("t.layers.0.", attn, PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 64}), norm, norm,
                            **NAMES)]
    return ModelSpec(architecture=cfg.architecture, hidden_size=H, vocab_size=70,
                     embedding=PartSpec("embedding", {"vocab_size": 70, "hidden_size": H}), layers=layers,
                     schedule=[ScheduleEntry(0, 0)], final_norm=norm,
                     lm_head=PartSpec("lm_head", {"vocab_size": 70, "hidden_size": H, "tied_to": None}),
                     positions={"sections": PartSpec("two_section_rotary", {"rotary_dim": 16, "theta": 1e4})},
                     max_position_embeddings=256, embedding_prefix="t.embed.", final_norm_prefix="t.norm.",
                     lm_head_prefix="t.head.")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_position_numbers_of_the_callers_own_two_a_token(tmp_path, dtype):
    register_part("position", "two_section_rotary", TwoSectionRotary)
    register_architecture("ToySectionForCausalLM", SectionConfig, section_spec)
    try:
        folder = B.Engine.write_random_folder(str(tmp_path / "t"), SectionConfig(), seed=9, std=0.2)
        eng = B.Engine.from_folder(folder, dtype=dtype, max_tokens=256)
        _, w = P.read_folder(folder)
        toks = [int(t) for t in np.random.default_rng(6).integers(0, 70, 40)]
        T = len(toks)
        ids = [(t, 5 + t // 3) for t in range(T)]

        inv = P.rope_inv_freq(16, 1e4)
        th = np.where(np.arange(8)[None, :] < 4, np.array([i[0] for i in ids], np.float32)[:, None],
                      np.array([i[1] for i in ids], np.float32)[:, None]).astype(np.float32) * inv[None, :]

        def rot(x):
            c, s_ = np.cos(th).astype(np.float32)[:, None, :], np.sin(th).astype(np.float32)[:, None, :]
            a, b = x[..., :8], x[..., 8:]
            return np.concatenate([a * c - b * s_, a * s_ + b * c], -1).astype(np.float32)

        x = P.embedding(w["t.embed.weight"], toks)
        p = "t.layers.0."
        n = P.rms_norm(x, w[p + "input_layernorm.weight"], 1e-5)
        q, k, v = (P.linear(n, w[p + f"self_attn.{m}_proj.weight"]).reshape(T, -1, 16) for m in "qkv")
        x = x + P.linear(P.attention(rot(q), rot(k), v, 3, 1).reshape(T, 48), w[p + "self_attn.o_proj.weight"])
        x = P.ffn_block(x, w, p, dict(eps=1e-5))
        ref = P.linear(P.rms_norm(x, w["t.norm.weight"], 1e-5), w["t.head.weight"])

        s = eng.alloc_slot()
        got = [eng.step([StepEntry(s, toks[:25], list(range(25)), position_ids=ids[:25])]).cpu().numpy()]
        for t in range(25, T):
            got.append(eng.step([StepEntry(s, [toks[t]], [0], position_ids=[ids[t]])]).cpu().numpy())
        got = np.concatenate(got)
        assert np.abs(got - ref).max() < (1e-4 if dtype == "float32" else 4e-2) * np.abs(ref).max()
        # a step must bring position numbers for all of its entries or for none, and one per token
        s2 = eng.alloc_slot()
        with pytest.raises(B.StepError, match="position"):
            eng.step([StepEntry(s, [1], [0], position_ids=[(40, 18)]), StepEntry(s2, [1], [0])])
        with pytest.raises(B.StepError, match="position numbers"):
            eng.step([StepEntry(s2, [1, 2], [0], position_ids=[(0, 5)])])
        assert eng.length(s2) == 0 and eng.length(s) == T
    finally:
        unregister_architecture("ToySectionForCausalLM")
        unregister_part("position", "two_section_rotary")


def test_attention_refuses_an_encoding_it_cannot_find_or_use():
    norm = PartSpec("rmsnorm", {"size": 32, "eps": 1e-5})

    def spec(position, positions):
        attn = PartSpec("gqa_attention", {"hidden_size": 32, "num_heads": 2, "num_kv_heads": 1, "head_dim": 16,
                                          "window": None, "position": position})
        return ModelSpec(architecture="x", hidden_size=32, vocab_size=50,
                         embedding=PartSpec("embedding", {"vocab_size": 50, "hidden_size": 32}),
                         layers=[prenorm_layer("x.0.", attn, None, norm, None, **NAMES)], schedule=[ScheduleEntry(0, 0)],
                         final_norm=norm, lm_head=PartSpec("lm_head", {"vocab_size": 50, "hidden_size": 32, "tied_to": None}),
                         positions=positions, max_position_embeddings=64, embedding_prefix="x.e.", final_norm_prefix="x.n.",
                         lm_head_prefix="x.h.")
    rope = {"rope": PartSpec("rope", {"rotary_dim": 16, "theta": 1e4, "pairing": "half"})}
    B.DecoderModel(spec("rope", rope))
    B.DecoderModel(spec(None, rope))
    with pytest.raises(B.ConfigError, match="position encoding 'rotary'"):
        B.DecoderModel(spec("rotary", rope))            # a misspelt name is an error, not attention without positions

    class Odd(B.parts.PositionEncoding):
        gives = "sinusoid_bias"
    register_part("position", "odd", Odd)
    try:
        with pytest.raises(B.ConfigError, match="cannot use"):
            B.DecoderModel(spec("p", {"p": PartSpec("odd", {})}))
    finally:
        unregister_part("position", "odd")


# --------------------- a mixer that keeps rows of two widths per token in the paged cache ----
class LatentMixer(Mixer):
    """One head; per token it keeps a 24-wide key and an 8-wide value in the cache (widths
    that differ), attends over the last `window` of them, and projects the 8-wide result out."""

    def __init__(self, hidden_size, window):
        self.H, self.window = hidden_size, window

    def weight_specs(self, prefix):
        return [TensorSpec(prefix + "q.weight", (24, self.H)), TensorSpec(prefix + "k.weight", (24, self.H)),
                TensorSpec(prefix + "v.weight", (8, self.H)), TensorSpec(prefix + "o.weight", (self.H, 8))]

    def load(self, tensors, prefix, rt):
        self.rt = rt
        self.q, self.k, self.v, self.o = (tensors[prefix + n + ".weight"].float() for n in "qkvo")

    def cache_need(self):
        return B.cache.CacheNeed(kv_heads=1, head_dim=24, window=self.window, value_dim=8)

    def first_visible(self, pos):
        return max(0, pos - self.window + 1)

    def forward(self, h, x, step, ctx):
        hf = h.float()
        q, k, v = hf @ self.q.T, hf @ self.k.T, hf @ self.v.T
        table = ctx.block_table.cpu()
        o = 0
        for b, n in enumerate(step.host_new):
            slot, start = step.host_slots[b], step.host_start[b]
            for i in range(n):
                pos = start + i
                pg = int(table[slot, pos // 64])
                ctx.keys[pg, 0].view(64, 24)[pos % 64] = k[o + i].to(ctx.keys.dtype)
                ctx.values[pg, 0].view(64, 8)[pos % 64] = v[o + i].to(ctx.values.dtype)
                lo = self.first_visible(pos)
                ks = torch.stack([ctx.keys[int(table[slot, j // 64]), 0].view(64, 24)[j % 64] for j in range(lo, pos + 1)]).float()
                vs = torch.stack([ctx.values[int(table[slot, j // 64]), 0].view(64, 8)[j % 64] for j in range(lo, pos + 1)]).float()
                p = torch.softmax(ks @ q[o + i] / 24 ** 0.5, 0)
                x[o + i] += (p @ vs) @ self.o.T
            o += n


def _chunk_start(length):
    return (length // 70) * 70


class ChunkedLatentMixer(LatentMixer):
    """The same mixer with another rule of what stays visible: a token sees the tokens of its own chunk of 70
    (`window` is the chunk's length here).  The cache learns the rule through `CacheNeed.live_from` and gives
    back the pages of finished chunks."""

    def cache_need(self):
        return B.cache.CacheNeed(kv_heads=1, head_dim=24, value_dim=8, live_from=_chunk_start)

    def first_visible(self, pos):
        return _chunk_start(pos)


@dataclass(frozen=True)
class LatentConfig:
    architecture = "ToyLatentForCausalLM"

    @classmethod
    def from_dict(cls, d):
        return cls()

    def to_dict(self):
        return {"architectures": [self.architecture]}


def latent_spec(cfg, mixer="latent"):
    H = 40
    norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-5})
    layers = [prenorm_layer(f"l.layers.{i}.", PartSpec(mixer, {"hidden_size": H, "window": 70}), None, norm, None, **NAMES)
              for i in range(2)]
    return ModelSpec(architecture=cfg.architecture, hidden_size=H, vocab_size=50,
                     embedding=PartSpec("embedding", {"vocab_size": 50, "hidden_size": H}), layers=layers,
                     schedule=[ScheduleEntry(0, 0), ScheduleEntry(1, 1)], final_norm=norm,
                     lm_head=PartSpec("lm_head", {"vocab_size": 50, "hidden_size": H, "tied_to": None}),
                     positions={}, max_position_embeddings=512, embedding_prefix="l.embed.", final_norm_prefix="l.norm.",
                     lm_head_prefix="l.head.")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rule", ["window", "chunks"])
def test_a_mixer_whose_keys_and_values_differ_in_width_uses_the_paged_cache(tmp_path, dtype, rule):
    """With the window's rule of what stays in the cache, and with a rule of the mixer's own (chunks)."""
    register_part("mixer", "latent", LatentMixer if rule == "window" else ChunkedLatentMixer)
    register_architecture("ToyLatentForCausalLM", LatentConfig, latent_spec)
    first_visible = (lambda t: max(0, t - 70 + 1)) if rule == "window" else _chunk_start
    try:
        folder = B.Engine.write_random_folder(str(tmp_path / "l"), LatentConfig(), seed=12, std=0.2)
        eng = B.Engine.from_folder(folder, dtype=dtype, max_tokens=512)
        g = eng.cache.groups[0]
        assert len(eng.cache.groups) == 1 and g.page_elems == 64 * (24 + 8) and g.keys(0).shape[1:] == (1, 64 * 24)
        assert g.values(1).shape[1:] == (1, 64 * 8) and g.storage_view(0).dim() == 2
        _, w = P.read_folder(folder)
        rd = (lambda a: bf(a)) if dtype == "bfloat16" else (lambda a: a)

        def plain(toks):
            T = len(toks)
            x = P.embedding(w["l.embed.weight"], toks)
            for l in range(2):
                p = f"l.layers.{l}.self_attn."
                n = rd(P.rms_norm(x, w[f"l.layers.{l}.input_layernorm.weight"], 1e-5))
                q, k, v = n @ w[p + "q.weight"].T, rd(n @ w[p + "k.weight"].T), rd(n @ w[p + "v.weight"].T)
                for t in range(T):
                    lo = first_visible(t)
                    sc = k[lo:t + 1] @ q[t] / np.sqrt(24.0)
                    pr = np.exp(sc - sc.max()); pr /= pr.sum()
                    x[t] = x[t] + (pr @ v[lo:t + 1]) @ w[p + "o.weight"].T
            return P.linear(rd(P.rms_norm(x, w["l.norm.weight"], 1e-5)), w["l.head.weight"])

        rng = np.random.default_rng(8)
        seqs = [[int(t) for t in rng.integers(0, 50, n)] for n in (150, 66)]
        refs = [plain(s) for s in seqs]
        for round_ in range(2):                                   # twice: pages come back and are used again
            slots = [eng.alloc_slot() for _ in seqs]
            cut = [100, 60]
            out = eng.step([StepEntry(sl, s[:c], list(range(c))) for sl, s, c in zip(slots, seqs, cut)]).cpu().numpy()
            got = [[out[:100]], [out[100:]]]
            pos, live = list(cut), [0, 1]
            while live:
                out = eng.step([StepEntry(slots[i], [seqs[i][pos[i]]], [0]) for i in live]).cpu().numpy()
                for r, i in enumerate(live):
                    got[i].append(out[r:r + 1]); pos[i] += 1
                for i in [i for i in live if pos[i] == len(seqs[i])]:
                    assert g.pool.held_count <= 3 * len(live)     # the window gives pages back while the sequence grows
                    eng.free_slot(slots[i]); live.remove(i)
            assert g.pool.held_count == 0
            for i in range(2):
                gi = np.concatenate(got[i])
                assert np.abs(gi - refs[i]).max() < (1e-4 if dtype == "float32" else 3e-2) * np.abs(refs[i]).max(), (round_, i)
    finally:
        unregister_architecture("ToyLatentForCausalLM")
        unregister_part("mixer", "latent")
