"""The plain implementation: a slow, whole-sequence Mistral forward in NumPy float32,
written from the reference's formulas, one function per part, no cache, no batching.
It shares no code with `braidinfer_amd` (it does not import it); tests compare the
engine with it.

Every function cites where the reference computes the same thing
(paths under crates/braidinfer-runtime/src/ or kernels/ of mcelrath/braidinfer).
Where the reference has nothing (sliding window) or deviates from the checkpoint
format (rotary pairing), the function's docstring says which convention is fixed.
"""
import json
import math
import os
import struct

import numpy as np

F = np.float32


# ---------------------------------------------------------------- reading a folder ----
def bf16_bytes_to_f32(raw):
    """bf16 -> f32 by shifting 16 bits (kernels/bf16_utils.h:7-12)."""
    u16 = np.frombuffer(raw, dtype="<u2").astype(np.uint32)
    return (u16 << 16).view(np.float32)


def read_safetensors(path):
    """Every tensor of one safetensors file as float32 arrays: 8 bytes header length, a JSON
    header {name: {dtype, shape, data_offsets}}, then the data
    (braidinfer-core/src/safetensors.rs:71-80)."""
    with open(path, "rb") as f:
        (hlen,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(hlen))
        data = f.read()
    tensors = {}
    for name, e in header.items():
        if name == "__metadata__":
            continue
        b, en = e["data_offsets"]
        raw = data[b:en]
        if e["dtype"] == "BF16":
            a = bf16_bytes_to_f32(raw)
        elif e["dtype"] == "F32":
            a = np.frombuffer(raw, dtype="<f4")
        else:
            raise ValueError(f"dtype {e['dtype']} of {name}")
        tensors[name] = a.reshape(e["shape"]).astype(F)
    return tensors


def read_folder(folder):
    """config.json as a dict and every tensor as float32 arrays, from model.safetensors or
    from the files that model.safetensors.index.json's weight_map names
    (braidinfer-core/src/safetensors.rs:102-159)."""
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    single = os.path.join(folder, "model.safetensors")
    if os.path.isfile(single):
        return cfg, read_safetensors(single)
    with open(os.path.join(folder, "model.safetensors.index.json")) as f:
        weight_map = json.load(f)["weight_map"]
    tensors = {}
    for fname in sorted(set(weight_map.values())):
        part = read_safetensors(os.path.join(folder, fname))
        for name, a in part.items():
            if weight_map.get(name) != fname or name in tensors:
                raise ValueError(f"{name} in {fname} disagrees with the index")
            tensors[name] = a
    return cfg, tensors


# ------------------------------------------------------------------ random weights ----
_M64 = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15


def _mix64(z):
    z &= _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def tensor_names(cfg):
    """The name table of a Mistral folder, in the order the random generator numbers the
    tensors: embedding; per layer the attention norm, q, k, v, o, the feed-forward norm,
    gate, up, down; the final norm; the head unless tied."""
    sz = sizes(cfg)
    H, I, V, nq, nkv, hd = sz["H"], sz["I"], sz["V"], sz["nq"], sz["nkv"], sz["hd"]
    out = [("model.embed_tokens.weight", (V, H))]
    for i in range(sz["L"]):
        p = f"model.layers.{i}."
        out += [(p + "input_layernorm.weight", (H,)),
                (p + "self_attn.q_proj.weight", (nq * hd, H)), (p + "self_attn.k_proj.weight", (nkv * hd, H)),
                (p + "self_attn.v_proj.weight", (nkv * hd, H)), (p + "self_attn.o_proj.weight", (H, nq * hd)),
                (p + "post_attention_layernorm.weight", (H,)),
                (p + "mlp.gate_proj.weight", (I, H)), (p + "mlp.up_proj.weight", (I, H)),
                (p + "mlp.down_proj.weight", (H, I))]
    out.append(("model.norm.weight", (H,)))
    if not sz["tied"]:
        out.append(("lm_head.weight", (V, H)))
    return out


def random_weights(cfg, seed, std=0.02, vector_jitter=0.0):
    """The random-weights mode's tensors as float32 arrays holding bfloat16 values, written
    with Python integers from the generator's definition (ours; the reference has no random
    weights): key = mix(mix(seed + G) + (t + 1) G) for tensor t of the name table;
    word(c) = mix(key + (c + 1) G); a matrix element i is (the twelve 16-bit fields of
    word(3i), word(3i+1), word(3i+2) added up, minus 393210) * (float32(std) * 2^-16); a norm
    weight is 1 + (2 u - 1) * jitter with u = (word(i) >> 40) * 2^-24; float32 is rounded to
    bfloat16 to nearest even (quant.rs:203-207)."""
    scale = F(F(std) * F(2.0 ** -16))
    out = {}
    for t, (name, shape) in enumerate(tensor_names(cfg)):
        key = _mix64(_mix64(seed + _GOLDEN) + (t + 1) * _GOLDEN)
        n = int(np.prod(shape))
        vals = np.empty(n, dtype=F)
        for i in range(n):
            if len(shape) == 1:
                u = F(_mix64(key + (i + 1) * _GOLDEN) >> 40) * F(2.0 ** -24)
                vals[i] = F(F(1.0) + F(F(F(u + u) - F(1.0)) * F(vector_jitter)))
            else:
                s = 0
                for c in (3 * i, 3 * i + 1, 3 * i + 2):
                    w = _mix64(key + (c + 1) * _GOLDEN)
                    s += (w & 0xFFFF) + ((w >> 16) & 0xFFFF) + ((w >> 32) & 0xFFFF) + (w >> 48)
                vals[i] = F(s - 393210) * scale
        bits = vals.view(np.uint32)
        rounded = ((bits + (((bits >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF))) >> np.uint32(16)) << np.uint32(16)
        out[name] = rounded.astype(np.uint32).view(F).reshape(shape)
    return out


def sizes(cfg):
    """Keys and defaults as config.rs:208-277 reads them, except tie_word_embeddings
    (false when absent) and sliding_window (read; config.rs never parses it)."""
    nq = cfg["num_attention_heads"]
    return dict(
        L=cfg["num_hidden_layers"], H=cfg["hidden_size"], nq=nq,
        nkv=cfg.get("num_key_value_heads", nq), hd=cfg.get("head_dim") or cfg["hidden_size"] // nq,
        I=cfg["intermediate_size"], V=cfg["vocab_size"], theta=float(cfg.get("rope_theta", 10000.0)),
        eps=float(cfg.get("rms_norm_eps", 1e-5)), window=cfg.get("sliding_window"),
        tied=bool(cfg.get("tie_word_embeddings", False)), pairing=cfg.get("rope_pairing", "half"),
        layer_types=cfg.get("layer_types"))


# ------------------------------------------------------------------------ the parts ----
def bf16_round(a):
    """float32 -> the nearest bfloat16 (ties to even), kept as float32 (quant.rs:203-207)."""
    bits = np.ascontiguousarray(a, dtype=F).view(np.uint32)
    r = ((bits + (((bits >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF))) >> np.uint32(16)) << np.uint32(16)
    return r.astype(np.uint32).view(F).reshape(np.shape(a))


def _same(a):
    return a


def rounding(act_dtype):
    """What the forward functions apply to every activation that a bfloat16 engine keeps in
    bfloat16: the normed rows, q, k and v as the projection leaves them, q and k after rotation
    (keys are cached so), the probabilities that multiply the values, the attention's output
    and the SwiGLU output.  The residual rows, scores, sums and logits stay float.
    None or "float32": nothing is rounded."""
    if act_dtype in (None, "float32"):
        return _same
    if act_dtype == "bfloat16":
        return bf16_round
    raise ValueError(f"act_dtype {act_dtype!r}")


def embedding(table, tokens):
    """x[t] = table[token[t]], no scaling (kernels/megakernel_ops.hip:1757-1768)."""
    return table[np.asarray(tokens, dtype=np.int64)].astype(F)


def rms_norm(x, w, eps):
    """y = x * rsqrt(mean(x^2) + eps) * w; eps inside the root, plain w
    (kernels/megakernel_ops.hip:862-904)."""
    x = x.astype(F)
    ms = (x * x).sum(axis=-1, keepdims=True, dtype=F) / F(x.shape[-1])
    return (x * (F(1.0) / np.sqrt(ms + F(eps))) * w.astype(F)).astype(F)


def linear(x, W):
    """y = x W^T, W stored [out, in], no bias (kernels/megakernel_ops.hip:166-276)."""
    return (x.astype(F) @ W.astype(F).T).astype(F)


def rope_inv_freq(rotary_dim, theta):
    """inv_freq[p] = 1 / theta^(2p / rotary_dim) in f32 (weights.rs:743-751)."""
    p = np.arange(rotary_dim // 2, dtype=F)
    expo = (F(2.0) * p / F(rotary_dim)).astype(F)
    return (F(1.0) / np.power(F(theta), expo, dtype=F)).astype(F)


def rope(x, positions, inv_freq, pairing):
    """Rotate pairs of each head by theta = f32(pos) * inv_freq[p]:
    a' = a cos - b sin, b' = a sin + b cos (kernels/megakernel_ops.hip:2019-2030).
    pairing "adjacent": (2p, 2p+1), as that kernel does; "half": (p, p + rd/2), the
    layout of MistralForCausalLM checkpoints (the convention the engine defaults to).
    x: [T, heads, hd]; only the first rd = 2 len(inv_freq) elements are rotated."""
    T, nh, hd = x.shape
    P = inv_freq.shape[0]
    th = (np.asarray(positions, dtype=F)[:, None] * inv_freq[None, :]).astype(F)   # [T, P]
    c, s = np.cos(th).astype(F)[:, None, :], np.sin(th).astype(F)[:, None, :]
    out = x.astype(F).copy()
    if pairing == "adjacent":
        a, b = x[..., 0:2 * P:2], x[..., 1:2 * P:2]
        out[..., 0:2 * P:2] = a * c - b * s
        out[..., 1:2 * P:2] = a * s + b * c
    else:
        a, b = x[..., :P], x[..., P:2 * P]
        out[..., :P] = a * c - b * s
        out[..., P:2 * P] = a * s + b * c
    return out.astype(F)


def attention(q, k, v, nq, nkv, window=None, scale=None, rnd=_same):
    """softmax over the keys a query may see of (q . k_j) * rsqrt(hd), times v
    (kernels/megakernel_ops.hip:2192-2194 kv head = q head / (nq/nkv) and the scale,
    :2310-2342 the softmax; causality is the loop bound j <= i, compile_attention.rs:285).
    Window W (ours; the reference has none): query i sees keys j with i - W < j <= i.
    q: [T, nq, hd], k, v: [T, nkv, hd] -> [T, nq, hd].
    `rnd` rounds the unnormalised probabilities exp(s - max) that multiply the values (the
    divisor stays the float sum of the unrounded ones)."""
    T, _, hd = q.shape
    scale = F(1.0 / math.sqrt(hd)) if scale is None else F(scale)
    out = np.zeros((T, nq, hd), dtype=F)
    g = nq // nkv
    i = np.arange(T)[:, None]
    j = np.arange(T)[None, :]
    allowed = j <= i
    if window is not None:
        allowed &= j > i - window
    for h in range(nq):
        kh = h // g
        s = (q[:, h, :].astype(F) @ k[:, kh, :].astype(F).T) * scale          # [T, T]
        s = np.where(allowed, s, F(-np.inf))
        m = s.max(axis=-1, keepdims=True)
        e = np.exp(s - m, dtype=F)
        if rnd is _same:
            p = e / e.sum(axis=-1, keepdims=True, dtype=F)
            out[:, h, :] = p.astype(F) @ v[:, kh, :].astype(F)
        else:
            out[:, h, :] = (rnd(e) @ v[:, kh, :].astype(F)) / e.sum(axis=-1, keepdims=True, dtype=F)
    return out


def silu(x):
    """silu(g) = g / (1 + exp(-g)) (kernels/megakernel_ops.hip:374-407)."""
    x = x.astype(F)
    return (x / (F(1.0) + np.exp(-x, dtype=F))).astype(F)


def swiglu(n, Wg, Wu, Wd, rnd=_same):
    """W_d (silu(W_g n) * (W_u n)) (kernels/megakernel_ops.hip:1538-1544, :1559-1602)."""
    return linear(rnd(silu(linear(n, Wg)) * linear(n, Wu)), Wd)


def attention_block(x, positions, w, prefix, sz, window, rnd=_same):
    """x + W_o attn(rope(W_q n), rope(W_k n), W_v n), n = norm(x)
    (megakernel/compile_attention.rs:78-376)."""
    T = x.shape[0]
    n = rnd(rms_norm(x, w[prefix + "input_layernorm.weight"], sz["eps"]))
    q = rnd(linear(n, w[prefix + "self_attn.q_proj.weight"])).reshape(T, sz["nq"], sz["hd"])
    k = rnd(linear(n, w[prefix + "self_attn.k_proj.weight"])).reshape(T, sz["nkv"], sz["hd"])
    v = rnd(linear(n, w[prefix + "self_attn.v_proj.weight"])).reshape(T, sz["nkv"], sz["hd"])
    inv = rope_inv_freq(sz["hd"], sz["theta"])
    q, k = rnd(rope(q, positions, inv, sz["pairing"])), rnd(rope(k, positions, inv, sz["pairing"]))
    o = rnd(attention(q, k, v, sz["nq"], sz["nkv"], window, rnd=rnd)).reshape(T, sz["nq"] * sz["hd"])
    return (x + linear(o, w[prefix + "self_attn.o_proj.weight"])).astype(F)


def ffn_block(x, w, prefix, sz, rnd=_same):
    """x + swiglu(norm(x)) (megakernel/compile_layers.rs:373-386)."""
    n = rnd(rms_norm(x, w[prefix + "post_attention_layernorm.weight"], sz["eps"]))
    return (x + swiglu(n, w[prefix + "mlp.gate_proj.weight"], w[prefix + "mlp.up_proj.weight"],
                       w[prefix + "mlp.down_proj.weight"], rnd)).astype(F)


def layer_window(sz, i):
    if sz["window"] is None:
        return None
    if sz["layer_types"] is None:
        return sz["window"]
    return sz["window"] if sz["layer_types"][i] == "sliding_attention" else None


def forward(cfg, w, tokens, positions=None, act_dtype=None):
    """Logits [T, V] of one whole sequence (layer loop megakernel/megakernel_compile.rs:115-236;
    final norm and lm_head :238-262).  `act_dtype="bfloat16"` rounds the activations a bfloat16
    engine keeps in bfloat16 (see `rounding`): what such an engine may differ by from the float
    result through rounding alone."""
    rnd = rounding(act_dtype)
    sz = sizes(cfg)
    T = len(tokens)
    positions = np.arange(T) if positions is None else np.asarray(positions)
    x = embedding(w["model.embed_tokens.weight"], tokens)
    for i in range(sz["L"]):
        p = f"model.layers.{i}."
        x = attention_block(x, positions, w, p, sz, layer_window(sz, i), rnd)
        x = ffn_block(x, w, p, sz, rnd)
    n = rnd(rms_norm(x, w["model.norm.weight"], sz["eps"]))
    head = w["model.embed_tokens.weight"] if sz["tied"] else w["lm_head.weight"]
    return linear(n, head)


# ------------------------------------------------------------------------- sampling ----
def argmax_lowest(v):
    """Index of the maximum; the lowest index wins ties (the engine's stated rule; the
    reference's host argmax keeps the last, generate.rs:493-500)."""
    return int(np.argmax(np.asarray(v)))


def filter_logits(l, top_k=0, top_p=1.0, min_p=0.0):
    """Top-k, then min-p, then top-p (sampling.rs:89-151): the logits with what is cut set
    to -inf.  Sorting is stable by (value descending, index ascending)."""
    l = np.array(l, dtype=F)
    n = l.shape[0]
    order = sorted(range(n), key=lambda i: (-l[i], i))
    if 0 < top_k < n:
        for i in order[top_k:]:
            l[i] = -np.inf
    if min_p > 0.0:
        mx = l.max()
        for i in range(n):
            if l[i] > -np.inf and np.exp(F(l[i] - mx), dtype=F) < F(min_p):
                l[i] = -np.inf
    if top_p < 1.0:
        idx = [i for i in order if l[i] > -np.inf]
        mx = l[idx[0]]
        pr = np.array([np.exp(F(l[i] - mx), dtype=F) for i in idx], dtype=F)
        pr = pr / pr.sum(dtype=F)
        cum, cut = F(0), len(idx)
        for r, p in enumerate(pr):
            cum = F(cum + p)
            if cum >= F(top_p):
                cut = r + 1
                break
        for i in idx[cut:]:
            l[i] = -np.inf
    return l


def sample(logits, u, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0, repetition_penalty=1.0,
           history=(), logit_bias=None):
    """The reference's sampler in its order (sampling.rs:49-171), with the uniform draw
    `u` given.  Sorting is stable by (value descending, index ascending)."""
    l = np.array(logits, dtype=F)
    n = l.shape[0]
    if logit_bias:
        for tok, d in logit_bias:
            if 0 <= tok < n:
                l[tok] = F(l[tok] + F(d))
    if repetition_penalty != 1.0:
        for tok in history:
            if 0 <= tok < n:
                l[tok] = F(l[tok] / F(repetition_penalty)) if l[tok] > 0 else F(l[tok] * F(repetition_penalty))
    if temperature == 0.0:
        return argmax_lowest(l)
    l = filter_logits((l / F(temperature)).astype(F), top_k, top_p, min_p)
    mx = l.max()
    pr = np.exp((l - mx).astype(F), dtype=F)
    pr = pr / pr.sum(dtype=F)
    cum = F(0)
    for i in range(n):
        cum = F(cum + pr[i])
        if F(u) <= cum:
            return i
    return argmax_lowest(pr)


def greedy_generate(cfg, w, prompt, max_new_tokens, stop_ids=()):
    """The reference's loop (generate.rs:314-439): argmax of the prompt's last logits,
    then one token at a time; a stop token ends the sequence and is not emitted."""
    toks = list(prompt)
    out = []
    for _ in range(max_new_tokens):
        nxt = argmax_lowest(forward(cfg, w, toks)[-1])
        if nxt in stop_ids:
            break
        out.append(nxt)
        toks.append(nxt)
    return out


def uniform(seed, sequence, draw):
    """The uniform number of draw `draw` of request `sequence` under `seed` (ours; the reference
    seeds a StdRng, sampling.rs:188-191, whose stream exists in Rust only): with
    mix'(x) = mix64(x + G) (splitmix64's step), key = mix'(mix'(seed) ^ (sequence * 0xD6E8FEB86659FD93)),
    u = (mix'(key ^ (draw * 0xCA5A826395121157)) >> 40) * 2^-24: 24 bits in [0, 1)."""
    def step(x):
        return _mix64((x + _GOLDEN) & _M64)
    key = step(step(seed & _M64) ^ ((sequence * 0xD6E8FEB86659FD93) & _M64))
    return (step(key ^ ((draw * 0xCA5A826395121157) & _M64)) >> 40) / float(1 << 24)


def sampled_generate(cfg, w, prompt, max_new_tokens, seed, sequence=0, stop_ids=(), **options):
    """The reference's sampled loop (sampling.rs:181-220): every new token is sampled from the
    logits of the last position with the history = prompt + everything generated so far, one
    uniform number a token; as in `greedy_generate` the first token comes from the prompt's last
    logits and a stop token ends the sequence without being emitted."""
    toks = list(prompt)
    out = []
    for k in range(max_new_tokens):
        nxt = sample(forward(cfg, w, toks)[-1], uniform(seed, sequence, k), history=toks, **options)
        if nxt in stop_ids:
            break
        out.append(nxt)
        toks.append(nxt)
    return out
