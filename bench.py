#!/usr/bin/env python3
"""Decode and prefill throughput of the Mistral shapes on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload headline|v0.1|24b] [--layers L] [--batch B]

A step is one decode step of the whole batch: the engine's step function over one token
per sequence, greedy sampling on the GPU, and the token ids read back (what the
generation loop does per step).  Prompts have random token ids and lengths uniform in the
workload's range; weights are random N(0, 0.02) bf16.  One JSON line goes to standard output.

Workloads (the benchmark description's shapes): `headline` Mistral-7B-v0.3, context 4,096,
batch 8, prompts in [128, 2048]; `v0.1` Mistral-7B-v0.1 with its window of 4,096, context
8,192, batch 8, prompts in [4096, 7168]; `24b` Mistral-Small-24B, context 32,768, batch 16,
prompts in [1024, 16384].  Beside the headline value the line carries: the decode step's
share of the published memory rate (`roofline`), further batch sizes and prompt lengths and the
headline batch with the reference's default sampling instead of greedy, and the decode rates of the two
other workloads, each in an engine of its own (`points`), what this GPU delivers to plain streaming kernels
and to the tile product of this library (`measured_peaks`), and where an eager decode step's kernel time goes
(`kernel_share`).  `warmup` counts every untimed decode step before the timed ones.
"""
import argparse
import json
import sys
import time

import numpy as np

PEAK_HBM = 8.0e12          # MI355X HBM3E, bytes/s
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

WORKLOADS = {
    "headline": dict(preset="mistral-7b-v0.3", context=4096, batch=8, prompt_min=128, prompt_max=2048),
    "v0.1": dict(preset="mistral-7b-v0.1", context=8192, batch=8, prompt_min=4096, prompt_max=7168),
    "24b": dict(preset="mistral-small-24b", context=32768, batch=16, prompt_min=1024, prompt_max=16384),
}


def measured_peaks(torch, K):
    """What plain kernels of this library get out of this GPU: a copy and a pure read of 2 GiB,
    and this library's own tile product (the kernel the prompts use) on 8,192 cubed in bf16: a
    figure of that kernel, not of the hardware."""
    out = {}
    n = 1 << 31
    src = torch.empty(n, dtype=torch.uint8, device="cuda")
    dst = torch.empty(n, dtype=torch.uint8, device="cuda")
    src.view(torch.int32).fill_(1)
    sums = torch.empty(64 * 1024, dtype=torch.float32, device="cuda")

    def timed(f, reps=5):
        f()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            f()
            b.record()
            torch.cuda.synchronize()
            best = min(best, a.elapsed_time(b) * 1e-3)
        return best
    out["hbm_copy_GBs"] = round(2 * n / timed(lambda: K.stream_copy(src, dst)) / 1e9, 1)
    out["hbm_read_GBs"] = round(n / timed(lambda: K.stream_read(src, sums)) / 1e9, 1)
    del src, dst
    M = 8192
    a = torch.randn(M, M, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    w = torch.randn(M, M, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    c = torch.empty(M, M, device="cuda", dtype=torch.bfloat16)
    out["own_tile_product_8192_TFLOPs"] = round(2.0 * M ** 3 / timed(lambda: K.gemm(a, w, c)) / 1e12, 1)
    return out


def kernel_share(torch, eng, entries_of, classes):
    """Where the kernel time of one decode step goes: the step is run eagerly (no graph) with
    every launcher of `braidinfer_amd.kernels` bracketed by events; shares by class of kernel."""
    from braidinfer_amd import kernels as K
    records = []
    saved = {}

    def wrap(name, f):
        def g(*a, **k):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            r = f(*a, **k)
            e.record()
            records.append((classes(name, a, k), s, e))
            return r
        return g
    names = ["embedding", "rmsnorm", "rope_table", "rope_kv_write", "silu_mul", "residual_add", "gather_rows", "convert",
             "gemm", "gemm_swiglu", "gemm_norm_prepare", "gemm_norm_scaled", "attention_simple",
             "attention_prefill_bf16", "attention_decode_bf16", "argmax"]
    was = eng.use_graphs
    eng.use_graphs = False
    try:
        for n in names:
            saved[n] = getattr(K, n)
            setattr(K, n, wrap(n, saved[n]))
        eng.step(entries_of())           # once to size the workspace
        records.clear()
        eng.step(entries_of())
        torch.cuda.synchronize()
    finally:
        for n, f in saved.items():
            setattr(K, n, f)
        eng.use_graphs = was
    total, by = 0.0, {}
    for cls, s, e in records:
        ms = s.elapsed_time(e)
        by[cls] = by.get(cls, 0.0) + ms
        total += ms
    share = {k: round(v / total, 4) for k, v in sorted(by.items(), key=lambda kv: -kv[1])}
    share["kernels_ms"] = round(total, 3)
    share["launches"] = len(records)
    return share


class Shape:
    """One preset in an engine of its own, with the decode and prefill measurements over it."""

    def __init__(self, torch, B, preset, layers, dtype, context, room, prompt_min, prompt_max):
        self.torch, self.B = torch, B
        from braidinfer_amd.sampling import Sampler
        self.full = B.preset(preset)
        self.layers = layers or self.full.num_hidden_layers
        self.cfg = cfg = B.preset(preset, num_hidden_layers=self.layers)
        self.preset, self.dtype, self.context = preset, dtype, context
        self.prompt_min, self.prompt_max = prompt_min, prompt_max
        t0 = time.time()
        self.eng = B.Engine.random(cfg, seed=0, dtype=dtype, max_tokens=room, max_seq_len=context)
        print(f"[bench] {preset}: engine with {self.layers} layers ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
        self.sampler = Sampler(self.eng.device, cfg.vocab_size)
        esz = 2 if dtype == "bfloat16" else 4
        self.H, self.I, self.V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
        self.nq, self.nkv, self.hd = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        H, I, V, nq, nkv, hd = self.H, self.I, self.V, self.nq, self.nkv, self.hd
        self.layer_params = (nq + 2 * nkv) * hd * H + H * nq * hd + 3 * H * I
        self.weight_bytes = (self.layers * self.layer_params + V * H) * esz + (2 * self.layers + 1) * H * 4
        self.kv_bytes_per_token = 2 * nkv * hd * esz * self.layers
        self.W = cfg.sliding_window

    def close(self):
        self.eng = self.sampler = None
        self.torch.cuda.empty_cache()

    def prefill(self, T, reps=4):
        torch, engine = self.torch, self.eng
        from braidinfer_amd import StepEntry
        rng = np.random.default_rng(5)
        prompt = [int(t) for t in rng.integers(0, self.V, T)]
        times = []
        for rep in range(reps):
            s = engine.alloc_slot()
            torch.cuda.synchronize()
            t = time.perf_counter()
            engine.step([StepEntry(s, prompt, [T - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            engine.free_slot(s)
        pt = min(times[1:])
        # attention counted causally (2 T^2 hd per head), and within the window where the model has one
        W, hd, nq, layers = self.W, self.hd, self.nq, self.layers
        if W:
            pairs = sum(min(t + 1, W) for t in range(T))
            attn = 4.0 * pairs * hd * nq * layers
        else:
            attn = 2.0 * T * T * hd * nq * layers
        flops = 2.0 * layers * self.layer_params * T + 2.0 * self.V * self.H + attn
        peak = PEAK_FLOPS["bf16" if self.dtype == "bfloat16" else "fp32"]
        return {"value": round(T / pt, 1), "tokens": T, "ms": round(pt * 1e3, 3), "frac": round(flops / pt / peak, 4)}

    def decode(self, batch, steps, warmup, seed, share=False, sampling=None):
        """Seconds a step, the bytes a step must read, the mean prompt length, the kernel shares.
        `sampling`: a SamplingParams for every request (the generation loop's sampled chain);
        None is greedy."""
        torch, eng, sampler = self.torch, self.eng, self.sampler
        from braidinfer_amd import StepEntry
        V, W = self.V, self.W
        rng = np.random.default_rng(seed)
        lens = [int(n) for n in rng.integers(self.prompt_min, self.prompt_max + 1, batch)]
        lens.sort(reverse=True)       # the generation loop's order within a batch: longest prompts first
        prompts = [[int(t) for t in rng.integers(0, V, n)] for n in lens]
        slots = [eng.alloc_slot() for _ in range(batch)]
        # prompts in chunks of at most 16k tokens a step, to bound the activations
        i = 0
        last = [None] * batch
        while i < batch:
            j, tot = i, 0
            while j < batch and (j == i or tot + lens[j] <= 16384):
                tot += lens[j]; j += 1
            out = eng.step([StepEntry(slots[b], prompts[b], [lens[b] - 1]) for b in range(i, j)])
            for r, b in enumerate(range(i, j)):
                last[b] = out[r:r + 1].clone()
            i = j
        state = None
        if sampling is not None:      # as the generation loop makes it: the state draws its own uniform numbers
            state = sampler.state([sampling] * batch, prompts, random=[(seed, b, 0) for b in range(batch)])
        toks = sampler.argmax(torch.cat(last)).tolist() if state is None else state.sample(torch.cat(last))

        # the generation loop's way: a chain, one step launched ahead of the read
        chain = eng.chain(slots, toks, state)

        def one():
            nonlocal toks
            if chain is None:
                lg = eng.step([StepEntry(slots[b], [toks[b]], [0]) for b in range(batch)])
                toks = sampler.argmax(lg).tolist() if state is None else state.sample(lg)
            else:
                chain.launch()
                toks = chain.read()
        if chain is not None:
            chain.launch()
        for _ in range(warmup):
            one()
        torch.cuda.synchronize()
        # keys a step has to read: the whole context, or the window where the model has one
        seen = lambda n: n if W is None else min(n, W)
        ctx0 = sum(seen(eng.length(s)) for s in slots)
        ctx1 = sum(seen(eng.length(s) + steps) for s in slots)
        t = time.perf_counter()
        for _ in range(steps):
            one()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t) / steps
        mean_ctx_total = (ctx0 + ctx1) / 2.0
        if chain is not None:
            toks = chain.read()          # the step launched ahead
            chain.close()
        shares = None
        if share:
            H, I, nq, nkv, hd = self.H, self.I, self.nq, self.nkv, self.hd
            products = {((nq + 2 * nkv) * hd, H): "qkv_product", (H, nq * hd): "o_product", (2 * I, H): "gate_up_product",
                        (H, I): "down_product", (V, H): "head_product"}

            def classes(name, a, k):
                if name == "gemm_wide_partial":
                    return products.get((a[2], a[1].shape[1] * 128 if a[1].dim() == 4 else a[1].shape[1]), "other_product")
                if name in ("gemm", "gemm_swiglu", "gemm_norm_prepare"):
                    w, out, glu = a[1], a[2], name == "gemm_swiglu"
                elif name == "gemm_norm_scaled":
                    w, out, glu = a[4], a[5], bool(k.get("swiglu"))
                elif name.startswith("attention"):
                    return "attention"
                else:
                    return {"rmsnorm": "norm", "rope_table": "rope", "rope_kv_write": "rope", "argmax": "sampling"}.get(name, name)
                n_out = out.shape[1] * (2 if glu else 1)
                k_in = w.shape[1] * 128 if w.dim() == 4 else w.shape[1]
                return products.get((n_out, k_in), "other_product")
            shares = kernel_share(torch, eng, lambda: [StepEntry(slots[b], [toks[b]], [0]) for b in range(batch)], classes)
        for s in slots:
            eng.free_slot(s)
        return dt, self.weight_bytes + mean_ctx_total * self.kv_bytes_per_token, float(np.mean(lens)), shares


def room_for(batches, prompt_max, context, untimed_and_timed, prefill_tokens):
    per_seq = -(-(min(prompt_max, context) + untimed_and_timed + 3) // 64) * 64
    return max(max(batches) * per_seq, -(-prefill_tokens // 64) * 64)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    # untimed steps before the timed ones: the first steps after the prompts run while the GPU's clocks
    # still settle (measured: up to 3 % on the step when a heavy job ran just before)
    ap.add_argument("--warmup", type=int, default=48)
    ap.add_argument("--workload", default="headline", choices=sorted(WORKLOADS),
                    help="which of the benchmark description's shapes (preset, context, batch, prompt lengths)")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (named in config)")
    ap.add_argument("--batch", type=int, default=None)
    ap.add_argument("--preset", default=None)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--context", type=int, default=None)
    ap.add_argument("--prompt-min", type=int, default=None)
    ap.add_argument("--prompt-max", type=int, default=None)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--no-points", action="store_true",
                    help="skip the further batch sizes, prompt lengths and workloads, the measured peaks and the kernel shares")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the prefill of --prefill-tokens (for profiles); prints its own line")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    wl = WORKLOADS[args.workload]
    for k, v in wl.items():
        if getattr(args, k) is None:
            setattr(args, k, v)
    headline = args.workload == "headline"

    import torch
    import braidinfer_amd as B
    from braidinfer_amd import kernels as K
    from braidinfer_amd.sampling import SamplingParams

    points_on = not args.no_points
    batches = sorted({1, args.batch, 64, 128}) if (points_on and headline) else [args.batch]
    room = room_for(batches, args.prompt_max, args.context, args.steps + args.warmup, args.prefill_tokens)
    sh = Shape(torch, B, args.preset, args.layers, args.dtype, args.context, room, args.prompt_min, args.prompt_max)
    cfg, layers = sh.cfg, sh.layers

    if args.prefill_only:
        print(json.dumps({"metric": "prefill tok/s", "layers": layers, "prefill": sh.prefill(args.prefill_tokens)}), flush=True)
        return 0

    dt, nbytes, mean_len, shares = sh.decode(args.batch, args.steps, args.warmup, seed=1, share=points_on)
    value = args.batch / dt
    line = {
        "metric": f"decode tok/s (batch {args.batch}, {args.preset} shape, {args.dtype}, prompts uniform in "
                  f"[{args.prompt_min}, {args.prompt_max}])",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {"model": args.preset, "layers": layers, "layers_of_shape": sh.full.num_hidden_layers,
                   "hidden": sh.H, "heads": sh.nq, "kv_heads": sh.nkv, "head_dim": sh.hd, "intermediate": sh.I, "vocab": sh.V,
                   "rope_theta": cfg.rope_theta, "rms_norm_eps": cfg.rms_norm_eps,
                   "sliding_window": cfg.sliding_window, "global_batch": args.batch, "seq_len": args.context,
                   "prompt_lens": f"uniform[{args.prompt_min},{args.prompt_max}]", "mean_prompt_len": round(mean_len, 1),
                   "weights": "random N(0,0.02) bf16", "parallelism": "single GPU"},
        "roofline": {"bound": "hbm", "achieved": round(nbytes / dt / 1e9, 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                     "frac": round(nbytes / dt / PEAK_HBM, 4)},
    }
    if points_on:
        points = {}
        half_steps, half_warm = max(8, args.steps // 2), max(2, args.warmup // 2)
        if headline:
            for b in (1, 64, 128):
                if b == args.batch:
                    points[f"decode_b{b}"] = round(value, 2)
                    continue
                d, _, _, _ = sh.decode(b, half_steps, half_warm, seed=10 + b)
                points[f"decode_b{b}"] = round(b / d, 2)
                print(f"[bench] batch {b}: {d * 1e3:.3f} ms/step", file=sys.stderr, flush=True)
            # the reference's default sampling (temperature 1, top-k 50: sampling.rs:21-33) at the headline batch
            d, _, _, _ = sh.decode(args.batch, half_steps, half_warm, seed=3, sampling=SamplingParams(seed=3))
            points[f"decode_b{args.batch}_sampled"] = round(args.batch / d, 2)
        line["prefill"] = sh.prefill(min(args.prefill_tokens, args.context))
        if headline:
            for T in (128, 512):
                points[f"prefill_{T}"] = sh.prefill(T)["value"]
            # longer prompts than the headline's context: an engine of its own for them
            sh.close()
            long_sh = Shape(torch, B, args.preset, args.layers, args.dtype, 32768, 32768, args.prompt_min, args.prompt_max)
            for T in (8192, 32768):
                r = long_sh.prefill(T, reps=3)
                points[f"prefill_{T}"] = r["value"]
                points[f"prefill_{T}_frac"] = r["frac"]
                print(f"[bench] prefill of {T}: {r['ms']:.1f} ms", file=sys.stderr, flush=True)
            long_sh.close()
            del long_sh
            # the two other workloads, whole (every layer of their shapes), each in an engine of its own
            for key, name in (("v01_decode_b8", "v0.1"), ("s24b_decode_b16", "24b")):
                o = WORKLOADS[name]
                other = Shape(torch, B, o["preset"], None, args.dtype, o["context"],
                              room_for([o["batch"]], o["prompt_max"], o["context"], half_steps + half_warm, 64),
                              o["prompt_min"], o["prompt_max"])
                d, nb, _, _ = other.decode(o["batch"], half_steps, half_warm, seed=1)
                points[key] = round(o["batch"] / d, 2)
                points[key + "_frac"] = round(nb / d / PEAK_HBM, 4)
                print(f"[bench] {name}: batch {o['batch']}: {d * 1e3:.3f} ms/step", file=sys.stderr, flush=True)
                other.close()
                del other
        if points:
            line["points"] = points
        line["kernel_share"] = shares
        peaks = measured_peaks(torch, K)
        peaks["decode_frac_of_read"] = round(nbytes / dt / 1e9 / peaks["hbm_read_GBs"], 4)
        peaks["prefill_frac_of_own_tile_product"] = \
            round(line["prefill"]["frac"] * PEAK_FLOPS["bf16"] / 1e12 / peaks["own_tile_product_8192_TFLOPs"], 4) \
            if args.dtype == "bfloat16" else None
        line["measured_peaks"] = peaks
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
