#!/usr/bin/env python3
"""Decode and prefill throughput of the Mistral-7B-v0.3 shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B]

A step is one decode step of the whole batch: the engine's step function over one token
per sequence, greedy sampling on the GPU, and the token ids read back (what the
generation loop does per step).  Prompts have lengths uniform in [128, 2048] and random
token ids; weights are random N(0, 0.02) bf16.  One JSON line goes to standard output.
"""
import argparse
import json
import sys
import time

import numpy as np

PEAK_HBM = 8.0e12          # MI355X HBM3E, bytes/s
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (named in config)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--preset", default="mistral-7b-v0.3")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--prompt-min", type=int, default=128)
    ap.add_argument("--prompt-max", type=int, default=2048)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the prefill of --prefill-tokens (for profiles); prints its own line")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    import braidinfer_amd as B
    from braidinfer_amd import StepEntry
    from braidinfer_amd.sampling import Sampler

    full = B.preset(args.preset)
    layers = args.layers or full.num_hidden_layers
    cfg = B.preset(args.preset, num_hidden_layers=layers)
    batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})
    room = max(max(batches) * (-(-(args.prompt_max + args.steps + args.warmup + 1) // 64) * 64),
               -(-args.prefill_tokens // 64) * 64)
    t0 = time.time()
    eng = B.Engine.random(cfg, seed=0, dtype=args.dtype, max_tokens=room, max_seq_len=args.context)
    print(f"[bench] engine with {layers} layers ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    sampler = Sampler(eng.device, cfg.vocab_size)
    esz = 2 if args.dtype == "bfloat16" else 4
    H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    nq, nkv, hd = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    layer_params = (nq + 2 * nkv) * hd * H + H * nq * hd + 3 * H * I
    weight_bytes = (layers * layer_params + V * H) * esz + (2 * layers + 1) * H * 4
    kv_bytes_per_token = 2 * nkv * hd * esz * layers

    def prefill(T, reps=4):
        rng = np.random.default_rng(5)
        prompt = [int(t) for t in rng.integers(0, V, T)]
        times = []
        for rep in range(reps):
            s = eng.alloc_slot()
            torch.cuda.synchronize()
            t = time.perf_counter()
            eng.step([StepEntry(s, prompt, [T - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            eng.free_slot(s)
        pt = min(times[1:])
        flops = 2.0 * layers * layer_params * T + 2.0 * V * H + 2.0 * T * T * hd * nq * layers
        peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
        return {"value": round(T / pt, 1), "tokens": T, "ms": round(pt * 1e3, 3), "frac": round(flops / pt / peak, 4)}

    if args.prefill_only:
        print(json.dumps({"metric": "prefill tok/s", "layers": layers, "prefill": prefill(args.prefill_tokens)}), flush=True)
        return 0

    def decode(batch, steps, warmup, seed):
        rng = np.random.default_rng(seed)
        lens = [int(n) for n in rng.integers(args.prompt_min, args.prompt_max + 1, batch)]
        prompts = [[int(t) for t in rng.integers(0, V, n)] for n in lens]
        slots = [eng.alloc_slot() for _ in range(batch)]
        # prompts in chunks of at most 16k tokens a step, to bound the activations
        logits, i = None, 0
        last = [None] * batch
        while i < batch:
            j, tot = i, 0
            while j < batch and (j == i or tot + lens[j] <= 16384):
                tot += lens[j]; j += 1
            out = eng.step([StepEntry(slots[b], prompts[b], [lens[b] - 1]) for b in range(i, j)])
            for r, b in enumerate(range(i, j)):
                last[b] = out[r:r + 1].clone()
            i = j
        toks = sampler.argmax(torch.cat(last)).tolist()

        def one():
            nonlocal toks
            lg = eng.step([StepEntry(slots[b], [toks[b]], [0]) for b in range(batch)])
            toks = sampler.argmax(lg).tolist()
        for _ in range(warmup):
            one()
        torch.cuda.synchronize()
        # keys a step has to read: the whole context, or the window where the model has one
        W = cfg.sliding_window
        seen = lambda n: n if W is None else min(n, W)
        ctx0 = sum(seen(eng.length(s)) for s in slots)
        ctx1 = sum(seen(eng.length(s) + steps) for s in slots)
        t = time.perf_counter()
        for _ in range(steps):
            one()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t) / steps
        mean_ctx_total = (ctx0 + ctx1) / 2.0
        for s in slots:
            eng.free_slot(s)
        return dt, weight_bytes + mean_ctx_total * kv_bytes_per_token, float(np.mean(lens))

    dt, nbytes, mean_len = decode(args.batch, args.steps, args.warmup, seed=1)
    value = args.batch / dt
    line = {
        "metric": f"decode tok/s (batch {args.batch}, {args.preset} shape, {args.dtype}, prompts uniform in "
                  f"[{args.prompt_min}, {args.prompt_max}])",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {"model": args.preset, "layers": layers, "layers_of_shape": full.num_hidden_layers,
                   "hidden": H, "heads": nq, "kv_heads": nkv, "head_dim": hd, "intermediate": I, "vocab": V,
                   "rope_theta": cfg.rope_theta, "rms_norm_eps": cfg.rms_norm_eps,
                   "sliding_window": cfg.sliding_window, "global_batch": args.batch, "seq_len": args.context,
                   "prompt_lens": f"uniform[{args.prompt_min},{args.prompt_max}]", "mean_prompt_len": round(mean_len, 1),
                   "weights": "random N(0,0.02) bf16", "parallelism": "single GPU"},
        "roofline": {"bound": "hbm", "achieved": round(nbytes / dt / 1e9, 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                     "frac": round(nbytes / dt / PEAK_HBM, 4)},
    }
    if not args.no_points:
        points = {}
        for b in (1, 64):
            if b == args.batch:
                points[f"decode_b{b}"] = round(value, 2)
                continue
            k = max(8, args.steps // 2)
            d, _, _ = decode(b, k, max(2, args.warmup // 2), seed=10 + b)
            points[f"decode_b{b}"] = round(b / d, 2)
            print(f"[bench] batch {b}: {d * 1e3:.3f} ms/step", file=sys.stderr, flush=True)
        line["points"] = points
        line["prefill"] = prefill(args.prefill_tokens)
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
