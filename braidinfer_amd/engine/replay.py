"""Trace replay: feeds given token ids through the engine step by step and writes the
logits asked for.  It samples nothing and owns nothing of its own: the model, the step
function, the cache and the kernels are the engine's, the ones generation uses.

The reference's nearest tools print statistics or hashes only: `trace_dump` (prefill a
prompt, N greedy steps, per-probe statistics, crates/braidinfer-runtime/src/bin/trace_dump.rs:49-117)
and the per-step logit hash of `BRAIDINFER_LOGIT_TRACE` (generate.rs:380-396).

Input, one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step with wanted places, `<out>/<step>.f32` holds float32 little-endian logits
[wanted, vocab] in the order of the entries and of `want`.  After every step a line
`done <step>` is printed and flushed.  With `--probes` a step also leaves
`<out>/<step>.probes.json`, statistics of the activations at the reference's probe points
(crates/braidinfer-runtime/src/tracer.rs:94-160: embed, L{i}.post_mixer, L{i}.post_ffn,
final_norm, logits).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Dict, IO, Optional

import numpy as np

from ..errors import BraidError, StepError
from .engine import Engine, StepEntry


def probe_stats(t) -> dict:
    """What the reference's `trace_dump` prints of a probed tensor (bin/trace_dump.rs:49-117):
    its size, mean, root mean square, largest magnitude and first values."""
    f = t.detach().float()
    n = f.numel()
    if n == 0:
        return {"shape": list(t.shape), "mean": 0.0, "rms": 0.0, "absmax": 0.0, "head": []}
    return {"shape": list(t.shape), "mean": float(f.mean()), "rms": float(f.pow(2).mean().sqrt()),
            "absmax": float(f.abs().max()), "head": [float(v) for v in f.reshape(-1)[:8].tolist()]}


class Replayer:
    def __init__(self, engine: Engine, out_dir: str, probes: bool = False):
        self.engine = engine
        self.out_dir = out_dir
        os.makedirs(out_dir, exist_ok=True)
        self.slot_of: Dict[str, int] = {}
        self.probes = probes

    def run_step(self, obj: dict) -> None:
        step_no = obj["step"]
        entries = []
        fresh = []
        try:
            for e in obj.get("entries", []):
                rid = str(e["id"])
                if rid not in self.slot_of:
                    self.slot_of[rid] = self.engine.alloc_slot()
                    fresh.append(rid)
                entries.append(StepEntry(self.slot_of[rid], e["tokens"], e.get("want", [])))
            if entries:
                stats = {}
                logits = self.engine.step(entries, probe=(lambda name, t: stats.__setitem__(name, probe_stats(t)))
                                          if self.probes else None)
                if self.probes:
                    with open(os.path.join(self.out_dir, f"{step_no}.probes.json"), "w") as f:
                        json.dump(stats, f, indent=1)
                if logits.shape[0] > 0:
                    arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                    tmp = os.path.join(self.out_dir, f".{step_no}.f32.tmp")
                    arr.tofile(tmp)
                    os.replace(tmp, os.path.join(self.out_dir, f"{step_no}.f32"))
        except BraidError:
            for rid in fresh:                       # a step that failed leaves nothing behind
                self.engine.free_slot(self.slot_of.pop(rid))
            raise
        for rid in obj.get("end", []):
            rid = str(rid)
            if rid not in self.slot_of:
                raise StepError(f"step {step_no}: request {rid!r} ends but was never started")
            self.engine.free_slot(self.slot_of.pop(rid))

    def run(self, lines: IO[str], out: IO[str]) -> None:
        for line in lines:
            line = line.strip()
            if not line:
                continue
            obj = json.loads(line)
            self.run_step(obj)
            out.write(f"done {obj['step']}\n")
            out.flush()


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description="replay token traces through the engine and write logits")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32", "bf16", "fp32"],
                    help="bfloat16 (bf16): the kernels and precisions of serving; float32 (fp32): everything in true 32-bit")
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--probes", action="store_true",
                    help="also write <step>.probes.json: statistics of the residual rows after the embedding, after "
                         "every layer's mixer and feed-forward, of the final norm and the logits")
    args = ap.parse_args(argv)
    try:
        # a replay takes any request the cache holds: the longest sequence is the cache's size, whatever
        # number of positions the model's configuration names (rotary angles are defined for every position)
        room = max(args.max_tokens, 64)
        engine = Engine.from_folder(args.model, dtype=args.dtype, device=args.device, max_tokens=room, max_seq_len=room)
        Replayer(engine, args.out, probes=args.probes).run(sys.stdin, sys.stdout)
    except BraidError as e:
        print(f"trace_run: {type(e).__name__}: {e}", file=sys.stderr, flush=True)
        return 1
    return 0
