"""The `generate` command line, in the manner of the reference's binary
(crates/braidinfer-runtime/src/bin/generate.rs:13-58, ENV_CONFIG.md):

    MODEL=/path/to/folder MAX_TOKENS=32 generate "prompt text"
    generate /path/to/folder "prompt text"

* `MODEL` (environment) or the first argument when it is an existing folder: the model
  folder (config.json, model.safetensors, optionally tokenizer.json).
* the remaining arguments, joined with spaces: the prompt (default "Hello, world!").
* `MAX_TOKENS`: new-token budget, default 64.  `MAX_SEQ_LEN`: cap on the context.
* `RAW`: kept for compatibility; the prompt is always continued as it is (the chat
  template of the reference's default mode is outside this library).
Output: the generated text on standard output (token ids when the folder has no
tokenizer), statistics on standard error, including the reference's `PPTG` line.

Flags beyond the reference: --prompt-ids, --batch-file, --temperature, --top-k, --top-p,
--min-p, --repetition-penalty, --seed, --dtype, --random-weights SEED --preset NAME
(--save-folder DIR, --shard-bytes N), --list-weights.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile
import time
from typing import List, Optional


def _load_tokenizer(folder: str):
    path = os.path.join(folder, "tokenizer.json")
    if not os.path.isfile(path):
        return None
    try:
        from tokenizers import Tokenizer
    except ImportError:
        return None
    return Tokenizer.from_file(path)


def _add_bos(folder: str) -> Optional[bool]:
    """`add_bos_token` of tokenizer_config.json; None when unspecified (reference:
    generate.rs:479-489 prepends the BOS unless this is false)."""
    try:
        with open(os.path.join(folder, "tokenizer_config.json")) as f:
            v = json.load(f).get("add_bos_token")
        return v if isinstance(v, bool) else None
    except (OSError, json.JSONDecodeError):
        return None


def main(argv: Optional[List[str]] = None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    ap = argparse.ArgumentParser(prog="generate", add_help=True,
                                 description="generate tokens with a model folder on one MI355X")
    ap.add_argument("--prompt-ids", action="append", default=[],
                    help="a prompt as comma-separated token ids; may be given several times (a batch)")
    ap.add_argument("--batch-file", help="a file with one prompt per line (comma-separated ids, or text with a tokenizer)")
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--min-p", type=float, default=0.0)
    ap.add_argument("--repetition-penalty", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=None)
    ap.add_argument("--dtype", choices=["bfloat16", "float32", "bf16", "fp32"], default="bfloat16",
                    help="bfloat16 (bf16) or float32 (fp32)")
    ap.add_argument("--random-weights", type=int, metavar="SEED", default=None,
                    help="make a model folder of random weights for --preset instead of reading MODEL")
    ap.add_argument("--preset", default="tiny-a")
    ap.add_argument("--save-folder", metavar="DIR", default=None,
                    help="with --random-weights: write the model folder here and keep it (default: a temporary folder)")
    ap.add_argument("--shard-bytes", type=int, default=None,
                    help="with --random-weights: cut the folder into files of about this size with an index")
    ap.add_argument("--list-weights", action="store_true", help="print the tensor names and shapes the model needs")
    ap.add_argument("--max-seq-len", type=int, default=None)
    ap.add_argument("rest", nargs="*")
    args = ap.parse_args(argv)

    import braidinfer_amd as B
    from braidinfer_amd.engine import DecoderModel

    rest = list(args.rest)
    model_dir = os.environ.get("MODEL")
    if model_dir is None and rest and os.path.isdir(rest[0]):
        model_dir = rest.pop(0)
    max_tokens = int(os.environ.get("MAX_TOKENS", "64"))
    max_seq_len = args.max_seq_len or (int(os.environ["MAX_SEQ_LEN"]) if os.environ.get("MAX_SEQ_LEN") else None)
    tmp = None
    try:
        if args.random_weights is not None:
            import torch
            cfg = B.preset(args.preset)
            if args.save_folder:
                where = args.save_folder
            else:
                where = tmp = tempfile.mkdtemp(prefix="braidinfer_random_")
            t0 = time.perf_counter()
            # the values are the same bits wherever they are made; the GPU makes them faster
            model_dir = B.Engine.write_random_folder(where, cfg, seed=args.random_weights, shard_bytes=args.shard_bytes,
                                                     device="cuda:0" if torch.cuda.is_available() else "cpu")
            print(f"random weights of {args.preset} (seed {args.random_weights}) written to {model_dir} in "
                  f"{time.perf_counter() - t0:.1f} s", file=sys.stderr)
        if model_dir is None:
            print("generate: no model: set MODEL, pass a folder, or use --random-weights SEED --preset NAME",
                  file=sys.stderr)
            return 2
        cfg = B.config_from_folder(model_dir)
        if args.list_weights:
            for s in DecoderModel(B.spec_of(cfg)).weight_specs():
                print(f"{s.name}\t{list(s.shape)}\t{s.kind}")
            return 0
        tok = _load_tokenizer(model_dir)
        prompts: List[List[int]] = []
        for p in args.prompt_ids:
            prompts.append([int(x) for x in p.replace(" ", "").split(",") if x])
        lines: List[str] = []
        if args.batch_file:
            with open(args.batch_file) as f:
                lines = [l.rstrip("\n") for l in f if l.strip()]
        if not prompts and not lines:
            lines = [" ".join(rest) if rest else "Hello, world!"]
        spec = B.spec_of(cfg)
        for line in lines:
            is_ids = all(c.isdigit() or c in ", " for c in line)
            if is_ids:
                prompts.append([int(x) for x in line.replace(",", " ").split()])
            elif tok is None:
                print("generate: the folder has no tokenizer.json (or the tokenizers package is missing); "
                      "give the prompt as --prompt-ids", file=sys.stderr)
                return 2
            else:
                ids = tok.encode(line, add_special_tokens=False).ids
                bos = spec.bos_token_id
                if _add_bos(model_dir) is not False and bos is not None and (not ids or ids[0] != bos):
                    ids = [bos] + ids
                prompts.append(ids)
        longest = max(len(p) for p in prompts) + max_tokens
        cap_seq = min(max_seq_len, 1 << 20) if max_seq_len else max(longest, 64)
        room = sum(-(-min(len(p) + max_tokens, cap_seq) // 64) * 64 for p in prompts)
        t0 = time.perf_counter()
        engine = B.Engine.from_folder(model_dir, dtype=args.dtype, max_tokens=max(room, 64), max_seq_len=cap_seq)
        print(f"LOAD PROFILE: Engine.from_folder = {(time.perf_counter() - t0) * 1e3:.0f} ms", file=sys.stderr)
        if engine.load_profile is not None:
            print(engine.load_profile.line(), file=sys.stderr)
        import resource
        print(f"host memory at its peak: {resource.getrusage(resource.RUSAGE_SELF).ru_maxrss / 1e6:.2f} GB",
              file=sys.stderr)
        print(f"max_seq_len: {engine.cache.max_seq_len}", file=sys.stderr)
        print(f"stop tokens: {list(engine.stop_token_ids)}", file=sys.stderr)
        t0 = time.perf_counter()
        outs, stats = engine.generate(prompts, max_new_tokens=max_tokens, temperature=args.temperature,
                                      seed=args.seed, top_k=args.top_k, top_p=args.top_p, min_p=args.min_p,
                                      repetition_penalty=args.repetition_penalty, return_stats=True)
        dt = time.perf_counter() - t0
        for o in outs:
            print(tok.decode(o) if tok is not None else " ".join(str(t) for t in o))
        sys.stdout.flush()
        n = sum(len(o) for o in outs)
        print(stats.pptg_line(), file=sys.stderr)
        print(f"{n} tokens in {dt:.2f}s = {n / dt if dt > 0 else 0.0:.1f} tok/s", file=sys.stderr)
        return 0
    except B.BraidError as e:
        print(f"generate: {type(e).__name__}: {e}", file=sys.stderr)
        return 1
    finally:
        if tmp:
            import shutil
            shutil.rmtree(tmp, ignore_errors=True)
