"""Command line of the package.

  python -m vllm_i64_amd.cli generate --model DIR --prompt 5,17,3 [--prompt ...] [--max-new-tokens N] [--temperature T] [--top-k K] [--top-p P]
  python -m vllm_i64_amd.cli trace --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N      (bin/trace_run)

trace replays a recorded schedule: it reads one JSON object a line from standard input,
  {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
runs the entries of a step as one batch through the engine (a request is admitted at its first entry and gives its slot and pages
back when it is listed in "end"), writes the logits at the wanted places to <out>/<step>.f32 (little-endian fp32 [wanted, vocab])
when any are wanted, and prints 'done <step>'.  It samples nothing."""
from __future__ import annotations

import argparse
import json
import os
import sys


def _ensure_built(dense_only: bool = True) -> None:
    """Compile the HIP library this process needs if it is not there (a fresh checkout)."""
    from . import _lib, build
    if not os.path.exists(_lib.DENSE_LIB_PATH):
        build.build_dense(verbose=False)
    if not dense_only and not os.path.exists(_lib.LIB_PATH):
        build.build(verbose=False)


def _load(args, max_seqs: int, max_tokens: int):
    import torch
    from .registry import architecture_of, load_model
    with open(os.path.join(args.model, "config.json"), "r", encoding="utf-8") as f:
        config = json.load(f)
    _ensure_built(dense_only=architecture_of(config).lower() in ("morilorn", "dogalorn", "zabutar", "fukatar"))
    if not torch.cuda.is_available():
        raise SystemExit("no GPU: this package has no CPU path")
    return load_model(args.model, dtype=args.dtype, device="cuda:0", max_seqs=max_seqs, max_tokens=max_tokens, config=config)


def trace_main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description="replay a recorded schedule of steps and write the logits asked for")
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True, help="tokens the live requests hold at most (rounded up per request to whole pages)")
    ap.add_argument("--max-seqs", type=int, default=4, help="requests that are live at the same time at most")
    args = ap.parse_args(argv)
    import numpy as np
    from .engine import Engine
    model = _load(args, args.max_seqs, args.max_tokens)
    eng = Engine(model)
    os.makedirs(args.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(str(e["id"]), e["tokens"], e.get("want", [])) for e in st["entries"]]
        logits = eng.step(entries, end=[str(r) for r in st.get("end", [])])
        if logits.shape[0]:
            a = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
            tmp = os.path.join(args.out, f".{st['step']}.part")
            a.tofile(tmp)
            os.replace(tmp, os.path.join(args.out, f"{st['step']}.f32"))
        print(f"done {st['step']}", flush=True)
    return 0


def generate_main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="generate", description="generate token ids from prompts of token ids")
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--prompt", action="append", required=True, help="token ids with commas between them; repeat for a batch")
    ap.add_argument("--max-new-tokens", type=int, default=16)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--max-seqs", type=int, default=4)
    ap.add_argument("--max-tokens", type=int, default=0, help="size of the cache pool in tokens (default: what the prompts need)")
    ap.add_argument("--max-batch-tokens", type=int, default=512)
    args = ap.parse_args(argv)
    from .engine import Engine, SamplingParams
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in args.prompt]
    need = sum((len(p) + args.max_new_tokens + 63) // 64 * 64 for p in sorted(prompts, key=len, reverse=True)[: args.max_seqs])
    model = _load(args, args.max_seqs, args.max_tokens or need)
    eng = Engine(model, max_batch_tokens=args.max_batch_tokens)
    params = SamplingParams(max_new_tokens=args.max_new_tokens, temperature=args.temperature, top_k=args.top_k, top_p=args.top_p, seed=args.seed)
    for out in eng.generate(prompts, params):
        print(",".join(str(t) for t in out), flush=True)
    return 0


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if not argv or argv[0] not in ("generate", "trace"):
        print(__doc__)
        return 2
    return (trace_main if argv[0] == "trace" else generate_main)(argv[1:])


if __name__ == "__main__":
    sys.exit(main())
