"""Trace replay: feed given token ids through a model step by step and write logits.

Nothing is sampled.  The program drives the framework's own model, step function, cache
manager and kernels -- the ones generation uses -- below the scheduler and the sampler.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps come on standard input, one JSON object a line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

All entries of a step form one batch.  For a step in which something is wanted the logits
at the wanted places are written to ``OUT/<step>.f32`` (little-endian float32,
``[wanted, vocab]``, in the order of the entries and of their ``want`` lists).  After
every step ``done <step>`` is printed and flushed.  Requests listed under ``end`` give
back their pages and slot after the step.  The page pool is made for ``--max-tokens``
tokens (each live request's count rounded up to whole pages), so pages are used again.
"""
from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path


def parse_args(argv=None):
    p = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    p.add_argument("--out", required=True, help="folder for the <step>.f32 files")
    p.add_argument("--max-tokens", type=int, required=True,
                   help="most tokens live requests hold at any time (each rounded up to whole pages)")
    p.add_argument("--page-size", type=int, default=16, help="tokens per cache page (default 16)")
    p.add_argument("--max-requests", type=int, default=8, help="most requests live at a time (default 8)")
    p.add_argument("--graphs", action="store_true", help="replay decode-only steps as captured HIP graphs")
    return p.parse_args(argv)


def run(args, lines, out=sys.stdout) -> int:
    from .batch import StepEntry
    from .config import EngineConfig
    from .loading import load_model, make_runner

    if args.max_tokens <= 0 or args.page_size <= 0:
        raise SystemExit("trace_run: --max-tokens and --page-size must be positive")
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    _, model = load_model(args.model, args.dtype)
    pages = -(-args.max_tokens // args.page_size) + 1          # + the sentinel page
    runner = make_runner(model, EngineConfig(page_size=args.page_size, num_pages=pages, max_slots=args.max_requests,
                                             dtype=args.dtype, use_graphs=args.graphs))
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = [StepEntry(e["id"], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])])
                   for e in rec.get("entries", [])]
        logits = runner.step(entries)
        if logits is not None:
            arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
            tmp = out_dir / f".{step}.f32.tmp"
            arr.tofile(tmp)
            tmp.replace(out_dir / f"{step}.f32")
        for req_id in rec.get("end", []):
            runner.release(req_id)
        print(f"done {step}", file=out, flush=True)
    return 0


def main(argv=None) -> int:
    args = parse_args(argv)
    return run(args, iter(sys.stdin.readline, ""))


if __name__ == "__main__":
    sys.exit(main())
