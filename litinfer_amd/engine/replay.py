"""Trace replay: feed given token ids through a model step by step and write
the logits.  Nothing is sampled.  It drives the framework's own engine (model,
step function, cache, kernels), the one that generation uses.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps come on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, OUT/<step>.f32 holds the logits at the
wanted places, in the order of the entries and of `want`, as little-endian
float32 [wanted, vocab].  After every step the line `done <step>` is printed.
"""
from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path


def _log(msg: str) -> None:
    print(f"[trace_run] {msg}", file=sys.stderr, flush=True)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="the most tokens live requests hold at any time (each rounded up to the page size)")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--max-seqs", type=int, default=16, help="requests that may be live at a time")
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--page-order-seed", "--shuffle-pages", dest="page_order_seed", type=int, default=None,
                    help="shuffle the order in which free pages are handed out, so that block tables are not contiguous")
    ap.add_argument("--plugin", action="append", default=[],
                    help="a module to import first (one that registers further parts or architectures)")
    args = ap.parse_args(argv)
    for mod in args.plugin:
        __import__(mod)

    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    _log("importing torch ...")
    import numpy as np
    import torch                                   # noqa: F401
    from . import Engine, StepEntry
    from ..kernels import build
    missing = [m for m in build.MODULES if build.find_built(m) is None]
    if missing:
        _log(f"building the HIP kernels ({', '.join(missing)}) ...")
        build.build_all(verbose=True, force=False)
    _log(f"loading {args.model} as {args.dtype} ...")
    pages = -(-max(1, args.max_tokens) // args.page_size)
    engine = Engine.from_dir(args.model, dtype=args.dtype, device=args.device, page_size=args.page_size,
                             num_pages=pages, max_seqs=args.max_seqs, page_order_seed=args.page_order_seed)
    _log(f"ready: {engine.spec.architecture}, {pages} pages of {args.page_size} tokens in each of "
         f"{len(engine.cache.groups)} cache group(s)")
    while True:
        line = sys.stdin.readline()
        if not line:
            break
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = [StepEntry(e["id"], e["tokens"], e.get("want", [])) for e in rec.get("entries", [])]
        if entries:
            logits = engine.step(entries)
            if logits is not None:
                arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                tmp = out_dir / f".{step}.f32.tmp"
                arr.tofile(tmp)
                tmp.replace(out_dir / f"{step}.f32")
            elif args.device.startswith("cuda"):
                torch.cuda.synchronize()
        for rid in rec.get("end", []):
            engine.finish(rid)
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
