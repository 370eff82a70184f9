"""Command line.

    python -m litinfer_amd generate --model DIR --prompt-ids 1,2,3 --max_steps 32
    python -m litinfer_amd generate --random config.json --seed 0 --prompt-ids 1,2,3
    python -m litinfer_amd random   --config config.json --seed 0 --out DIR
    python -m litinfer_amd replay   --model DIR --dtype float32 --out DIR --max-tokens 256 < steps.jsonl
    python -m litinfer_amd bench    [the options of bench.py]

`--plugin MODULE` (before or after the sub-command, repeatable) imports a module
first: one that registers further parts or architectures, which every
sub-command then finds in the registry like the built-in one.

The options of `generate` carry the names and meanings of the reference's
driver script (test/test_infer.py:173-191): --model, --prompt, --max_steps,
--top_p, --top_k, --temperature, --test (forces top_p=1, top_k=1,
temperature=1, i.e. greedy).  The library's contract is token ids in, token ids
out; --prompt TEXT needs the checkpoint's tokenizer.json and the `tokenizers`
package, --prompt-ids works always.
"""
from __future__ import annotations

import argparse
import json
import sys


def _cmd_generate(a) -> int:
    from .models import load
    if a.test:
        a.top_p, a.top_k, a.temperature = 1.0, 1, 1.0
    if (a.model is None) == (a.random is None):
        print("generate: give either --model DIR or --random CONFIG.json", file=sys.stderr)
        return 2
    tmp = None
    if a.random is not None:                      # random weights of that configuration, written to a folder that goes again
        import tempfile
        import torch
        from .weights import write_random_model
        with open(a.random) as f:
            cfg = json.load(f)
        tmp = tempfile.TemporaryDirectory(prefix="litinfer_random_")
        stored = torch.float32 if a.dtype == "float32" else torch.bfloat16
        a.model = str(write_random_model(tmp.name, cfg, a.weights_seed, stored))
    try:
        return _generate(a, load)
    finally:
        if tmp is not None:
            tmp.cleanup()


def _generate(a, load) -> int:
    tokenizer = None
    if a.prompt_ids is not None:
        ids = [int(t) for t in a.prompt_ids.replace(",", " ").split()]
    elif a.prompt_file is not None:
        with open(a.prompt_file) as f:
            ids = [int(t) for t in json.load(f)]
    else:
        from pathlib import Path
        tok_path = Path(a.model) / "tokenizer.json"
        if not tok_path.exists():
            print("generate: --prompt needs tokenizer.json in the model folder; "
                  "use --prompt-ids instead", file=sys.stderr)
            return 2
        from tokenizers import Tokenizer
        tokenizer = Tokenizer.from_file(str(tok_path))
        ids = tokenizer.encode(a.prompt).ids
    model = load(a.model, device=a.device, dtype=a.dtype, page_size=a.page_size, num_pages=a.num_pages,
                 max_batch_tokens=a.max_batch_tokens, chunk_size=a.chunk_size, seed=a.seed)
    tokens, metrics = model.generate_profile(ids, max_new_tokens=a.max_steps, top_k=a.top_k,
                                             top_p=a.top_p, temperature=a.temperature)
    print(json.dumps({"tokens": tokens, **{k: round(v, 6) if isinstance(v, float) else v
                                           for k, v in metrics.items()}}))
    if tokenizer is not None:
        print(tokenizer.decode(tokens))
    return 0


def _cmd_random(a) -> int:
    import torch
    from .weights import write_random_model
    with open(a.config) as f:
        cfg = json.load(f)
    dt = {"bfloat16": torch.bfloat16, "float32": torch.float32}[a.dtype]
    out = write_random_model(a.out, cfg, a.seed, dt)
    print(f"wrote {out}/config.json and {out}/model.safetensors")
    return 0


def load_plugins(argv):
    """Import every module named by `--plugin MODULE` (or `--plugin=MODULE`) and
    return the arguments without these options."""
    import importlib
    rest, i = [], 0
    while i < len(argv):
        arg = argv[i]
        if arg == "--plugin":
            if i + 1 >= len(argv):
                raise SystemExit("--plugin needs a module name")
            importlib.import_module(argv[i + 1])
            i += 2
        elif arg.startswith("--plugin="):
            importlib.import_module(arg.split("=", 1)[1])
            i += 1
        else:
            rest.append(arg)
            i += 1
    return rest


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m litinfer_amd")
    sub = ap.add_subparsers(dest="cmd", required=True)
    g = sub.add_parser("generate", help="generate tokens from a prompt")
    g.add_argument("--model", default=None, type=str)
    g.add_argument("--random", default=None, type=str, metavar="CONFIG.json",
                   help="instead of --model: random weights for this configuration")
    g.add_argument("--weights-seed", default=0, type=int, help="seed of the random weights (--random)")
    g.add_argument("--device", default="cuda:0", type=str)
    g.add_argument("--prompt", default="Who are you?", type=str)
    g.add_argument("--prompt-ids", default=None, type=str, help="token ids, comma or space separated")
    g.add_argument("--prompt-file", default=None, type=str, help="JSON list of token ids")
    g.add_argument("--max_steps", "--max-new-tokens", dest="max_steps", default=128, type=int)
    g.add_argument("--top_p", "--top-p", dest="top_p", default=0.8, type=float)
    g.add_argument("--top_k", "--top-k", dest="top_k", default=50, type=int)
    g.add_argument("--temperature", default=1.0, type=float)
    g.add_argument("--test", action="store_true", help="greedy: top_p=1, top_k=1, temperature=1")
    g.add_argument("--seed", "--sample-seed", dest="seed", default=0, type=int, help="seed of the sampler")
    g.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    g.add_argument("--page-size", default=16, type=int)
    g.add_argument("--num-pages", default=None, type=int)
    g.add_argument("--max-batch-tokens", default=2048, type=int)
    g.add_argument("--chunk-size", default=512, type=int)
    g.set_defaults(fn=_cmd_generate)
    r = sub.add_parser("random", help="write a model folder with random weights")
    r.add_argument("--config", required=True)
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--out", required=True)
    r.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    r.set_defaults(fn=_cmd_random)
    p = sub.add_parser("replay", help="trace replay (same as bin/trace_run)", add_help=False)
    p.set_defaults(fn=None)
    b = sub.add_parser("bench", help="throughput measurements (same as bench.py)", add_help=False)
    b.set_defaults(fn=None)
    argv = list(sys.argv[1:] if argv is None else argv)
    argv = load_plugins(argv)
    if argv and argv[0] == "replay":
        from .engine.replay import main as replay_main
        return replay_main(argv[1:])
    if argv and argv[0] == "bench":
        from .benchmark import main as bench_main
        return bench_main(argv[1:])
    a = ap.parse_args(argv)
    return a.fn(a)


if __name__ == "__main__":
    sys.exit(main())
