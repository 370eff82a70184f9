"""bin/trace_run as a user drives it: JSON steps on standard input, logits in
files, compared with the plain implementation for every schedule."""
import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import helpers
import schedules
from tiny_configs import TINY_A, TINY_B

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
TOL = {"float32": 2e-5, "bfloat16": 1.5e-2}


def replay(model_dir, dtype, requests, steps, out_dir, max_tokens):
    proc = subprocess.Popen([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dir),
                             "--dtype", dtype, "--out", str(out_dir), "--max-tokens", str(max_tokens)],
                            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    rows = {rid: [] for rid in requests}
    vocab = None
    for i, (entries, end) in enumerate(steps):
        rec = {"step": i, "end": end, "entries": [
            {"id": rid, "tokens": list(requests[rid][a:a + n]), "want": list(range(n))} for rid, a, n in entries]}
        proc.stdin.write(json.dumps(rec) + "\n")
        proc.stdin.flush()
        assert proc.stdout.readline().strip() == f"done {i}"
        flat = np.fromfile(Path(out_dir) / f"{i}.f32", dtype="<f4")
        total = sum(n for _, _, n in entries)
        vocab = flat.size // total
        flat = flat.reshape(total, vocab)
        o = 0
        for rid, a, n in entries:
            rows[rid].append(flat[o:o + n])
            o += n
    proc.stdin.close()
    assert proc.wait(timeout=60) == 0
    return {rid: np.concatenate(v) for rid, v in rows.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cfg,seed", [(TINY_A, 0), (TINY_B, 1)])
def test_trace_run_schedules(tmp_path, cfg, seed, dtype):
    stored = torch.float32 if dtype == "float32" else torch.bfloat16
    d = helpers.make_model(tmp_path, cfg, seed, stored)
    reqs = helpers.random_requests(cfg["vocab_size"], [40, 100, 5, 64, 33, 70], seed + 20)
    ref = helpers.plain_logits(d, reqs)
    for kind in ("whole", "tail", "chunks", "mixed"):
        steps = getattr(schedules, kind)(reqs)
        out = replay(d, dtype, reqs, steps, tmp_path / f"out_{kind}", schedules.max_live_tokens(reqs, steps))
        worst = max(schedules.rel_err(out[r], ref[r]) for r in reqs)
        print(f"[observed] trace_run {dtype} {kind}: {worst:.3e}")
        assert worst < TOL[dtype], f"{kind}: {worst}"


def test_trace_run_writes_nothing_when_nothing_is_wanted(tmp_path):
    d = helpers.make_model(tmp_path, TINY_A, 0, torch.float32)
    proc = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(d), "--dtype",
                           "float32", "--out", str(tmp_path / "o"), "--max-tokens", "64"],
                          input='{"step": 3, "entries": [{"id": "a", "tokens": [1, 2], "want": []}], "end": []}\n'
                                '{"step": 4, "entries": [{"id": "a", "tokens": [3], "want": [0]}], "end": ["a"]}\n',
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr
    assert proc.stdout.split("\n")[:2] == ["done 3", "done 4"]
    assert not (tmp_path / "o" / "3.f32").exists()
    assert np.fromfile(tmp_path / "o" / "4.f32", dtype="<f4").size == TINY_A["vocab_size"]
