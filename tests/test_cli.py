"""The command line as a user runs it, in a subprocess: `python -m litinfer_amd
random | generate | replay`.  The options of `generate` are those of the reference's
driver (test/test_infer.py:173-191: --model, --max_steps, --top_k, --top_p,
--temperature, --test), and, like it, the test compares the tokens with another
implementation's greedy tokens (:277-278), here the plain one."""
import json
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import helpers
import plain_impl as P
from tiny_configs import TINY_A, TINY_B

ROOT = Path(__file__).resolve().parent.parent


def cli(*args, stdin=None, check=True):
    env = dict(os.environ, PYTHONPATH=os.pathsep.join([str(ROOT), str(ROOT / "tests"),
                                                       os.environ.get("PYTHONPATH", "")]))
    p = subprocess.run([sys.executable, "-m", "litinfer_amd", *map(str, args)], input=stdin, env=env,
                       capture_output=True, text=True, timeout=300)
    if check:
        assert p.returncode == 0, f"exit code {p.returncode}\n{p.stdout}\n{p.stderr}"
    return p


def last_json(out: str):
    return json.loads([l for l in out.splitlines() if l.startswith("{")][-1])


def test_random_writes_a_model_folder_that_the_plain_implementation_reads(tmp_path):
    (tmp_path / "c.json").write_text(json.dumps(TINY_A))
    out = tmp_path / "m"
    cli("random", "--config", tmp_path / "c.json", "--seed", 5, "--out", out, "--dtype", "float32")
    assert (out / "config.json").exists() and (out / "model.safetensors").exists()
    same = helpers.make_model(tmp_path / "same", TINY_A, 5)
    assert (out / "model.safetensors").read_bytes() == (same / "model.safetensors").read_bytes()
    cfg, w = P.load_folder(out)
    assert P.forward(cfg, w, [1, 2, 3]).shape == (3, 256)


def test_generate_without_a_gpu_fails_loudly_and_bad_options_are_refused(tmp_path):
    d = helpers.make_model(tmp_path, TINY_A, 0)
    p = cli("generate", "--model", d, "--device", "cpu", "--prompt-ids", "1,2,3", "--max_steps", 4, check=False)
    assert p.returncode != 0 and ("no CPU path" in p.stderr or "not on the GPU" in p.stderr)
    p = cli("generate", "--prompt-ids", "1,2,3", check=False)                 # neither --model nor --random
    assert p.returncode == 2 and "--model DIR or --random" in p.stderr
    p = cli("--plugin", "no_such_module_anywhere", "generate", "--model", d, check=False)
    assert p.returncode != 0 and "no_such_module_anywhere" in p.stderr


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generate_gives_the_plain_implementations_greedy_tokens(tmp_path, dtype):
    d = helpers.make_model(tmp_path, TINY_B, 1, torch.float32 if dtype == "float32" else torch.bfloat16)
    pcfg, w = P.load_folder(d)
    prompt = helpers.random_requests(320, [40], 3)["r0"]
    want = P.greedy_generate(pcfg, w, prompt, 12, eos=TINY_B["eos_token_id"])
    out = last_json(cli("generate", "--model", d, "--test", "--max_steps", 12, "--dtype", dtype, "--page-size", 8,
                        "--chunk-size", 24, "--prompt-ids", ",".join(map(str, prompt))).stdout)
    if dtype == "float32":
        assert out["tokens"] == want
    else:
        # bfloat16 may part ways with the plain tokens where two logits are close.  Every token is checked
        # against the plain logits of the engine's OWN prefix: it is their argmax, or it loses to the argmax
        # by less than the bfloat16 tolerance (relative to the row's largest logit); and where the engine
        # stopped early, the plain side (nearly) chose an end token there
        got = out["tokens"]
        assert 0 < len(got) <= 12
        rows = P.forward(pcfg, w, prompt + got)[len(prompt) - 1:]
        near = 0
        for i, row in enumerate(rows):
            if i < len(got):
                chosen = row[got[i]]
            elif len(got) < 12:
                chosen = max(row[e] for e in TINY_B["eos_token_id"])
            else:
                break
            margin = (row.max() - chosen) / np.abs(row).max()
            assert margin < 1.5e-2, f"token {i}: the engine's choice loses by {margin:.3e} of the row's largest logit"
            near += margin > 0
        print(f"[observed] bfloat16 generate: {len(got)} tokens, {near} of them not the plain argmax")
        assert got[:4] == want[:4]
    assert out["generated_tokens"] == len(out["tokens"]) and out["prefill_seconds"] > 0
    # the prompt from a file, sampling options under the reference's names
    (tmp_path / "p.json").write_text(json.dumps(prompt))
    a = last_json(cli("generate", "--model", d, "--max_steps", 6, "--dtype", dtype, "--prompt-file", tmp_path / "p.json",
                      "--top_k", 20, "--top_p", 0.9, "--temperature", 0.8, "--seed", 4).stdout)
    b = last_json(cli("generate", "--model", d, "--max_steps", 6, "--dtype", dtype, "--prompt-file", tmp_path / "p.json",
                      "--top-k", 20, "--top-p", 0.9, "--temperature", 0.8, "--sample-seed", 4).stdout)
    assert a["tokens"] == b["tokens"] and len(a["tokens"]) <= 6
    assert a["tokens"][:1] == out["tokens"][:1]          # the first token is the argmax whatever the options


@pytest.mark.gpu
def test_generate_with_random_weights_in_one_call(tmp_path):
    (tmp_path / "c.json").write_text(json.dumps(TINY_A))
    d = helpers.make_model(tmp_path / "m", TINY_A, 9)
    pcfg, w = P.load_folder(d)
    want = P.greedy_generate(pcfg, w, [7, 8, 9, 10], 8)
    out = last_json(cli("generate", "--random", tmp_path / "c.json", "--weights-seed", 9, "--dtype", "float32",
                        "--test", "--max_steps", 8, "--prompt-ids", "7 8 9 10").stdout)
    assert out["tokens"] == want


@pytest.mark.gpu
def test_a_toy_architecture_from_a_plugin_generates_through_the_command_line(tmp_path):
    """The toy state mixer of tests/toy_parts.py: registered by `--plugin toy_parts`,
    found by `random`, `generate` and `replay` through the one registry."""
    import toy_parts
    cfg = dict(TINY_A, architectures=["ToyStateLM"], toy_decay=0.8)
    (tmp_path / "c.json").write_text(json.dumps(cfg))
    d = tmp_path / "toy"
    cli("--plugin", "toy_parts", "random", "--config", tmp_path / "c.json", "--seed", 2, "--out", d, "--dtype", "float32")
    p = cli("generate", "--model", d, "--prompt-ids", "1,2,3", check=False)            # without the plugin: unknown
    assert p.returncode != 0 and "unknown architecture 'ToyStateLM'" in p.stderr
    pcfg, w = P.load_folder(d)
    prompt = helpers.random_requests(256, [19], 8)["r0"]
    toks = list(prompt)
    for _ in range(10):
        toks.append(int(np.argmax(toy_parts.plain_toy_state_logits(pcfg, w, toks, 0.8)[-1])))
    out = last_json(cli("generate", "--plugin", "toy_parts", "--model", d, "--test", "--max_steps", 10,
                        "--dtype", "float32", "--chunk-size", 8, "--prompt-ids", ",".join(map(str, prompt))).stdout)
    assert out["tokens"] == toks[len(prompt):]
    # and replay of the same model, pages handed out in a shuffled order
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": prompt[:11], "want": [10]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": prompt[11:], "want": [len(prompt) - 12]}], "end": ["a"]}]
    cli("replay", "--plugin", "toy_parts", "--model", d, "--dtype", "float32", "--out", tmp_path / "o",
        "--max-tokens", 64, "--shuffle-pages", 3, stdin="".join(json.dumps(s) + "\n" for s in steps))
    ref = toy_parts.plain_toy_state_logits(pcfg, w, prompt, 0.8)
    for i, row in ((0, 10), (1, len(prompt) - 1)):
        got = np.fromfile(tmp_path / "o" / f"{i}.f32", dtype="<f4")
        assert np.abs(got - ref[row]).max() / np.abs(ref[row]).max() < 2e-5


@pytest.mark.gpu
def test_a_toy_mixer_with_pages_and_state_generates_through_the_command_line(tmp_path):
    """The toy mixer that keeps keys and values in pages and a tail of its inputs in a state slot
    (tests/toy_parts.py), through `--plugin`: random weights, greedy generation in portions, replay."""
    import toy_parts
    cfg = dict(TINY_A, architectures=["ToyTailLM"], toy_decay=0.0)
    (tmp_path / "c.json").write_text(json.dumps(cfg))
    d = tmp_path / "toy"
    cli("--plugin", "toy_parts", "random", "--config", tmp_path / "c.json", "--seed", 3, "--out", d, "--dtype", "float32")
    pcfg, w = P.load_folder(d)
    prompt = helpers.random_requests(256, [23], 9)["r0"]
    toks = list(prompt)
    for _ in range(10):
        toks.append(int(np.argmax(toy_parts.plain_toy_tail_logits(pcfg, w, toks)[-1])))
    out = last_json(cli("generate", "--plugin", "toy_parts", "--model", d, "--test", "--max_steps", 10,
                        "--dtype", "float32", "--chunk-size", 7, "--page-size", 8,
                        "--prompt-ids", ",".join(map(str, prompt))).stdout)
    assert out["tokens"] == toks[len(prompt):]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": prompt[:2], "want": [1]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": prompt[2:13], "want": [0, 10]},
                                     {"id": "b", "tokens": prompt[5:9], "want": [3]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": prompt[13:], "want": [len(prompt) - 14]}], "end": ["a"]}]
    cli("replay", "--plugin", "toy_parts", "--model", d, "--dtype", "float32", "--out", tmp_path / "o",
        "--max-tokens", 128, "--shuffle-pages", 3, stdin="".join(json.dumps(s) + "\n" for s in steps))
    ref = toy_parts.plain_toy_tail_logits(pcfg, w, prompt)
    other = toy_parts.plain_toy_tail_logits(pcfg, w, prompt[5:9])
    vocab = ref.shape[1]
    got = {i: np.fromfile(tmp_path / "o" / f"{i}.f32", dtype="<f4").reshape(-1, vocab) for i in range(3)}
    for rows, want in ((got[0], ref[[1]]), (got[1], np.stack([ref[2], ref[12], other[3]])), (got[2], ref[[-1]])):
        assert np.abs(rows - want).max() / np.abs(want).max() < 2e-5
