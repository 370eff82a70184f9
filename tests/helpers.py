"""Shared helpers of the tests: model folders in temporary places, token
streams, the plain reference's logits."""
from __future__ import annotations

import json
from pathlib import Path
from typing import Dict, Sequence

import numpy as np
import torch

import plain_impl
from litinfer_amd.weights import write_random_model


def make_model(tmp_path, config: dict, seed: int, dtype=torch.float32, name="model") -> Path:
    return write_random_model(Path(tmp_path) / name, config, seed=seed, dtype=dtype)


def random_requests(vocab: int, lengths: Sequence[int], seed: int) -> Dict[str, list]:
    rng = np.random.default_rng(seed)
    return {f"r{i}": rng.integers(0, vocab, n).tolist() for i, n in enumerate(lengths)}


def plain_logits(model_dir, requests) -> Dict[str, np.ndarray]:
    """float64 logits of every token of every request, from the stored weights."""
    cfg, w = plain_impl.load_folder(model_dir, np.float64)
    return {rid: plain_impl.forward(cfg, w, toks) for rid, toks in requests.items()}


def gpu_available() -> bool:
    return torch.cuda.is_available()
