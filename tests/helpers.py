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


def round_to_bfloat16(a: np.ndarray) -> np.ndarray:
    """Nearest-even rounding of float32-representable values to bfloat16, by hand on the bits
    (finite values only), returned in the input's dtype."""
    bits = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return bits.astype(np.uint32).view(np.float32).reshape(a.shape).astype(a.dtype)


def plain_logits(model_dir, requests, matrices_as_bfloat16: bool = False) -> Dict[str, np.ndarray]:
    """float64 logits of every token of every request, from the stored weights; with
    `matrices_as_bfloat16` from the stored matrices rounded once to bfloat16 (what a bfloat16
    engine binds from a checkpoint stored in another precision), vectors as stored."""
    cfg, w = plain_impl.load_folder(model_dir, np.float64)
    if matrices_as_bfloat16:
        w = {n: round_to_bfloat16(a) if a.ndim == 2 else a for n, a in w.items()}
    return {rid: plain_impl.forward(cfg, w, toks) for rid, toks in requests.items()}


def gpu_available() -> bool:
    return torch.cuda.is_available()
