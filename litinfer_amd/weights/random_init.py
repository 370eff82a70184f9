"""Random weights from a configuration and a seed.

Each tensor has a generator of its own, seeded from (seed, tensor name), so a
tensor's values do not depend on which other tensors exist or on the order of
generation.  How a tensor is drawn is what its part says (`ParamSpec.init`):
matrices and biases N(0, 0.02), the weights of a norm 1 + N(0, 0.02), zeros or
ones.  Values are drawn in float32 and rounded once to the stored dtype.
"""
from __future__ import annotations

import hashlib
import json
from pathlib import Path
from typing import Dict, Iterator, Tuple

import torch

from ..config import lookup
from .loader import ParamSpec
from .safetensors_io import write_safetensors

STD = 0.02


def _tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensor(seed: int, name: str, spec: ParamSpec, dtype: torch.dtype,
                  device="cpu") -> torch.Tensor:
    g = torch.Generator(device=device)
    g.manual_seed(_tensor_seed(seed, name))
    if spec.integer:
        return torch.randint(0, 2 ** 15, spec.shape, generator=g, device=device, dtype=torch.int32)
    if spec.init in ("zeros", "ones"):
        return torch.full(spec.shape, float(spec.init == "ones"), device=device, dtype=dtype)
    t = torch.randn(spec.shape, generator=g, device=device, dtype=torch.float32) * STD
    if spec.init == "one_plus_normal":
        t += 1.0
    return t.to(dtype)


def random_tensors(expected: Dict[str, ParamSpec], seed: int, dtype: torch.dtype,
                   device="cpu") -> Iterator[Tuple[str, torch.Tensor]]:
    for name in sorted(expected):
        yield name, random_tensor(seed, name, expected[name], dtype, device)


def write_random_model(model_dir, config: Dict, seed: int, dtype: torch.dtype = torch.bfloat16) -> Path:
    """Write config.json and model.safetensors for the architecture that
    `config` (the content of a config.json) names.  Optional tensors (biases)
    are written too."""
    from ..engine.model import expected_params_of_spec
    from ..config import architecture_name
    arch = lookup(architecture_name(config))
    cfg = arch.config_from_dict(config)
    spec = arch.model_spec(cfg)
    spec.validate()
    expected = expected_params_of_spec(spec)
    model_dir = Path(model_dir)
    model_dir.mkdir(parents=True, exist_ok=True)
    out_cfg = dict(config)
    out_cfg.setdefault("architectures", [arch.name])
    out_cfg["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32",
                              torch.float16: "float16"}[dtype]
    with open(model_dir / "config.json", "w", encoding="utf-8") as f:
        json.dump(out_cfg, f, indent=1)
    write_safetensors(model_dir / "model.safetensors", random_tensors(expected, seed, dtype),
                      metadata={"format": "pt", "seed": seed})
    return model_dir
