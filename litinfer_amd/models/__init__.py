from pathlib import Path

from .causal_lm import CausalLM
from .qwen2 import Qwen2


def load(model_path, **kw):
    """The entry point for a model folder: the class that the registry entry of the
    architecture in config.json names, the generic `CausalLM` when it names none."""
    from ..config import architecture_name, lookup, read_config_json
    arch = lookup(architecture_name(read_config_json(Path(model_path))))
    return (arch.entry or CausalLM)(model_path, **kw)


__all__ = ["CausalLM", "Qwen2", "load"]
