from pathlib import Path

from .qwen2 import Qwen2

_ENTRY_POINTS = {"Qwen2ForCausalLM": Qwen2, "qwen2": Qwen2}


def load(model_path, **kw):
    """The entry point of whatever architecture config.json names."""
    from ..config import architecture_name, read_config_json
    name = architecture_name(read_config_json(Path(model_path)))
    if name not in _ENTRY_POINTS:
        raise KeyError(f"no entry point for architecture '{name}'; known: {sorted(_ENTRY_POINTS)}")
    return _ENTRY_POINTS[name](model_path, **kw)


__all__ = ["Qwen2", "load"]
