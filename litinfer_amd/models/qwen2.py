"""`Qwen2(model_path)`, the name under which the reference offers its entry point
(python/llaisys/models/qwen2.py:23-29, python/llaisys/models/__init__.py:1).  The
class is the generic one: which model it builds is decided by config.json."""
from .causal_lm import CausalLM

Qwen2 = CausalLM

__all__ = ["Qwen2"]
