from .spec import ExecEntry, LayerSpec, ModelSpec, PartSpec
from .registry import (Architecture, architecture_name, load_config, lookup, read_config_json,
                       register_architecture, registered_architectures)
from .qwen2 import ConfigError, Qwen2Config, qwen2_model_spec

from .qwen2 import QWEN2_WEIGHT_ALIASES

register_architecture("Qwen2ForCausalLM", Qwen2Config.from_dict, qwen2_model_spec, aliases=("qwen2",),
                      weight_aliases=QWEN2_WEIGHT_ALIASES)

__all__ = ["ExecEntry", "LayerSpec", "ModelSpec", "PartSpec", "Architecture", "architecture_name",
           "load_config", "lookup", "read_config_json", "register_architecture",
           "registered_architectures", "ConfigError", "Qwen2Config", "qwen2_model_spec"]
