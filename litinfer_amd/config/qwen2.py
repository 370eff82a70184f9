"""Typed configuration of the Qwen2 dense decoder, read from config.json.

Keys and defaults follow the reference's reader
(python/llaisys/models/qwen2.py:243-299); the keys it does not read
(tie_word_embeddings, use_sliding_window, sliding_window, max_window_layers,
hidden_act, rope_scaling) are read and checked here.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .spec import ExecEntry, LayerSpec, ModelSpec, PartSpec


class ConfigError(ValueError):
    pass


def _need_int(cfg: Dict[str, Any], key: str) -> int:
    if key not in cfg or cfg[key] is None:
        raise ConfigError(f"config.json: required key '{key}' is missing")
    v = cfg[key]
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"config.json: '{key}' must be a positive integer, found {v!r}")
    return v


@dataclass(frozen=True)
class Qwen2Config:
    num_hidden_layers: int
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    use_sliding_window: bool
    sliding_window: Optional[int]
    max_window_layers: int
    eos_token_ids: Tuple[int, ...]
    torch_dtype: str

    architecture = "Qwen2ForCausalLM"

    @classmethod
    def from_dict(cls, cfg: Dict[str, Any]) -> "Qwen2Config":
        nl = _need_int(cfg, "num_hidden_layers")
        hs = _need_int(cfg, "hidden_size")
        nh = _need_int(cfg, "num_attention_heads")
        inter = _need_int(cfg, "intermediate_size")
        voc = _need_int(cfg, "vocab_size")
        maxpos = _need_int(cfg, "max_position_embeddings")
        nkv = cfg.get("num_key_value_heads")
        nkv = nh if nkv is None else _need_int(cfg, "num_key_value_heads")
        dh = cfg.get("head_dim")
        dh = hs // nh if dh is None else _need_int(cfg, "head_dim")
        if nh % nkv != 0:
            raise ConfigError(f"config.json: num_attention_heads ({nh}) is not a multiple of "
                              f"num_key_value_heads ({nkv})")
        if dh <= 0 or dh % 2 != 0:
            raise ConfigError(f"config.json: head_dim must be positive and even, found {dh}")
        eps = float(cfg.get("rms_norm_eps", 1e-6))
        if eps < 0:
            raise ConfigError(f"config.json: rms_norm_eps must not be negative, found {eps}")
        theta = float(cfg.get("rope_theta", 10000.0))
        if theta <= 0:
            raise ConfigError(f"config.json: rope_theta must be positive, found {theta}")
        act = cfg.get("hidden_act")
        if act is not None and act != "silu":
            raise ConfigError(f"config.json: hidden_act '{act}' is not supported (only 'silu')")
        if cfg.get("rope_scaling") is not None:
            raise ConfigError("config.json: rope_scaling is not supported")
        use_win = bool(cfg.get("use_sliding_window", False))
        win = cfg.get("sliding_window")
        if use_win:
            if isinstance(win, bool) or not isinstance(win, int) or win <= 0:
                raise ConfigError("config.json: use_sliding_window needs a positive integer "
                                  f"sliding_window, found {win!r}")
        mwl = cfg.get("max_window_layers")
        mwl = nl if mwl is None else int(mwl)
        if mwl < 0:
            raise ConfigError(f"config.json: max_window_layers must not be negative, found {mwl}")
        eos = cfg.get("eos_token_id", None)
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, list):
            eos_ids = tuple(int(e) for e in eos)
        else:
            eos_ids = (int(eos),)
        eos_ids = tuple(e for e in eos_ids if e >= 0)
        return cls(num_hidden_layers=nl, hidden_size=hs, num_attention_heads=nh,
                   num_key_value_heads=nkv, head_dim=dh, intermediate_size=inter,
                   vocab_size=voc, max_position_embeddings=maxpos, rms_norm_eps=eps,
                   rope_theta=theta, tie_word_embeddings=bool(cfg.get("tie_word_embeddings", False)),
                   use_sliding_window=use_win, sliding_window=(int(win) if win is not None else None),
                   max_window_layers=mwl, eos_token_ids=eos_ids,
                   torch_dtype=str(cfg.get("torch_dtype", "bfloat16")))

    def to_dict(self) -> Dict[str, Any]:
        """The config.json that reads back to this configuration."""
        d: Dict[str, Any] = {
            "architectures": [self.architecture], "model_type": "qwen2", "hidden_act": "silu",
            "num_hidden_layers": self.num_hidden_layers, "hidden_size": self.hidden_size,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads, "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size, "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps, "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "use_sliding_window": self.use_sliding_window,
            "sliding_window": self.sliding_window, "max_window_layers": self.max_window_layers,
            "torch_dtype": self.torch_dtype,
        }
        if self.eos_token_ids:
            d["eos_token_id"] = (self.eos_token_ids[0] if len(self.eos_token_ids) == 1
                                 else list(self.eos_token_ids))
        return d

    def window_of_layer(self, layer: int) -> int:
        """0 = all keys.  A layer with index >= max_window_layers uses the
        window when use_sliding_window is set."""
        if self.use_sliding_window and self.sliding_window and layer >= self.max_window_layers:
            return self.sliding_window
        return 0


# other names under which the reference takes three of the tensors
# (python/llaisys/models/qwen2.py:139-149): stored name -> the model's name
QWEN2_WEIGHT_ALIASES = {
    "transformer.wte.weight": "model.embed_tokens.weight",
    "model.lm_head.weight": "lm_head.weight",
    "transformer.ln_f.weight": "model.norm.weight",
}


def qwen2_model_spec(c: Qwen2Config) -> ModelSpec:
    """The Qwen2 decoder as data: per layer RMSNorm -> grouped-query attention
    with biased q/k/v and half-split rotary positions -> residual -> RMSNorm ->
    SwiGLU -> residual (src/llaisys/models/qwen2.cpp:272-317), a final RMSNorm
    (:319) and a linear head without bias (:337)."""
    layers = []
    for l in range(c.num_hidden_layers):
        p = f"model.layers.{l}."
        norm_args = {"size": c.hidden_size, "eps": c.rms_norm_eps}
        layers.append(LayerSpec(block="prenorm", parts={
            "norm1": PartSpec("rmsnorm", p + "input_layernorm.", dict(norm_args)),
            "mixer": PartSpec("gqa_attention", p + "self_attn.", {
                "hidden_size": c.hidden_size, "num_heads": c.num_attention_heads,
                "num_kv_heads": c.num_key_value_heads, "head_dim": c.head_dim,
                "qkv_bias": True, "out_bias": False, "window": c.window_of_layer(l),
                "scale": None,
                "position": PartSpec("rope_neox", "", {"head_dim": c.head_dim,
                                                       "rotary_dim": c.head_dim,
                                                       "theta": c.rope_theta}),
            }),
            "norm2": PartSpec("rmsnorm", p + "post_attention_layernorm.", dict(norm_args)),
            "feed_forward": PartSpec("swiglu_mlp", p + "mlp.", {
                "hidden_size": c.hidden_size, "intermediate_size": c.intermediate_size}),
        }))
    return ModelSpec(
        architecture=c.architecture, hidden_size=c.hidden_size, vocab_size=c.vocab_size,
        max_positions=c.max_position_embeddings,
        embedding=PartSpec("token_embedding", "model.embed_tokens.",
                           {"vocab_size": c.vocab_size, "hidden_size": c.hidden_size}),
        layers=tuple(layers),
        order=tuple(ExecEntry(l) for l in range(c.num_hidden_layers)),
        final_norm=PartSpec("rmsnorm", "model.norm.", {"size": c.hidden_size, "eps": c.rms_norm_eps}),
        head=PartSpec("linear_head", "lm_head.", {
            "vocab_size": c.vocab_size, "hidden_size": c.hidden_size,
            "tied_to": "model.embed_tokens.weight" if c.tie_word_embeddings else None,
            "tie_if_absent": True}),
        eos_token_ids=c.eos_token_ids)
