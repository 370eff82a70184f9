"""A toy architecture defined outside the framework: a recurrent mixer whose state
lives in the request's state slot, in a model that is otherwise the tiny decoder.
Importing this module registers the part and the architecture; nothing in the
framework's files knows of them.  The tests import it, and the command line takes it
as `--plugin toy_parts`.  It is a toy, written with torch: it shows the interfaces,
it is no model of anyone's."""
from dataclasses import dataclass, replace

import numpy as np
import torch

import plain_impl as P
from litinfer_amd.config import LayerSpec, ModelSpec, PartSpec, Qwen2Config, qwen2_model_spec, register_architecture
from litinfer_amd.parts import Mixer, StateNeed, register_part
from litinfer_amd.weights import ParamSpec


class ToyStateMixer(Mixer):
    """s_t = decay * s_{t-1} + xn_t, y_t = s_t W^T + b: a recurrent mixer whose state
    lives in the request's state slot.  The bias is drawn as zeros, which only a
    part can say of its own tensor."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.h = spec.args["hidden_size"]
        self.decay = spec.args["decay"]
        self.w = self.b = None

    def cache_need(self):
        return StateNeed((self.h,), torch.float32)

    def expected_params(self):
        return {self.prefix + "w": ParamSpec((self.h, self.h)),
                self.prefix + "b": ParamSpec((self.h,), init="zeros")}

    def load_params(self, get):
        self.w = get(self.prefix + "w").to(torch.float32).to(self.rt.device)
        self.b = get(self.prefix + "b").to(torch.float32).to(self.rt.device)

    def forward(self, xn, residual, ctx, cache):
        residual = residual.tensor()
        for s in range(ctx.num_segments):
            q0, n, slot = int(ctx.host_q_start[s]), int(ctx.host_q_len[s]), int(ctx.host_state_slots[s])
            state = cache.state[slot]
            for t in range(q0, q0 + n):
                state.mul_(self.decay).add_(xn[t].float())
                residual[t] += state @ self.w.T + self.b


@dataclass(frozen=True)
class ToyConfig:
    hidden_size: int
    vocab_size: int
    decay: float
    inner: Qwen2Config

    @classmethod
    def from_dict(cls, raw):
        return cls(raw["hidden_size"], raw["vocab_size"], raw["toy_decay"], Qwen2Config.from_dict(raw))


def toy_state_spec(c: ToyConfig) -> ModelSpec:
    base = qwen2_model_spec(c.inner)
    l0 = base.layers[0]
    toy = LayerSpec("prenorm", dict(l0.parts, mixer=PartSpec("toy_state", "model.layers.0.toy.",
                                                             {"hidden_size": c.hidden_size, "decay": c.decay})))
    return replace(base, architecture="ToyStateLM", layers=(toy,) + base.layers[1:])


register_part("mixer", "toy_state", ToyStateMixer)
register_architecture("ToyStateLM", ToyConfig.from_dict, toy_state_spec)


def plain_toy_state_logits(pcfg, w, ids, decay):
    """The toy model's logits for a whole sequence, from the plain implementation's
    parts (two layers: the toy mixer in the first, the tiny decoder's second)."""
    ids = np.asarray(ids)
    eps = pcfg.get("rms_norm_eps", 1e-6)
    pos = np.arange(len(ids))
    x = P.embedding(ids, w["model.embed_tokens.weight"])
    xn = P.rms_norm(x, w["model.layers.0.input_layernorm.weight"], eps)
    s = np.zeros(x.shape[1])
    y = np.zeros_like(x)
    for t in range(len(ids)):
        s = decay * s + xn[t]
        y[t] = s @ w["model.layers.0.toy.w"].T + w["model.layers.0.toy.b"]
    x = x + y
    xn = P.rms_norm(x, w["model.layers.0.post_attention_layernorm.weight"], eps)
    p = "model.layers.0.mlp."
    x = x + P.swiglu(xn @ w[p + "gate_proj.weight"].T, xn @ w[p + "up_proj.weight"].T) @ w[p + "down_proj.weight"].T
    x, _ = P.decoder_layer(x, pos, w, "model.layers.1.", pcfg, 0)
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]
    return P.rms_norm(x, w["model.norm.weight"], eps) @ head.T
