"""Toy architectures defined outside the framework: a recurrent mixer whose state
lives in the request's state slot, and a mixer that keeps keys and values in pages AND
a short tail of its last inputs in a state slot, each in a model that is otherwise the tiny decoder.
Importing this module registers the part and the architecture; nothing in the
framework's files knows of them.  The tests import it, and the command line takes it
as `--plugin toy_parts`.  It is a toy, written with torch: it shows the interfaces,
it is no model of anyone's."""
from dataclasses import dataclass, replace

import numpy as np
import torch

import plain_impl as P
from litinfer_amd.config import LayerSpec, ModelSpec, PartSpec, Qwen2Config, qwen2_model_spec, register_architecture
from litinfer_amd.parts import Mixer, PagedNeed, PagedTensor, StateNeed, register_part
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


# ------------------------------------------------ pages and a state of fixed size in one mixer
TAIL = 3
TAPS = (0.5, -0.25, 0.125)          # weights of the inputs 1, 2 and 3 tokens back


class ToyTailAttention(Mixer):
    """u_t = xn_t + sum_j TAPS[j] * xn_{t-1-j} (a short causal filter over the last TAIL inputs, which
    are kept in the request's state slot between steps); q, k, v = u_t Wq, u_t Wk, u_t Wv; one head of
    causal softmax attention over ALL earlier k, v, which are kept in pages; output y_t Wo.  Written
    with torch: it is a toy that shows the interface of a mixer with both kinds of cache, not a kernel."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.h, self.r = spec.args["hidden_size"], spec.args["rank"]

    def cache_need(self):
        return (PagedNeed((PagedTensor("k", (self.r,), torch.float32), PagedTensor("v", (self.r,), torch.float32))),
                StateNeed((TAIL, self.h), torch.float32, name="tail"))

    def expected_params(self):
        p = self.prefix
        return {p + "wq": ParamSpec((self.r, self.h)), p + "wk": ParamSpec((self.r, self.h)),
                p + "wv": ParamSpec((self.r, self.h)), p + "wo": ParamSpec((self.h, self.r))}

    def load_params(self, get):
        self.wq, self.wk, self.wv, self.wo = (get(self.prefix + n).to(torch.float32).to(self.rt.device)
                                              for n in ("wq", "wk", "wv", "wo"))

    def forward(self, xn, residual, ctx, cache):
        x = xn.float()
        u = torch.empty_like(x)
        tails = cache.states["tail"]                                   # [max_seqs, TAIL, hidden], oldest first
        for s in range(ctx.num_segments):
            q0, n, slot = int(ctx.host_q_start[s]), int(ctx.host_q_len[s]), int(ctx.host_state_slots[s])
            ext = torch.cat([tails[slot], x[q0:q0 + n]])               # the tail, then this step's inputs
            u[q0:q0 + n] = ext[TAIL:] + sum(c * ext[TAIL - 1 - j:len(ext) - 1 - j] for j, c in enumerate(TAPS))
            tails[slot] = ext[-TAIL:]
        kp, vp = cache.tensors["k"], cache.tensors["v"]                # [pages, page_size, rank]
        slots = ctx.slot_map(cache.group).long()
        kp.view(-1, self.r)[slots] = u @ self.wk.T                     # written before they are read
        vp.view(-1, self.r)[slots] = u @ self.wv.T
        q = u @ self.wq.T
        table = ctx.attention_meta(cache.group).block_table.cpu()
        out = residual.tensor()
        for s in range(ctx.num_segments):
            q0, n, have = int(ctx.host_q_start[s]), int(ctx.host_q_len[s]), int(ctx.host_ctx_len[s])
            blocks = table[s, :-(-have // cache.page_size)].long().to(kp.device)
            k, v = kp[blocks].reshape(-1, self.r)[:have], vp[blocks].reshape(-1, self.r)[:have]
            score = q[q0:q0 + n] @ k.T / self.r ** 0.5
            pos = torch.arange(have - n, have, device=score.device)[:, None]
            score = score.masked_fill(torch.arange(have, device=score.device)[None, :] > pos, float("-inf"))
            out[q0:q0 + n] += torch.softmax(score, dim=-1) @ v @ self.wo.T


def toy_tail_spec(c: ToyConfig) -> ModelSpec:
    base = qwen2_model_spec(c.inner)
    l0 = base.layers[0]
    toy = LayerSpec("prenorm", dict(l0.parts, mixer=PartSpec("toy_tail", "model.layers.0.tail.",
                                                             {"hidden_size": c.hidden_size, "rank": 12})))
    return replace(base, architecture="ToyTailLM", layers=(toy,) + base.layers[1:])


register_part("mixer", "toy_tail", ToyTailAttention)
register_architecture("ToyTailLM", ToyConfig.from_dict, toy_tail_spec)


def plain_toy_tail_logits(pcfg, w, ids):
    """The toy tail model's logits for a whole sequence, from the plain implementation's parts."""
    ids = np.asarray(ids)
    eps = pcfg.get("rms_norm_eps", 1e-6)
    t = len(ids)
    pos = np.arange(t)
    x = P.embedding(ids, w["model.embed_tokens.weight"])
    xn = P.rms_norm(x, w["model.layers.0.input_layernorm.weight"], eps)
    u = xn.copy()
    for j, c in enumerate(TAPS):
        u[1 + j:] += c * xn[:t - 1 - j]
    p = "model.layers.0.tail."
    q, k, v = u @ w[p + "wq"].T, u @ w[p + "wk"].T, u @ w[p + "wv"].T
    score = q @ k.T / np.sqrt(k.shape[1])
    score[np.triu_indices(t, 1)] = -np.inf
    e = np.exp(score - score.max(-1, keepdims=True))
    x = x + (e / e.sum(-1, keepdims=True)) @ v @ w[p + "wo"].T
    xn = P.rms_norm(x, w["model.layers.0.post_attention_layernorm.weight"], eps)
    p = "model.layers.0.mlp."
    x = x + P.swiglu(xn @ w[p + "gate_proj.weight"].T, xn @ w[p + "up_proj.weight"].T) @ w[p + "down_proj.weight"].T
    x, _ = P.decoder_layer(x, pos, w, "model.layers.1.", pcfg, 0)
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]
    return P.rms_norm(x, w["model.norm.weight"], eps) @ head.T
