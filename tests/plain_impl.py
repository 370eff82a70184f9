"""Plain, slow implementation of the Qwen2 dense decoder, written from the
formulas of the reference's operator loops.  Whole sequences, no cache, one
function per part, NumPy only.  It shares no code with the product package:
the tests compare the engine against it.

Every function works in the dtype of its inputs (float32 or float64); the
tests usually feed float64 copies of the stored weights so that this file is
the more exact side of a comparison.
"""
from __future__ import annotations

import json
import math
import struct
from pathlib import Path

import numpy as np


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------
def embedding(ids, table):
    """out[t, :] = table[ids[t], :], a row copy without scaling; an id outside
    the table is an error (src/ops/embedding/op.cpp:32-40)."""
    ids = np.asarray(ids)
    if ids.size and (ids.min() < 0 or ids.max() >= table.shape[0]):
        raise IndexError("embedding: index out of range")
    return table[ids]


def rms_norm(x, w, eps):
    """y = w * x / sqrt(mean(x^2) + eps): eps inside the root, added to the
    mean; the weight multiplies directly (src/ops/rms_norm/op.cpp:13-23)."""
    ss = (x * x).sum(axis=-1, keepdims=True)
    inv = 1.0 / np.sqrt(ss / x.shape[-1] + eps)
    return w * x * inv


def linear(x, w, b=None):
    """y = x W^T + b with W stored [out, in] (src/ops/linear/cpu/linear_cpu.cpp:32-37,
    52-58); the bias is skipped when absent (src/ops/linear/op.cpp:55)."""
    y = x @ w.T
    if b is not None:
        y = y + b
    return y


def rope_neox(x, pos, theta):
    """Half-split rotary encoding of x [T, heads, dh] at integer positions pos [T]
    (src/ops/rope/op.cpp:13-20 rotation, :32-39 angles):
    angle_j = pos / theta^(2j/dh); y[j] = a cos - b sin; y[j+dh/2] = b cos + a sin
    with a = x[j], b = x[j+dh/2]."""
    dh = x.shape[-1]
    half = dh // 2
    j = np.arange(half, dtype=x.dtype)
    ang = np.asarray(pos, dtype=x.dtype)[:, None] / (np.asarray(theta, dtype=x.dtype) ** (2 * j / dh))
    c = np.cos(ang)[:, None, :]
    s = np.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:]
    return np.concatenate([a * c - b * s, b * c + a * s], axis=-1)


def attention(q, k, v, q_pos, k_pos, scale, window=0):
    """Causal grouped-query attention (src/ops/paged_attention/op.cpp:20-64):
    query head h reads kv head h // (nh/nkv) (:20); the query at absolute
    position p sees the keys at positions t <= p (:22,:28); scores are
    scaled after the dot product (:42); softmax over the visible keys.
    `window` > 0 adds the rule p - t < window (the reference has no window;
    the rule is: a windowed layer's query sees itself and the window-1 keys
    before it).  q [Tq, nh, dh], k/v [Tk, nkv, dh]."""
    tq, nh, dh = q.shape
    nkv = k.shape[1]
    g = nh // nkv
    q_pos = np.asarray(q_pos)[:, None]
    k_pos = np.asarray(k_pos)[None, :]
    visible = k_pos <= q_pos
    if window and window > 0:
        visible &= (q_pos - k_pos) < window
    out = np.zeros_like(q)
    for h in range(nh):
        kh = h // g
        s = (q[:, h, :] @ k[:, kh, :].T) * scale
        s = np.where(visible, s, -np.inf)
        m = s.max(axis=-1, keepdims=True)
        e = np.exp(s - m)
        out[:, h, :] = (e / e.sum(axis=-1, keepdims=True)) @ v[:, kh, :]
    return out


def swiglu(gate, up):
    """out = up * gate / (1 + exp(-gate)) (src/ops/swiglu/op.cpp:19-22)."""
    return up * (gate / (1.0 + np.exp(-gate)))


def argmax_first(logits):
    """Index of the maximum, the lowest index on ties
    (src/ops/argmax/op.cpp:26-33)."""
    return int(np.argmax(logits))


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
def layer_window(cfg, layer):
    """Window of a layer: layers with index >= max_window_layers use
    sliding_window when use_sliding_window is set; 0 means all keys.  (The
    reference reads none of these keys; python/llaisys/models/qwen2.py:243-299.)"""
    if cfg.get("use_sliding_window", False) and cfg.get("sliding_window") is not None:
        if layer >= cfg.get("max_window_layers", cfg["num_hidden_layers"]):
            return int(cfg["sliding_window"])
    return 0


def head_dim_of(cfg):
    """head_dim defaults to hidden_size // num_attention_heads
    (python/llaisys/models/qwen2.py:282)."""
    return int(cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"])


def decoder_layer(x, pos, w, prefix, cfg, window, kv_from=None):
    """One pre-norm block in the reference's order (src/llaisys/models/qwen2.cpp:272-317):
    xn = norm1(x); q,k,v = linear(xn)+bias (:613-615); rope on q and k only
    (:628-629); attention with scale 1/sqrt(dh) (:690); o projection without
    bias (:699); x += o (:287-290); xn = norm2(x) (:297); mlp (:744-759);
    x += y (:309-312).  Returns (x, (k, v)); `kv_from`, if given, is another
    layer's (k, v) that this layer attends to instead of its own."""
    nh = cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads", nh)
    dh = head_dim_of(cfg)
    eps = cfg.get("rms_norm_eps", 1e-6)
    theta = cfg.get("rope_theta", 10000.0)
    t = x.shape[0]
    xn = rms_norm(x, w[prefix + "input_layernorm.weight"], eps)
    q = linear(xn, w[prefix + "self_attn.q_proj.weight"], w.get(prefix + "self_attn.q_proj.bias"))
    q = rope_neox(q.reshape(t, nh, dh), pos, theta)
    if kv_from is None:
        k = linear(xn, w[prefix + "self_attn.k_proj.weight"], w.get(prefix + "self_attn.k_proj.bias"))
        v = linear(xn, w[prefix + "self_attn.v_proj.weight"], w.get(prefix + "self_attn.v_proj.bias"))
        k = rope_neox(k.reshape(t, nkv, dh), pos, theta)
        v = v.reshape(t, nkv, dh)
    else:
        k, v = kv_from
    a = attention(q, k, v, pos, pos, 1.0 / math.sqrt(dh), window)
    x = x + linear(a.reshape(t, nh * dh), w[prefix + "self_attn.o_proj.weight"])
    xn = rms_norm(x, w[prefix + "post_attention_layernorm.weight"], eps)
    g = linear(xn, w[prefix + "mlp.gate_proj.weight"])
    u = linear(xn, w[prefix + "mlp.up_proj.weight"])
    x = x + linear(swiglu(g, u), w[prefix + "mlp.down_proj.weight"])
    return x, (k, v)


def forward(cfg, w, ids, start_pos=0, order=None):
    """Logits [T, V] of one whole sequence (src/llaisys/models/qwen2.cpp:261-346):
    embedding, the layers, final norm (:319), lm_head without bias (:337); the
    output matrix is the embedding table when the checkpoint is tied
    (python/llaisys/models/qwen2.py:196-199).  Positions count from start_pos
    (:618-624).  `order` is a list of (layer, source) pairs: run `layer`, and if
    `source` is not None attend to the keys and values that entry `source` of
    the list made."""
    ids = np.asarray(ids)
    pos = np.arange(start_pos, start_pos + len(ids))
    x = embedding(ids, w["model.embed_tokens.weight"])
    n_layers = cfg["num_hidden_layers"]
    if order is None:
        order = [(l, None) for l in range(n_layers)]
    made = []
    for layer, source in order:
        x, kv = decoder_layer(x, pos, w, f"model.layers.{layer}.", cfg, layer_window(cfg, layer),
                              kv_from=None if source is None else made[source])
        made.append(kv)
    x = rms_norm(x, w["model.norm.weight"], cfg.get("rms_norm_eps", 1e-6))
    if cfg.get("tie_word_embeddings", False) or "lm_head.weight" not in w:
        head = w["model.embed_tokens.weight"]
    else:
        head = w["lm_head.weight"]
    return linear(x, head)


def greedy_generate(cfg, w, prompt, n_new, eos=()):
    """Greedy continuation by recomputing the whole sequence for each token; an
    end token stops and is not appended (python/llaisys/models/qwen2.py:363,393)."""
    seq = list(prompt)
    out = []
    for _ in range(n_new):
        tok = argmax_first(forward(cfg, w, seq)[-1])
        if tok in eos:
            break
        out.append(tok)
        seq.append(tok)
    return out


# --------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------
def sampling_candidates(logits, temperature, top_k, top_p):
    """The reference engine's filter (src/llaisys/models/qwen2.cpp:890-920):
    divide by the temperature, order descending, keep the first top_k when
    0 < top_k < V, then when 0 < top_p < 1 keep the shortest prefix whose
    softmax mass reaches top_p, and take the softmax of the survivors.  Ties
    are ordered by ascending index here (the reference leaves them open).
    Returns (ids ascending, probabilities in that order)."""
    z = np.asarray(logits, dtype=np.float64) / temperature
    order = np.lexsort((np.arange(z.size), -z))
    if 0 < top_k < z.size:
        order = order[:top_k]
    if 0.0 < top_p < 1.0:
        p = np.exp(z[order] - z[order[0]])
        p /= p.sum()
        cum = np.cumsum(p)
        cutoff = int(np.argmax(cum >= top_p)) + 1 if (cum >= top_p).any() else len(order)
        order = order[:cutoff]
    p = np.exp(z[order] - z[order[0]])
    p /= p.sum()
    asc = np.argsort(order)
    return order[asc], p[asc]


def sample_with_uniform(logits, temperature, top_k, top_p, u):
    """Inverse-CDF draw over the surviving ids in ascending order: the first id
    whose running probability sum reaches u (0 <= u < 1).  temperature <= 0 is
    greedy (src/llaisys/models/qwen2.cpp:893-895)."""
    if temperature <= 0.0:
        return argmax_first(logits)
    ids, p = sampling_candidates(logits, temperature, top_k, top_p)
    cum = np.cumsum(p)
    i = int(np.searchsorted(cum, u * cum[-1], side="left"))
    return int(ids[min(i, len(ids) - 1)])


# --------------------------------------------------------------------------
# reading a model folder without the product's loader
# --------------------------------------------------------------------------
_ST_DTYPES = {"F32": np.float32, "F64": np.float64, "F16": np.float16, "I32": np.int32, "I64": np.int64}


def read_safetensors(path, dtype=np.float64):
    """File layout as the reference reads it by hand
    (python/llaisys/models/qwen2.py:112-129): u64 little-endian header length,
    a JSON header, then the data; each entry has dtype, shape and data_offsets.
    BF16 is widened through its upper 16 bits (:104-107, without the
    reference's narrowing to half)."""
    raw = Path(path).read_bytes()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + hlen])
    base = 8 + hlen
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        b, e = meta["data_offsets"]
        buf = raw[base + b: base + e]
        if meta["dtype"] == "BF16":
            a = (np.frombuffer(buf, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
        else:
            a = np.frombuffer(buf, dtype=_ST_DTYPES[meta["dtype"]])
        out[name] = a.reshape(meta["shape"]).astype(dtype)
    return out


def load_folder(folder, dtype=np.float64):
    folder = Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    return cfg, read_safetensors(folder / "model.safetensors", dtype)
