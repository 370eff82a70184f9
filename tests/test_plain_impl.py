"""What fixes the plain implementation beside the reference's text: special
cases that reduce to a library routine, invariants, and the shapes and special
inputs of the reference's own operator tests.  Each is chosen so that a
plausible mistake (a wrong sign or pairing, a norm in the wrong place, tiled
instead of interleaved kv heads) fails it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_impl as P
from tiny_configs import TINY_A, TINY_B

RNG = np.random.default_rng(0)


def test_embedding_is_a_row_copy_and_checks_range():
    table = RNG.standard_normal((512, 40))
    for idx in ([1], RNG.integers(0, 512, 50)):               # shapes of test/ops/embedding.py:45-48
        assert np.array_equal(P.embedding(idx, table), table[np.asarray(idx)])
    with pytest.raises(IndexError):
        P.embedding([512], table)
    with pytest.raises(IndexError):
        P.embedding([-1], table)


def test_rms_norm():
    x = RNG.standard_normal((7, 64)) * 3
    w = RNG.standard_normal(64)
    ref = F.rms_norm(torch.from_numpy(x), (64,), torch.from_numpy(w), 1e-5).numpy()   # library routine
    assert np.allclose(P.rms_norm(x, w, 1e-5), ref, rtol=1e-12)
    y = P.rms_norm(x, np.ones(64), 0.0)
    assert np.allclose((y * y).mean(-1), 1.0)                                        # unit mean square
    assert np.allclose(P.rms_norm(5 * x, w, 0.0), P.rms_norm(x, w, 0.0))             # scale invariant
    assert np.array_equal(P.rms_norm(np.zeros((1, 4)), np.ones(4), 1e-6), np.zeros((1, 4)))  # eps inside the root
    # eps is added to the MEAN of squares: for one element x the result is w x / sqrt(x^2 + eps)
    assert np.isclose(P.rms_norm(np.array([[3.0]]), np.array([2.0]), 7.0)[0, 0], 6.0 / 4.0)


def test_linear_is_x_wt_plus_b():
    x, w, b = RNG.standard_normal((2, 4)), RNG.standard_normal((3, 4)), RNG.standard_normal(3)
    ref = F.linear(torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(b)).numpy()
    assert np.allclose(P.linear(x, w, b), ref)
    assert np.allclose(P.linear(x, w), P.linear(x, w, np.zeros(3)))                  # no bias = zero bias
    assert np.allclose(P.linear(x[:1], w, b), P.linear(x, w, b)[:1])                 # one row = a row of many


def test_rope_pairing_sign_and_relative_property():
    one = np.array([[[1.0, 0.0, 0.0, 0.0]]])
    y = P.rope_neox(one, [1], 10000.0)[0, 0]
    assert np.allclose(y, [math.cos(1), 0, math.sin(1), 0])      # half-split pairs (0,2),(1,3); +sin on the partner
    x = RNG.standard_normal((6, 3, 16))
    assert np.array_equal(P.rope_neox(x, [0] * 6, 1e4), x)       # position 0 is the identity
    r = P.rope_neox(x, np.arange(6) + 100, 1e4)
    assert np.allclose(x[..., :8] ** 2 + x[..., 8:] ** 2, r[..., :8] ** 2 + r[..., 8:] ** 2)   # pairs keep length
    # the second frequency is theta^(-2/dh): angle of pair 1 at position 1
    ang = 1.0 / 1e4 ** (2 / 16)
    e1 = np.zeros((1, 1, 16)); e1[0, 0, 1] = 1
    assert np.isclose(P.rope_neox(e1, [1], 1e4)[0, 0, 9], math.sin(ang))
    q, k = RNG.standard_normal((1, 1, 16)), RNG.standard_normal((1, 1, 16))
    dots = [float((P.rope_neox(q, [p + 5], 1e4) * P.rope_neox(k, [p], 1e4)).sum()) for p in (0, 3, 40)]
    assert np.allclose(dots, dots[0])                             # only the distance counts


def torch_attention(q, k, v, scale):
    """The reference's own test formula (test/ops/self_attention.py:11-28)."""
    q, k, v = (torch.from_numpy(a).transpose(0, 1) for a in (q, k, v))
    L, S = q.size(-2), k.size(-2)
    mask = torch.ones(L, S, dtype=torch.bool).tril(diagonal=S - L)
    k = k.repeat_interleave(q.size(0) // k.size(0), 0)
    v = v.repeat_interleave(q.size(0) // v.size(0), 0)
    w = (q @ k.transpose(-2, -1) * scale).masked_fill(~mask, float("-inf"))
    return (torch.softmax(w, -1) @ v).transpose(0, 1).numpy()


@pytest.mark.parametrize("qlen,kvlen,nh,nkv,hd", [(2, 2, 1, 1, 4), (5, 11, 4, 2, 8)])   # self_attention.py:71-81
def test_attention_against_the_reference_test_formula(qlen, kvlen, nh, nkv, hd):
    q, k, v = (RNG.standard_normal(s) for s in ((qlen, nh, hd), (kvlen, nkv, hd), (kvlen, nkv, hd)))
    scale = 1 / math.sqrt(hd)
    got = P.attention(q, k, v, np.arange(kvlen - qlen, kvlen), np.arange(kvlen), scale)
    assert np.allclose(got, torch_attention(q, k, v, scale))


def test_attention_reduces_to_the_library_routine():
    q, k, v = (RNG.standard_normal((9, 4, 16)) for _ in range(3))
    t = lambda a: torch.from_numpy(a).transpose(0, 1)
    ref = F.scaled_dot_product_attention(t(q), t(k), t(v), is_causal=True).transpose(0, 1).numpy()
    assert np.allclose(P.attention(q, k, v, np.arange(9), np.arange(9), 0.25), ref)


def test_attention_special_cases():
    q, k, v = RNG.standard_normal((1, 4, 8)), RNG.standard_normal((1, 2, 8)), RNG.standard_normal((1, 2, 8))
    out = P.attention(q, k, v, [0], [0], 1.0)
    assert np.allclose(out[0, 0], v[0, 0]) and np.allclose(out[0, 1], v[0, 0])       # heads 0,1 -> kv head 0
    assert np.allclose(out[0, 2], v[0, 1]) and np.allclose(out[0, 3], v[0, 1])       # interleaved, not tiled
    k5, v5 = np.zeros((5, 1, 8)), RNG.standard_normal((5, 1, 8))
    out = P.attention(RNG.standard_normal((1, 1, 8)), k5, v5, [4], np.arange(5), 1.0)
    assert np.allclose(out[0, 0], v5[:, 0].mean(0))                                  # equal scores: the mean


def test_window_rule():
    q, k, v = (RNG.standard_normal((12, 2, 8)) for _ in range(3))
    pos = np.arange(12)
    full = P.attention(q, k, v, pos, pos, 0.3)
    assert np.array_equal(P.attention(q, k, v, pos, pos, 0.3, window=12), full)      # window >= length
    assert np.allclose(P.attention(q, k, v, pos, pos, 0.3, window=1), v)             # sees itself only
    w3 = P.attention(q, k, v, pos, pos, 0.3, window=3)
    assert np.allclose(w3[5], P.attention(q[5:6], k[3:6], v[3:6], [5], [3, 4, 5], 0.3)[0])   # p-2..p
    assert not np.allclose(w3[5], P.attention(q[5:6], k[2:6], v[2:6], [5], [2, 3, 4, 5], 0.3)[0])


def test_swiglu():
    g, u = RNG.standard_normal((2, 3)) * 4, RNG.standard_normal((2, 3))
    assert np.allclose(P.swiglu(g, u), (F.silu(torch.from_numpy(g)) * torch.from_numpy(u)).numpy())
    assert np.array_equal(P.swiglu(np.zeros(3), u[0]), np.zeros(3))
    assert np.allclose(P.swiglu(np.full(3, 40.0), u[0]), 40.0 * u[0])
    assert np.allclose(P.swiglu(np.full(3, -40.0), u[0]), 0.0, atol=1e-15)


def test_argmax_takes_the_first_maximum():
    assert P.argmax_first(np.array([1.0, 5.0, 5.0, 2.0])) == 1


def _tiny_weights(cfg, seed, dtype=np.float64):
    """Random tensors under the names of the reference's checkpoint table
    (python/llaisys/models/qwen2.py:139-194), written out here: the tests of the plain
    implementation take nothing from the product package."""
    rng = np.random.default_rng(seed)
    h, nh, inter, voc = cfg["hidden_size"], cfg["num_attention_heads"], cfg["intermediate_size"], cfg["vocab_size"]
    nkv = cfg.get("num_key_value_heads", nh)
    dh = cfg.get("head_dim") or h // nh
    shapes = {"model.embed_tokens.weight": (voc, h), "model.norm.weight": (h,)}
    if not cfg.get("tie_word_embeddings", False):
        shapes["lm_head.weight"] = (voc, h)
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        shapes.update({p + "input_layernorm.weight": (h,), p + "post_attention_layernorm.weight": (h,),
                       p + "self_attn.q_proj.weight": (nh * dh, h), p + "self_attn.q_proj.bias": (nh * dh,),
                       p + "self_attn.k_proj.weight": (nkv * dh, h), p + "self_attn.k_proj.bias": (nkv * dh,),
                       p + "self_attn.v_proj.weight": (nkv * dh, h), p + "self_attn.v_proj.bias": (nkv * dh,),
                       p + "self_attn.o_proj.weight": (h, nh * dh), p + "mlp.gate_proj.weight": (inter, h),
                       p + "mlp.up_proj.weight": (inter, h), p + "mlp.down_proj.weight": (h, inter)})
    out = {}
    for name, shape in shapes.items():
        a = rng.standard_normal(shape) * 0.05
        out[name] = (a + 1 if name.endswith("norm.weight") else a).astype(dtype)
    return out


def test_model_closed_forms():
    for cfg in (TINY_A, TINY_B):
        w = _tiny_weights(cfg, 1)
        eps = cfg["rms_norm_eps"]
        head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
        # with zero output projections every block adds nothing: logits = head(norm(E[ids]))
        w0 = {n: (np.zeros_like(a) if n.endswith(("o_proj.weight", "down_proj.weight")) else a) for n, a in w.items()}
        ids = [3, 1, 4, 1, 5]
        want = P.rms_norm(w0["model.embed_tokens.weight"][ids], w0["model.norm.weight"], eps) @ head.T
        assert np.allclose(P.forward(cfg, w0, ids), want)
        # a prompt of one token: each attention output is its value row, whatever q and k are
        x = w["model.embed_tokens.weight"][[7]]
        nh, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
        dh = cfg["head_dim"]
        for l in range(cfg["num_hidden_layers"]):
            p = f"model.layers.{l}."
            xn = P.rms_norm(x, w[p + "input_layernorm.weight"], eps)
            v = (xn @ w[p + "self_attn.v_proj.weight"].T + w[p + "self_attn.v_proj.bias"]).reshape(nkv, dh)
            a = np.repeat(v, nh // nkv, axis=0).reshape(1, nh * dh)
            x = x + a @ w[p + "self_attn.o_proj.weight"].T
            xn = P.rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
            g, u = xn @ w[p + "mlp.gate_proj.weight"].T, xn @ w[p + "mlp.up_proj.weight"].T
            x = x + P.swiglu(g, u) @ w[p + "mlp.down_proj.weight"].T
        assert np.allclose(P.forward(cfg, w, [7]), P.rms_norm(x, w["model.norm.weight"], eps) @ head.T)


def test_attention_layer_in_closed_form_with_complex_rotations():
    """A layer whose query and key matrices are zero, so that q and k are their BIASES at every
    token, and whose feed-forward adds nothing: the scores then follow from the biases and the
    distance alone.  Written out independently of this file's functions, the pair (j, j + dh/2) of a
    head as one complex number z_j that the position p turns by exp(i p theta^(-2j/dh)):
    score(p, t) = Re sum_j q_j conj(k_j) exp(i (p - t) angle_j) / sqrt(dh).  It fails if the biases
    are left out or added after the rotation, if the rotation's sign or pairing is another, if the
    scale is 1 / sqrt(hidden / heads) (the sizes differ here), if query head h reads kv head h % 2
    instead of h // 2, or if the blocks' norms stand elsewhere (src/llaisys/models/qwen2.cpp:613-629,
    :690; src/ops/rope/op.cpp:13-20; src/ops/paged_attention/op.cpp:20-42)."""
    cfg = {"num_hidden_layers": 1, "hidden_size": 20, "num_attention_heads": 4, "num_key_value_heads": 2,
           "head_dim": 6, "intermediate_size": 8, "vocab_size": 11, "rope_theta": 100.0, "rms_norm_eps": 1e-5,
           "tie_word_embeddings": True, "max_position_embeddings": 64}
    w = _tiny_weights(cfg, 5)
    pre = "model.layers.0."
    for n in ("q_proj.weight", "k_proj.weight"):
        w[pre + "self_attn." + n][:] = 0
    for n in ("q_proj.bias", "k_proj.bias", "v_proj.bias"):
        w[pre + "self_attn." + n] = RNG.standard_normal(w[pre + "self_attn." + n].shape)
    w[pre + "mlp.down_proj.weight"][:] = 0
    ids = [3, 9, 4, 4, 1]
    nh, nkv, dh, half = 4, 2, 6, 3
    E, eps = w["model.embed_tokens.weight"], cfg["rms_norm_eps"]
    x = E[ids]
    xn = w[pre + "input_layernorm.weight"] * x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)
    v = (xn @ w[pre + "self_attn.v_proj.weight"].T + w[pre + "self_attn.v_proj.bias"]).reshape(len(ids), nkv, dh)
    bq = w[pre + "self_attn.q_proj.bias"].reshape(nh, dh)
    bk = w[pre + "self_attn.k_proj.bias"].reshape(nkv, dh)
    zq, zk = bq[:, :half] + 1j * bq[:, half:], bk[:, :half] + 1j * bk[:, half:]
    angle = 100.0 ** (-2.0 * np.arange(half) / dh)

    def logits(kv_of_head):
        attn = np.zeros((len(ids), nh, dh))
        for h in range(nh):
            kh = kv_of_head(h)
            for p in range(len(ids)):
                s = np.array([(zq[h] * np.conj(zk[kh]) * np.exp(1j * (p - t) * angle)).real.sum() / math.sqrt(dh)
                              for t in range(p + 1)])
                pr = np.exp(s - s.max())
                attn[p, h] = (pr / pr.sum()) @ v[:p + 1, kh]
        y = x + attn.reshape(len(ids), nh * dh) @ w[pre + "self_attn.o_proj.weight"].T
        return w["model.norm.weight"] * y / np.sqrt((y * y).mean(-1, keepdims=True) + eps) @ E.T

    got = P.forward(cfg, w, ids)
    assert np.allclose(got, logits(lambda h: h // 2), atol=1e-12)
    assert not np.allclose(got, logits(lambda h: h % 2), atol=1e-6)          # interleaved heads would show
    no_bias = dict(w)
    no_bias[pre + "self_attn.q_proj.bias"] = np.zeros(nh * dh)
    assert not np.allclose(P.forward(cfg, no_bias, ids), got, atol=1e-6)      # the biases do act


def test_model_depends_on_distances_only():
    w = _tiny_weights(TINY_A, 2)
    ids = RNG.integers(0, 256, 20).tolist()
    assert np.allclose(P.forward(TINY_A, w, ids, start_pos=0), P.forward(TINY_A, w, ids, start_pos=37), atol=1e-10)


def test_window_changes_only_what_lies_beyond_it():
    w = _tiny_weights(TINY_B, 3)
    ids = RNG.integers(0, 320, 60).tolist()
    windowed = P.forward(TINY_B, w, ids)
    full = P.forward(dict(TINY_B, use_sliding_window=False), w, ids)
    assert np.allclose(windowed[:32], full[:32]) and not np.allclose(windowed[40:], full[40:])
    assert [P.layer_window(TINY_B, l) for l in range(3)] == [0, 32, 32]


def test_shared_cache_order():
    w = _tiny_weights(TINY_A, 4)
    ids = RNG.integers(0, 256, 9).tolist()
    plain = P.forward(TINY_A, w, ids)
    assert np.allclose(P.forward(TINY_A, w, ids, order=[(0, None), (1, None)]), plain)
    shared = P.forward(TINY_A, w, ids, order=[(0, None), (1, 0), (0, None)])
    assert shared.shape == plain.shape and not np.allclose(shared, plain)


def test_sampler_filters_and_limits():
    lg = np.array([2.0, 1.0, 3.0, 3.0, -1.0, 0.5, 2.5, 0.0])
    assert P.sample_with_uniform(lg, 0.0, 0, 1.0, 0.7) == 2                   # greedy: the first maximum
    assert P.sample_with_uniform(lg, 1e-4, 0, 1.0, 0.3) == 2                  # T -> 0+: the argmax ...
    assert P.sample_with_uniform(lg, 1e-4, 0, 1.0, 0.7) == 3                  # ... or its equal
    ids, p = P.sampling_candidates(lg, 1.0, 3, 1.0)
    assert ids.tolist() == [2, 3, 6] and np.isclose(p.sum(), 1)               # ties by ascending index
    ids, p = P.sampling_candidates(lg, 1.0, 0, 0.5)
    assert ids.tolist() == [2, 3]                                             # shortest prefix reaching 0.5
    ids, _ = P.sampling_candidates(lg, 1.0, 1, 0.99)
    assert ids.tolist() == [2]
    ids, p = P.sampling_candidates(lg, 2.0, 0, 1.0)
    assert np.allclose(p, np.exp(lg / 2) / np.exp(lg / 2).sum())
    # inverse CDF over ascending ids
    cum = np.cumsum(p)
    for u in (0.0, 0.2, 0.55, 0.999):
        assert P.sample_with_uniform(lg, 2.0, 0, 1.0, u) == int(np.searchsorted(cum, u))
    draws = [P.sample_with_uniform(lg, 1.0, 0, 1.0, u) for u in RNG.random(20000)]
    freq = np.bincount(draws, minlength=8) / 20000
    assert np.abs(freq - np.exp(lg) / np.exp(lg).sum()).max() < 0.01
