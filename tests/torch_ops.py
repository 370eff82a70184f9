"""A stand-in for the HIP kernels, written with torch on the CPU, for tests
that check the engine's bookkeeping (batches, pages, block tables, schedules)
where there is no GPU.  It is a test double: the package has no CPU path, and
the tests patch these functions over `litinfer_amd.kernels.ops` themselves.
Each function follows the documented contract of the kernel it stands for,
with the cache addressed through the block table exactly as on the device."""
from __future__ import annotations

import math

import torch


def require_gpu(device):
    return None


def embedding(ids, table, out, id_src=None, feedback=None):
    ids = ids.long()
    if id_src is not None:
        ids = torch.where(id_src >= 0, feedback.long()[id_src.clamp(min=0).long()], ids)
    out.copy_(table[ids].float())


def rmsnorm(x, weight, eps, out):
    xf = x.float()
    inv = torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps)
    out.copy_((weight * xf * inv).to(out.dtype))


def gather_rows(x, rows, out):
    out.copy_(x[rows.long()])


def cast(src, dst):
    dst.copy_(src.view(dst.shape).to(dst.dtype))


def swiglu(gate_up, out):
    inter = out.shape[1]
    g, u = gate_up[:, :inter].float(), gate_up[:, inter:].float()
    out.copy_((u * (g / (1 + torch.exp(-g)))).to(out.dtype))


def rope_table(positions, theta, rotary_dim, cos, sin):
    j = torch.arange(rotary_dim // 2, dtype=torch.float32)
    ang = positions.float()[:, None] / torch.pow(torch.tensor(theta, dtype=torch.float32),
                                                  2 * j / rotary_dim)
    cos.copy_(torch.cos(ang))
    sin.copy_(torch.sin(ang))


def rope_apply(qkv, n_heads, head_dim, rotary_dim, cos, sin):
    t = qkv.shape[0]
    x = qkv[:, :n_heads * head_dim].reshape(t, n_heads, head_dim).float().clone()
    half = rotary_dim // 2
    a, b = x[..., :half].clone(), x[..., half:rotary_dim].clone()
    c, s = cos[:, None, :], sin[:, None, :]
    x[..., :half] = a * c - b * s
    x[..., half:rotary_dim] = b * c + a * s
    qkv[:, :n_heads * head_dim] = x.reshape(t, -1).to(qkv.dtype)


def kv_store(qkv, nh, nkv, dh, slot_map, k, v, page_size):
    t = qkv.shape[0]
    kk = qkv[:, nh * dh:(nh + nkv) * dh].reshape(t, nkv, dh)
    vv = qkv[:, (nh + nkv) * dh:(nh + 2 * nkv) * dh].reshape(t, nkv, dh)
    page = (slot_map // page_size).long()
    off = (slot_map % page_size).long()
    k[page, :, off, :] = kk
    v[page, :, off, :] = vv


def rope_kv_store(qkv, nh, nkv, dh, rotary_dim, cos, sin, slot_map, k, v, page_size):
    rope_apply(qkv, nh + nkv, dh, rotary_dim, cos, sin)
    kv_store(qkv, nh, nkv, dh, slot_map, k, v, page_size)


def linear(x, w, bias, out, accumulate=False, ws=None):
    y = x.float() @ w.float().T
    if bias is not None:
        y = y + bias
    if accumulate:
        out += y
    else:
        out.copy_(y.to(out.dtype))


def linear_skinny(x, w, bias, out, accumulate=False, swiglu=False):
    y = x.float() @ w.float().T
    if swiglu:
        n = out.shape[1]
        g, u = y[:, :n], y[:, n:]
        out.copy_((u * (g / (1 + torch.exp(-g)))).to(out.dtype))
        return
    if bias is not None:
        y = y + bias
    if accumulate:
        out += y
    else:
        out.copy_(y.to(out.dtype))


def check_attention_sizes(num_heads, num_kv_heads, head_dim):
    assert num_heads % num_kv_heads == 0 and head_dim % 2 == 0


def paged_attention(qkv, out, k, v, meta, nh, nkv, dh, page_size, window, scale, ws=None):
    g = nh // nkv
    for s in range(meta.num_segments):
        q0, ql, cl = int(meta.host_q_start[s]), int(meta.host_q_len[s]), int(meta.host_ctx_len[s])
        table = meta.block_table[s].long()
        for i in range(ql):
            p = cl - ql + i
            lo = max(0, p - window + 1) if window > 0 else 0
            pos = torch.arange(lo, p + 1)
            pages = table[pos // page_size]
            assert (pages >= 0).all(), "attention addressed a page that was given back"
            off = pos % page_size
            for h in range(nh):
                kh = h // g
                qv = qkv[q0 + i, h * dh:(h + 1) * dh].float()
                kk = k[pages, kh, off, :].float()
                vv = v[pages, kh, off, :].float()
                sc = (kk @ qv) * scale
                w = torch.softmax(sc, dim=0)
                out[q0 + i, h * dh:(h + 1) * dh] = (w @ vv).to(out.dtype)


def swiglu_takes(m, k, w_dtype):
    return w_dtype is torch.bfloat16 and m > 0 and (k % 8 == 0 if m <= 64 else k % 64 == 0)


RESIDUAL_NORM_MAX_PARTS = 512


class RowScale:
    def __init__(self, sq_parts, nparts, eps):
        self.sq_parts, self.nparts, self.eps = sq_parts, int(nparts), float(eps)


def residual_norm_parts(n):
    return -(-n // (32 if n >= 8192 else 16))


def few_rows_preferred(m, n, k):
    if m <= 12 or (m <= 16 and n * k * 2 < (100 << 20)):
        return True
    return m <= 32 and k % 8 == 0 and n * k * 2 <= (56 << 20) and (k <= 4096 or n * k * 2 <= (32 << 20))


def residual_norm_takes(m, n, k, w_dtype):
    return w_dtype is torch.bfloat16 and 0 < m <= 32 and k % 8 == 0 and residual_norm_parts(n) <= RESIDUAL_NORM_MAX_PARTS


def linear_residual_norm(x, w, bias, out, gamma, xg, sq_parts):
    linear(x, w, bias, out, True)
    xg.copy_((gamma * out).to(xg.dtype))
    per = 32 if out.shape[1] >= 8192 else 16
    parts = residual_norm_parts(out.shape[1])
    r = 16 if out.shape[0] <= 16 else 32
    for p in range(parts):                               # one share a block of columns, 16 places each (32 above 16 rows)
        sq_parts[p * r:p * r + out.shape[0]] = (out[:, p * per:(p + 1) * per] ** 2).sum(dim=1)
    return parts


def linear_then_norm(x, w, bias, out, gamma, eps, xn, ws):
    return False                                         # the stand-ins cut no product along K


def _row_factors(row_scale, m, k):
    r = 16 if m <= 16 else 32
    sq = row_scale.sq_parts[:row_scale.nparts * r].view(row_scale.nparts, r)[:, :m].sum(dim=0)
    return (1.0 / torch.sqrt(sq / k + row_scale.eps))[:, None]


def linear_swiglu(x, w, out, row_scale=None):
    if row_scale is None:
        return linear_skinny(x, w, None, out, False, swiglu=True)
    y = (x.float() @ w.float().T) * _row_factors(row_scale, x.shape[0], x.shape[1])
    n = out.shape[1]
    g, u = y[:, :n], y[:, n:]
    out.copy_((u * (g / (1 + torch.exp(-g)))).to(out.dtype))


def rope_store_takes(m, k, w_dtype, dh, rotary_dim):
    return w_dtype is torch.bfloat16 and 0 < m <= 32 and k % 8 == 0 and dh % 16 == 0 and rotary_dim == dh


def linear_rope_store_parts(*args, **kwargs):
    return False                 # (the stand-in never cuts a product along K)


def linear_rope_store(x, w, bias, out, nh, nkv, dh, cos, sin, slot_map, k, v, page_size, row_scale=None):
    y = x.float() @ w.float().T
    if row_scale is not None:
        y = y * _row_factors(row_scale, x.shape[0], x.shape[1])
    if bias is not None:
        y = y + bias
    # rotated from the 32-bit sums and rounded once, as the fused kernel does
    t = y.shape[0]
    heads = y.view(t, nh + 2 * nkv, dh)
    rot = heads[:, :nh + nkv]
    a, b = rot[..., :dh // 2].clone(), rot[..., dh // 2:].clone()
    c, s = cos[:, None, :], sin[:, None, :]
    rot[..., :dh // 2], rot[..., dh // 2:] = a * c - b * s, b * c + a * s
    out.copy_(y.to(out.dtype))
    kv_store(out, nh, nkv, dh, slot_map, k, v, page_size)


def argmax_rows(logits, out):
    out.copy_(torch.argmax(logits, dim=-1).to(torch.int32))


ALL = ["require_gpu", "embedding", "rmsnorm", "gather_rows", "cast", "swiglu", "rope_table",
       "rope_apply", "kv_store", "rope_kv_store", "linear", "linear_skinny", "swiglu_takes", "linear_swiglu", "rope_store_takes", "linear_rope_store", "linear_rope_store_parts", "check_attention_sizes",
       "RowScale", "few_rows_preferred", "RESIDUAL_NORM_MAX_PARTS", "residual_norm_parts", "residual_norm_takes", "linear_residual_norm", "linear_then_norm",
       "paged_attention", "argmax_rows"]


def sample_rows(logits, temperature, top_k, top_p, uniform, out):
    import numpy as np
    lg = logits.double().numpy()
    for r in range(lg.shape[0]):
        t = float(temperature[r])
        if not t > 0:
            out[r] = int(np.argmax(lg[r]))
            continue
        z = lg[r] / t
        order = np.lexsort((np.arange(z.size), -z))
        k, p = int(top_k[r]), float(top_p[r])
        if 0 < k < z.size:
            order = order[:k]
        if 0 < p < 1:
            e = np.exp(z[order] - z[order[0]])
            cum = np.cumsum(e / e.sum())
            order = order[:int(np.argmax(cum >= p)) + 1] if (cum >= p).any() else order
        keep = np.sort(order)
        e = np.exp(z[keep] - z[keep].max())
        cum = np.cumsum(e)
        i = int(np.searchsorted(cum, float(uniform[r]) * cum[-1], side="left"))
        out[r] = int(keep[min(i, keep.size - 1)])


ALL.append("sample_rows")


def sample_prepare(rows, table, temperature, top_k, top_p, uniform):
    """The device's per-slot sampling table (csrc/sampling.hip, sample_prepare_kernel) written out on the host."""
    import numpy as np
    from litinfer_amd.sampling import uniform as stream_uniform
    nslots = table.shape[0]
    for i, word in enumerate(rows.tolist()):
        slot, flags = word & 0xffffff, (word >> 24) & 0x7f
        t, p, k, u = 0.0, 1.0, 0, 0.0
        if slot < nslots and not flags & 1:
            row = table[slot]
            t = float(row[0:1].view(torch.float32))
            p = float(row[1:2].view(torch.float32))
            k = int(row[2])
            if t > 0:
                seed = (int(row[3]) & 0xffffffff) | ((int(row[4]) & 0xffffffff) << 32)
                u = stream_uniform(seed, int(row[5]) & 0xffffffff)
                row[5] += 1
            else:
                t = 0.0
        temperature[i], top_k[i], top_p[i], uniform[i] = t, k, p, u


ALL.append("sample_prepare")
