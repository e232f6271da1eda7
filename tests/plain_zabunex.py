"""A plain, slow Zabunex: every mechanism as one function of whole sequences, written
from the design's equations, sharing no code with the engine.  Everything is computed
in one floating-point type (float64 unless asked otherwise) on the CPU.

A model is ``(config, weights)``: the ``config.json`` as a dict and a dict of tensors
under the folder's own names.  Notation: ``T`` tokens of one sequence, positions
``0 .. T-1``; linear weights are ``[out, in]``.
"""

from __future__ import annotations

import json
import math
import os

import torch


# ---- small pieces ------------------------------------------------------------------------
def rms_norm(x, w, eps):
    """Rows of ``x`` divided by their root mean square (eps under the root), times ``w``."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w


def relu_squared(x):
    return torch.relu(x) ** 2


def softplus(x):
    return torch.log1p(torch.exp(-x.abs())) + torch.clamp(x, min=0)


def silu(x):
    return x * torch.sigmoid(x)


def distance_bucket(n: int, n_buckets: int, max_distance: int) -> int:
    """Row of the bias table for a key ``n`` tokens back: the first half of the rows is one
    distance each, the second half spaced evenly in the logarithm up to ``max_distance``."""
    half = n_buckets // 2
    if n < half:
        return n
    return min(n_buckets - 1, half + int(math.floor(math.log(n / half) / math.log(max_distance / half) * (n_buckets - half))))


def short_convolution(u, w, bias=None):
    """``y[t, c] = sum_j w[c, j] * u[t - taps + 1 + j, c]`` with zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    padded = torch.cat([u.new_zeros(taps - 1, C), u])
    y = u.new_zeros(T, C)
    for j in range(taps):
        y = y + padded[j : j + T] * w[:, j]
    return y if bias is None else y + bias


def rotate_leading(x, dims, base, factor):
    """``x`` [T, heads, size]: of every head the first ``dims`` entries are rotated, entry
    ``i`` with entry ``i + dims/2``, by the angle ``t * base^(-2i/dims) / factor``."""
    T = x.shape[0]
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) / factor for i in range(half)], dtype=x.dtype)
    angle = torch.arange(T, dtype=x.dtype)[:, None] * freq[None, :]
    c, s = angle.cos()[:, None, :], angle.sin()[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


def query_temperature(T, coef, every, dtype):
    p = torch.arange(T)
    return (1 + coef * torch.log((torch.div(p + 1, every, rounding_mode="floor") + 1).to(dtype))).to(dtype)


def attend(q, k, v, scale, visible, bias=None, sink=False):
    """``q`` [T, H, d], ``k`` [T, G, d], ``v`` [T, G, dv]; ``visible(i, j)`` for ``j <= i``;
    ``bias(i - j, head)`` is added to the scaled score; with ``sink`` the softmax has one
    more term of score 0 and no value.  Written key by key on purpose."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = q.new_zeros(T, H, v.shape[-1])
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            js = [j for j in range(i + 1) if visible(i, j)]
            s = torch.stack([(q[i, h] * k[j, g]).sum() * scale + (bias(i - j, h) if bias is not None else 0.0) for j in js])
            m = s.max()
            if sink:
                m = torch.clamp(m, min=0.0)
            e = torch.exp(s - m)
            denom = e.sum() + (torch.exp(-m) if sink else 0.0)
            w = e / denom
            out[i, h] = (w[:, None] * v[js, g]).sum(dim=0)
    return out


def attend_fast(q, k, v, scale, mask, bias=None, sink=False):
    """The same as ``attend`` with whole matrices: ``mask`` [T, T] bool, ``bias`` [H, T, T]."""
    T, H, _ = q.shape
    G = k.shape[1]
    kk = k.repeat_interleave(H // G, dim=1)
    vv = v.repeat_interleave(H // G, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, kk) * scale
    if bias is not None:
        s = s + bias
    s = s.masked_fill(~mask[None], float("-inf"))
    m = s.max(dim=-1, keepdim=True).values
    if sink:
        m = torch.clamp(m, min=0.0)
    e = torch.exp(s - m)
    denom = e.sum(dim=-1, keepdim=True)
    if sink:
        denom = denom + torch.exp(-m)
    return torch.einsum("hij,jhd->ihd", e / denom, vv)


# ---- mixers ------------------------------------------------------------------------------
def biased_attention(h, w, prefix, m, eps, fast=True):
    """The mixer 'attention': values are the keys before their norm, a norm over the whole
    of q and of k, a temperature on q, a bias by distance, a sink."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = h @ w[prefix + "q"].T
    k = h @ w[prefix + "k"].T
    v = k.view(T, G, m["vdim"])
    q = rms_norm(q, w[prefix + "q.norm"], eps)
    k = rms_norm(k, w[prefix + "k.norm"], eps).view(T, G, d)
    q = (q * query_temperature(T, m["q_temp"]["coef"], m["q_temp"]["every"], h.dtype)[:, None]).view(T, H, d)
    rel = w[prefix + "rel"]
    B, D = rel.shape[0], m["bias_max"]
    if fast:
        idx = torch.tensor([[distance_bucket(i - j, B, D) if j <= i else 0 for j in range(T)] for i in range(T)])
        bias = rel[idx].permute(2, 0, 1)  # [H, T, T]
        mask = torch.ones(T, T, dtype=torch.bool).tril()
        o = attend_fast(q, k, v, m["scale"], mask, bias, sink=True)
    else:
        o = attend(q, k, v, m["scale"], lambda i, j: True, lambda n, hh: rel[distance_bucket(n, B, D), hh], sink=True)
    return o.reshape(T, -1) @ w[prefix + "o"].T


def chunked_attention(h, w, prefix, m, eps, fast=True):
    """The left half of 'parallel': short convolutions on q, k, v, the whole-projection
    norms, a rotation of the leading entries with stretched positions, keys of the query's
    own chunk only."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_convolution(h @ w[prefix + "q"].T, w[prefix + "q.conv"])
    k = short_convolution(h @ w[prefix + "k"].T, w[prefix + "k.conv"])
    v = short_convolution(h @ w[prefix + "v"].T, w[prefix + "v.conv"])
    q = rms_norm(q, w[prefix + "q.norm"], eps).view(T, H, d)
    k = rms_norm(k, w[prefix + "k.norm"], eps).view(T, G, d)
    rot = m["rot"]
    q = rotate_leading(q, rot["dims"], rot["base"], rot["scaling"]["factor"])
    k = rotate_leading(k, rot["dims"], rot["base"], rot["scaling"]["factor"])
    size = m["mask"]["size"]
    if fast:
        i = torch.arange(T)
        mask = (i[None, :] <= i[:, None]) & ((i[None, :] // size) == (i[:, None] // size))
        o = attend_fast(q, k, v.view(T, G, dv), m["scale"], mask)
    else:
        o = attend(q, k, v.view(T, G, dv), m["scale"], lambda a, b: a // size == b // size)
    return o.reshape(T, -1) @ w[prefix + "o"].T


def selective_scan(x, Bm, Cm, dt_raw, dt_bias, a_log, skip, S=None):
    """``x`` [T, heads, P], ``Bm``, ``Cm`` [T, G, N], ``dt_raw`` [T, heads]; token by token
    ``S <- exp(-exp(a_log) dt) S + dt B x^T`` and ``y = S^T C + skip x`` with
    ``dt = softplus(dt_raw + dt_bias)``.  Returns ``y`` and the last state [heads, N, P]."""
    T, heads, P = x.shape
    G, N = Bm.shape[1:]
    dt = softplus(dt_raw + dt_bias)
    rate = torch.exp(a_log)
    S = x.new_zeros(heads, N, P) if S is None else S.clone()
    y = x.new_zeros(T, heads, P)
    for t in range(T):
        for hd in range(heads):
            g = hd // (heads // G)
            S[hd] = torch.exp(-rate[hd] * dt[t, hd]) * S[hd] + dt[t, hd] * torch.outer(Bm[t, g], x[t, hd])
            y[t, hd] = S[hd].T @ Cm[t, g] + skip[hd] * x[t, hd]
    return y, S


def gated_part_norm(y, z, w, eps, parts):
    """``y * silu(z)``, then every one of ``parts`` equal parts of a row divided by its own
    root mean square, times ``w``."""
    T, n = y.shape
    y = (y * silu(z)).view(T, parts, n // parts)
    y = y / torch.sqrt((y * y).mean(dim=-1, keepdim=True) + eps)
    return y.reshape(T, n) * w


def state_space(h, w, prefix, m, eps):
    """The right half of 'parallel': a selective state-space recurrence with scalar decay a
    head."""
    T = h.shape[0]
    heads, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = heads * P
    a = h @ w[prefix + "in"].T
    z, xbc, dt = a[:, :inner], a[:, inner : 2 * inner + 2 * G * N], a[:, 2 * inner + 2 * G * N :]
    xbc = silu(short_convolution(xbc, w[prefix + "conv"], w[prefix + "conv.b"]))
    x = xbc[:, :inner].view(T, heads, P)
    Bm = xbc[:, inner : inner + G * N].view(T, G, N)
    Cm = xbc[:, inner + G * N :].view(T, G, N)
    y, _ = selective_scan(x, Bm, Cm, dt, w[prefix + "dt_bias"], w[prefix + "A_log"], w[prefix + "D"])
    y = gated_part_norm(y.reshape(T, inner), z, w[prefix + "norm"], eps, m["norm_groups"])
    return y @ w[prefix + "o"].T


def parallel_mixer(h, w, prefix, m, eps, fast=True):
    left = chunked_attention(h, w, prefix + "left.", m["left"], eps, fast)
    right = state_space(h, w, prefix + "right.", m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def dense_feed_forward(h, w, prefix):
    return relu_squared(h @ w[prefix + "up"].T) @ w[prefix + "down"].T


# ---- the model ---------------------------------------------------------------------------
def forward(config, weights, tokens, dtype=torch.float64, fast=True, layers_out=None):
    """Logits [T, vocab] of one sequence; ``layers_out`` (a list) receives the stream after
    every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        if layer["type"] == "attention":
            a = biased_attention(x, w, p + "mix.", layer["mixer"], eps, fast)
        elif layer["type"] == "parallel":
            a = parallel_mixer(x, w, p + "mix.", layer["mixer"], eps, fast)
        else:
            raise ValueError(f"layer {i}: unknown type {layer['type']!r}")
        x = x + rms_norm(a, w[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward {layer['mlp']['kind']!r}")
            x = x + rms_norm(dense_feed_forward(x, w, p + "mlp."), w[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T


def read_model_folder(folder):
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    return config, load_file(os.path.join(folder, "model.safetensors"))


# ---- small models of the tests' own ----------------------------------------------------------
def attention_layer(heads, kv_heads, dim, scale, bias_max, coef, every, ff=None):
    return dict(type="attention",
                mixer=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=scale, bias_max=bias_max,
                           q_temp=dict(coef=coef, every=every)),
                mlp=None if ff is None else dict(kind="dense", ff=ff))


def parallel_layer(left, right, left_scale, right_scale, ff=None):
    return dict(type="parallel", mixer=dict(left=left, right=right, left_scale=left_scale, right_scale=right_scale),
                mlp=None if ff is None else dict(kind="dense", ff=ff))


def left_cfg(heads, kv_heads, dim, vdim, scale, conv, chunk, rot_dims, base=10000.0, factor=1.0):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, conv=conv, mask=dict(size=chunk),
                rot=dict(base=base, dims=rot_dims, scaling=dict(factor=factor)))


def right_cfg(heads, vdim, state, groups, conv, norm_groups):
    return dict(heads=heads, vdim=vdim, state=state, groups=groups, conv=conv, norm_groups=norm_groups)


def model_cfg(width, vocab, layers, eps=1e-5):
    return dict(architecture="Zabunex", vocab=vocab, width=width, norm=dict(eps=eps), layers=layers)


def tensor_shapes(cfg, bias_rows):
    """Name -> shape of every tensor of a folder; ``bias_rows[i]``: rows of layer i's bias table."""
    d = cfg["width"]
    out = {"embed": (cfg["vocab"], d)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (d,)
        out[p + "norm2"] = (d,)
        if layer["type"] == "attention":
            nq, nk = m["heads"] * m["dim"], m["kv_heads"] * m["dim"]
            out.update({p + "mix.q": (nq, d), p + "mix.k": (nk, d), p + "mix.q.norm": (nq,), p + "mix.k.norm": (nk,),
                        p + "mix.rel": (bias_rows[i], m["heads"]), p + "mix.o": (d, m["heads"] * m["vdim"])})
        else:
            l, r = m["left"], m["right"]
            nq, nk, nv = l["heads"] * l["dim"], l["kv_heads"] * l["dim"], l["kv_heads"] * l["vdim"]
            q = p + "mix.left."
            out.update({q + "q": (nq, d), q + "k": (nk, d), q + "v": (nv, d), q + "q.norm": (nq,), q + "k.norm": (nk,),
                        q + "q.conv": (nq, l["conv"]), q + "k.conv": (nk, l["conv"]), q + "v.conv": (nv, l["conv"]),
                        q + "o": (d, l["heads"] * l["vdim"])})
            inner, gn = r["heads"] * r["vdim"], r["groups"] * r["state"]
            q = p + "mix.right."
            out.update({q + "in": (2 * inner + 2 * gn + r["heads"], d), q + "conv": (inner + 2 * gn, r["conv"]),
                        q + "conv.b": (inner + 2 * gn,), q + "dt_bias": (r["heads"],), q + "A_log": (r["heads"],),
                        q + "D": (r["heads"],), q + "norm": (inner,), q + "o": (d, inner)})
        if layer.get("mlp") is not None:
            out[p + "mlp.up"] = (layer["mlp"]["ff"], d)
            out[p + "mlp.down"] = (d, layer["mlp"]["ff"])
    out["final.norm"] = (d,)
    out["head"] = (cfg["vocab"], d)
    return out


def random_weights(cfg, bias_rows, seed, std=0.12, stored=torch.bfloat16):
    """Matrices N(0, std), norm weights around 1, bias tables and convolutions of a size that
    counts, decays and step sizes spread over a range; rounded to ``stored`` so that engine
    and plain model hold the same numbers."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg, bias_rows).items():
        last = name.rsplit(".", 1)[-1]
        if last == "rel":
            t = 1.5 * torch.randn(shape, generator=gen)
        elif last == "conv":
            t = 0.5 * torch.randn(shape, generator=gen)
        elif last in ("b", "dt_bias"):
            t = 0.5 * torch.randn(shape, generator=gen)
        elif last == "A_log":
            t = torch.rand(shape, generator=gen) * 2.0 - 2.0
        elif len(shape) == 1:
            t = 1.0 + 0.2 * torch.randn(shape, generator=gen)
        else:
            t = std * torch.randn(shape, generator=gen)
        out[name] = t.to(stored).float()
    return out


def write_model_folder(folder, cfg, weights, dtype=torch.bfloat16):
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(dtype).contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return folder


# equal layers of each kind, grouped heads everywhere
ZAB_A = model_cfg(64, 331, [
    attention_layer(4, 2, 16, 0.25, 40, 0.3, 16, ff=96),
    parallel_layer(left_cfg(4, 2, 16, 16, 0.25, 3, 24, 8, factor=2.0), right_cfg(4, 16, 16, 2, 4, 2), 0.7, 1.2, ff=80),
    attention_layer(4, 2, 16, 0.25, 40, 0.3, 16, ff=96),
])
ZAB_A_BIAS = {0: 12, 2: 12}
# the recurrent layer first; value heads of another size than the keys', one group, one
# norm part, a temperature that changes with every position, chunks shorter than a page, a
# rotation of the whole head without stretching, a layer without a feed-forward
ZAB_B = model_cfg(48, 257, [
    parallel_layer(left_cfg(2, 1, 24, 8, 0.2, 2, 7, 24, base=500.0), right_cfg(3, 8, 8, 1, 2, 1), 1.0, -0.5),
    attention_layer(6, 2, 8, 0.35, 17, -0.2, 1, ff=64),
    parallel_layer(left_cfg(4, 4, 8, 24, 0.3, 4, 33, 2, factor=4.0), right_cfg(2, 24, 16, 2, 3, 4), 0.4, 0.9, ff=40),
])
ZAB_B_BIAS = {1: 10}
# sizes that are multiples of little: head sizes that pages pad, a state of 24 numbers, a
# convolution of one tap and one of five, a chunk of exactly a page, a single bias row per
# distance up to the table's half
ZAB_C = model_cfg(40, 199, [
    attention_layer(3, 3, 20, 0.22, 100, 0.45, 48, ff=52),
    parallel_layer(left_cfg(3, 3, 12, 20, 0.29, 5, 16, 4, base=2.0e5, factor=6.0), right_cfg(5, 12, 24, 5, 1, 3), 0.55, 1.25, ff=36),
    attention_layer(2, 1, 12, 0.3, 9, 0.0, 5),
])
ZAB_C_BIAS = {0: 6, 2: 16}
