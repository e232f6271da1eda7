"""A plain, slow Kavuvik on the CPU: one function per mechanism, written from the design's
equations with nothing of the framework.  Keys and values of every head are made
explicitly from the latent (no algebraic shortcut), the experts run token by token, and
everything is float64 unless ``round_to`` asks for the roundings of a 16-bit engine.

Notation: ``x`` the stream, ``h`` a normed input, ``c`` a latent, ``r`` the shared rotated
key part, ``H`` heads, ``dn`` / ``dr`` / ``dv`` the unrotated, rotated and value sizes.
"""

import json
import os

import torch

F = torch.float64


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def rotate_pairs(x, positions, base, dims):
    """Rotates the first ``dims`` entries of the last axis: entry i with entry i + dims/2
    by the angle position * base^(-2i/dims); the rest passes."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    angle = positions.to(F)[:, None] * freq[None, :]
    cos, sin = torch.cos(angle), torch.sin(angle)
    for _ in range(x.dim() - 2):
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat((u * cos - v * sin, v * cos + u * sin, x[..., dims:]), dim=-1)


def visible(n, window):
    """[query, key] booleans: key j is seen from i if 0 <= i - j (< window)."""
    i = torch.arange(n)
    gap = i[:, None] - i[None, :]
    ok = gap >= 0
    if window is not None:
        ok &= gap < window
    return ok


def latent_attention(h, w, m, eps, positions, rnd=lambda t: t):
    """``w``: the mixer's tensors by their short names; ``m``: the mixer's config dict."""
    n = h.shape[0]
    H, dn, dr, dv, kr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rnd(rms_norm(h @ w["dq"].T, w["dq.norm"], eps))
    q = rnd(cq @ w["uq"].T).view(n, H, dn + dr)
    down = h @ w["dkv"].T
    c = rnd(rms_norm(down[:, :kr], w["dkv.norm"], eps))
    r = rnd(down[:, kr:])
    keys = (c @ w["uk"].T).view(n, H, dn)
    values = (c @ w["uv"].T).view(n, H, dv)
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    q_rot = rnd(rotate_pairs(q[..., dn:], positions, base, dims))
    r_rot = rnd(rotate_pairs(r, positions, base, dims))
    window = m["mask"]["size"] if m.get("mask") else None
    ok = visible(n, window)
    out = torch.zeros(n, H, dv, dtype=F)
    for head in range(H):
        score = (q[:, head, :dn] @ keys[:, head].T + q_rot[:, head] @ r_rot.T) * m["scale"]
        score = score.masked_fill(~ok, float("-inf"))
        out[:, head] = torch.softmax(score, dim=-1) @ values[:, head]
    out = rnd(rnd(out.reshape(n, H * dv)) * torch.sigmoid(h @ w["g"].T))
    return out @ w["o"].T


def route(h, w_router, top):
    """Chosen experts [n, top] and their weights: sigmoid scores, the largest ``top``,
    divided by their sum."""
    score = torch.sigmoid(h @ w_router.T)
    chosen_score, chosen = torch.topk(score, top, dim=-1)
    return chosen, chosen_score / (chosen_score.sum(-1, keepdim=True) + 1e-20)


def clamped_expert(h, gate, up, down, limit, rnd=lambda t: t):
    g = torch.clamp(h @ gate.T, max=limit)
    u = torch.clamp(h @ up.T, min=-limit, max=limit)
    return rnd(g * torch.sigmoid(1.702 * g) * (u + 1)) @ down.T


def mixture(h, w, f, rnd=lambda t: t):
    """``w``: the feed-forward's tensors by short name (``e3.gate`` ...); ``f``: its config."""
    chosen, weight = route(h, w["router"], f["router"]["top"])
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for j in range(chosen.shape[1]):
            e = int(chosen[t, j])
            out[t] += weight[t, j] * clamped_expert(h[t : t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"],
                                                    f["expert"]["limit"], rnd)[0]
    if f.get("shared"):
        out = out + clamped_expert(h, w["shared.gate"], w["shared.up"], w["shared.down"], f["shared"]["limit"], rnd)
    return out


def part(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, ids, round_to=None, stream_after=None):
    """Logits [len(ids), vocab] (float64).  ``round_to``: a 16-bit type whose roundings of
    normed inputs, projections and activations are imitated; ``stream_after``: a list that
    receives the stream after every layer."""
    rnd = (lambda t: t.to(round_to).to(F)) if round_to is not None else (lambda t: t)
    W = {k: v.to(F) for k, v in weights.items()}
    ids = torch.as_tensor(ids)
    positions = torch.arange(len(ids))
    eps = cfg["norm"]["eps"]
    x = W["embed"][ids] * cfg["embedding"]["scale"]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        delta = latent_attention(rnd(rms_norm(x, W[p + "norm1"], eps)), part(W, p + "mix."), layer["mixer"], eps, positions, rnd)
        if layer.get("mlp"):
            delta = delta + mixture(rnd(rms_norm(x, W[p + "norm2"], eps)), part(W, p + "mlp."), layer["mlp"], rnd)
        x = x + delta
        if stream_after is not None:
            stream_after.append(x.clone())
    return rnd(rms_norm(x, W["final.norm"], eps)) @ W["head"].T * cfg["logit_scale"]


# -- tensors and folders ------------------------------------------------------------------


def tensor_shapes(cfg):
    d, v = cfg["width"], cfg["vocab"]
    shapes = {"embed": (v, d), "final.norm": (d,), "head": (v, d)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
        shapes[p + "norm1"] = (d,)
        shapes[p + "mix.dq"] = (m["q_rank"], d)
        shapes[p + "mix.dq.norm"] = (m["q_rank"],)
        shapes[p + "mix.uq"] = (H * (dn + dr), m["q_rank"])
        shapes[p + "mix.dkv"] = (m["kv_rank"] + dr, d)
        shapes[p + "mix.dkv.norm"] = (m["kv_rank"],)
        shapes[p + "mix.uk"] = (H * dn, m["kv_rank"])
        shapes[p + "mix.uv"] = (H * dv, m["kv_rank"])
        shapes[p + "mix.g"] = (H * dv, d)
        shapes[p + "mix.o"] = (d, H * dv)
        f = layer.get("mlp")
        if not f:
            continue
        shapes[p + "norm2"] = (d,)
        shapes[p + "mlp.router"] = (f["router"]["experts"], d)
        names = [f"e{e}" for e in range(f["router"]["experts"])] + (["shared"] if f.get("shared") else [])
        for name in names:
            ff = f["shared"]["ff"] if name == "shared" else f["expert"]["ff"]
            shapes[p + f"mlp.{name}.gate"] = (ff, d)
            shapes[p + f"mlp.{name}.up"] = (ff, d)
            shapes[p + f"mlp.{name}.down"] = (d, ff)
    return shapes


def random_weights(cfg, seed, std=0.08, stored=torch.bfloat16):
    """N(0, std) matrices (the routers wider, so that choices are not close calls), norm
    weights around 1; rounded to ``stored`` so that engine and plain model hold the same numbers."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if len(shape) == 1:
            t = 1.0 + 0.1 * torch.randn(shape, generator=gen)
        else:
            t = (0.5 if name.endswith("router") else std) * torch.randn(shape, generator=gen)
        out[name] = t.to(stored).float()
    return out


def write_model_folder(folder, cfg, weights, dtype=torch.bfloat16):
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(dtype).contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def mixer_cfg(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base=10000.0, dims=None, window=None):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank, scale=scale,
             rot=dict(base=base, dims=rot_dim if dims is None else dims))
    if window is not None:
        m["mask"] = dict(size=window)
    return m


def moe_cfg(experts, top, ff, limit, shared_ff=None, shared_limit=None):
    f = dict(kind="moe", router=dict(experts=experts, top=top), expert=dict(ff=ff, limit=limit))
    if shared_ff is not None:
        f["shared"] = dict(ff=shared_ff, limit=shared_limit)
    return f


def model_cfg(width, vocab, layers, embedding_scale=1.0, logit_scale=1.0, eps=1e-5):
    return dict(architecture="Kavuvik", vocab=vocab, width=width, embedding=dict(scale=embedding_scale),
                norm=dict(eps=eps), logit_scale=logit_scale,
                layers=[dict(type="latent_attention", mixer=m, mlp=f) for m, f in layers])


# two equal layers; a window shorter than a page and a half
KAV_A = model_cfg(64, 97, [
    (mixer_cfg(2, 16, 16, 24, 40, 32, 0.2, window=20), moe_cfg(5, 2, 24, 0.7, 40, 1.5)),
    (mixer_cfg(2, 16, 16, 24, 40, 32, 0.2, window=20), moe_cfg(5, 2, 24, 0.7, 40, 1.5)),
], embedding_scale=2.0, logit_scale=0.5)

# three layers that differ in everything: no window and no feed-forward; one head, a part of
# the rotated dimensions rotating, one expert a token and no shared one; all experts chosen
KAV_B = model_cfg(80, 131, [
    (mixer_cfg(3, 8, 8, 8, 16, 24, 0.3, base=500.0, dims=4), None),
    (mixer_cfg(1, 32, 16, 16, 24, 48, 0.15, window=33), moe_cfg(4, 1, 16, 2.0)),
    (mixer_cfg(4, 16, 32, 8, 48, 16, 0.25, base=50000.0, window=7), moe_cfg(3, 3, 32, 0.5, 8, 0.25)),
], embedding_scale=1.0, logit_scale=3.0, eps=1e-6)

# sizes that are multiples of nothing
KAV_C = model_cfg(36, 53, [
    (mixer_cfg(3, 10, 6, 6, 12, 20, 0.4, dims=6, window=70), moe_cfg(7, 3, 10, 1.0, 14, 1.0)),
    (mixer_cfg(5, 6, 2, 10, 18, 9, 0.4, dims=2), moe_cfg(2, 1, 6, 3.0, 6, 0.1)),
], embedding_scale=0.5, logit_scale=1.5)
