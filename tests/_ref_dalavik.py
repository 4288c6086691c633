"""A plain, slow implementation of the Dalavik design in float64: whole sequences, dense masks,
one function per mechanism.  It shares no code with ``lumen``; the tests compare the framework's
kernels and engine with it.

Weights are a dict {checkpoint tensor name: tensor}; the configuration is the checkpoint's
``config.json`` as a dict.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x, w, groups, eps):
    """The last axis in ``groups`` equal consecutive parts, each divided by its own RMS; then w."""
    shp = x.shape
    y = rms_unit(x.reshape(*shp[:-1], groups, shp[-1] // groups), eps).reshape(shp)
    return y * w


def rotate_pairs(x, pos, dims, base):
    """Interleaved rotary on the first ``dims`` entries of the last axis: (x[2i], x[2i+1]) turns
    by the angle pos * base^(-2i / dims).  x [T, ..., n], pos [T]."""
    out = x.clone()
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = pos.to(F64).view(-1, *([1] * (x.dim() - 1))) * f
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * torch.cos(a) - v * torch.sin(a)
    out[..., 1:dims:2] = v * torch.cos(a) + u * torch.sin(a)
    return out


def dense_ff(h, w, p):
    return (torch.relu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def token_side(x, tokens, w, layer, dim, eps):
    """Per-layer token input: a slice of a second embedding, gated by the stream."""
    p = f"l{layer}.side."
    e = w["side.embed"][tokens][:, layer * dim:(layer + 1) * dim]
    g = gelu_tanh(x @ w[p + "gate"].T) * e
    y = g @ w[p + "proj"].T
    return x + rms_unit(y, eps) * w[p + "norm"]


def latent_kv(h, w, p, m, eps, pos):
    """The cached pair of a latent-attention layer: the normed latent and the rotated shared key."""
    R = m["kv_rank"]
    z = h @ w[p + "dkv"].T
    c = rms_unit(z[:, :R], eps) * w[p + "dkv.norm"]
    kr = rotate_pairs(z[:, R:], pos, m["rot"]["dims"], m["rot"]["base"])
    return c, kr


def latent_attention(h, w, p, m, eps, pos, kv):
    """kv = (c [T, R], kr [T, rot_dim]) of this layer or of the layer it borrows from."""
    T = h.shape[0]
    H, D, Dr, Dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, kr = kv
    cq = rms_unit(h @ w[p + "dq"].T, eps) * w[p + "dq.norm"]
    q = (cq @ w[p + "uq"].T).view(T, H, D + Dr)
    qn = q[..., :D]
    qr = rotate_pairs(q[..., D:], pos, m["rot"]["dims"], m["rot"]["base"])
    k = (c @ w[p + "uk"].T).view(T, H, D)
    v = (c @ w[p + "uv"].T).view(T, H, Dv)
    s = (torch.einsum("ihd,jhd->hij", qn, k) + torch.einsum("ihd,jd->hij", qr, kr)) * m["scale"]
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    s = s.masked_fill(~mask, -math.inf)
    a = torch.softmax(s, -1)
    o = torch.einsum("hij,jhd->ihd", a, v).reshape(T, H * Dv)
    return o @ w[p + "o"].T


def talking_attention(h, w, p, m, eps, pos):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, D)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, D)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, Dv)
    q = rms_unit(q, eps) * w[p + "q.norm"]
    k = rms_unit(k, eps) * w[p + "k.norm"]
    qt = m.get("q_temp")
    if qt:
        temp = 1.0 + qt["coef"] * torch.log(torch.floor((pos.to(F64) + 1) / qt["every"]) + 1.0)
        q = q * temp.view(T, 1, 1)
    rep = H // G
    k = k.repeat_interleave(rep, 1)
    v = v.repeat_interleave(rep, 1)
    s = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    cap = m.get("softcap")
    if cap:
        s = cap * torch.tanh(s / cap)
    dist = (pos.view(T, 1) - pos.view(1, T)).clamp(min=0).to(F64)
    s = s - w[p + "r1"].view(H, 1, 1) * torch.log(1.0 + w[p + "r2"].view(H, 1, 1) * dist)
    s = torch.einsum("hg,gij->hij", w[p + "talk"], s)
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    s = s.masked_fill(~mask, -math.inf)
    sink = w[p + "sink"].view(H, 1, 1).expand(H, T, 1)
    a = torch.softmax(torch.cat([s, sink], -1), -1)[..., :T]
    o = torch.einsum("hij,jhd->ihd", a, v).reshape(T, H * Dv)
    return o @ w[p + "o"].T


def forward(cfg: dict, weights: dict, tokens, layers_out=None):
    """Logits [T, vocab] of one whole sequence from position 0."""
    w = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in weights.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.shape[0]
    pos = torch.arange(T)
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    side = cfg.get("token_side")
    x = w["embed"][tokens]
    kvs = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", L["mixer"]
        if L["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                kvs[i] = latent_kv(x, w, p, m, eps, pos)
                src = i
            y = latent_attention(x, w, p, m, eps, pos, kvs[src])
        elif L["type"] == "attention":
            y = talking_attention(x, w, p, m, eps, pos)
        else:
            raise ValueError(L["type"])
        x = x + group_norm(y, w[f"l{i}.norm1"], groups, eps)
        if L.get("mlp"):
            x = x + group_norm(dense_ff(x, w, f"l{i}.mlp."), w[f"l{i}.norm2"], groups, eps)
        if side:
            x = token_side(x, tokens, w, i, side["dim"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return group_norm(x, w["final.norm"], groups, eps) @ w["embed"].T
