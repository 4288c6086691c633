"""Slow, plain oracle of the Gedatar design for the tests: whole sequences, float64, one function
per mechanism, token loops for the recurrences, dense masks for attention.  Shares no code with
``lumen`` (only torch): it is what the framework's kernels, caches and scheduler are compared to.

Notation: T tokens, W width, H heads, G key/value heads, D head size; weights are [out, in].
"""
import math

import torch
import torch.nn.functional as F

F64 = torch.float64


def ref_dyt(x, w, b, alpha):
    return torch.tanh(alpha * x) * w + b


def ref_unit_rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def ref_canon(h, cw):
    """h [T, W] -> h + causal depthwise conv; cw [W, taps], the last tap multiplies h_t."""
    T, taps = h.shape[0], cw.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                out[t] += cw[:, j] * h[s]
    return out


def ref_token_shift(h, mu):
    """The mixes h + (h_prev - h) * mu[s]; mu [n, W] -> [n, T, W]."""
    hp = torch.zeros_like(h)
    hp[1:] = h[:-1]
    return torch.stack([h + (hp - h) * m for m in mu])


def ref_wkv(r, k, v, w, u):
    """r, k, v, w [T, H, D], u [H, D] -> read-outs [T, H, D] (before the head norm)."""
    T, H, D = r.shape
    S = torch.zeros(H, D, D, dtype=r.dtype)
    o = torch.zeros_like(r)
    for t in range(T):
        for h in range(H):
            kv = torch.outer(k[t, h], v[t, h])
            o[t, h] = (S[h] + u[h][:, None] * kv).T @ r[t, h]
            S[h] = w[t, h][:, None] * S[h] + kv
    return o


def ref_delta(r, k, v, w, a, key_eps=1e-6):
    T, H, D = r.shape
    S = torch.zeros(H, D, D, dtype=r.dtype)
    o = torch.zeros_like(r)
    for t in range(T):
        for h in range(H):
            un = k[t, h] / torch.sqrt(k[t, h].pow(2).sum() + key_eps)
            S[h] = (w[t, h][:, None] * S[h] - torch.outer(a[t, h] * un, un @ S[h])
                    + torch.outer(k[t, h], v[t, h]))
            o[t, h] = S[h].T @ r[t, h]
    return o


def ref_attention(q, k, scale, chunk, eps, sink=True):
    """q [T, H, D], k [T, G, D] (the values are k itself) -> [T, H, D]."""
    T, H, D = q.shape
    G = k.shape[1]
    qn, kn = ref_unit_rms(q, eps), ref_unit_rms(k, eps)
    out = torch.zeros_like(q)
    for i in range(T):
        js = [j for j in range(i + 1) if not chunk or j // chunk == i // chunk]
        for h in range(H):
            g = h // (H // G)
            e = torch.exp(torch.stack([(qn[i, h] @ kn[j, g]) * scale for j in js]))
            p = e / (e.sum() + (1.0 if sink else 0.0))
            out[i, h] = sum(pj * k[j, g] for pj, j in zip(p, js))
    return out


def ref_route(z, top):
    """Dense routing weights [T, E]: softmax over each row's `top` largest logits."""
    out = torch.zeros_like(z)
    for t in range(z.shape[0]):
        idx = sorted(range(z.shape[1]), key=lambda e: (-float(z[t, e]), e))[:top]
        e = torch.exp(z[t, idx] - z[t, idx].max())
        out[t, idx] = e / e.sum()
    return out


def ref_ffn(h, gate, up, down):
    return (F.silu(h @ gate.T) * (h @ up.T)) @ down.T


class RefModel:
    """Whole-sequence forward of a configuration (lumen ModelConfig) from a name -> tensor dict."""

    def __init__(self, cfg, tensors):
        self.cfg = cfg
        self.t = {k: v.detach().to("cpu", F64) for k, v in tensors.items()}

    def norm(self, x, name):
        return ref_dyt(x, self.t[name], self.t[name + ".b"], self.t[name + ".alpha"])

    def mixer(self, i, h):
        t, cfg = self.t, self.cfg
        L = cfg.layer_specs[i]
        m, p, eps = L["mixer"], f"l{i}.mix.", cfg.rms_norm_eps
        T = h.shape[0]
        if L["type"] == "attention":
            H, G, D = m["heads"], m["kv_heads"], m["dim"]
            o = ref_attention((h @ t[p + "q"].T).view(T, H, D), (h @ t[p + "k"].T).view(T, G, D),
                              m["scale"], m["mask"]["size"], eps)
            return o.reshape(T, -1) @ t[p + "o"].T
        H, D = m["heads"], m["dim"]
        sh = lambda x: x.view(T, H, D)  # noqa: E731
        if L["type"] == "wkv":
            mr, mk, mv, mg, mw = ref_token_shift(h, torch.stack([t[p + "mu." + s] for s in "rkvgw"]))
            w = torch.exp(-torch.exp(torch.tanh(mw @ t[p + "w1"].T) @ t[p + "w2"].T + t[p + "w0"]))
            o = ref_wkv(sh(mr @ t[p + "r"].T), sh(mk @ t[p + "k"].T), sh(mv @ t[p + "v"].T), sh(w),
                        t[p + "u"])
            gate = F.silu(mg @ t[p + "g"].T)
        else:
            w = torch.exp(-math.exp(-0.5) * torch.sigmoid(
                torch.tanh(h @ t[p + "w1"].T) @ t[p + "w2"].T + t[p + "w0"]))
            a = torch.sigmoid(h @ t[p + "a"].T + t[p + "a.b"])
            o = ref_delta(sh(h @ t[p + "r"].T), sh(h @ t[p + "k"].T), sh(h @ t[p + "v"].T), sh(w),
                          sh(a))
            gate = torch.sigmoid(h @ t[p + "g"].T)
        o = ref_unit_rms(o, eps).reshape(T, H * D) * t[p + "norm"] * gate
        return o @ t[p + "o"].T

    def feed_forward(self, i, h):
        t = self.t
        f, p = self.cfg.layer_specs[i]["mlp"], f"l{i}.mlp."
        if f["kind"] == "dense":
            return ref_ffn(h, t[p + "gate"], t[p + "up"], t[p + "down"])
        wts = ref_route(h @ t[p + "router"].T + t[p + "router.b"], f["router"]["top"])
        out = torch.zeros_like(h)
        for e in range(f["router"]["experts"]):
            q = p + f"e{e}."
            out += wts[:, e:e + 1] * ref_ffn(h, t[q + "gate"], t[q + "up"], t[q + "down"])
        if f.get("shared"):
            q = p + "shared."
            out += ref_ffn(h, t[q + "gate"], t[q + "up"], t[q + "down"])
        return out

    def forward(self, tokens, layers_out=None):
        """Logits [T, V] of one sequence from position 0."""
        x = self.t["embed"][torch.as_tensor(tokens, dtype=torch.long)]
        for i, L in enumerate(self.cfg.layer_specs):
            p = f"l{i}."
            h = ref_canon(self.norm(x, p + "norm1"), self.t[p + "canon1"])
            x = x + self.norm(self.mixer(i, h), p + "norm1b")
            if L.get("mlp"):
                x = x + self.norm(self.feed_forward(i, self.norm(x, p + "norm2")), p + "norm2b")
            if layers_out is not None:
                layers_out.append(x.clone())
        return self.norm(x, "final.norm") @ self.t["head"].T
