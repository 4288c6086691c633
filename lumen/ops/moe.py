"""Mixture-of-experts routing and gated activations (HIP: ``csrc/seqmix/moe.hip``).

Two ways to run a layer's experts, both on library GEMMs over weights stacked once at load (the
gate|up rows of every expert and of the shared expert in one [E * 2ff + 2ffs, W] weight, the down
projections side by side in one [W, E * ff + ffs] weight):

* ``moe_dense``: TWO GEMMs over all tokens and all experts.  Between them ``gated_act``
  multiplies each expert's activation by the token's routing weight (zero for experts the token
  did not choose), so the second GEMM's reduction over [experts x ff] IS the weighted sum of the
  chosen experts -- no gather / scatter, no host-visible token counts, graph-capturable.  Decode
  steps use it: at a few rows per step the cost is reading the expert weights, which a batch
  touches almost all of anyway.
* ``moe_grouped``: tokens sorted by expert, one pair of GEMMs per expert on its rows (slices of
  the same stacked weights), weighted rows added back in fp32.  It does top / E of the dense
  form's expert FLOPs but needs the per-expert row counts on the host (one synchronisation), so
  it serves prefill-sized steps outside graph capture.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F


def route_topk_ref(z: torch.Tensor, top: int) -> torch.Tensor:
    val, idx = torch.sort(z.float(), dim=-1, descending=True, stable=True)  # ties: lowest index
    val, idx = val[:, :top], idx[:, :top]
    return torch.zeros_like(z, dtype=torch.float32).scatter_(1, idx, torch.softmax(val, -1))


def route_topk(z: torch.Tensor, top: int) -> torch.Tensor:
    """Router logits z [T, E] (fp32) -> dense routing weights [T, E] (fp32): the softmax over
    each row's ``top`` largest logits at their places, zero elsewhere (ties: lowest index)."""
    from ._seqmix import call, use_seqmix

    if not use_seqmix(z):
        return route_topk_ref(z, top)
    assert z.dtype == torch.float32 and z.is_contiguous()
    T, E = z.shape
    if E > 1024:
        raise ValueError(f"route_topk supports at most 1024 experts, got {E}")
    out = torch.empty_like(z)
    call("sm_route_topk", z, out, T, E, top)
    return out


GATE_ACTS = {"silu": 0, "relu": 1, "gelu_tanh": 2}
_ACT_FN = {"silu": F.silu, "relu": F.relu, "gelu_tanh": lambda z: F.gelu(z, approximate="tanh")}


def gated_act_ref(gu, wts, E, ff, ffs, act="silu"):
    T = gu.shape[0]
    fn = _ACT_FN[act]
    parts = []
    if E:
        g = gu[:, :E * 2 * ff].float().view(T, E, 2, ff)
        parts.append((fn(g[:, :, 0]) * g[:, :, 1] * wts.float()[:, :, None]).reshape(T, E * ff))
    if ffs:
        s = gu[:, E * 2 * ff:].float().view(T, 2, ffs)
        parts.append(fn(s[:, 0]) * s[:, 1])
    return torch.cat(parts, 1).to(gu.dtype)


def gated_act(gu: torch.Tensor, wts: Optional[torch.Tensor], E: int, ff: int,
              ffs: int, act: str = "silu") -> torch.Tensor:
    """act(gate) * up over stacked [gate | up] blocks (``act``: silu, i.e. SwiGLU, relu or
    gelu_tanh): ``gu`` [T, E * 2 * ff + 2 * ffs] holds E expert blocks (gate rows then up rows,
    ff each) and one unweighted block of ffs (a dense feed-forward, or the shared expert);
    expert e's activation is scaled by ``wts[:, e]``.  Returns [T, E * ff + ffs]."""
    from ._seqmix import DT, call, use_seqmix

    if not use_seqmix(gu):
        return gated_act_ref(gu, wts, E, ff, ffs, act)
    assert gu.is_contiguous() and gu.shape[1] == E * 2 * ff + 2 * ffs
    out = torch.empty(gu.shape[0], E * ff + ffs, dtype=gu.dtype, device=gu.device)
    call("sm_gated_act", DT[gu.dtype], gu, wts, out, gu.shape[0], E, ff, ffs, GATE_ACTS[act])
    return out


def moe_dense(h, wts, gu_w, down_w, E: int, ff: int, ffs: int) -> torch.Tensor:
    return F.linear(gated_act(F.linear(h, gu_w), wts, E, ff, ffs), down_w)


def moe_grouped(h, wts, gu_w, down_w, E: int, ff: int, ffs: int) -> torch.Tensor:
    """Same result as ``moe_dense`` (to rounding) running each expert on its own rows only."""
    T = h.shape[0]
    tok, exp = (wts > 0).nonzero(as_tuple=True)           # (host sync) pairs in token order
    order = torch.argsort(exp, stable=True)
    tok, exp = tok[order], exp[order]
    counts = torch.bincount(exp, minlength=E).tolist()
    x = h.index_select(0, tok)
    wsel = wts[tok, exp].unsqueeze(1)
    out = torch.zeros(T, h.shape[1], dtype=torch.float32, device=h.device)
    ys = torch.empty(x.shape[0], h.shape[1], dtype=h.dtype, device=h.device)
    a = 0
    for e, n in enumerate(counts):
        if n:
            gu = F.linear(x[a:a + n], gu_w[e * 2 * ff:(e + 1) * 2 * ff])
            torch.matmul(gated_act(gu, None, 0, 0, ff), down_w[:, e * ff:(e + 1) * ff].t(),
                         out=ys[a:a + n])
            a += n
    out.index_add_(0, tok, ys.float() * wsel)
    if ffs:
        gu = F.linear(h, gu_w[E * 2 * ff:])
        out += F.linear(gated_act(gu, None, 0, 0, ffs), down_w[:, E * ff:]).float()
    return out.to(h.dtype)


# steps with at least this many rows per expert-FLOP saved take the grouped form
GROUPED_MIN_ROWS = 256


def moe(h, wts, gu_w, down_w, E: int, top: int, ff: int, ffs: int) -> torch.Tensor:
    """Weighted sum of each row's chosen experts (+ the shared expert): [T, W] in h's dtype."""
    grouped = (h.shape[0] >= GROUPED_MIN_ROWS and top * 2 <= E
               and not (h.is_cuda and torch.cuda.is_current_stream_capturing()))
    return (moe_grouped if grouped else moe_dense)(h, wts, gu_w, down_w, E, ff, ffs)
