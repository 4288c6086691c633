"""Mixture-of-experts routing and gated activations (HIP: ``csrc/seqmix/moe.hip``).

The experts of a layer are run as TWO library GEMMs over all tokens: the gate|up rows of every
expert (and of the shared expert) stacked into one weight, and the down projections stacked
along their input dimension.  Between them ``gated_act`` multiplies each expert's activation by
the token's routing weight (zero for experts the token did not choose), so the second GEMM's
reduction over [experts x ff] IS the weighted sum of the chosen experts -- no gather / scatter,
no host-visible token counts, graph-capturable.  It spends experts / top times the FLOPs of a
grouped GEMM on the expert part, which is the price of staying on the library GEMM.
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


def gated_act_ref(gu, wts, E, ff, ffs):
    T = gu.shape[0]
    parts = []
    if E:
        g = gu[:, :E * 2 * ff].float().view(T, E, 2, ff)
        parts.append((F.silu(g[:, :, 0]) * g[:, :, 1] * wts.float()[:, :, None]).reshape(T, E * ff))
    if ffs:
        s = gu[:, E * 2 * ff:].float().view(T, 2, ffs)
        parts.append(F.silu(s[:, 0]) * s[:, 1])
    return torch.cat(parts, 1).to(gu.dtype)


def gated_act(gu: torch.Tensor, wts: Optional[torch.Tensor], E: int, ff: int,
              ffs: int) -> torch.Tensor:
    """SwiGLU over stacked [gate | up] blocks: ``gu`` [T, E * 2 * ff + 2 * ffs] holds E expert
    blocks (gate rows then up rows, ff each) and one unweighted block of ffs (a dense
    feed-forward, or the shared expert); expert e's activation is scaled by ``wts[:, e]``.
    Returns [T, E * ff + ffs]."""
    from ._seqmix import DT, call, use_seqmix

    if not use_seqmix(gu):
        return gated_act_ref(gu, wts, E, ff, ffs)
    assert gu.is_contiguous() and gu.shape[1] == E * 2 * ff + 2 * ffs
    out = torch.empty(gu.shape[0], E * ff + ffs, dtype=gu.dtype, device=gu.device)
    call("sm_gated_act", DT[gu.dtype], gu, wts, out, gu.shape[0], E, ff, ffs)
    return out
