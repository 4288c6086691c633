"""Causal depthwise convolution over time on a layer's normed input, with per-sequence tails.

``dyt_canon``: h = DyT(x) on every row, then out_t = h_t + sum_j w[:, j] * h_(t - taps + 1 + j)
with zeros before a sequence's start.  The last ``taps - 1`` normed rows of every sequence live
in ``tail`` [slots, taps - 1, W] (fp32), so a step may begin anywhere in a sequence: rows before
the step's first row come from the tail (positions below 0 read as zero, whatever a reused slot
still holds), and the tail is moved on to the step's last rows afterwards.  (HIP:
``csrc/seqmix/norm_conv.hip``, norm and convolution in one pass over x.)
"""
from __future__ import annotations

import torch

from .norm import dyt_ref
from .segments import SegBatch


def dyt_canon_ref(x, norm, conv_w, tail, seg: SegBatch, out_dtype):
    taps = conv_w.shape[1]
    K = taps - 1
    h = dyt_ref(x, norm, torch.float32)
    out = torch.empty_like(h)
    cu, slots, starts = seg.cu.tolist(), seg.slot.tolist(), seg.start.tolist()
    w = conv_w.float()
    for s in range(seg.S):
        a, b, sl, p0 = cu[s], cu[s + 1], slots[s], starts[s]
        if b == a:
            continue
        hist = tail[sl].clone() if K else h.new_zeros(0, h.shape[1])
        for i in range(K):                     # tail row i is position p0 - K + i
            if p0 - K + i < 0:
                hist[i] = 0
        ext = torch.cat([hist, h[a:b]], 0)     # row K + t is the segment's row t
        acc = h[a:b].clone()
        for j in range(taps):
            acc += w[:, j] * ext[j:j + (b - a)]
        out[a:b] = acc
        if K:
            tail[sl] = ext[-K:]
    return out.to(out_dtype)


def dyt_canon(x: torch.Tensor, norm, conv_w: torch.Tensor, tail: torch.Tensor, seg: SegBatch,
              out_dtype) -> torch.Tensor:
    from ._seqmix import DT, call, use_seqmix

    if not use_seqmix(x):
        return dyt_canon_ref(x, norm, conv_w, tail, seg, out_dtype)
    T, W = x.shape
    taps = conv_w.shape[1]
    assert x.dtype == torch.float32 and x.is_contiguous() and conv_w.dtype == torch.float32
    assert tail.dtype == torch.float32 and tail.shape[1:] == (max(taps - 1, 0), W) or taps == 1
    out = torch.empty(T, W, dtype=out_dtype, device=x.device)
    call("sm_dyt_canon", DT[out_dtype], x, norm[0], norm[1], norm[2], conv_w, tail, out, seg.cu,
         seg.slot, seg.start, seg.row_seg, T, W, taps)
    if taps > 1:
        call("sm_canon_tail", x, norm[0], norm[1], norm[2], tail, seg.cu, seg.slot, seg.start,
             seg.S, W, taps)
    return out
