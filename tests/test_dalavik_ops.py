"""The mechanisms of the Dalavik design, each alone, against plain float64 formulas written here
or in tests/_ref_dalavik.py (no code shared with ``lumen``).  CPU tensors take the ops' torch
path; marked ``gpu``, the same cases run the HIP kernels in fp32 and bf16.

Where random inputs would hide a fault the inputs are made so that it shows: one far key that
must win among hundreds, keys beyond a row's position holding huge values, a sink that halves the
output, a head mixing that swaps heads, a temperature that steps between neighbouring rows."""
import math

import pytest
import torch

import _ref_dalavik as ref

from lumen.ops.attention import head_norm_write, latent_write, row_attention
from lumen.ops.embedding import gated_token_slice
from lumen.ops.moe import gated_act
from lumen.ops.norm import group_rms_norm, group_rms_residual
from lumen.ops.rope import interleaved_inv_freq, rotate_interleaved_
from lumen.ops.segments import SegBatch

F64 = torch.float64
CASES = [("cpu", torch.float32), pytest.param("cuda", torch.float32, marks=pytest.mark.gpu),
         pytest.param("cuda", torch.bfloat16, marks=pytest.mark.gpu)]


def tol(dtype):
    return 2e-5 if dtype == torch.float32 else 2e-2


def close(got, want, dtype, scale=None):
    got, want = got.detach().cpu().to(F64), want.to(F64)
    s = scale if scale is not None else max(1.0, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= tol(dtype) * s, f"max error {err:.3e} (scale {s:.3f})"


def rnd(*shape, seed=0, dtype=torch.float32, device="cpu", scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(*shape, generator=g)).to(dtype).to(device)


# ---- norms ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("W,groups", [(96, 3), (64, 1), (64, 2), (80, 5), (256, 8), (30, 3),
                                      (1024, 4), (1536, 1)])
def test_group_rms_norm(device, dtype, W, groups):
    x = rnd(7, W, seed=1, dtype=dtype, device=device, scale=3.0)
    w = rnd(W, seed=2, device=device) + 1.0
    want = ref.group_norm(x.cpu().to(F64), w.cpu().to(F64), groups, 1e-5)
    close(group_rms_norm(x, w, groups, 1e-5, dtype), want, dtype)
    # a column slice of a wider buffer (the fused projection's output)
    wide = rnd(7, W + 40, seed=3, dtype=dtype, device=device)
    want = ref.group_norm(wide[:, 8:8 + W].cpu().to(F64), w.cpu().to(F64), groups, 1e-5)
    close(group_rms_norm(wide[:, 8:8 + W], w, groups, 1e-5, dtype), want, dtype)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("W,groups", [(96, 3), (64, 1), (80, 5), (512, 2)])
def test_group_rms_residual(device, dtype, W, groups):
    x = rnd(9, W, seed=4, device=device)
    y = rnd(9, W, seed=5, dtype=dtype, device=device, scale=0.01)      # eps matters at this size
    w = rnd(W, seed=6, device=device) + 1.0
    want = x.cpu().to(F64) + ref.group_norm(y.cpu().to(F64), w.cpu().to(F64), groups, 1e-4)
    cast = None if dtype == torch.float32 else dtype
    x2, xb = group_rms_residual(x, y, w, groups, 1e-4, cast)
    assert x2 is x and x.dtype == torch.float32
    close(x, want, torch.float32 if dtype == torch.float32 else dtype)
    if cast is None:
        assert xb is None
    else:
        assert xb.dtype == dtype and torch.equal(xb.float(), x.to(dtype).float())


# ---- feed-forward activation and the token side gate ---------------------------------------------
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("ff", [40, 37])
def test_relu_gated_activation(device, dtype, ff):
    gu = rnd(11, 2 * ff, seed=7, dtype=dtype, device=device)
    g, u = gu[:, :ff].cpu().to(F64), gu[:, ff:].cpu().to(F64)
    close(gated_act(gu, None, 0, 0, ff, "relu"), torch.relu(g) * u, dtype)
    close(gated_act(gu, None, 0, 0, ff, "gelu_tanh"), ref.gelu_tanh(g) * u, dtype)


@pytest.mark.parametrize("device,dtype", CASES)
def test_gated_token_slice(device, dtype):
    z = rnd(13, 6, seed=8, dtype=dtype, device=device, scale=2.0)
    table = rnd(50, 30, seed=9, dtype=dtype, device=device)
    toks = torch.randint(0, 50, (13,), generator=torch.Generator().manual_seed(10)).to(device)
    for col0 in (0, 6, 24):
        want = ref.gelu_tanh(z.cpu().to(F64)) * table.cpu().to(F64)[toks.cpu()][:, col0:col0 + 6]
        close(gated_token_slice(z, table, toks, col0), want, dtype)
    with pytest.raises(ValueError):
        gated_token_slice(z, table, toks, 25)


# ---- rotary --------------------------------------------------------------------------------------
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("dims,width", [(8, 8), (4, 6), (16, 16)])
def test_rotate_interleaved(device, dtype, dims, width):
    H, D = 3, 10
    x = rnd(6, H * (D + width), seed=11, dtype=dtype, device=device)
    pos = torch.tensor([0, 1, 2, 77, 1000, 4095], dtype=torch.int32, device=device)
    xf = x.cpu().to(F64).view(6, H, D + width)
    want = xf.clone()
    want[..., D:] = ref.rotate_pairs(xf[..., D:], pos.cpu(), dims, 900.0)
    rotate_interleaved_(x, pos, H, D + width, D, dims, interleaved_inv_freq(dims, 900.0, device))
    close(x.view(6, H, D + width), want, dtype)
    # position 0 turns nothing, and what lies outside the slice never moves
    assert torch.equal(x.view(6, H, -1)[0].cpu().to(F64), xf[0])
    assert torch.equal(x.view(6, H, -1)[..., :D].cpu().to(F64), xf[..., :D])


# ---- cache writes --------------------------------------------------------------------------------
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("R,Dr,dims", [(32, 8, 8), (22, 6, 4), (128, 64, 64)])
def test_latent_write(device, dtype, R, Dr, dims):
    T = 9
    z = rnd(T, 5 + R + Dr, seed=12, dtype=dtype, device=device, scale=2.0)[:, 5:]
    wn = rnd(R, seed=13, device=device) + 1.0
    pos = torch.tensor([0, 1, 2, 3, 40, 41, 500, 7, 8], dtype=torch.int32, device=device)
    slots = torch.tensor([5, 4, 63, -1, 0, 17, 33, 2, -1], device=device)
    cache = torch.full((4, 16, R + Dr), 9.0, dtype=dtype, device=device)
    vt = torch.full((4, R, 16), 9.0, dtype=dtype, device=device)
    latent_write(z, wn, interleaved_inv_freq(dims, 300.0, device), pos, slots, cache, R, dims, 1e-5,
                 vt)
    zf = z.cpu().to(F64)
    c = ref.rms_unit(zf[:, :R], 1e-5) * wn.cpu().to(F64)
    kr = ref.rotate_pairs(zf[:, R:], pos.cpu(), dims, 300.0)
    rows = cache.view(64, R + Dr).cpu()
    used = set()
    for t, s in enumerate(slots.tolist()):
        if s >= 0:
            used.add(s)
            close(rows[s], torch.cat([c[t], kr[t]]), dtype)
    for s in set(range(64)) - used:                      # skipped rows and the rest stay untouched
        assert bool((rows[s] == 9.0).all())
    # the transposed copy holds the same latents, [block][R][token in block]
    assert torch.equal(vt.transpose(1, 2).reshape(64, R).cpu(), rows[:, :R])


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,G,D,Dv", [(6, 2, 24, 16), (3, 3, 20, 12), (1, 1, 128, 64), (8, 1, 8, 40)])
def test_head_norm_write(device, dtype, H, G, D, Dv):
    T = 5
    qkv = rnd(T, (H + G) * D + G * Dv, seed=14, dtype=dtype, device=device, scale=1.5)
    before = qkv.cpu().to(F64)
    wq, wk = rnd(D, seed=15, device=device) + 1.0, rnd(D, seed=16, device=device) + 1.0
    slots = torch.tensor([3, -1, 30, 0, 31], device=device)
    kc = torch.full((2, 16, G, D), 7.0, dtype=dtype, device=device)
    vc = torch.full((2, 16, G, Dv), 7.0, dtype=dtype, device=device)
    head_norm_write(qkv, wq, wk, slots, kc, vc, H, G, D, Dv, 1e-6)
    q = ref.rms_unit(before[:, :H * D].view(T, H, D), 1e-6) * wq.cpu().to(F64)
    k = ref.rms_unit(before[:, H * D:(H + G) * D].view(T, G, D), 1e-6) * wk.cpu().to(F64)
    v = before[:, (H + G) * D:].view(T, G, Dv)
    close(qkv[:, :H * D].view(T, H, D), q, dtype)
    for t, s in enumerate(slots.tolist()):
        if s >= 0:
            close(kc.view(32, G, D)[s], k[t], dtype)
            close(vc.view(32, G, Dv)[s], v[t], dtype)
    assert bool((kc.view(32, -1)[1] == 7.0).all()) and bool((vc.view(32, -1)[5] == 7.0).all())


# ---- row attention -------------------------------------------------------------------------------
def dense_attention(q, k, v, pos_q, hg, scale, softcap=0.0, q_temp=None, r1=None, r2=None,
                    talk=None, sink=None):
    """q [T, H, Dk] at positions pos_q against keys k [n, G, Dk] / values v [n, G, Dv] at positions
    0 .. n-1 of the same sequence; float64, dense mask."""
    q, k, v = q.to(F64), k.to(F64)[:, hg], v.to(F64)[:, hg]
    T, H, _ = q.shape
    n = k.shape[0]
    temp = torch.ones(T, dtype=F64)
    if q_temp:
        temp = 1.0 + q_temp[0] * torch.log(torch.floor((pos_q.to(F64) + 1) / q_temp[1]) + 1.0)
    s = torch.einsum("thd,nhd->htn", q, k) * scale * temp.view(1, T, 1)
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    dist = (pos_q.view(T, 1) - torch.arange(n).view(1, n)).to(F64)
    if r1 is not None:
        s = s - r1.to(F64).view(H, 1, 1) * torch.log(1.0 + r2.to(F64).view(H, 1, 1) * dist.clamp(min=0))
    if talk is not None:
        s = torch.einsum("hg,gtn->htn", talk.to(F64), s)
    s = s.masked_fill((dist < 0).view(1, T, n), -math.inf)
    if sink is not None:
        s = torch.cat([s, sink.to(F64).view(H, 1, 1).expand(H, T, 1)], -1)
    a = torch.softmax(s, -1)[..., :n]
    return torch.einsum("htn,nhd->thd", a, v)


def paged(seq_rows, bs, nb, width, dtype, device, seed, fill=1e4):
    """Scatter each sequence's rows [n, width] into a scrambled block pool; every row of the pool
    that no sequence owns, and every owned row past a sequence's end, holds ``fill``."""
    g = torch.Generator().manual_seed(seed)
    order = torch.randperm(nb, generator=g).tolist()
    pool = torch.full((nb, bs, width), fill, dtype=torch.float32)
    tables = []
    for rows in seq_rows:
        need = (rows.shape[0] + bs - 1) // bs
        blocks = [order.pop() for _ in range(need)]
        tables.append(blocks)
        for j in range(rows.shape[0]):
            pool[blocks[j // bs], j % bs] = rows[j].float()
    mb = max(len(t) for t in tables)
    tb = torch.zeros(len(tables), mb, dtype=torch.int32)
    for i, t in enumerate(tables):
        tb[i, :len(t)] = torch.tensor(t, dtype=torch.int32)
    return pool.to(dtype).to(device), tb.to(device)


def segments(spans, tables, device):
    """spans: [(sequence, first position, rows)] -> SegBatch with one segment per span."""
    cu, row_seg, pos = [0], [], []
    for i, (_, p0, n) in enumerate(spans):
        cu.append(cu[-1] + n)
        row_seg += [i] * n
        pos += list(range(p0, p0 + n))
    i32 = dict(dtype=torch.int32, device=device)
    tb = torch.stack([tables[s] for s, _, _ in spans])
    return SegBatch(torch.tensor(cu, **i32), torch.zeros(len(spans), **i32),
                    torch.tensor([p0 for _, p0, _ in spans], **i32), torch.tensor(row_seg, **i32),
                    torch.tensor(pos, **i32), tb.contiguous(), None)


SPANS = [(0, 0, 19), (1, 130, 1), (2, 60, 37), (0, 19, 1), (1, 131, 2), (2, 97, 1), (2, 98, 1)]
LENS = [20, 133, 99]


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,G,D,Dv,bs", [(6, 2, 24, 16, 8), (3, 3, 20, 12, 16), (4, 1, 32, 48, 8),
                                         (9, 3, 16, 8, 16), (32, 4, 64, 64, 16)])
def test_row_attention_grouped_with_everything(device, dtype, H, G, D, Dv, bs):
    """Grouped-query rows of prompts' portions and decoded tokens in one step, every score
    shaping switched on, scrambled block tables, poison past every sequence's end."""
    ks = [rnd(n, G * D, seed=20 + i, dtype=dtype) for i, n in enumerate(LENS)]
    vs = [rnd(n, G * Dv, seed=30 + i, dtype=dtype) for i, n in enumerate(LENS)]
    kc, tb = paged(ks, bs, 40, G * D, dtype, device, 1)
    vc, _ = paged(vs, bs, 40, G * Dv, dtype, device, 1)
    seg = segments(SPANS, tb, device)
    T = seg.T
    q = rnd(T, H * D + 3, seed=40, dtype=dtype, device=device)[:, :H * D].view(T, H, D)
    r1, r2 = torch.rand(H, device=device) * 0.4, torch.rand(H, device=device) + 0.05
    talk = (torch.eye(H) + 0.3 * rnd(H, H, seed=41)).to(device)
    sink = rnd(H, seed=42, device=device)
    out = torch.zeros(T, H, Dv, dtype=dtype, device=device)
    kw = dict(softcap=5.0, q_temp=(0.3, 20), r1=r1, r2=r2, talk=talk, sink=sink)
    row_attention(q, None, kc.view(40, bs, G, D), vc.view(40, bs, G, Dv), Dv, out, seg, H, G, 0.3, **kw)
    hg = torch.arange(H) // (H // G)
    at = 0
    for s, p0, n in SPANS:
        pos = torch.arange(p0, p0 + n)
        want = dense_attention(q[at:at + n].cpu(), ks[s][:p0 + n].view(-1, G, D),
                               vs[s][:p0 + n].view(-1, G, Dv), pos, hg, 0.3,
                               **{k: (v.cpu() if torch.is_tensor(v) else v) for k, v in kw.items()})
        close(out[at:at + n], want, dtype, scale=1.0)
        at += n


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,D1,D2,R,bs", [(3, 32, 8, 32, 8), (7, 22, 6, 22, 16), (12, 64, 24, 64, 16),
                                          (5, 128, 32, 128, 16), (20, 192, 24, 192, 8),
                                          (9, 512, 64, 512, 16)])
@pytest.mark.parametrize("transposed", [False, True])
def test_row_attention_latent_two_part_query(device, dtype, H, D1, D2, R, bs, transposed):
    """One shared cache row per token, the value its first R columns, the query in two parts
    with strides of their own (head-major and token-major), the output written head-major; with
    and without the per-block transposed copy of the values that switches the matrix-core value
    product on where it has a kernel (16-bit, R a multiple of 64)."""
    assert D1 == R
    rows = [rnd(n, R + D2, seed=50 + i, dtype=dtype) for i, n in enumerate(LENS)]
    cache, tb = paged(rows, bs, 40, R + D2, dtype, device, 2)
    seg = segments(SPANS, tb, device)
    T = seg.T
    qa = rnd(H, T, D1, seed=60, dtype=dtype, device=device)                  # [H, T, D1]
    qb = rnd(T, H, 11 + D2, seed=61, dtype=dtype, device=device)[:, :, 11:]  # [T, H, D2], strided
    out = torch.zeros(H, T, R, dtype=dtype, device=device)
    vt = cache[:, :, :R].transpose(1, 2).contiguous() if transposed else None
    sink = rnd(H, seed=62, device=device) if transposed else None
    row_attention(qa.transpose(0, 1), qb, cache, cache, R, out.transpose(0, 1), seg, H, 1, 0.2,
                  sink=sink, vt=vt)
    q = torch.cat([qa.transpose(0, 1), qb], -1).cpu()
    hg = torch.zeros(H, dtype=torch.long)
    at = 0
    for s, p0, n in SPANS:
        kv = rows[s][:p0 + n]
        want = dense_attention(q[at:at + n], kv.view(-1, 1, R + D2), kv[:, :R].reshape(-1, 1, R),
                               torch.arange(p0, p0 + n), hg, 0.2,
                               sink=sink.cpu() if sink is not None else None)
        close(out.transpose(0, 1)[at:at + n], want, dtype, scale=max(1.0, (D1 + D2) ** 0.5 / 8))
        at += n


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("far", [0, 3, 63, 64, 511, 512])
def test_far_key_wins_among_hundreds(device, dtype, far):
    """700 cached keys, one of them (at a tile or block border, or the very first) aligned with
    the query and scaled so that it takes nearly all the weight: prompt rows and decoded rows
    far behind it must return ITS value."""
    n, H, D, Dv, bs = 700, 2, 16, 8, 16
    k = rnd(n, D, seed=70, dtype=torch.float32, scale=0.1)
    v = rnd(n, Dv, seed=71, dtype=torch.float32)
    d = torch.zeros(D)
    d[5] = 1.0
    k[far] = 4.0 * d
    kc, tb = paged([k.to(dtype)], bs, 50, D, dtype, device, 3)
    vc, _ = paged([v.to(dtype)], bs, 50, Dv, dtype, device, 3)
    spans = [(0, 600, 40), (0, 640, 1), (0, 699, 1)]
    seg = segments(spans, tb, device)
    q = (8.0 * d).to(dtype).to(device).expand(seg.T, H, D).contiguous()
    out = torch.zeros(seg.T, H, Dv, dtype=dtype, device=device)
    row_attention(q, None, kc.view(50, bs, 1, D), vc.view(50, bs, 1, Dv), Dv, out, seg, H, 1, 1.0)
    want = v[far].to(dtype).to(F64).expand(seg.T, H, Dv)
    close(out, want, dtype, scale=1.0)
    # and a row just BEFORE the key must not see it
    if far > 0:
        seg2 = segments([(0, far - 1, 1), (0, far, 1)], tb, device)
        out2 = torch.zeros(2, H, Dv, dtype=dtype, device=device)
        row_attention(q[:2].contiguous(), None, kc.view(50, bs, 1, D), vc.view(50, bs, 1, Dv), Dv,
                      out2, seg2, H, 1, 1.0)
        got = out2.cpu().to(F64)
        assert float((got[1] - want[0]).abs().max()) < 0.05
        assert float((got[0] - want[0]).abs().max()) > 0.05


@pytest.mark.parametrize("device,dtype", CASES)
def test_sink_counts_once_and_has_no_value(device, dtype):
    """All keys score 0 and the sink is ln(n): the softmax denominator doubles, so the output is
    half the values' mean -- whatever the scale, cap, bias or head mixing would do to a key."""
    n, H, D, Dv, bs = 50, 2, 8, 8, 16
    v = rnd(n, Dv, seed=80, dtype=dtype)
    kc, tb = paged([torch.zeros(n, D)], bs, 8, D, dtype, device, 4, fill=0.0)
    vc, _ = paged([v], bs, 8, Dv, dtype, device, 4)
    seg = segments([(0, n - 1, 1)], tb, device)
    q = rnd(1, H, D, seed=81, dtype=dtype, device=device)
    sink = torch.tensor([math.log(n), -1e4], device=device)
    out = torch.zeros(1, H, Dv, dtype=dtype, device=device)
    row_attention(q, None, kc.view(8, bs, 1, D), vc.view(8, bs, 1, Dv), Dv, out, seg, H, 1, 7.0,
                  softcap=2.0, sink=sink, talk=torch.eye(H, device=device))
    mean = v.to(F64).mean(0)
    close(out[0, 0], mean / 2, dtype, scale=1.0)
    close(out[0, 1], mean, dtype, scale=1.0)               # a sink far below: no effect


@pytest.mark.parametrize("device,dtype", CASES)
def test_head_mixing_swaps_heads_and_temperature_steps(device, dtype):
    n, H, D, Dv, bs = 45, 2, 8, 8, 8
    k = rnd(n, D, seed=90, dtype=dtype)
    v = rnd(n, Dv, seed=91, dtype=dtype)
    kc, tb = paged([k], bs, 8, D, dtype, device, 5)
    vc, _ = paged([v], bs, 8, Dv, dtype, device, 5)
    seg = segments([(0, 36, 4)], tb, device)               # positions 36 .. 39, step at p + 1 = 40
    q = rnd(4, H, D, seed=92, dtype=dtype, device=device, scale=2.0)
    out = torch.zeros(4, H, Dv, dtype=dtype, device=device)
    out_sw = torch.zeros_like(out)
    caches = (kc.view(8, bs, 1, D), vc.view(8, bs, 1, Dv))
    row_attention(q, None, *caches, Dv, out, seg, H, 1, 0.5, q_temp=(0.9, 40))
    swap = torch.tensor([[0.0, 1.0], [1.0, 0.0]], device=device)
    row_attention(q, None, *caches, Dv, out_sw, seg, H, 1, 0.5, q_temp=(0.9, 40), talk=swap)
    close(out_sw[:, 0], out[:, 1].cpu().to(F64), dtype, scale=1.0)
    close(out_sw[:, 1], out[:, 0].cpu().to(F64), dtype, scale=1.0)
    hg = torch.zeros(H, dtype=torch.long)
    for i, p in enumerate(range(36, 40)):
        t = 1.0 + 0.9 * math.log((p + 1) // 40 + 1.0)
        assert (t > 1.0) == (p == 39)
        want = dense_attention(q[i:i + 1].cpu(), k[:p + 1].view(-1, 1, D), v[:p + 1].view(-1, 1, Dv),
                               torch.tensor([p]), hg, 0.5 * t)
        close(out[i:i + 1], want, dtype, scale=1.0)


@pytest.mark.parametrize("device,dtype", CASES)
def test_distance_bias_prefers_near_keys(device, dtype):
    """Equal scores everywhere; a strong bias r1 ln(1 + r2 d) leaves the row's own key nearly all
    the weight on head 0 and changes nothing on head 1 (r1 = 0)."""
    n, H, D, Dv, bs = 130, 2, 8, 8, 16
    v = rnd(n, Dv, seed=95, dtype=dtype)
    kc, tb = paged([torch.zeros(n, D)], bs, 10, D, dtype, device, 6, fill=0.0)
    vc, _ = paged([v], bs, 10, Dv, dtype, device, 6)
    seg = segments([(0, 100, 3), (0, 129, 1)], tb, device)
    q = rnd(4, H, D, seed=96, dtype=dtype, device=device)
    out = torch.zeros(4, H, Dv, dtype=dtype, device=device)
    r1 = torch.tensor([30.0, 0.0], device=device)
    r2 = torch.tensor([1.0, 5.0], device=device)
    row_attention(q, None, kc.view(10, bs, 1, D), vc.view(10, bs, 1, Dv), Dv, out, seg, H, 1, 1.0,
                  r1=r1, r2=r2)
    for i, p in enumerate([100, 101, 102, 129]):
        close(out[i, 0], v[p].to(F64), dtype, scale=1.0)
        close(out[i, 1], v[:p + 1].to(F64).mean(0), dtype, scale=1.0)
