"""The sequence-mixing ops against the float64 oracle of tests/_ref_gedatar.py, one mechanism at
a time, on steps cut into segments: whole sequences, pieces down to two tokens and single rows,
state slots holding stale values and cache blocks in scrambled order.  The HIP kernels
(lumen/csrc/seqmix) run every case (marked ``gpu``); the ops' torch path, which the CPU engine
uses, runs the mixed-pieces fp32 case of each."""
import math

import pytest
import torch

from _ref_gedatar import (F64, ref_attention, ref_canon, ref_delta, ref_dyt, ref_route,
                          ref_token_shift, ref_unit_rms, ref_wkv)

DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(autouse=True)
def _device(request):
    """Tests whose parameters start with the device run there; all others on the GPU."""
    global DEV
    DEV = request.node.callspec.params.get("dev", "cuda") if hasattr(request.node, "callspec") \
        else "cuda"
    yield
    DEV = "cuda"


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2.5e-2, atol=2.5e-2)


def cut_steps(lengths, pieces, seed):
    """Steps for sequences of ``lengths``: each step holds at most one piece per sequence; piece
    sizes cycle through ``pieces``.  Yields lists of (seq, lo, hi)."""
    g = torch.Generator().manual_seed(seed)
    at = [0] * len(lengths)
    k = 0
    while any(a < n for a, n in zip(at, lengths)):
        step = []
        for s, n in enumerate(lengths):
            if at[s] >= n or (len(lengths) > 1 and torch.rand((), generator=g) < 0.25):
                continue
            c = min(pieces[k % len(pieces)], n - at[s])
            k += 1
            step.append((s, at[s], at[s] + c))
            at[s] += c
        if step:
            yield step


def seg_of(step, slots, tables=None, bs=16, tiled=False, tile_size=64):
    from lumen.ops.segments import SegBatch, tile_list

    i32 = dict(dtype=torch.int32, device=DEV)
    cu, row_seg, pos, cs = [0], [], [], []
    for i, (s, lo, hi) in enumerate(step):
        cu.append(cu[-1] + hi - lo)
        row_seg += [i] * (hi - lo)
        pos += list(range(lo, hi))
        if tables is not None:
            cs += [tables[s][p // bs] * bs + p % bs for p in range(lo, hi)]
    tb = None
    if tables is not None:
        mb = max(len(t) for t in tables)
        tb = torch.tensor([tables[s] + [0] * (mb - len(tables[s])) for s, _, _ in step], **i32)
    sb = SegBatch(torch.tensor(cu, **i32), torch.tensor([slots[s] for s, _, _ in step], **i32),
                  torch.tensor([lo for _, lo, _ in step], **i32), torch.tensor(row_seg, **i32),
                  torch.tensor(pos, **i32), tb,
                  torch.tensor(cs, dtype=torch.long, device=DEV) if tables is not None else None)
    if tiled:       # every segment through the matrix-core tiles (where the op has them)
        sb.q_tiles = torch.tensor(tile_list(cu, len(step), tile_size), **i32).view(-1, 2)
        sb.tile_rows, sb.tile_size = cu[-1], tile_size
    return sb


def gather(step, per_seq):
    return torch.cat([per_seq[s][lo:hi] for s, lo, hi in step], 0)


def scatter(step, rows, outs):
    r = 0
    for s, lo, hi in step:
        outs[s][lo:hi] = rows[r:r + hi - lo].to("cpu", F64)
        r += hi - lo


LENGTHS = [37, 5, 70, 2]
SLOTS = [3, 0, 5, 1]
PIECES = [[1000], [7, 2, 1, 16, 3], [1], [2]]
GPU = pytest.mark.gpu
# (device, dtype, pieces): every combination on the GPU, one on the CPU path
CASES = [pytest.param("cuda", d, p, marks=GPU, id=f"cuda-{str(d)[6:]}-{i}")
         for d in DTYPES for i, p in enumerate(PIECES)] + [
    pytest.param("cpu", torch.float32, PIECES[1], id="cpu-float32-1")]
DEVS = ["cpu", pytest.param("cuda", marks=GPU)]


@pytest.mark.parametrize("dev,dtype,pieces", CASES)
@pytest.mark.parametrize("taps,W", [(1, 96), (2, 96), (4, 96), (3, 50), (10, 24)])
def test_dyt_canon_segments(dev, dtype, pieces, taps, W):
    """(Widths that are / are not a multiple of 4 and more than 8 taps take different kernels.)"""
    from lumen.ops.conv import dyt_canon

    torch.manual_seed(taps)
    norm = (torch.randn(W) * 0.2 + 1, torch.randn(W) * 0.1, torch.tensor(0.7))
    cw = torch.randn(W, taps) * 0.4
    xs = [torch.randn(n, W) for n in LENGTHS]
    ref = [ref_canon(ref_dyt(x.to(F64), *[t.to(F64) for t in norm]), cw.to(F64)) for x in xs]
    tail = torch.full((8, max(taps - 1, 0), W), 7.0, device=DEV)   # stale values in every slot
    nd = tuple(t.to(DEV) for t in norm)
    got = [torch.zeros(n, W, dtype=F64) for n in LENGTHS]
    for step in cut_steps(LENGTHS, pieces, 1):
        out = dyt_canon(gather(step, xs).to(DEV), nd, cw.to(DEV), tail, seg_of(step, SLOTS), dtype)
        scatter(step, out, got)
    for g, r in zip(got, ref):
        torch.testing.assert_close(g, r, **tol(dtype))


@pytest.mark.parametrize("dev,dtype", [("cpu", torch.float32)] + [
    pytest.param("cuda", d, marks=GPU) for d in DTYPES])
@pytest.mark.parametrize("W", [80, 42])
def test_dyt_and_residual(dev, dtype, W):
    from lumen.ops.norm import dyt, dyt_residual

    torch.manual_seed(0)
    T = 33
    n1 = (torch.randn(W) + 1, torch.randn(W) * 0.1, torch.tensor(0.4))
    n2 = (torch.randn(W) + 1, torch.randn(W) * 0.1, torch.tensor(1.3))
    x, y = torch.randn(T, W), torch.randn(T, W).to(dtype)
    d = lambda n: tuple(t.to(DEV) for t in n)  # noqa: E731
    r64 = lambda n: [t.to(F64) for t in n]  # noqa: E731
    xr = x.to(F64) + ref_dyt(y.to(F64), *r64(n1))
    xg, h = dyt_residual(x.clone().to(DEV), y.to(DEV), d(n1), d(n2), dtype)
    torch.testing.assert_close(xg.cpu().to(F64), xr, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(h.cpu().to(F64), ref_dyt(xr, *r64(n2)), **tol(dtype))
    xg2, none = dyt_residual(x.clone().to(DEV), y.to(DEV), d(n1), None, dtype)
    assert none is None
    torch.testing.assert_close(xg2.cpu().to(F64), xr, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(dyt(x.to(DEV), d(n2), dtype).cpu().to(F64),
                               ref_dyt(x.to(F64), *r64(n2)), **tol(dtype))


@pytest.mark.parametrize("dev,dtype,pieces", CASES)
@pytest.mark.parametrize("W", [72, 30])
def test_token_shift_segments(dev, dtype, pieces, W):
    from lumen.ops.recurrent import token_shift

    torch.manual_seed(2)
    mu = torch.rand(5, W)
    hs = [torch.randn(n, W).to(dtype) for n in LENGTHS]
    ref = [ref_token_shift(h.to(F64), mu.to(F64)) for h in hs]
    prev = torch.full((8, W), -3.0, device=DEV)
    got = [torch.zeros(5, n, W, dtype=F64) for n in LENGTHS]
    for step in cut_steps(LENGTHS, pieces, 2):
        out = token_shift(gather(step, hs).to(DEV), mu.to(DEV), prev, seg_of(step, SLOTS))
        r = 0
        for s, lo, hi in step:
            got[s][:, lo:hi] = out[:, r:r + hi - lo].to("cpu", F64)
            r += hi - lo
    for g, r in zip(got, ref):
        torch.testing.assert_close(g, r, **tol(dtype))


def _scan_inputs(H, D, dtype, seed, n_in):
    g = torch.Generator().manual_seed(seed)
    mk = lambda n, s=1.0: (torch.randn(n, H * D, generator=g) * s).to(dtype)  # noqa: E731
    return [[mk(n, 0.7) for _ in range(n_in)] for n in LENGTHS], g


@pytest.mark.parametrize("dev,dtype,pieces", CASES)
@pytest.mark.parametrize("H,D", [(2, 32), (3, 48), (1, 64), (2, 80), (1, 256)])
def test_wkv_scan_segments(dev, dtype, pieces, H, D):
    from lumen.ops.recurrent import wkv_scan

    ins, g = _scan_inputs(H, D, dtype, D, 5)         # r k v wl gate
    w0 = torch.linspace(-3, 0.5, H * D)
    u = torch.randn(H * D, generator=g) * 0.5
    nw = torch.randn(H * D, generator=g) * 0.2 + 1
    eps = 1e-5
    ref = []
    for r, k, v, wl, gl in ins:
        f = lambda t: t.to(F64).view(-1, H, D)  # noqa: E731
        w = torch.exp(-torch.exp(wl.to(F64) + w0.to(F64))).view(-1, H, D)
        o = ref_unit_rms(ref_wkv(f(r), f(k), f(v), w, u.to(F64).view(H, D)), eps)
        ref.append(o.reshape(-1, H * D) * nw.to(F64) * torch.nn.functional.silu(gl.to(F64)))
    state = torch.full((8, H, D, D), 9.0, device=DEV)
    got = [torch.zeros(n, H * D, dtype=F64) for n in LENGTHS]
    for step in cut_steps(LENGTHS, pieces, 3):
        a = [gather(step, [x[i] for x in ins]).to(DEV) for i in range(5)]
        out = wkv_scan(a[0], a[1], a[2], a[3], a[4], w0.to(DEV), u.to(DEV), nw.to(DEV), state,
                       seg_of(step, SLOTS), H, D, eps)
        scatter(step, out, got)
    for gg, r in zip(got, ref):
        torch.testing.assert_close(gg, r, **tol(dtype))


@pytest.mark.parametrize("dev,dtype,pieces", CASES)
@pytest.mark.parametrize("H,D", [(2, 32), (3, 48), (1, 128), (1, 200)])
def test_delta_scan_segments(dev, dtype, pieces, H, D):
    from lumen.ops.recurrent import delta_scan

    ins, g = _scan_inputs(H, D, dtype, D + 1, 6)     # r k v wl al gl
    w0 = torch.randn(H * D, generator=g)
    ab = torch.randn(H * D, generator=g) * 0.3
    nw = torch.randn(H * D, generator=g) * 0.2 + 1
    eps, cdec, keps = 1e-5, 0.61, 1e-6
    ref = []
    for r, k, v, wl, al, gl in ins:
        f = lambda t: t.to(F64).view(-1, H, D)  # noqa: E731
        w = torch.exp(-cdec * torch.sigmoid(wl.to(F64) + w0.to(F64))).view(-1, H, D)
        a = torch.sigmoid(al.to(F64) + ab.to(F64)).view(-1, H, D)
        o = ref_unit_rms(ref_delta(f(r), f(k), f(v), w, a, keps), eps)
        ref.append(o.reshape(-1, H * D) * nw.to(F64) * torch.sigmoid(gl.to(F64)))
    state = torch.full((8, H, D, D), 9.0, device=DEV)
    got = [torch.zeros(n, H * D, dtype=F64) for n in LENGTHS]
    for step in cut_steps(LENGTHS, pieces, 4):
        a = [gather(step, [x[i] for x in ins]).to(DEV) for i in range(6)]
        out = delta_scan(a[0], a[1], a[2], a[3], a[4], a[5], w0.to(DEV), ab.to(DEV), nw.to(DEV),
                         state, seg_of(step, SLOTS), H, D, eps, cdec, keps)
        scatter(step, out, got)
    for gg, r in zip(got, ref):
        torch.testing.assert_close(gg, r, **tol(dtype))


@pytest.mark.gpu
def test_scan_strided_inputs_match_contiguous():
    """Column slices of one fused projection (row stride > H * D) give the same result."""
    from lumen.ops.recurrent import wkv_scan

    torch.manual_seed(5)
    H, D, T = 2, 32, 19
    z = torch.randn(T, 5 * H * D, device=DEV, dtype=torch.bfloat16)
    parts = [z[:, i * H * D:(i + 1) * H * D] for i in range(5)]
    w0, u, nw = (torch.randn(H * D, device=DEV) for _ in range(3))
    step = [(0, 0, T)]
    outs = []
    for ps in (parts, [p.contiguous() for p in parts]):
        st = torch.zeros(2, H, D, D, device=DEV)
        outs.append(wkv_scan(*ps, w0, u, nw, st, seg_of(step, [1]), H, D, 1e-5))
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("dev,dtype,pieces", CASES)
@pytest.mark.parametrize("H,G,D,chunk,bs", [(4, 2, 32, 24, 16), (2, 2, 64, 16, 16),
                                             (6, 1, 40, 33, 8), (3, 3, 20, 0, 16)])
def test_chunk_sink_attention_segments(dev, dtype, pieces, H, G, D, chunk, bs):
    from lumen.ops.attention import chunk_sink_attention, write_key_cache

    torch.manual_seed(H * D + chunk)
    scale, eps = 0.3, 1e-5
    qs = [torch.randn(n, H * D).to(dtype) for n in LENGTHS]
    ks = [torch.randn(n, G * D).to(dtype) for n in LENGTHS]
    ref = [ref_attention(q.to(F64).view(-1, H, D), k.to(F64).view(-1, G, D), scale, chunk, eps)
           .reshape(-1, H * D) for q, k in zip(qs, ks)]
    # scrambled block tables
    nb = sum((n + bs - 1) // bs for n in LENGTHS)
    perm = torch.randperm(nb + 3).tolist()
    tables, at = [], 0
    for n in LENGTHS:
        c = (n + bs - 1) // bs
        tables.append(perm[at:at + c])
        at += c
    cache = torch.full((nb + 3, bs, G, D), 50.0, device=DEV, dtype=dtype)
    got = [torch.zeros(n, H * D, dtype=F64) for n in LENGTHS]
    for step in cut_steps(LENGTHS, pieces, 5):
        sg = seg_of(step, SLOTS, tables, bs, tiled=(H + chunk) % 2 == 0)
        write_key_cache(gather(step, ks).to(DEV), cache, sg.cache_slots)
        out = chunk_sink_attention(gather(step, qs).to(DEV), cache, sg, H, G, D, scale, chunk, eps)
        scatter(step, out, got)
    for gg, r in zip(got, ref):
        torch.testing.assert_close(gg, r, **tol(dtype))


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("pieces", [[1000], [1], [3, 1, 2]])
def test_attention_chunk_edges_and_sink_show(dev, pieces):
    """One key per chunk is made to dominate (an aligned query / key pair among small random
    ones), so a mask that is one position off, or a missing sink, moves the output by far more
    than the tolerance: the kernel must match the oracle and differ from both wrong variants."""
    from lumen.ops.attention import chunk_sink_attention, write_key_cache

    H = G = 1
    D, chunk, T, bs, scale = 32, 8, 40, 16, 0.12
    torch.manual_seed(11)
    k = torch.randn(T, D) * 0.3
    q = torch.randn(T, D) * 0.3
    d0 = torch.zeros(D)
    d0[3] = 1.0
    for c0 in range(0, T, chunk):
        k[c0] += 6 * d0                     # first key of every chunk points along d0
    q[:] += 6 * d0                          # every query looks along d0
    q64, k64 = q.to(F64).view(T, 1, D), k.to(F64).view(T, 1, D)
    ref = ref_attention(q64, k64, scale, chunk, 1e-6).view(T, D)
    cache = torch.zeros(4, bs, 1, D, device=DEV)
    got = [torch.zeros(T, D, dtype=F64)]
    for step in cut_steps([T], pieces, 0):   # prompt rows and decoded rows, chunk edges at and
        sg = seg_of(step, [0], [[2, 0, 3]], bs)   # between block borders (chunk 8, blocks of 16)
        write_key_cache(gather(step, [k]).to(DEV), cache, sg.cache_slots)
        scatter(step, chunk_sink_attention(gather(step, [q]).to(DEV), cache, sg, H, G, D, scale,
                                           chunk, 1e-6), got)
    out = got[0]
    torch.testing.assert_close(out, ref, rtol=1e-5, atol=1e-5)
    for wrong in (ref_attention(q64, k64, scale, chunk + 1, 1e-6),
                  ref_attention(q64, k64, scale, chunk - 1, 1e-6),
                  ref_attention(q64, k64, scale, 0, 1e-6),
                  ref_attention(q64, k64, scale, chunk, 1e-6, sink=False)):
        assert float((wrong.view(T, D) - ref).abs().max()) > 0.05


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("E,top", [(6, 3), (12, 2), (5, 1), (70, 4), (4, 4)])
def test_route_topk(dev, E, top):
    from lumen.ops.moe import route_topk

    torch.manual_seed(E)
    z = torch.randn(45, E)
    z[0, :] = 0.25                          # all equal: lowest indices win
    got = route_topk(z.to(DEV), top).cpu()
    torch.testing.assert_close(got.to(F64), ref_route(z.to(F64), top), rtol=1e-5, atol=1e-6)
    assert ((got > 0).sum(1) == top).all()


@pytest.mark.parametrize("dev,dtype", [("cpu", torch.float32)] + [
    pytest.param("cuda", d, marks=GPU) for d in DTYPES])
@pytest.mark.parametrize("E,ff,ffs", [(0, 0, 96), (5, 24, 40), (3, 16, 0), (4, 12, 20)])
def test_gated_act(dev, dtype, E, ff, ffs):
    from lumen.ops.moe import gated_act

    torch.manual_seed(ff + ffs)
    T = 21
    gu = torch.randn(T, E * 2 * ff + 2 * ffs).to(dtype)
    wts = torch.rand(T, E) * (torch.rand(T, E) > 0.5) if E else None
    parts = []
    g64 = gu.to(F64)
    for e in range(E):
        b = g64[:, e * 2 * ff:(e + 1) * 2 * ff]
        parts.append(torch.nn.functional.silu(b[:, :ff]) * b[:, ff:] * wts[:, e:e + 1].to(F64))
    if ffs:
        b = g64[:, E * 2 * ff:]
        parts.append(torch.nn.functional.silu(b[:, :ffs]) * b[:, ffs:])
    got = gated_act(gu.to(DEV), wts.to(DEV) if E else None, E, ff, ffs).cpu().to(F64)
    torch.testing.assert_close(got, torch.cat(parts, 1), **tol(dtype))


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("kind", ["wkv", "delta"])
@pytest.mark.parametrize("pieces", [[1000], [64, 1], [2]])
def test_far_token_reaches_through_the_state(dev, kind, pieces):
    """A write 250 tokens back, on slowly decaying channels, must still dominate the read-out: the
    early token's key / value are large, a late query is aligned with that key.  A state that is
    lost, reset or decayed by the wrong factor anywhere on the way changes the result by far more
    than the tolerance (the oracle without the early token differs by > 0.5)."""
    from lumen.ops.recurrent import delta_scan, wkv_scan

    torch.manual_seed(7)
    H, D, T, far, late = 2, 32, 260, 4, 255
    mk = lambda s: torch.randn(T, H * D) * s  # noqa: E731
    r, k, v, gl = mk(0.1), mk(0.1), mk(0.1), mk(1.0)
    wl = torch.zeros(T, H * D)
    al = torch.full((T, H * D), -6.0)                  # removal rate ~ 0
    key = torch.zeros(H * D)
    key[5], key[D + 9] = 4.0, 4.0
    k[far] += key
    v[far] += 3.0
    r[late] += key
    w0 = torch.full((H * D,), -7.0)                    # decay ~ 1 per step
    u = torch.zeros(H * D)
    ab = torch.zeros(H * D)
    nw = torch.ones(H * D)
    eps = 1e-6

    def ref_of(k_, v_):
        f = lambda t: t.to(F64).view(T, H, D)  # noqa: E731
        if kind == "wkv":
            w = torch.exp(-torch.exp(wl.to(F64) + w0.to(F64))).view(T, H, D)
            o = ref_wkv(f(r), f(k_), f(v_), w, u.to(F64).view(H, D))
            gate = torch.nn.functional.silu(gl.to(F64))
        else:
            w = torch.exp(-0.61 * torch.sigmoid(wl.to(F64) + w0.to(F64))).view(T, H, D)
            o = ref_delta(f(r), f(k_), f(v_), w, torch.sigmoid(al.to(F64) + ab.to(F64)).view(T, H, D))
            gate = torch.sigmoid(gl.to(F64))
        return ref_unit_rms(o, eps).reshape(T, H * D) * gate

    ref = ref_of(k, v)
    k0, v0 = k.clone(), v.clone()
    k0[far] -= key
    v0[far] -= 3.0
    assert float((ref_of(k0, v0)[late] - ref[late]).abs().max()) > 0.5
    state = torch.full((3, H, D, D), 5.0, device=DEV)
    got = [torch.zeros(T, H * D, dtype=F64)]
    for step in cut_steps([T], pieces, 0):
        a = [gather(step, [x]).to(DEV) for x in (r, k, v, wl, al, gl)]
        sg = seg_of(step, [2])
        if kind == "wkv":
            out = wkv_scan(a[0], a[1], a[2], a[3], a[5], w0.to(DEV), u.to(DEV), nw.to(DEV), state,
                           sg, H, D, eps)
        else:
            out = delta_scan(a[0], a[1], a[2], a[3], a[4], a[5], w0.to(DEV), ab.to(DEV),
                             nw.to(DEV), state, sg, H, D, eps, 0.61, 1e-6)
        scatter(step, out, got)
    torch.testing.assert_close(got[0], ref, rtol=2e-4, atol=2e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("pieces", [[1000], [64, 1, 70, 2, 33]])
@pytest.mark.parametrize("tile_size", [64, 128])
@pytest.mark.parametrize("H,G,D,chunk,bs", [(4, 2, 128, 48, 16), (2, 1, 96, 100, 16),
                                             (3, 3, 32, 0, 8), (2, 2, 64, 5, 16),
                                             (1, 1, 256, 64, 16), (2, 1, 192, 31, 4)])
def test_tile_attention_matches_oracle(dtype, pieces, tile_size, H, G, D, chunk, bs):
    """The matrix-core prefill kernel: several 64-row tiles per segment, chunks that start inside
    a tile, span tiles or are smaller than a key tile, segments that start mid-sequence; and the
    row kernel on the same rows gives the same result to rounding."""
    from lumen.ops.attention import chunk_sink_attention, write_key_cache

    torch.manual_seed(D + chunk)
    lengths, slots = [150, 33, 200], [0, 1, 2]
    scale, eps = 0.6 / math.sqrt(D), 1e-5
    qs = [(torch.randn(n, H * D) * 1.5).to(dtype) for n in lengths]
    ks = [(torch.randn(n, G * D) * 1.5).to(dtype) for n in lengths]
    ref = [ref_attention(q.to(F64).view(-1, H, D), k.to(F64).view(-1, G, D), scale, chunk, eps)
           .reshape(-1, H * D) for q, k in zip(qs, ks)]
    nb = sum((n + bs - 1) // bs for n in lengths)
    perm = torch.randperm(nb + 2).tolist()
    tables, at = [], 0
    for n in lengths:
        c = (n + bs - 1) // bs
        tables.append(perm[at:at + c])
        at += c
    cache = torch.full((nb + 2, bs, G, D), 30.0, device=DEV, dtype=dtype)
    got = [torch.zeros(n, H * D, dtype=F64) for n in lengths]
    rows = [torch.zeros(n, H * D, dtype=F64) for n in lengths]
    for step in cut_steps(lengths, pieces, 6):
        sg = seg_of(step, slots, tables, bs, tiled=True, tile_size=tile_size)
        write_key_cache(gather(step, ks).to(DEV), cache, sg.cache_slots)
        qd = gather(step, qs).to(DEV)
        scatter(step, chunk_sink_attention(qd, cache, sg, H, G, D, scale, chunk, eps), got)
        sg.q_tiles, sg.tile_rows = None, 0
        scatter(step, chunk_sink_attention(qd, cache, sg, H, G, D, scale, chunk, eps), rows)
    t = dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(rtol=3e-3, atol=3e-3)
    for g_, r_, ref_ in zip(got, rows, ref):
        torch.testing.assert_close(g_, ref_, **t)
        torch.testing.assert_close(g_, r_, **t)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("E,top,ff,ffs", [(6, 2, 24, 40), (4, 1, 16, 0), (5, 3, 8, 8)])
def test_moe_dense_and_grouped_match_oracle(dev, E, top, ff, ffs):
    """Both ways of running the experts (all experts with zero weights / each expert on its own
    rows) against a per-expert loop; ``moe`` picks by step size."""
    from lumen.ops import moe as M

    torch.manual_seed(E * top)
    T, W = 300, 64
    h = torch.randn(T, W)
    gu = torch.randn(E * 2 * ff + 2 * ffs, W) * 0.2
    dn = torch.randn(W, E * ff + ffs) * 0.2
    z = torch.randn(T, E)
    wr = ref_route(z.to(F64), top)
    ref = torch.zeros(T, W, dtype=F64)
    for e in range(E + (1 if ffs else 0)):
        n = ff if e < E else ffs
        b = gu[e * 2 * ff:e * 2 * ff + 2 * n].to(F64)
        y = (torch.nn.functional.silu(h.to(F64) @ b[:n].T) * (h.to(F64) @ b[n:].T)) \
            @ dn[:, e * ff:e * ff + n].to(F64).T
        ref += y * (wr[:, e:e + 1] if e < E else 1.0)
    hd, gd, dd = h.to(DEV), gu.to(DEV), dn.to(DEV)
    wts = M.route_topk(z.to(DEV), top)
    for fn in (M.moe_dense, M.moe_grouped):
        torch.testing.assert_close(fn(hd, wts, gd, dd, E, ff, ffs).cpu().to(F64), ref, rtol=1e-4,
                                   atol=1e-4)
    torch.testing.assert_close(M.moe(hd, wts, gd, dd, E, top, ff, ffs).cpu().to(F64), ref,
                               rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("pieces,tiled", [([1000], True), ([1000], False), ([150, 1], False),
                                           ([128, 40, 2], True)])
def test_attention_far_key_among_hundreds(dev, pieces, tiled):
    """One early key (position 3) is aligned with the queries near the end of a 200-token prompt,
    among some two hundred small random keys: rows far away must still find it -- in a prompt, in its
    portions and when decoded -- and the oracle without that key differs by far more than the
    tolerance."""
    from lumen.ops.attention import chunk_sink_attention, write_key_cache

    torch.manual_seed(21)
    H, G, D, T, bs, chunk, scale = 2, 1, 32, 200, 16, 512, 0.2
    dtype = torch.bfloat16 if (tiled and dev == "cuda") else torch.float32
    k = (torch.randn(T, D) * 0.2)
    q = (torch.randn(T, H * D) * 0.2)
    d0 = torch.zeros(D)
    d0[7] = 1.0
    k[3] += 5 * d0
    q[190:, :D] += 5 * d0                   # head 0 of the last rows looks for it
    k, q = k.to(dtype), q.to(dtype)
    q64, k64 = q.to(F64).view(T, H, D), k.to(F64).view(T, G, D)
    ref = ref_attention(q64, k64, scale, chunk, 1e-6).reshape(T, H * D)
    k0 = k64.clone()
    k0[3, 0] -= 5 * d0.to(F64)
    without = ref_attention(q64, k0, scale, chunk, 1e-6).reshape(T, H * D)
    assert float((without[190:, :D] - ref[190:, :D]).abs().max()) > 0.3
    nb = (T + bs - 1) // bs
    table = torch.randperm(nb + 1).tolist()[:nb]
    cache = torch.zeros(nb + 1, bs, G, D, device=DEV, dtype=dtype)
    got = [torch.zeros(T, H * D, dtype=F64)]
    for step in cut_steps([T], pieces, 0):
        sg = seg_of(step, [0], [table], bs, tiled=tiled)
        write_key_cache(gather(step, [k]).to(DEV), cache, sg.cache_slots)
        scatter(step, chunk_sink_attention(gather(step, [q]).to(DEV), cache, sg, H, G, D, scale,
                                           chunk, 1e-6), got)
    t = dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(got[0], ref, **t)
