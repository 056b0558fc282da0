"""The mechanisms of the Foderax design, each alone, against plain float64 formulas written here
or in tests/_ref_foderax.py (no code shared with ``lumen``).  CPU tensors take the ops' torch
path; marked ``gpu``, the same cases run the HIP kernels in fp32 and bf16.

Where random inputs would hide a fault the inputs are made so that it shows: a bias so negative
that only one aligned key far back carries weight, a sink that takes half the weight, a gate of
exactly 0 or 1, states left in a slot by another sequence, the best expert sitting in a group
that is dropped."""
import math

import pytest
import torch

import _ref_foderax as ref
from test_dalavik_ops import CASES, F64, close, paged, rnd, segments

from lumen.ops.attention import diff_head_combine, row_attention
from lumen.ops.embedding import embed_scaled, soft_cap
from lumen.ops.moe import route_groups
from lumen.ops.norm import depth_mix_norm
from lumen.ops.recurrent import min_gru_scan
from lumen.ops.rope import interleaved_inv_freq, rotary_write
from lumen.ops.segments import TILE_ROWS, SegBatch, tile_list


# ---- start of the stream, soft cap ------------------------------------------------------------------
@pytest.mark.parametrize("device,dtype", CASES)
def test_embed_scaled_and_soft_cap(device, dtype):
    V, W = 50, 24
    table = rnd(V, W, seed=7, dtype=dtype, device=device)
    toks = torch.tensor([0, 49, 3, 3, 17], device=device)
    out = torch.empty(5, W, dtype=torch.float32, device=device)
    got = embed_scaled(toks, table, 13.5, out)
    assert got.dtype == torch.float32
    close(got, table.cpu().to(F64)[toks.cpu()] * 13.5, torch.float32, scale=13.5)
    z = rnd(7, 33, seed=8, dtype=dtype, device=device, scale=20.0)
    got = soft_cap(z, 15.0)
    assert got.dtype == torch.float32
    close(got, ref.soft_cap(z.cpu().to(F64), 15.0), torch.float32, scale=15.0)


# ---- layer scales, history, depth-weighted average, next norm ----------------------------------------
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("W,n,k", [(80, 1, 1), (192, 3, 2), (30, 2, 3), (1024, 5, 3), (4100, 2, 2)])
def test_depth_mix_norm(device, dtype, W, n, k):
    T, L = 6, 6
    hist = rnd(L + 1, T, W, seed=1, device=device)
    before = hist.cpu().to(F64)
    x = rnd(T, W, seed=2, device=device, scale=2.0)
    ys = [rnd(T, W, seed=3 + i, dtype=dtype, device=device, scale=1.5) for i in range(k)]
    scales = [rnd(W, seed=10 + i, device=device) for i in range(k)]
    mix = rnd(n + 1, seed=20, device=device)
    w = rnd(W, seed=21, device=device, scale=0.1)
    new = x.cpu().to(F64) + sum(y.cpu().to(F64) * s.cpu().to(F64) for y, s in zip(ys, scales))
    want = sum(mix.cpu().to(F64)[j] * before[j] for j in range(n)) + mix.cpu().to(F64)[n] * new
    xn, h = depth_mix_norm(hist, n, x, ys, scales, mix, (1.0 + w).contiguous(), 1e-5, dtype)
    assert xn.dtype == torch.float32 and h.dtype == dtype
    close(hist[n], new, torch.float32)                         # the layer's own result is kept
    assert torch.equal(hist[:n].cpu().to(F64), before[:n])
    assert torch.equal(hist[n + 1:].cpu().to(F64), before[n + 1:])
    close(xn, want, torch.float32)
    close(h, ref.offset_rms_norm(want, w.cpu().to(F64), 1e-5), dtype)
    xn2, none = depth_mix_norm(hist, n, x, ys, scales, mix, None, 1e-5, dtype)
    assert none is None
    close(xn2, want, torch.float32)


# ---- rotary in both layouts, keys and values into the caches -----------------------------------------
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("half", [True, False])
@pytest.mark.parametrize("nq,nk,D,dims,vw", [(6, 1, 24, 24, 40), (3, 3, 10, 6, 14), (8, 4, 16, 8, 24),
                                             (2, 2, 128, 64, 256), (4, 0, 12, 4, 0), (5, 1, 8, 0, 8)])
def test_rotary_write(device, dtype, half, nq, nk, D, dims, vw):
    T = 5
    n = nq + nk
    extra = 5
    z = rnd(T, n * D + vw + extra, seed=9, dtype=dtype, device=device, scale=1.5)
    before = z.cpu().to(F64)
    pos = torch.tensor([0, 1, 97, 31, 400], dtype=torch.int32, device=device)
    slots = torch.tensor([3, -1, 30, 0, 31], device=device)
    inv = interleaved_inv_freq(dims, 5000.0, device)
    kc = torch.full((2, 16, max(nk, 1), D), 7.0, dtype=dtype, device=device) if nk else None
    vc = torch.full((2, 16, 1, max(vw, 1)), 7.0, dtype=dtype, device=device) if nk else None
    rotary_write(z, pos, slots, kc, vc, nq, nk, D, dims, inv, half)
    heads = before[:, :n * D].view(T, n, D)
    want = []
    for t in range(T):
        p = int(pos[t])
        row = heads[t:t + 1].transpose(0, 1)                  # [n, 1, D] as a "sequence" of one
        f = torch.tensor([5000.0 ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
        a = p * f
        c, s = torch.cos(a), torch.sin(a)
        r = row.clone()
        if dims:
            if half:
                u, v = row[..., :dims // 2], row[..., dims // 2:dims]
                r[..., :dims // 2], r[..., dims // 2:dims] = u * c - v * s, v * c + u * s
            else:
                u, v = row[..., 0:dims:2], row[..., 1:dims:2]
                r[..., 0:dims:2], r[..., 1:dims:2] = u * c - v * s, v * c + u * s
        want.append(r.transpose(0, 1))
    want = torch.cat(want, 0).reshape(T, n * D)
    close(z[:, :n * D], want, dtype, scale=16.0)       # fp32 angles: 400 rad carry 2e-5 rad
    assert torch.equal(z[:, n * D:].cpu().to(F64), before[:, n * D:])      # values and the rest stay
    if nk:
        for t, sl in enumerate(slots.tolist()):
            if sl >= 0:
                assert torch.equal(kc.view(32, -1)[sl], z[t, nq * D:n * D])
                assert torch.equal(vc.view(32, -1)[sl], z[t, n * D:n * D + vw])
        assert bool((kc.view(32, -1)[1] == 7.0).all()) and bool((vc.view(32, -1)[5] == 7.0).all())
    if dims >= 4:
        # the two layouts pair different entries: the other one gives another answer
        other = z.clone()
        other[:, :n * D] = before[:, :n * D].to(dtype).to(device)
        rotary_write(other, pos, slots, None, None, n, 0, D, dims, inv, not half)
        assert float((other[:, :n * D].cpu().to(F64) - want).abs().max()) > 0.05


# ---- the gated recurrence ---------------------------------------------------------------------------
def gru_segments(spans, slots, device, tile=0):
    cu, row_seg = [0], []
    for i, (_, n) in enumerate(spans):
        cu.append(cu[-1] + n)
        row_seg += [i] * n
    i32 = dict(dtype=torch.int32, device=device)
    seg = SegBatch(torch.tensor(cu, **i32), torch.tensor(slots, **i32),
                   torch.tensor([p0 for p0, _ in spans], **i32), torch.tensor(row_seg, **i32),
                   torch.zeros(cu[-1], **i32))
    return seg, cu


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("width", [72, 30, 224, 1000])
@pytest.mark.parametrize("tiled", [False, True])
def test_min_gru_scan(device, dtype, width, tiled):
    """Prompt portions longer and shorter than a tile, a fresh sequence in a slot that holds
    another one's state, continued sequences, decoded rows after the portions: every row against
    the sequential float64 recurrence."""
    spans = [(0, 300), (40, 131), (0, 2), (7, 1), (0, 1), (99, 1)]     # (start position, rows)
    n_pre = 3 if tiled else 0
    slots = [2, 0, 5, 1, 4, 3]
    seg, cu = gru_segments(spans, slots, device)
    if tiled:                                                       # portions first, then one-row segments
        tiles = tile_list(cu, n_pre, 128)
        seg.q_tiles = torch.tensor(tiles, dtype=torch.int32, device=device).view(-1, 2)
        seg.tile_rows, seg.tile_size = cu[n_pre], 128
    T = cu[-1]
    zxg = rnd(T, 3 * width + 8, seed=1, dtype=dtype, device=device, scale=2.0)
    bz, bx = rnd(width, seed=2, device=device), rnd(width, seed=3, device=device)
    state = rnd(7, width, seed=4, device=device)
    s0 = state.cpu().to(F64)
    out = min_gru_scan(zxg, bz, bx, state, seg, width, 0.5)
    assert out.dtype == dtype and tuple(out.shape) == (T, width)
    f = zxg.cpu().to(F64)
    z = torch.sigmoid(f[:, :width] + bz.cpu().to(F64))
    u = f[:, width:2 * width] + bx.cpu().to(F64)
    c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = f[:, 2 * width:3 * width]
    for i, (p0, n) in enumerate(spans):
        S = s0[slots[i]].clone() if p0 > 0 else torch.zeros(width, dtype=F64)
        rows = []
        for t in range(cu[i], cu[i + 1]):
            S = (1 - z[t]) * S + z[t] * c[t]
            rows.append(S * g[t] * torch.sigmoid(g[t]))
        want = torch.stack(rows)
        close(out[cu[i]:cu[i + 1]], want, dtype, scale=max(4.0, float(want.abs().max())))
        close(state[slots[i]], S, torch.float32, scale=4.0)        # the state moves on, in fp32
    assert torch.equal(state[6].cpu().to(F64), s0[6])               # nobody's slot is untouched


@pytest.mark.parametrize("device,dtype", CASES)
def test_min_gru_candidate_is_continuous_at_zero(device, dtype):
    """z = 1 (a huge gate logit): the state IS the candidate, u + 1/2 from 0 upwards and
    sigmoid(u) below, meeting at 1/2."""
    width = 8
    u = torch.tensor([-30.0, -1.0, -1e-3, 0.0, 1e-3, 1.0, 2.5, 30.0])
    zxg = torch.cat([torch.full((1, width), 60.0), u.view(1, -1), torch.full((1, width), 40.0)], 1)
    zxg = zxg.to(dtype).to(device)
    seg, _ = gru_segments([(0, 1)], [0], device)
    state = torch.full((1, width), 9.0, device=device)
    zero = torch.zeros(width, device=device)
    out = min_gru_scan(zxg, zero, zero, state, seg, width, 0.5)
    uu = zxg[0, width:2 * width].cpu().to(F64)
    want = torch.where(uu >= 0, uu + 0.5, torch.sigmoid(uu)) * 40.0    # silu(40) = 40
    close(out[0], want, dtype, scale=float(want.abs().max()))


# ---- attention whose weights are sigmoids --------------------------------------------------------------
SPANS = [(0, 0, 19), (1, 130, 1), (2, 60, 37), (0, 19, 1), (1, 131, 2), (2, 97, 1), (2, 98, 1)]
LENS = [20, 133, 99]
# prompt portions first (one of them longer than a tile), decoded rows after them: the layout of an
# engine step, with the tile list that sends the portions to the matrix-core kernel
SPANS_TILED = [(0, 0, 19), (2, 60, 37), (1, 3, 129), (1, 132, 1), (0, 19, 1), (2, 97, 1)]


def step_segments(tiled, tb, device):
    if not tiled:
        return segments(SPANS, tb, device), SPANS
    seg = segments(SPANS_TILED, tb, device)
    cu = seg.cu.tolist()
    seg.q_tiles = torch.tensor(tile_list(cu, 3), dtype=torch.int32, device=device).view(-1, 2)
    seg.tile_rows, seg.tile_size = cu[3], TILE_ROWS
    return seg, SPANS_TILED


def dense_sigmoid_attention(q, k, v, pos_q, hg, scale, pb):
    q, k, v = q.to(F64), k.to(F64)[:, hg], v.to(F64)[:, hg]
    T, H, _ = q.shape
    n = k.shape[0]
    s = torch.einsum("thd,nhd->htn", q, k) * scale + pb.to(F64).view(H, 1, 1)
    seen = (pos_q.view(T, 1) - torch.arange(n).view(1, n)) >= 0
    return torch.einsum("htn,nhd->thd", torch.sigmoid(s) * seen, v)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,G,D,Dv,bs", [(6, 1, 24, 40, 8), (3, 3, 10, 14, 16), (4, 2, 32, 16, 8),
                                         (16, 4, 128, 128, 16), (2, 2, 96, 192, 16),
                                         (6, 2, 64, 64, 8), (2, 1, 48, 96, 16)])
@pytest.mark.parametrize("tiled", [False, True])
def test_sigmoid_weight_attention(device, dtype, H, G, D, Dv, bs, tiled):
    ks = [rnd(n, G * D, seed=20 + i, dtype=dtype) for i, n in enumerate(LENS)]
    vs = [rnd(n, G * Dv, seed=30 + i, dtype=dtype) for i, n in enumerate(LENS)]
    kc, tb = paged(ks, bs, 40, G * D, dtype, device, 1)
    vc, _ = paged(vs, bs, 40, G * Dv, dtype, device, 1)
    seg, SPANS = step_segments(tiled, tb, device)
    T = seg.T
    q = rnd(T, H * D + 8, seed=40, dtype=dtype, device=device)[:, :H * D].view(T, H, D)
    pb = rnd(H, seed=41, device=device) - 2.0
    out = torch.zeros(T, H, Dv, dtype=dtype, device=device)
    row_attention(q, None, kc.view(40, bs, G, D), vc.view(40, bs, G, Dv), Dv, out, seg, H, G,
                  D ** -0.5, sigmoid_bias=pb)
    hg = torch.arange(H) // (H // G)
    at = 0
    for s, p0, n in SPANS:
        want = dense_sigmoid_attention(q[at:at + n].cpu(), ks[s][:p0 + n].view(-1, G, D),
                                       vs[s][:p0 + n].view(-1, G, Dv), torch.arange(p0, p0 + n),
                                       hg, D ** -0.5, pb.cpu())
        close(out[at:at + n], want, dtype, scale=max(1.0, float(want.abs().max())))
        at += n
    with pytest.raises(ValueError):                                 # nothing to normalise: no sink
        row_attention(q, None, kc.view(40, bs, G, D), vc.view(40, bs, G, Dv), Dv, out, seg, H, G,
                      1.0, sigmoid_bias=pb, sink=pb)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("far", [0, 3, 63, 64, 511, 512])
def test_sigmoid_weights_are_not_normalised(device, dtype, far):
    """700 cached keys; a bias of -16 silences all of them but one (at a tile or block border, or
    the very first), which is aligned with the query and scores +16: its weight is 1, not 1 / n,
    and rows far behind it -- in a prompt's portion or decoded, split over several workgroups or
    not -- return ITS value; two such keys return the SUM of their values."""
    n, H, D, Dv, bs = 700, 2, 16, 8, 16
    k = rnd(n, D, seed=70, dtype=torch.float32, scale=0.05)
    v = rnd(n, Dv, seed=71, dtype=torch.float32)
    d = torch.zeros(D)
    d[5] = 1.0
    k[far] = 4.0 * d
    k[far + 100] = 4.0 * d
    kc, tb = paged([k.to(dtype)], bs, 50, D, dtype, device, 3)
    vc, _ = paged([v.to(dtype)], bs, 50, Dv, dtype, device, 3)
    spans = [(0, far + 1, 40), (0, far + 50, 1), (0, 640, 1), (0, 699, 1)]
    seg = segments(spans, tb, device)
    q = (8.0 * d).to(dtype).to(device).expand(seg.T, H, D).contiguous()
    out = torch.zeros(seg.T, H, Dv, dtype=dtype, device=device)
    pb = torch.full((H,), -16.0, device=device)
    row_attention(q, None, kc.view(50, bs, 1, D), vc.view(50, bs, 1, Dv), Dv, out, seg, H, 1, 1.0,
                  sigmoid_bias=pb)
    one = v[far].to(dtype).to(F64)
    two = one + v[far + 100].to(dtype).to(F64)
    close(out[:41], one.expand(41, H, Dv), dtype, scale=1.0)
    close(out[41:], two.expand(2, H, Dv), dtype, scale=1.0)
    # a row just BEFORE the key sees nothing that counts: its output is (nearly) zero
    if far > 0:
        seg2 = segments([(0, far - 1, 1)], tb, device)
        out2 = torch.ones(1, H, Dv, dtype=dtype, device=device)
        row_attention(q[:1].contiguous(), None, kc.view(50, bs, 1, D), vc.view(50, bs, 1, Dv), Dv,
                      out2, seg2, H, 1, 1.0, sigmoid_bias=pb)
        assert float(out2.abs().max()) < 0.02


# ---- several score maps over shared values ------------------------------------------------------------
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,G,D,Dv,bs", [(4, 2, 16, 24, 8), (3, 1, 6, 10, 16), (8, 2, 64, 64, 16),
                                         (2, 2, 128, 256, 16), (3, 1, 48, 96, 8), (4, 1, 32, 64, 16),
                                         (6, 3, 96, 192, 16)])
@pytest.mark.parametrize("tiled", [False, True])
def test_two_maps_share_values(device, dtype, H, G, D, Dv, bs, tiled):
    """2 H query heads on 2 G key heads over G value heads (v_div = 2), laid out [key head][map]
    [head of the group]: every map is a softmax attention of its own over the same values."""
    rep = H // G
    ks = [rnd(n, 2 * G * D, seed=20 + i, dtype=dtype) for i, n in enumerate(LENS)]
    vs = [rnd(n, G * Dv, seed=30 + i, dtype=dtype) for i, n in enumerate(LENS)]
    kc, tb = paged(ks, bs, 40, 2 * G * D, dtype, device, 1)
    vc, _ = paged(vs, bs, 40, G * Dv, dtype, device, 1)
    seg, SPANS = step_segments(tiled, tb, device)
    T = seg.T
    q = rnd(T, 2 * H, D, seed=40, dtype=dtype, device=device, scale=2.0)
    out = torch.zeros(T, 2 * H, Dv, dtype=dtype, device=device)
    row_attention(q, None, kc.view(40, bs, 2 * G, D), vc.view(40, bs, G, Dv), Dv, out, seg, 2 * H,
                  2 * G, 0.3, v_div=2)
    at = 0
    for s, p0, n in SPANS:
        kk = ks[s][:p0 + n].to(F64).view(-1, G, 2, D)
        vv = vs[s][:p0 + n].to(F64).view(-1, G, Dv)
        qq = q[at:at + n].cpu().to(F64).view(n, G, 2, rep, D)
        sc = torch.einsum("tgmrd,ngmd->tgmrn", qq, kk) * 0.3
        seen = (torch.arange(p0, p0 + n).view(n, 1) - torch.arange(p0 + n).view(1, -1)) >= 0
        sc = sc.masked_fill(~seen.view(n, 1, 1, 1, -1), -math.inf)
        want = torch.einsum("tgmrn,ngd->tgmrd", torch.softmax(sc, -1), vv).reshape(n, 2 * H, Dv)
        close(out[at:at + n], want, dtype, scale=1.0)
        at += n


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("G,rep,Dv", [(2, 2, 24), (1, 3, 10), (2, 4, 64), (1, 1, 256), (3, 1, 500)])
def test_diff_head_combine(device, dtype, G, rep, Dv):
    T, H = 7, G * rep
    a = rnd(T, G * 2 * rep * Dv, seed=1, dtype=dtype, device=device)
    gate = rnd(T, H * Dv + 8, seed=2, dtype=dtype, device=device, scale=2.0)[:, 3:3 + H * Dv]
    lam, diff, eps = 0.37, 0.2, 1e-5
    af = a.cpu().to(F64).view(T, G, 2, rep, Dv)
    o = af[:, :, 0] - lam * af[:, :, 1]
    o = ref.rms_unit(o, eps) * (1.0 - diff)
    want = o.reshape(T, H * Dv) * torch.sigmoid(gate.cpu().to(F64))
    close(diff_head_combine(a, lam, 1.0 - diff, eps, gate, G, rep, Dv), want, dtype, scale=3.0)
    close(diff_head_combine(a, lam, 1.0 - diff, eps, None, G, rep, Dv), o.reshape(T, H * Dv), dtype,
          scale=3.0)


# ---- latent attention: sink and per-head gate -----------------------------------------------------------
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("R,transposed", [(32, False), (128, True), (20, False), (64, True)])
def test_latent_rows_with_sink_and_gate(device, dtype, R, transposed):
    """All keys score 0 and the sink is ln(n): the denominator doubles, so a head's output is half
    the values' mean -- times sigmoid(gate): gates of -1e4, 0 and ln 3 give 0, 1/2 and 3/4 of it.
    Through the row kernel and (with the per-block transposed copy) the matrix-core kernel, a
    decoded row whose keys are split over workgroups and prompt rows."""
    n, H, bs = 150, 3, 16
    rows = rnd(n, R, seed=80, dtype=dtype)
    cache, tb = paged([rows], bs, 12, R, dtype, device, 4, fill=0.0)
    vt = cache.transpose(1, 2).contiguous() if transposed else None
    spans = [(0, n - 1, 1), (0, 30, 50)]
    seg = segments(spans, tb, device)
    T = seg.T
    q = torch.zeros(H, T, R, dtype=dtype, device=device)
    gate = torch.tensor([-1e4, 0.0, math.log(3.0)], dtype=dtype, device=device).expand(T, H).contiguous()
    out = torch.zeros(H, T, R, dtype=dtype, device=device)
    pos = seg.positions.cpu()
    sink = torch.log(pos.to(F64) + 1.0)                          # differs per row: one call per row kind
    for lo, hi in ((0, 1), (1, T)):
        sub = segments([spans[0]] if lo == 0 else [spans[1]], tb, device)
        if lo == 0:
            sk = torch.full((H,), float(sink[0]), device=device)
            row_attention(q[:, :1].transpose(0, 1), None, cache, cache, R, out[:, :1].transpose(0, 1),
                          sub, H, 1, 0.2, sink=sk, vt=vt, gate=gate[:1])
    mean = rows.to(F64).mean(0)
    want = 0.5 * mean.view(1, R) * torch.tensor([0.0, 0.5, 0.75], dtype=F64).view(H, 1)
    close(out[:, 0], want, dtype, scale=1.0)
    # prompt rows, one sink for all: row at position p has p + 1 keys of weight 1 and the sink
    sk = torch.full((H,), math.log(40.0), device=device)
    sub = segments([spans[1]], tb, device)
    row_attention(q[:, 1:].transpose(0, 1), None, cache, cache, R, out[:, 1:].transpose(0, 1), sub, H,
                  1, 0.2, sink=sk, vt=vt, gate=gate[1:])
    for i, p in enumerate(range(30, 80)):
        m = rows[:p + 1].to(F64).sum(0) / (p + 1 + 40.0)
        close(out[2, 1 + i], 0.75 * m, dtype, scale=1.0)
        assert float(out[0, 1 + i].abs().max()) == 0.0


# ---- the router -----------------------------------------------------------------------------------------
def dense_route(z, top, n, keep):
    T, E = z.shape
    s = torch.softmax(z.to(F64), -1)
    c = s
    if n > 1 and keep < n:
        sg = s.view(T, n, E // n)
        best = torch.sort(sg.max(-1).values, dim=-1, descending=True, stable=True).indices[:, :keep]
        allow = torch.zeros(T, n, dtype=torch.bool).scatter_(1, best, True)
        c = sg.masked_fill(~allow.view(T, n, 1), -math.inf).reshape(T, E)
    idx = torch.sort(c, dim=-1, descending=True, stable=True).indices[:, :top]
    return torch.zeros(T, E, dtype=F64).scatter_(1, idx, torch.gather(s, 1, idx))


@pytest.mark.parametrize("device", ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)])
@pytest.mark.parametrize("E,top,n,keep", [(12, 3, 2, 1), (8, 3, 4, 2), (5, 2, 1, 1), (6, 6, 6, 6),
                                          (32, 4, 8, 3), (256, 8, 8, 4), (9, 4, 3, 3), (1, 1, 1, 1)])
def test_softmax_router_with_group_limit(device, E, top, n, keep):
    z = rnd(64, E, seed=5, device=device, scale=2.0)
    got = route_groups(z, None, top, n, keep, 1.0, rank_top=1, score="softmax", normalize=False)
    want = dense_route(z.cpu(), top, n, keep)
    close(got, want, torch.float32, scale=1.0)
    assert bool(((got > 0).sum(-1) == top).all())
    # the weights are the scores themselves: they do not sum to one unless every expert is chosen
    if top < E:
        assert float(got.sum(-1).max()) < 1.0


@pytest.mark.parametrize("device", ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)])
def test_best_expert_in_a_dropped_group(device):
    """Group 0 holds the single best expert, group 1 the next three; with one group kept a group
    ranks by its BEST member, so group 0 wins and all three choices come from it -- a rank by the
    sum of two members would keep group 1 instead."""
    z = torch.tensor([[4.5, 0.0, -1.0, -2.0, 4.0, 3.9, 3.8, -3.0]], device=device)
    got = route_groups(z, None, 3, 2, 1, 1.0, rank_top=1, score="softmax", normalize=False)
    s = torch.softmax(z.cpu().to(F64), -1)
    assert sorted(got[0].nonzero().view(-1).tolist()) == [0, 1, 2]
    close(got[0, :3], s[0, :3], torch.float32, scale=1.0)
    other = route_groups(z, None, 3, 2, 1, 1.0, rank_top=2, score="softmax", normalize=False)
    assert sorted(other[0].nonzero().view(-1).tolist()) == [4, 5, 6]
