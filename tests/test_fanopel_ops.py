"""The mechanisms of the Fanopel design, each alone, against plain float64 formulas written here
or in tests/_ref_fanopel.py (no code shared with ``lumen``).  CPU tensors take the ops' torch
path; marked ``gpu``, the same cases run the HIP kernels in fp32 and bf16.

Where random inputs would hide a fault the inputs are made so that it shows: a key exactly at the
window's edge or among the kept first tokens that must (or must not) take all the weight, tiles
of keys between the kept tokens and the window holding huge values, a correction that makes every
choice score negative, the best expert sitting in a group that is dropped."""
import math

import pytest
import torch

import _ref_fanopel as ref
from test_dalavik_ops import CASES, F64, close, paged, rnd, segments

from lumen.ops.attention import row_attention, row_norm_write
from lumen.ops.embedding import embed_positions
from lumen.ops.moe import (grouped_mm_ok, moe_dense, moe_grouped, moe_grouped_mm, route_groups,
                           scaled_act)
from lumen.ops.norm import scaled_residual_layer_norm, weight_layer_norm


# ---- layer norm with a weight, scaled residual ---------------------------------------------------
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("W", [112, 30, 64, 257, 1024, 4100])
def test_weight_layer_norm(device, dtype, W):
    x = rnd(7, W, seed=1, device=device, scale=3.0) + 50.0        # a mean far from 0
    w = rnd(W, seed=2, device=device) + 1.0
    want = ref.weight_layer_norm(x.cpu().to(F64), w.cpu().to(F64), 1e-5)
    got = weight_layer_norm(x, w, 1e-5, dtype)
    assert got.dtype == dtype
    close(got, want, dtype)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("W,mult", [(112, 0.7), (96, 1.0), (33, 0.25), (2048, 0.5)])
def test_scaled_residual_layer_norm(device, dtype, W, mult):
    x = rnd(9, W, seed=3, device=device)
    y = rnd(9, W, seed=4, dtype=dtype, device=device, scale=2.0)
    w = rnd(W, seed=5, device=device) + 1.0
    xs = x.cpu().to(F64) + mult * y.cpu().to(F64)
    x2, h = scaled_residual_layer_norm(x, y, mult, w, 1e-6, dtype)
    assert x2 is x and x.dtype == torch.float32 and h.dtype == dtype
    close(x, xs, torch.float32)                                    # the stream itself stays fp32
    close(h, ref.weight_layer_norm(xs, w.cpu().to(F64), 1e-6), dtype)
    # without a following norm only the stream moves on
    x3, none = scaled_residual_layer_norm(x, y, mult, None, 1e-6, dtype)
    assert none is None
    close(x3, xs + mult * y.cpu().to(F64), torch.float32)


@pytest.mark.parametrize("device,dtype", CASES)
def test_tiny_variance_feels_eps(device, dtype):
    """Rows that are almost constant: the variance is of the order of eps, which sits inside the
    root."""
    W = 48
    x = (5.0 + 1e-3 * rnd(4, W, seed=6)).to(device)
    w = torch.ones(W, device=device)
    want = ref.weight_layer_norm(x.cpu().to(F64), w.cpu().to(F64), 1e-6)
    assert float(want.abs().max()) < 0.9 * float(ref.weight_layer_norm(x.cpu().to(F64), w.cpu().to(F64), 0.0).abs().max())
    close(weight_layer_norm(x, w, 1e-6, torch.float32), want, torch.float32, scale=100.0)


@pytest.mark.parametrize("device,dtype", CASES)
def test_embed_positions(device, dtype):
    V, P, W = 50, 40, 24
    table = rnd(V, W, seed=7, dtype=dtype, device=device)
    ptab = rnd(P, W, seed=8, dtype=dtype, device=device)
    toks = torch.tensor([0, 49, 3, 3, 17], device=device)
    pos = torch.tensor([0, 39, 1, 2, 0], dtype=torch.int32, device=device)
    got = embed_positions(toks, pos, table, ptab)
    assert got.dtype == torch.float32
    want = table.cpu().to(F64)[toks.cpu()] + ptab.cpu().to(F64)[pos.cpu().long()]
    close(got, want, torch.float32)                                # the sum is not rounded to 16 bits


# ---- q / k norm over the whole projection, keys twice into the caches ---------------------------
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,G,D", [(6, 3, 24), (3, 3, 20), (1, 1, 128), (8, 1, 8), (5, 5, 7)])
def test_row_norm_write(device, dtype, H, G, D):
    T, HD, GD = 5, H * D, G * D
    extra = H + (-(HD + GD + H) % 8)                               # gate columns + padding
    z = rnd(T, HD + GD + extra, seed=9, dtype=dtype, device=device, scale=1.5)
    before = z.cpu().to(F64)
    wq, wk = rnd(HD, seed=10, device=device) + 1.0, rnd(GD, seed=11, device=device) + 1.0
    slots = torch.tensor([3, -1, 30, 0, 31], device=device)
    kc = torch.full((2, 16, G, D), 7.0, dtype=dtype, device=device)
    vc = torch.full((2, 16, G, D), 7.0, dtype=dtype, device=device)
    row_norm_write(z, wq, wk, slots, kc, vc, HD, GD, 1e-6)
    q = ref.rms_unit(before[:, :HD], 1e-6) * wq.cpu().to(F64)      # ONE root mean square per row
    k = ref.rms_unit(before[:, HD:HD + GD], 1e-6) * wk.cpu().to(F64)
    close(z[:, :HD], q, dtype)
    assert torch.equal(z[:, HD:].cpu().to(F64), before[:, HD:])    # keys and gate columns stay
    for t, s in enumerate(slots.tolist()):
        if s >= 0:
            close(kc.view(32, GD)[s], k[t], dtype)
            assert torch.equal(vc.view(32, GD)[s].cpu().to(F64), before[t, HD:HD + GD])
    assert bool((kc.view(32, -1)[1] == 7.0).all()) and bool((vc.view(32, -1)[5] == 7.0).all())
    if H > 1:
        # heads of unequal size: per-head norms would give another answer
        per_head = ref.rms_unit(before[:, :HD].view(T, H, D), 1e-6).reshape(T, HD) * wq.cpu().to(F64)
        assert float((per_head - q).abs().max()) > 0.05


# ---- row attention: window, kept first keys, linear distance bias, output gate -------------------
def dense_window_attention(q, k, v, pos_q, hg, scale, softcap, slopes, window, keep, gate):
    """q [T, H, D] at positions pos_q against keys / values [n, G, D] at positions 0 .. n-1 of the
    same sequence; float64, dense mask."""
    q, k, v = q.to(F64), k.to(F64)[:, hg], v.to(F64)[:, hg]
    T, H, _ = q.shape
    n = k.shape[0]
    s = torch.einsum("thd,nhd->htn", q, k) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    j = torch.arange(n).view(1, n)
    dist = pos_q.view(T, 1) - j
    if slopes is not None:
        s = s - slopes.to(F64).view(H, 1, 1) * dist.to(F64)
    seen = (dist >= 0) & ((dist < window) | (j < keep)) if window else dist >= 0
    s = s.masked_fill(~seen.view(1, T, n), -math.inf)
    o = torch.einsum("htn,nhd->thd", torch.softmax(s, -1), v)
    if gate is not None:
        o = o * torch.sigmoid(gate.to(F64)).view(T, H, 1)
    return o


SPANS = [(0, 0, 19), (1, 130, 1), (2, 60, 37), (0, 19, 1), (1, 131, 2), (2, 97, 1), (2, 98, 1),
         (3, 640, 3), (3, 699, 1)]
LENS = [20, 133, 99, 700]


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,G,D,bs,window,keep", [
    (6, 3, 24, 8, 21, 3), (3, 3, 20, 16, 70, 1), (4, 1, 32, 8, 9, 5), (9, 3, 16, 16, 64, 0),
    (32, 4, 64, 16, 65, 64), (2, 2, 40, 16, 130, 70), (4, 2, 128, 16, 1, 2), (5, 1, 12, 8, 1000, 4)])
def test_row_attention_window_bias_gate(device, dtype, H, G, D, bs, window, keep):
    """Rows of prompts' portions and decoded tokens in one step, scrambled block tables, poison
    past every sequence's end; windows shorter and longer than a tile and than the sequences,
    kept keys none, a few, a whole tile and more."""
    ks = [rnd(n, G * D, seed=20 + i, dtype=dtype) for i, n in enumerate(LENS)]
    vs = [rnd(n, G * D, seed=30 + i, dtype=dtype) for i, n in enumerate(LENS)]
    kc, tb = paged(ks, bs, 140, G * D, dtype, device, 1)
    vc, _ = paged(vs, bs, 140, G * D, dtype, device, 1)
    seg = segments(SPANS, tb, device)
    T = seg.T
    pad = -(H * D + H) % 8
    z = rnd(T, H * D + H + pad, seed=40, dtype=dtype, device=device)
    q, gate = z[:, :H * D].view(T, H, D), z[:, H * D:H * D + H]
    slopes = torch.tensor([2.0 ** (-6.0 * (h + 1) / H) for h in range(H)], device=device)
    out = torch.zeros(T, H, D, dtype=dtype, device=device)
    row_attention(q, None, kc.view(140, bs, G, D), vc.view(140, bs, G, D), D, out, seg, H, G, 0.3,
                  softcap=5.0, slopes=slopes, window=window, keep_first=keep, gate=gate)
    hg = torch.arange(H) // (H // G)
    at = 0
    for s, p0, n in SPANS:
        pos = torch.arange(p0, p0 + n)
        want = dense_window_attention(q[at:at + n].cpu(), ks[s][:p0 + n].view(-1, G, D),
                                      vs[s][:p0 + n].view(-1, G, D), pos, hg, 0.3, 5.0,
                                      slopes.cpu(), window, keep, gate[at:at + n].cpu())
        close(out[at:at + n], want, dtype, scale=1.0)
        at += n


def tiled_segments(spans, n_prompt, tables, device, rows):
    """As ``segments``, with the first ``n_prompt`` spans cut into tiles of ``rows`` rows: the
    form in which the engine hands a step's prompt portions to the matrix-core kernel."""
    from lumen.ops.segments import tile_list

    seg = segments(spans, tables, device)
    cu = seg.cu.tolist()
    seg.q_tiles = torch.tensor(tile_list(cu, n_prompt, rows), dtype=torch.int32,
                               device=device).view(-1, 2)
    seg.tile_rows, seg.tile_size = cu[n_prompt], rows
    return seg


TILE_SPANS = [(0, 0, 20), (2, 60, 39), (3, 310, 390), (1, 100, 33), (4, 0, 1), (5, 7, 2),
              (6, 0, 300),                                         # prompt portions ...
              (7, 130, 1), (8, 299, 1)]                            # ... then decoded rows
TILE_LENS = [20, 133, 99, 700, 1, 9, 300, 131, 300]             # by sequence


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows", [64, 128])
@pytest.mark.parametrize("H,G,D,bs,window,keep", [
    (4, 2, 32, 8, 21, 3), (3, 3, 64, 16, 70, 1), (4, 1, 96, 16, 150, 5), (8, 2, 128, 16, 64, 0),
    (2, 2, 128, 16, 65, 64), (2, 1, 192, 16, 130, 70), (2, 2, 256, 32, 1, 2), (6, 3, 64, 4, 1000, 4),
    (2, 1, 64, 16, 0, 0), (2, 2, 32, 16, 33, 31), (2, 2, 32, 16, 32, 33), (4, 4, 64, 16, 300, 200)])
def test_prompt_portions_on_the_matrix_cores(dtype, rows, H, G, D, bs, window, keep):
    """The tiled kernel takes a step's prompt portions (whole prompts, portions that start far
    into a sequence, portions of one and two rows, a portion longer than the window so that key
    tiles between the kept keys and the window are skipped), the row kernel the decoded rows
    behind them; both against the dense formula.  window 0: plain causal attention."""
    device = "cuda"
    ks = [rnd(n, G * D, seed=20 + i, dtype=dtype) for i, n in enumerate(TILE_LENS)]
    vs = [rnd(n, G * D, seed=40 + i, dtype=dtype) for i, n in enumerate(TILE_LENS)]
    nb = sum((n + bs - 1) // bs for n in TILE_LENS) + 3
    kc, tb = paged(ks, bs, nb, G * D, dtype, device, 1)
    vc, _ = paged(vs, bs, nb, G * D, dtype, device, 1)
    seg = tiled_segments(TILE_SPANS, 7, tb, device, rows)
    T = seg.T
    pad = -(H * D + H) % 8
    z = rnd(T, H * D + H + pad, seed=60, dtype=dtype, device=device)
    q, gate = z[:, :H * D].view(T, H, D), z[:, H * D:H * D + H]
    slopes = torch.tensor([2.0 ** (-6.0 * (h + 1) / H) for h in range(H)], device=device)
    out = torch.zeros(T, H, D, dtype=dtype, device=device)
    sc = 0.3 * (32.0 / D) ** 0.5
    row_attention(q, None, kc.view(nb, bs, G, D), vc.view(nb, bs, G, D), D, out, seg, H, G, sc,
                  softcap=5.0, slopes=slopes, window=window, keep_first=keep, gate=gate)
    hg = torch.arange(H) // (H // G)
    at = 0
    for s, p0, n in TILE_SPANS:
        pos = torch.arange(p0, p0 + n)
        want = dense_window_attention(q[at:at + n].cpu(), ks[s][:p0 + n].view(-1, G, D),
                                      vs[s][:p0 + n].view(-1, G, D), pos, hg, sc, 5.0,
                                      slopes.cpu(), window, keep, gate[at:at + n].cpu())
        close(out[at:at + n], want, dtype, scale=1.0)
        at += n
    # the same rows through the row kernel alone: the two kernels agree to rounding
    seg.q_tiles, seg.tile_rows = None, 0
    out2 = torch.zeros_like(out)
    row_attention(q, None, kc.view(nb, bs, G, D), vc.view(nb, bs, G, D), D, out2, seg, H, G, sc,
                  softcap=5.0, slopes=slopes, window=window, keep_first=keep, gate=gate)
    close(out, out2.cpu().to(F64), dtype, scale=1.0)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("window,keep", [(150, 3), (64, 1), (65, 0), (200, 64), (30, 65), (1, 1)])
@pytest.mark.parametrize("rows", ["decoded", "prompt", "tiled"])
def test_window_and_kept_edges(device, dtype, window, keep, rows):
    """One key carries a spike the query is aligned with.  Placed at the last position inside the
    window, at the first one outside it, at the last kept position and at the first one behind the
    kept ones: the row returns that key's value exactly when it may see it.  The keys the row may
    NOT see between the kept ones and the window are poisoned."""
    n, H, D, bs = 600, 2, 16, 16
    p = 577
    d = torch.zeros(D)
    d[5] = 1.0
    lo = p - window + 1
    places = {"in": lo, "out": lo - 1, "kept": keep - 1, "not_kept": keep}
    for name, at in places.items():
        if at < 0 or at > p:
            continue
        seen = at >= lo or at < keep
        if (name in ("in", "kept")) != seen and name in ("in", "kept"):
            continue
        k = rnd(n, D, seed=70, dtype=torch.float32, scale=0.1)
        v = rnd(n, D, seed=71, dtype=torch.float32)
        k[at] = 4.0 * d
        if lo - 1 > keep:
            hidden = [j for j in range(keep, lo) if j != at]
            k[hidden] = 50.0 * d                                   # would win if it were seen
        kc, tb = paged([k.to(dtype)], bs, 50, D, dtype, device, 3)
        vc, _ = paged([v.to(dtype)], bs, 50, D, dtype, device, 3)
        spans = [(0, p, 1)] if rows == "decoded" else [(0, p - 30, 31)]
        seg = (tiled_segments(spans, 1, tb, device, 128) if rows == "tiled"
               else segments(spans, tb, device))
        q = (8.0 * d).to(dtype).to(device).expand(seg.T, H, D).contiguous()
        out = torch.zeros(seg.T, H, D, dtype=dtype, device=device)
        row_attention(q, None, kc.view(50, bs, 1, D), vc.view(50, bs, 1, D), D, out, seg, H, 1, 1.0,
                      window=window, keep_first=keep)
        got = out[-1].cpu().to(F64)
        hit = float((got - v[at].to(dtype).to(F64)).abs().max()) < 0.05
        assert hit == seen, f"key {at} ({name}): window [{lo}, {p}], kept below {keep}"


@pytest.mark.parametrize("device,dtype", CASES)
def test_linear_bias_uses_true_distance(device, dtype):
    """Equal scores everywhere.  A strong slope leaves the row's own key all the weight (head 0); no
    slope averages what the row sees (head 1); a mild slope weighs a kept first key by its TRUE
    distance, not by its place among the seen keys (head 2)."""
    n, H, D, bs, window, keep = 300, 3, 8, 16, 10, 2
    v = rnd(n, D, seed=95, dtype=dtype)
    kc, tb = paged([torch.zeros(n, D)], bs, 20, D, dtype, device, 6, fill=0.0)
    vc, _ = paged([v], bs, 20, D, dtype, device, 6)
    seg = segments([(0, 100, 3), (0, 299, 1)], tb, device)
    q = rnd(4, H, D, seed=96, dtype=dtype, device=device)
    out = torch.zeros(4, H, D, dtype=dtype, device=device)
    slopes = torch.tensor([30.0, 0.0, 0.01], device=device)
    row_attention(q, None, kc.view(20, bs, 1, D), vc.view(20, bs, 1, D), D, out, seg, H, 1, 1.0,
                  slopes=slopes, window=window, keep_first=keep)
    vf = v.to(F64)
    for i, p in enumerate([100, 101, 102, 299]):
        js = torch.tensor(list(range(keep)) + list(range(p - window + 1, p + 1)))
        close(out[i, 0], vf[p], dtype, scale=1.0)
        close(out[i, 1], vf[js].mean(0), dtype, scale=1.0)
        wt = torch.softmax(-0.01 * (p - js).to(F64), 0)
        close(out[i, 2], (wt[:, None] * vf[js]).sum(0), dtype, scale=1.0)


@pytest.mark.parametrize("device,dtype", CASES)
def test_gate_scales_each_head(device, dtype):
    n, H, D, bs = 90, 4, 8, 8
    k = rnd(n, D, seed=97, dtype=dtype)
    kc, tb = paged([k], bs, 12, D, dtype, device, 7)
    seg = segments([(0, 80, 3), (0, 89, 1)], tb, device)
    q = rnd(4, H, D, seed=98, dtype=dtype, device=device)
    base = torch.zeros(4, H, D, dtype=dtype, device=device)
    out = torch.zeros_like(base)
    cache = kc.view(12, bs, 1, D)
    row_attention(q, None, cache, cache, D, base, seg, H, 1, 0.4)
    gate = torch.tensor([[0.0, -1e4, 1e4, math.log(3.0)]] * 4, dtype=dtype, device=device)
    row_attention(q, None, cache, cache, D, out, seg, H, 1, 0.4, gate=gate)
    b = base.cpu().to(F64)
    g = torch.sigmoid(gate.cpu().to(F64))                          # of the rounded logits
    close(out, b * g.view(4, H, 1), dtype, scale=1.0)
    assert float(out[:, 1].abs().max()) == 0.0


# ---- router --------------------------------------------------------------------------------------
def oracle_route(z, corr, top, n, keep, scale):
    """ref.route on given logits: an identity router weight turns h into the logits."""
    E = z.shape[1]
    w = {"r.router": torch.eye(E, dtype=F64), "r.correction": corr.to(F64)}
    r = {"experts": E, "top": top, "scale": scale, "groups": {"count": n, "keep": keep}}
    return ref.route(z.to(F64), w, "r.", r)


@pytest.mark.parametrize("device", ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)])
@pytest.mark.parametrize("E,top,n,keep", [(12, 4, 4, 2), (5, 2, 1, 1), (16, 3, 4, 4), (8, 8, 2, 2),
                                          (6, 2, 6, 3), (64, 6, 8, 3), (130, 5, 10, 2),
                                          (256, 8, 8, 4), (9, 1, 3, 1)])
def test_route_groups_matches_oracle(device, E, top, n, keep):
    z = rnd(37, E, seed=50, device=device, scale=2.0)
    corr = rnd(E, seed=51, device=device, scale=0.3)
    got = route_groups(z, corr, top, n, keep, 1.7)
    want = oracle_route(z.cpu(), corr.cpu(), top, n, keep, 1.7)
    close(got, want, torch.float32, scale=1.0)
    assert bool(((got > 0).sum(-1) == top).all())
    close(got.sum(-1), torch.full((37,), 1.7, dtype=F64), torch.float32)


@pytest.mark.parametrize("device", ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)])
def test_route_negative_choices_and_dropped_group(device):
    """Every corrected score is negative, so an expert outside the kept groups (which must count
    as minus infinity, not as 0) would win every time if it counted as 0; and the single best
    expert sits in a group whose second best is poor, so its group is dropped."""
    E, n, keep, top = 8, 4, 2, 3
    s = torch.tensor([[0.90, 0.05, 0.60, 0.55, 0.50, 0.52, 0.10, 0.12]])
    z = torch.log(s / (1 - s)).to(device)
    corr = torch.full((E,), -2.0, device=device)
    got = route_groups(z, corr, top, n, keep, 1.0).cpu()
    # group sums of the two largest: (0.95, 1.15, 1.02, 0.22) - 4 -> groups 1 and 2 are kept
    chosen = [2, 3, 5]
    want = torch.zeros(1, E, dtype=F64)
    want[0, chosen] = s[0, chosen].to(F64) / s[0, chosen].to(F64).sum()
    close(got, want, torch.float32, scale=1.0)
    close(got, oracle_route(z.cpu(), corr.cpu(), top, n, keep, 1.0), torch.float32, scale=1.0)
    # the weights come from the scores WITHOUT the correction: a lopsided correction changes the
    # choice, not the weights' formula
    corr2 = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 5.0, 5.0], device=device)
    got2 = route_groups(z, corr2, 2, 1, 1, 2.0).cpu()
    want2 = torch.zeros(1, E, dtype=F64)
    want2[0, [6, 7]] = 2.0 * s[0, [6, 7]].to(F64) / s[0, [6, 7]].to(F64).sum()
    close(got2, want2, torch.float32, scale=1.0)


@pytest.mark.parametrize("device", ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)])
def test_route_ties_go_to_the_lowest_index(device):
    z = torch.zeros(3, 12, device=device)
    corr = torch.zeros(12, device=device)
    got = route_groups(z, corr, 3, 4, 2, 1.0).cpu()
    want = torch.zeros(3, 12)
    want[:, :3] = 1.0 / 3
    close(got, want.to(F64), torch.float32, scale=1.0)


def test_route_groups_rejects_bad_shapes():
    z, c = torch.zeros(2, 12), torch.zeros(12)
    for top, n, keep in [(4, 5, 2), (7, 4, 2), (0, 4, 2), (2, 4, 5)]:
        with pytest.raises(ValueError):
            route_groups(z, c, top, n, keep, 1.0)


# ---- experts -------------------------------------------------------------------------------------
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("E,ff,ffs", [(3, 40, 0), (4, 37, 0), (0, 0, 48), (2, 16, 24)])
def test_squared_relu_scaled_by_routing_weight(device, dtype, E, ff, ffs):
    T = 11
    u = rnd(T, E * ff + ffs, seed=60, dtype=dtype, device=device, scale=2.0)
    wts = None
    uf = u.cpu().to(F64)
    parts = []
    if E:
        wts = torch.rand(T, E, generator=torch.Generator().manual_seed(61)).to(device)
        wts[:, 0] = 0.0                                            # an expert nobody chose
        parts.append((torch.relu(uf[:, :E * ff]) ** 2).view(T, E, ff) * wts.cpu().to(F64)[:, :, None])
        parts[0] = parts[0].reshape(T, E * ff)
    if ffs:
        parts.append(torch.relu(uf[:, E * ff:]) ** 2)
    close(scaled_act(u, wts, E, ff, ffs, "relu2"), torch.cat(parts, 1), dtype)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("E,top,n,keep,ff", [(6, 2, 3, 2, 24), (5, 3, 1, 1, 20)])
def test_experts_dense_and_grouped_match_oracle(device, dtype, E, top, n, keep, ff):
    """Both ways to run the experts (two stacked GEMMs over all experts; per expert on its own
    rows) against the oracle's loop over experts."""
    T, W = 300, 32
    h = rnd(T, W, seed=62, dtype=dtype, device=device)
    w = {"m.router": rnd(E, W, seed=63, scale=0.5), "m.correction": rnd(E, seed=64, scale=0.2)}
    for e in range(E):
        w[f"m.e{e}.up"] = rnd(ff, W, seed=65 + e, dtype=dtype, scale=W ** -0.5)
        w[f"m.e{e}.down"] = rnd(W, ff, seed=75 + e, dtype=dtype, scale=ff ** -0.5)
    f = {"kind": "moe", "expert": {"ff": ff},
         "router": {"experts": E, "top": top, "scale": 1.3, "groups": {"count": n, "keep": keep}}}
    want = ref.moe_ff(h.cpu().to(F64), {k: v.to(F64) for k, v in w.items()}, "m.", f)
    up = torch.cat([w[f"m.e{e}.up"] for e in range(E)], 0).to(device)
    down = torch.cat([w[f"m.e{e}.down"] for e in range(E)], 1).to(device)
    z = h.float() @ w["m.router"].to(device).t()
    r = route_groups(z, w["m.correction"].to(device), top, n, keep, 1.3)
    for fn in (moe_dense, moe_grouped):
        got = fn(h, r, up, down, E, ff, 0, "relu2", gated=False)
        assert got.dtype == dtype
        close(got, want, dtype)
    if grouped_mm_ok(h, ff):                               # 16 bits on the GPU: no host in the loop
        got = moe_grouped_mm(h, r, up, down, E, top, ff, 0, "relu2", gated=False)
        assert got.dtype == dtype
        close(got, want, dtype)


@pytest.mark.parametrize("device,dtype", CASES)
def test_router_logits_are_fp32_sums_of_exact_products(device, dtype):
    from lumen.ops.moe import router_logits

    h = rnd(300, 136, seed=90, dtype=dtype, device=device, scale=2.0)
    w = rnd(12, 136, seed=91, dtype=dtype, device=device)
    z = router_logits(h, w)
    assert z.dtype == torch.float32
    close(z, h.cpu().to(F64) @ w.cpu().to(F64).T, torch.float32)   # fp32 accuracy in every dtype


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("E,top,n,keep,ff,W,T", [(40, 2, 1, 1, 16, 64, 1000), (64, 4, 8, 2, 8, 40, 1200),
                                                 (33, 1, 1, 1, 24, 128, 1100)])
def test_grouped_gemm_form_with_idle_experts(dtype, E, top, n, keep, ff, W, T):
    """The sync-free grouped form as ``moe`` picks it for many experts and few chosen: a correction
    of -10 keeps a third of the experts from ever being chosen, so their groups are empty; one
    expert takes every row."""
    from lumen.ops.moe import moe

    device = "cuda"
    h = rnd(T, W, seed=70, dtype=dtype, device=device)
    w = {"m.router": rnd(E, W, seed=71, scale=0.5), "m.correction": rnd(E, seed=72, scale=0.2)}
    w["m.correction"][::3] = -10.0
    w["m.correction"][1] = 10.0
    for e in range(E):
        w[f"m.e{e}.up"] = rnd(ff, W, seed=100 + e, dtype=dtype, scale=W ** -0.5)
        w[f"m.e{e}.down"] = rnd(W, ff, seed=200 + e, dtype=dtype, scale=ff ** -0.5)
    f = {"kind": "moe", "expert": {"ff": ff},
         "router": {"experts": E, "top": top, "scale": 1.3, "groups": {"count": n, "keep": keep}}}
    want = ref.moe_ff(h.cpu().to(F64), {k: v.to(F64) for k, v in w.items()}, "m.", f)
    up = torch.cat([w[f"m.e{e}.up"] for e in range(E)], 0).to(device)
    down = torch.cat([w[f"m.e{e}.down"] for e in range(E)], 1).to(device)
    r = route_groups(h.float() @ w["m.router"].to(device).t(), w["m.correction"].to(device), top, n,
                     keep, 1.3)
    assert int((r[:, ::3] > 0).sum()) == 0 and bool((r[:, 1] > 0).all())
    assert grouped_mm_ok(h, ff) and T * (E - 3 * top) >= 32768     # moe() takes the grouped GEMM
    close(moe(h, r, up, down, E, top, ff, 0, "relu2", gated=False), want, dtype)
    close(moe_grouped_mm(h, r, up, down, E, top, ff, 0, "relu2", gated=False), want, dtype)
