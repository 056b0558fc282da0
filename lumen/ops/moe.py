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
* ``moe_grouped_mm``: the same arithmetic on the library's grouped GEMM (16-bit dtypes): the
  sorted (row, expert) pairs have a static count, the group offsets stay on the device, nothing
  synchronises and a layer's experts are three launches.
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


def router_logits(h: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """fp32 router logits h [T, W] @ w [E, W]^T for h and w in the model dtype.  16-bit values
    multiply exactly in fp32, so on the GPU the product runs on the matrix cores with fp32
    accumulation and an fp32 result -- the arithmetic of an fp32 GEMM on the widened operands
    without the pass that widens them."""
    if h.is_cuda and h.dtype == w.dtype and h.dtype in (torch.bfloat16, torch.float16):
        return torch.mm(h, w.t(), out_dtype=torch.float32)
    return h.float() @ w.float().t()


def route_groups_ref(z, correction, top, n_groups, keep, scale, sum_eps=1e-20, rank_top=2,
                     score="sigmoid", normalize=True):
    T, E = z.shape
    s = torch.softmax(z.float(), -1) if score == "softmax" else torch.sigmoid(z.float())
    c = s + correction.float() if correction is not None else s
    if n_groups > 1 and keep < n_groups:
        per = E // n_groups
        cg = c.view(T, n_groups, per)
        rank = torch.sort(cg, dim=-1, descending=True).values[..., :min(rank_top, per)].sum(-1)
        best = torch.sort(rank, dim=-1, descending=True, stable=True).indices[:, :keep]
        allow = torch.zeros(T, n_groups, dtype=torch.bool, device=z.device).scatter_(1, best, True)
        c = cg.masked_fill(~allow.view(T, n_groups, 1), float("-inf")).reshape(T, E)
    idx = torch.sort(c, dim=-1, descending=True, stable=True).indices[:, :top]
    chosen = torch.gather(s, 1, idx)
    wt = (chosen / (chosen.sum(-1, keepdim=True) + sum_eps) if normalize else chosen) * scale
    return torch.zeros_like(s).scatter_(1, idx, wt)


def route_groups(z: torch.Tensor, correction: Optional[torch.Tensor], top: int, n_groups: int,
                 keep: int, scale: float = 1.0, sum_eps: float = 1e-20, rank_top: int = 2,
                 score: str = "sigmoid", normalize: bool = True) -> torch.Tensor:
    """Router logits z [T, E] (fp32) -> dense routing weights [T, E] (fp32) of a router with a
    choice correction and a limit to the best groups: the scores are s = sigmoid(z), or with
    ``score`` = "softmax" the softmax of z over all experts; the
    choice ranks c = s + ``correction`` [E] (None: c = s); the experts form ``n_groups`` equal groups of
    neighbours, a group ranks by the sum of its ``rank_top`` largest c, and only experts of the
    ``keep`` best groups can be chosen (``keep`` = ``n_groups``: no limit); the ``top`` eligible
    experts with the largest c get s_e / (sum of the chosen s + ``sum_eps``) * ``scale`` at their
    places (``normalize`` False: s_e * ``scale``, the scores as they are), all others zero.  Ties
    go to the lowest index.  ``rank_top`` = 1 ranks a group by its best member."""
    from ._seqmix import call, use_seqmix

    T, E = z.shape
    if n_groups < 1 or E % n_groups or not 1 <= keep <= n_groups:
        raise ValueError(f"{E} experts do not form {n_groups} equal groups of which {keep} are kept")
    if not 1 <= top <= keep * (E // n_groups):
        raise ValueError(f"top {top} exceeds the {keep * (E // n_groups)} eligible experts")
    if score not in ("sigmoid", "softmax"):
        raise ValueError(f"unknown router score {score!r}")
    if not use_seqmix(z):
        return route_groups_ref(z, correction, top, n_groups, keep, scale, sum_eps, rank_top,
                                score, normalize)
    assert z.dtype == torch.float32 and z.is_contiguous()
    assert correction is None or (correction.dtype == torch.float32 and correction.is_contiguous())
    if E > 1024:
        raise ValueError(f"route_groups supports at most 1024 experts, got {E}")
    out = torch.empty_like(z)
    call("sm_route_groups", z, correction, out, T, E, top, n_groups, keep, rank_top, scale, sum_eps,
         int(score == "softmax"), int(bool(normalize)))
    return out


GATE_ACTS = {"silu": 0, "relu": 1, "gelu_tanh": 2, "relu2": 3}
_ACT_FN = {"silu": F.silu, "relu": F.relu, "gelu_tanh": lambda z: F.gelu(z, approximate="tanh"),
           "relu2": lambda z: F.relu(z) ** 2}


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


def scaled_act_ref(u, wts, E, ff, ffs, act="relu2"):
    T = u.shape[0]
    fn = _ACT_FN[act]
    parts = []
    if E:
        parts.append((fn(u[:, :E * ff].float()).view(T, E, ff) * wts.float()[:, :, None])
                     .reshape(T, E * ff))
    if ffs:
        parts.append(fn(u[:, E * ff:].float()))
    return torch.cat(parts, 1).to(u.dtype)


def scaled_act(u: torch.Tensor, wts: Optional[torch.Tensor], E: int, ff: int, ffs: int,
               act: str = "relu2") -> torch.Tensor:
    """act(u) over the stacked up projections of experts WITHOUT a gate (``act``: as for
    ``gated_act``, plus relu2 = relu(.)^2): ``u`` [T, E * ff + ffs] holds E expert blocks of ff and
    one unweighted block of ffs; expert e's activation is scaled by ``wts[:, e]``.  Same shape
    out."""
    from ._seqmix import DT, call, use_seqmix

    if not use_seqmix(u):
        return scaled_act_ref(u, wts, E, ff, ffs, act)
    assert u.is_contiguous() and u.shape[1] == E * ff + ffs
    out = torch.empty_like(u)
    call("sm_scaled_act", DT[u.dtype], u, wts, out, u.shape[0], E, ff, ffs, GATE_ACTS[act])
    return out


def _act(z, wts, E, ff, ffs, act, gated):
    return (gated_act if gated else scaled_act)(z, wts, E, ff, ffs, act)


def moe_dense(h, wts, gu_w, down_w, E: int, ff: int, ffs: int, act: str = "silu",
              gated: bool = True) -> torch.Tensor:
    return F.linear(_act(F.linear(h, gu_w), wts, E, ff, ffs, act, gated), down_w)


def moe_grouped(h, wts, gu_w, down_w, E: int, ff: int, ffs: int, act: str = "silu",
                gated: bool = True) -> torch.Tensor:
    """Same result as ``moe_dense`` (to rounding) running each expert on its own rows only."""
    T = h.shape[0]
    k = 2 if gated else 1                                 # rows of the first weight per ff
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
            gu = F.linear(x[a:a + n], gu_w[e * k * ff:(e + 1) * k * ff])
            torch.matmul(_act(gu, None, 0, 0, ff, act, gated), down_w[:, e * ff:(e + 1) * ff].t(),
                         out=ys[a:a + n])
            a += n
    out.index_add_(0, tok, ys.float() * wsel)
    if ffs:
        gu = F.linear(h, gu_w[E * k * ff:])
        out += F.linear(_act(gu, None, 0, 0, ffs, act, gated), down_w[:, E * ff:]).float()
    return out.to(h.dtype)


def grouped_mm_ok(h: torch.Tensor, ff: int) -> bool:
    """Can ``moe_grouped_mm`` run: the library's grouped GEMM (one launch for all experts, group
    offsets read on the device) exists, a 16-bit dtype on the GPU, 16-byte aligned rows."""
    return (h.is_cuda and h.dtype in (torch.bfloat16, torch.float16)
            and hasattr(torch, "_grouped_mm") and ff % 8 == 0 and h.shape[1] % 8 == 0)


def moe_grouped_mm(h, wts, gu_w, down_w, E: int, top: int, ff: int, ffs: int, act: str = "silu",
                   gated: bool = True) -> torch.Tensor:
    """``moe_grouped`` without the host in the loop: every row has exactly ``top`` chosen
    experts, so the (row, expert) pairs are a [T * top] list of static size; sorted by expert they
    feed ONE grouped GEMM per projection whose group offsets stay on the device.  No
    synchronisation, three launches per layer instead of three per expert."""
    T, W = h.shape
    k = 2 if gated else 1
    val, idx = torch.topk(wts, top, dim=1)                         # [T, top]: weights, experts
    exp = idx.reshape(-1)
    order = torch.argsort(exp, stable=True)
    tok = torch.div(order, top, rounding_mode="floor")
    offs = torch.cumsum(torch.bincount(exp, minlength=E), 0).to(torch.int32)
    x = h.index_select(0, tok)
    u = torch._grouped_mm(x, gu_w[:E * k * ff].view(E, k * ff, W).transpose(1, 2), offs=offs)
    a = _act(u, val.reshape(-1)[order].reshape(-1, 1).contiguous(), 1, ff, 0, act, gated)
    y = torch._grouped_mm(a, down_w[:, :E * ff].view(W, E, ff).permute(1, 2, 0), offs=offs)
    out = torch.zeros(T, W, dtype=torch.float32, device=h.device)
    out.index_add_(0, tok, y.float())
    if ffs:
        gu = F.linear(h, gu_w[E * k * ff:])
        out += F.linear(_act(gu, None, 0, 0, ffs, act, gated), down_w[:, E * ff:]).float()
    return out.to(h.dtype)


# When the grouped form pays.  Measured on MI355X (bf16, width 2048, 16 experts of 1408, top 4):
# the two stacked GEMMs of the dense form run at ~850 TFLOP/s, the grouped GEMMs at ~300, and
# sorting the (row, expert) pairs costs ~0.4 ms per layer whatever the size.  The grouped form does
# top / E of the dense form's FLOPs at about a third of its rate, so it needs E > 3 top to save
# anything, and enough rows for the saving to cover the sorting.
GROUPED_RATE_RATIO = 3
GROUPED_MIN_SAVING = 32768          # rows x (E - GROUPED_RATE_RATIO * top)


def moe(h, wts, gu_w, down_w, E: int, top: int, ff: int, ffs: int, act: str = "silu",
        gated: bool = True) -> torch.Tensor:
    """Weighted sum of each row's chosen experts (+ the shared expert): [T, W] in h's dtype.
    ``gated``: an expert is W_down (act(W_gate h) * W_up h) with [gate | up] rows stacked per
    expert in ``gu_w``; else W_down act(W_up h) with the up rows alone."""
    spare = E - GROUPED_RATE_RATIO * top
    grouped = (spare > 0 and h.shape[0] * spare >= GROUPED_MIN_SAVING
               and not (h.is_cuda and torch.cuda.is_current_stream_capturing()))
    if grouped and grouped_mm_ok(h, ff):
        return moe_grouped_mm(h, wts, gu_w, down_w, E, top, ff, ffs, act, gated)
    return (moe_grouped if grouped else moe_dense)(h, wts, gu_w, down_w, E, ff, ffs, act, gated)
