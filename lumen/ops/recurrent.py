"""Linear-recurrence token mixers with a per-sequence matrix state (HIP:
``csrc/seqmix/recurrent.hip``).

Both scans carry one fp32 state S [heads, D, D] (key channel x value channel) per sequence in
``state`` [slots, heads, D, D]; a segment whose ``start`` is 0 begins from zero whatever its
(reused) slot holds.  Inputs are rows of 16-bit or fp32 GEMM outputs (column slices of a fused
projection are fine: only the last dimension must be contiguous); decays, gates of the
recurrence, unit keys and the state are fp32.  The per-head RMS norm of the read-out, the
channel weight and the output gate are fused into the scan, which returns [T, heads * D] in the
compute dtype, ready for the output projection.

``wkv_scan``  (RWKV-style, bonus u for the current token):
    w_t = exp(-exp(wl_t + w0));   o_t = (S + diag(u) k_t v_t^T)^T r_t;   S <- diag(w_t) S + k_t v_t^T
    out = o / rms(o) * norm_w * silu(g)
``delta_scan`` (generalised delta rule; decay_scale and key_eps are the design's constants):
    w_t = exp(-decay_scale * sigmoid(wl_t + w0));  a_t = sigmoid(al_t + a_b)
    u_t = k_t / sqrt(sum k_t^2 + key_eps)
    S <- diag(w_t) S - (a_t * u_t)(u_t^T S) + k_t v_t^T;   o_t = S^T r_t   (the NEW state)
    out = o / rms(o) * norm_w * sigmoid(gl)
``token_shift``: the five inputs h + (h_prev - h) * mu_s of an RWKV-style mixer, h_prev being the
previous row of the same sequence (``prev`` [slots, W] across steps, zeros at position 0).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from .segments import SegBatch


def _head_out(o, eps, norm_w, gate, H, D, dtype):
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps)
    return (o.reshape(-1, H * D) * norm_w.float() * gate).to(dtype)


def token_shift_ref(h, mu, prev, seg: SegBatch):
    hf = h.float()
    hp = torch.empty_like(hf)
    cu, slots, starts = seg.cu.tolist(), seg.slot.tolist(), seg.start.tolist()
    for s in range(seg.S):
        a, b = cu[s], cu[s + 1]
        if b == a:
            continue
        hp[a] = prev[slots[s]] if starts[s] > 0 else 0
        hp[a + 1:b] = hf[a:b - 1]
        prev[slots[s]] = hf[b - 1]
    return (hf[None] + (hp - hf)[None] * mu.float()[:, None, :]).to(h.dtype)


def token_shift(h: torch.Tensor, mu: torch.Tensor, prev: torch.Tensor, seg: SegBatch):
    """h [T, W], mu [n, W] fp32 -> [n, T, W] shifted mixes in h's dtype; ``prev`` moves on."""
    from ._seqmix import DT, call, use_seqmix

    if not use_seqmix(h):
        return token_shift_ref(h, mu, prev, seg)
    T, W = h.shape
    assert h.is_contiguous() and mu.dtype == torch.float32 and prev.dtype == torch.float32
    out = torch.empty(mu.shape[0], T, W, dtype=h.dtype, device=h.device)
    call("sm_token_shift", DT[h.dtype], h, mu, prev, out, seg.cu, seg.slot, seg.start,
         seg.row_seg, T, W, mu.shape[0])
    call("sm_shift_tail", DT[h.dtype], h, prev, seg.cu, seg.slot, seg.S, W)
    return out


def wkv_scan_ref(r, k, v, wl, g, w0, u, norm_w, state, seg: SegBatch, H, D, eps):
    T = r.shape[0]
    f = lambda t: t.float().reshape(T, H, D)  # noqa: E731
    r_, k_, v_ = f(r), f(k), f(v)
    w = torch.exp(-torch.exp(f(wl) + w0.float().view(H, D)))
    uu = u.float().view(H, D)
    o = torch.empty(T, H, D, dtype=torch.float32, device=r.device)
    cu, slots, starts = seg.cu.tolist(), seg.slot.tolist(), seg.start.tolist()
    for s in range(seg.S):
        a, b = cu[s], cu[s + 1]
        if b == a:
            continue
        S = state[slots[s]].clone() if starts[s] > 0 else torch.zeros_like(state[slots[s]])
        for t in range(a, b):
            kv = k_[t][:, :, None] * v_[t][:, None, :]
            o[t] = torch.einsum("hkv,hk->hv", S + uu[:, :, None] * kv, r_[t])
            S = w[t][:, :, None] * S + kv
        state[slots[s]] = S
    return _head_out(o, eps, norm_w, F.silu(g.float()), H, D, r.dtype)


def delta_scan_ref(r, k, v, wl, al, gl, w0, a_b, norm_w, state, seg: SegBatch, H, D, eps,
                   decay_scale, key_eps):
    T = r.shape[0]
    f = lambda t: t.float().reshape(T, H, D)  # noqa: E731
    r_, k_, v_ = f(r), f(k), f(v)
    w = torch.exp(-decay_scale * torch.sigmoid(f(wl) + w0.float().view(H, D)))
    a_ = torch.sigmoid(f(al) + a_b.float().view(H, D))
    un = k_ / torch.sqrt((k_ * k_).sum(-1, keepdim=True) + key_eps)
    o = torch.empty(T, H, D, dtype=torch.float32, device=r.device)
    cu, slots, starts = seg.cu.tolist(), seg.slot.tolist(), seg.start.tolist()
    for s in range(seg.S):
        a, b = cu[s], cu[s + 1]
        if b == a:
            continue
        S = state[slots[s]].clone() if starts[s] > 0 else torch.zeros_like(state[slots[s]])
        for t in range(a, b):
            uS = torch.einsum("hk,hkv->hv", un[t], S)
            S = (w[t][:, :, None] * S - (a_[t] * un[t])[:, :, None] * uS[:, None, :]
                 + k_[t][:, :, None] * v_[t][:, None, :])
            o[t] = torch.einsum("hkv,hk->hv", S, r_[t])
        state[slots[s]] = S
    return _head_out(o, eps, norm_w, torch.sigmoid(gl.float()), H, D, r.dtype)


def _ld(t: torch.Tensor) -> int:
    assert t.dim() == 2 and t.stride(1) == 1, "rows must be contiguous in their last dimension"
    return t.stride(0)


def _check_state(state, H, D):
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, D, D)
    if D > 256:
        raise ValueError(f"recurrent head size {D} > 256 is not supported")


def wkv_scan(r, k, v, wl, g, w0, u, norm_w, state, seg: SegBatch, H: int, D: int, eps: float):
    from ._seqmix import DT, call, use_seqmix

    if not use_seqmix(r):
        return wkv_scan_ref(r, k, v, wl, g, w0, u, norm_w, state, seg, H, D, eps)
    _check_state(state, H, D)
    T = r.shape[0]
    out = torch.empty(T, H * D, dtype=r.dtype, device=r.device)
    call("sm_wkv", DT[r.dtype], r, _ld(r), k, _ld(k), v, _ld(v), wl, _ld(wl), g, _ld(g), w0, u,
         norm_w, state, out, H * D, seg.cu, seg.slot, seg.start, seg.S, H, D, eps)
    return out


def delta_scan(r, k, v, wl, al, gl, w0, a_b, norm_w, state, seg: SegBatch, H: int, D: int,
               eps: float, decay_scale: float, key_eps: float):
    from ._seqmix import DT, call, use_seqmix

    if not use_seqmix(r):
        return delta_scan_ref(r, k, v, wl, al, gl, w0, a_b, norm_w, state, seg, H, D, eps,
                              decay_scale, key_eps)
    _check_state(state, H, D)
    T = r.shape[0]
    out = torch.empty(T, H * D, dtype=r.dtype, device=r.device)
    call("sm_gdelta", DT[r.dtype], r, _ld(r), k, _ld(k), v, _ld(v), wl, _ld(wl), al, _ld(al), gl,
         _ld(gl), w0, a_b, norm_w, state, out, H * D, seg.cu, seg.slot, seg.start, seg.S, H, D,
         eps, decay_scale, key_eps)
    return out


# ---- minGRU: an element-wise linear recurrence; gate and candidate depend on one token alone -------
# Per channel, from S = 0 at a sequence's first token:
#     z_t = sigmoid(zl_t + b_z);  u_t = xl_t + b_x;  c_t = u_t + shift (u_t >= 0) | sigmoid(u_t)
#     S_t = (1 - z_t) S_(t-1) + z_t c_t;            out_t = S_t * silu(gl_t)
# zl, xl, gl are column blocks of one fused projection's rows; gates, candidate and state are fp32
# (``state`` [slots, width] carries S across steps); the result is stored in the compute dtype.
def min_gru_scan_ref(zxg, b_z, b_x, state, seg: SegBatch, width, shift):
    T = zxg.shape[0]
    f = zxg.float()
    z = torch.sigmoid(f[:, :width] + b_z.float())
    u = f[:, width:2 * width] + b_x.float()
    c = torch.where(u >= 0, u + shift, torch.sigmoid(u))
    g = f[:, 2 * width:3 * width]
    out = torch.empty(T, width, dtype=torch.float32, device=zxg.device)
    cu, slots, starts = seg.cu.tolist(), seg.slot.tolist(), seg.start.tolist()
    for s in range(seg.S):
        a, b = cu[s], cu[s + 1]
        if b == a:
            continue
        S = state[slots[s]].clone() if starts[s] > 0 else torch.zeros_like(state[slots[s]])
        for t in range(a, b):
            S = (1.0 - z[t]) * S + z[t] * c[t]
            out[t] = S
        state[slots[s]] = S
    return (out * F.silu(g)).to(zxg.dtype)


def min_gru_scan(zxg: torch.Tensor, b_z: torch.Tensor, b_x: torch.Tensor, state: torch.Tensor,
                 seg: SegBatch, width: int, shift: float = 0.5) -> torch.Tensor:
    """zxg [T, >= 3 * width] = [z logits | candidate pre-activations | output-gate logits] (a
    fused projection's rows, unit column stride), biases [width] fp32 -> [T, width] in zxg's dtype,
    ready for the output projection; ``state`` [slots, width] fp32 moves on by the step's rows (a
    segment that starts at position 0 begins from zero whatever its slot holds)."""
    from ._seqmix import DT, call, min_gru_sub, use_seqmix

    if zxg.shape[1] < 3 * width:
        raise ValueError(f"zxg has {zxg.shape[1]} columns, expected at least {3 * width}")
    if not use_seqmix(zxg):
        return min_gru_scan_ref(zxg, b_z, b_x, state, seg, width, shift)
    assert zxg.stride(1) == 1 and state.dtype == torch.float32 and state.is_contiguous()
    assert b_z.dtype == torch.float32 and b_x.dtype == torch.float32 and state.shape[1] == width
    T = zxg.shape[0]
    out = torch.empty(T, width, dtype=zxg.dtype, device=zxg.device)
    # a step's prompt portions: every tile of rows reduced to its affine map S -> A S + B, then
    # replayed from its true start state, so a long portion is not one serial walk; the decoded
    # rows after them (one-row segments) and steps without tiles: one thread per channel
    Tp = seg.tile_rows if seg.q_tiles is not None else 0
    if Tp:
        n = seg.q_tiles.shape[0]
        ab = torch.empty(n * min_gru_sub() * 2 * width, dtype=torch.float32, device=zxg.device)
        call("sm_min_gru", DT[zxg.dtype], zxg, zxg.stride(0), b_z, b_x, state, out, seg.cu,
             seg.slot, seg.start, 0, width, float(shift), ab, seg.q_tiles, n, seg.tile_size)
    if T > Tp:
        P = seg.S - (T - Tp) if Tp else 0              # decode rows are one-row segments
        call("sm_min_gru", DT[zxg.dtype], zxg, zxg.stride(0), b_z, b_x, state, out, seg.cu[P:],
             seg.slot[P:], seg.start[P:], seg.S - P, width, float(shift), None, None, 0, 0)
    return out
