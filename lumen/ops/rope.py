"""Rotary embeddings (HIP kernel ``kernels/rope.hip``; torch reference on CPU).

Training: ``qkv_rope_split`` turns the fused QKV GEMM output [B*S, (nh+2nkv)*D] into rotated
q [B,nh,S,D], k [B,nkv,S,D] and v [B,nkv,S,D] in one pass (rotate_half convention of
transformers' Llama, theta from the config).  Serving: ``rope_inplace`` rotates q/k heads inside
the token-major QKV buffer at arbitrary positions.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from ._native import native, use_native

_TABLES: Dict[tuple, Tuple[torch.Tensor, torch.Tensor]] = {}


def rope_tables(D: int, max_pos: int, theta: float, device) -> Tuple[torch.Tensor, torch.Tensor]:
    """f32 cos/sin tables [max_pos, D/2] (built once per device on the host, f64 math)."""
    key = (D, max_pos, float(theta), str(device))
    t = _TABLES.get(key)
    if t is None:
        inv = 1.0 / (theta ** (torch.arange(0, D, 2, dtype=torch.float64) / D))
        ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * inv[None, :]
        t = (ang.cos().float().to(device).contiguous(), ang.sin().float().to(device).contiguous())
        _TABLES[key] = t
    return t


def _rotate_ref(x, cos, sin, inverse=False):
    # x [..., S, D]; cos/sin [S, D/2]
    half = x.shape[-1] // 2
    a, b = x[..., :half].float(), x[..., half:].float()
    sgn = -1.0 if inverse else 1.0
    oa = a * cos - sgn * b * sin
    ob = b * cos + sgn * a * sin
    return torch.cat([oa, ob], -1).to(x.dtype)


def qkv_rope_split_ref(qkv, B, S, nh, nkv, D, cos_t, sin_t, pos=None):
    x = qkv.view(B, S, nh + 2 * nkv, D)
    q = x[:, :, :nh].transpose(1, 2)
    k = x[:, :, nh:nh + nkv].transpose(1, 2)
    v = x[:, :, nh + nkv:].transpose(1, 2).contiguous()
    if pos is None:
        cos, sin = cos_t[:S], sin_t[:S]
        cos, sin = cos[None, None], sin[None, None]
    else:
        p = pos.view(B, S).long()
        cos, sin = cos_t[p][:, None], sin_t[p][:, None]
    return _rotate_ref(q, cos, sin).contiguous(), _rotate_ref(k, cos, sin).contiguous(), v


class _QKVRope(torch.autograd.Function):
    @staticmethod
    def forward(ctx, qkv, B, S, nh, nkv, D, cos_t, sin_t, pos):
        C = native()
        qkv = qkv.contiguous()
        dev, dt = qkv.device, qkv.dtype
        q = torch.empty(B, nh, S, D, device=dev, dtype=dt)
        k = torch.empty(B, nkv, S, D, device=dev, dtype=dt)
        v = torch.empty(B, nkv, S, D, device=dev, dtype=dt)
        C.qkv_rope(False, qkv, q, k, v, pos, cos_t, sin_t, S, nh, nkv, D)
        ctx.dims = (B, S, nh, nkv, D)
        ctx.save_for_backward(cos_t, sin_t, pos if pos is not None else torch.empty(0))
        ctx.has_pos = pos is not None
        ctx.qkv_shape = qkv.shape
        return q, k, v

    @staticmethod
    def backward(ctx, dq, dk, dv):
        C = native()
        B, S, nh, nkv, D = ctx.dims
        cos_t, sin_t, pos = ctx.saved_tensors
        ref = dq if dq is not None else (dk if dk is not None else dv)
        dqkv = torch.empty(ctx.qkv_shape, device=ref.device, dtype=ref.dtype)
        z = lambda h: torch.zeros(B, h, S, D, device=ref.device, dtype=ref.dtype)  # noqa: E731
        dq = dq.contiguous() if dq is not None else z(nh)
        dk = dk.contiguous() if dk is not None else z(nkv)
        dv = dv.contiguous() if dv is not None else z(nkv)
        C.qkv_rope(True, dqkv, dq, dk, dv, pos if ctx.has_pos else None, cos_t, sin_t, S, nh, nkv, D)
        return dqkv, None, None, None, None, None, None, None, None


def qkv_rope_split(qkv: torch.Tensor, B: int, S: int, nh: int, nkv: int, D: int,
                   cos_t: torch.Tensor, sin_t: torch.Tensor, pos: Optional[torch.Tensor] = None):
    if use_native(qkv):
        if pos is not None:
            pos = pos.to(torch.int32).contiguous()
        return _QKVRope.apply(qkv, B, S, nh, nkv, D, cos_t, sin_t, pos)
    return qkv_rope_split_ref(qkv, B, S, nh, nkv, D, cos_t, sin_t, pos)


def rope_inplace(x2d: torch.Tensor, pos: torch.Tensor, nheads: int, D: int,
                 cos_t: torch.Tensor, sin_t: torch.Tensor, col_offset: int = 0) -> None:
    """Rotate `nheads` heads starting at column `col_offset` of token-major x2d [T, W] in place."""
    T = x2d.shape[0]
    if T == 0:
        return
    if use_native(x2d):
        sub = x2d[:, col_offset:]
        native().rope_inplace(sub, pos.to(torch.int32).contiguous(), cos_t, sin_t, T,
                              x2d.stride(0), nheads, D)
        return
    view = x2d[:, col_offset:col_offset + nheads * D].view(T, nheads, D)
    p = pos.long()
    cos, sin = cos_t[p][:, None], sin_t[p][:, None]
    view.copy_(_rotate_ref(view, cos, sin))


_NEG_SIN = {}


def _neg(sin_t):
    k = (sin_t.data_ptr(), sin_t.shape, str(sin_t.device))
    t = _NEG_SIN.get(k)
    if t is None:
        t = (-sin_t).contiguous()
        _NEG_SIN[k] = t
    return t


class _RopeQKV(torch.autograd.Function):
    """In-place RoPE on the q and k heads of the fused QKV buffer (training path of the HIP
    flash attention); backward = the inverse rotation (sin -> -sin) applied in place."""

    @staticmethod
    def forward(ctx, qkv, pos, nqk, D, cos_t, sin_t):
        native().rope_inplace(qkv, pos, cos_t, sin_t, qkv.shape[0], qkv.stride(0), nqk, D)
        ctx.mark_dirty(qkv)
        ctx.save_for_backward(pos)
        ctx.meta = (nqk, D, cos_t, sin_t)
        return qkv

    @staticmethod
    def backward(ctx, g):
        (pos,) = ctx.saved_tensors
        nqk, D, cos_t, sin_t = ctx.meta
        # g is the flash-attention backward's fresh dQKV buffer (sole consumer): rotate it in
        # place instead of copying 3*T*H*2 bytes
        if getattr(g, "_lumen_rope_undone", False):  # the flash-attention backward did it
            return g, None, None, None, None, None
        g = g if g.is_contiguous() else g.contiguous()
        native().rope_inplace(g, pos, cos_t, _neg(sin_t), g.shape[0], g.stride(0), nqk, D)
        return g, None, None, None, None, None


def rope_qkv_(qkv: torch.Tensor, pos: torch.Tensor, nh: int, nkv: int, D: int, cos_t, sin_t):
    """Rotate q and k heads of qkv [T, (nh+2nkv)*D] in place (autograd-aware)."""
    if use_native(qkv):
        return _RopeQKV.apply(qkv, pos.to(torch.int32).contiguous(), nh + nkv, D, cos_t, sin_t)
    T = qkv.shape[0]
    out = qkv.clone()
    view = out[:, :(nh + nkv) * D].view(T, nh + nkv, D)
    p = pos.long()
    rot = _rotate_ref(view, cos_t[p][:, None], sin_t[p][:, None])
    return torch.cat([rot.reshape(T, -1), out[:, (nh + nkv) * D:]], 1)


# ---- interleaved rotary at arbitrary positions ---------------------------------------------------
# The pair (x[2i], x[2i + 1]) of a head's slice [off, off + dims) turns by the angle
# position * base^(-2i / dims); what lies outside the slice passes unchanged.  The frequencies are
# computed once on the host in float64 and rounded to fp32; the angle and the rotation are fp32.
_INV_FREQ: Dict[tuple, torch.Tensor] = {}


def interleaved_inv_freq(dims: int, base: float, device) -> torch.Tensor:
    key = (int(dims), float(base), str(device))
    t = _INV_FREQ.get(key)
    if t is None:
        t = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(dims // 2)],
                         dtype=torch.float64).float().to(device)
        _INV_FREQ[key] = t
    return t


def rotate_interleaved_ref(x, positions, heads, head_stride, off, dims, inv_freq):
    T = x.shape[0]
    a = positions.float().view(T, 1, 1) * inv_freq.float().view(1, 1, -1)
    cs, sn = torch.cos(a), torch.sin(a)
    v = torch.as_strided(x, (T, heads, dims), (x.stride(0), head_stride, 1),
                         x.storage_offset() + off)
    u0, u1 = v[..., 0::2].float(), v[..., 1::2].float()
    r0, r1 = u0 * cs - u1 * sn, u1 * cs + u0 * sn
    v[..., 0::2] = r0.to(x.dtype)
    v[..., 1::2] = r1.to(x.dtype)
    return x


def rotate_interleaved_(x: torch.Tensor, positions: torch.Tensor, heads: int, head_stride: int,
                        off: int, dims: int, inv_freq: torch.Tensor) -> torch.Tensor:
    """In place: rows of x [T, >= (heads - 1) * head_stride + off + dims] (unit column stride),
    head h's slice starting at column h * head_stride + off; ``positions`` [T] int32."""
    from ._seqmix import DT, call, use_seqmix

    if dims % 2:
        raise ValueError(f"rotary dims must be even, got {dims}")
    if not use_seqmix(x):
        return rotate_interleaved_ref(x, positions, heads, head_stride, off, dims, inv_freq)
    assert x.stride(1) == 1 and positions.dtype == torch.int32
    call("sm_rotate_heads", DT[x.dtype], x, x.stride(0), head_stride, heads, off, dims, inv_freq,
         positions, x.shape[0])
    return x


# ---- rotary on the heads of a fused projection, keys and values into their paged caches ----------
# One pass over a row of z = [q heads | k heads | values]: every q and k head of size D turns on
# its first ``dims`` entries by the angle position * inv_freq[i] -- pairs (2i, 2i + 1) in the pair
# layout, (i, i + dims / 2) in the half layout --, q in place, the turned k (also kept in z) and
# the values as projected go to the cache rows ``slots``.  Angles and rotation are fp32.
def rotary_write_ref(z, positions, slots, kcache, vcache, nq, nk, D, dims, inv_freq, half):
    T = z.shape[0]
    n = nq + nk
    heads = z[:, :n * D].reshape(T, n, D).to(torch.float32, copy=True)
    if dims:
        a = positions.float().view(T, 1, 1) * inv_freq.float().view(1, 1, -1)
        cs, sn = torch.cos(a), torch.sin(a)
        if half:
            u0, u1 = heads[..., :dims // 2].clone(), heads[..., dims // 2:dims].clone()
            heads[..., :dims // 2] = u0 * cs - u1 * sn
            heads[..., dims // 2:dims] = u1 * cs + u0 * sn
        else:
            u0, u1 = heads[..., 0:dims:2].clone(), heads[..., 1:dims:2].clone()
            heads[..., 0:dims:2] = u0 * cs - u1 * sn
            heads[..., 1:dims:2] = u1 * cs + u0 * sn
    z[:, :n * D] = heads.reshape(T, n * D).to(z.dtype)
    if kcache is not None:
        ok = slots >= 0
        kcache.view(-1, nk * D)[slots[ok]] = z[:, nq * D:n * D][ok].to(kcache.dtype)
        vw = vcache.shape[2:].numel()
        vcache.view(-1, vw)[slots[ok]] = z[:, n * D:n * D + vw][ok].to(vcache.dtype)


def rotary_write(z: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor,
                 kcache: Optional[torch.Tensor], vcache: Optional[torch.Tensor], nq: int, nk: int,
                 D: int, dims: int, inv_freq: torch.Tensor, half: bool) -> None:
    """z [T, >= (nq + nk) * D + value columns] (a fused projection's output; further columns are
    left alone): the nq query heads and nk key heads (size D each, back to back from column 0)
    are rotated in place on their first ``dims`` entries, ``half`` choosing the half layout over
    the pair layout; the rotated keys go to ``kcache`` [blocks, block, ...] (rows of nk * D) and
    the columns after the keys to ``vcache`` (rows of its own width) at ``slots`` (int64; -1
    skips).  ``kcache`` None (nk must be 0): a layer that reads another's caches turns its queries
    only."""
    from ._seqmix import DT, call, use_seqmix

    if dims % 2 or dims > D:
        raise ValueError(f"rotary dims {dims} must be even and at most the head size {D}")
    vw = vcache.shape[2:].numel() if vcache is not None else 0
    if kcache is None and nk:
        raise ValueError("key heads without a key cache")
    if z.shape[1] < (nq + nk) * D + vw:
        raise ValueError(f"z has {z.shape[1]} columns, expected at least {(nq + nk) * D + vw}")
    if kcache is not None and kcache.shape[2:].numel() != nk * D:
        raise ValueError(f"cache rows of {kcache.shape[2:].numel()} do not hold keys of {nk * D}")
    if not use_seqmix(z):
        return rotary_write_ref(z, positions, slots, kcache, vcache, nq, nk, D, dims, inv_freq,
                                half)
    assert z.stride(1) == 1 and positions.dtype == torch.int32
    assert kcache is None or (kcache.is_contiguous() and vcache.is_contiguous()
                              and kcache.dtype == z.dtype and vcache.dtype == z.dtype)
    assert inv_freq.dtype == torch.float32 and inv_freq.numel() >= dims // 2
    call("sm_rotary_write", DT[z.dtype], z, z.stride(0), positions, slots, kcache, vcache,
         z.shape[0], nq, nk, D, dims, inv_freq, int(bool(half)), vw)
