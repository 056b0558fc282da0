"""Fused residual-add + RMSNorm (HIP kernel ``kernels/rmsnorm.hip``; torch reference on CPU).

``rms_norm(x, w, eps, residual)`` returns ``(y, s)`` with ``s = x + residual`` (the new residual
stream, ``x`` itself when no residual is given) and ``y = s * rsqrt(mean(s^2) + eps) * w``.
Mirrors transformers' LlamaRMSNorm (used by the model loaded at
reference training/train_baseline.py:122) with the residual add of the decoder layer fused in.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from ._native import native, use_native

def _occupancy_cap(C) -> None:
    """(No-op.)  An occupancy cap through reserved dynamic LDS per workgroup measured no gain;
    the knob stays reachable for scripts/probes/rmsnorm_probe.py via ``C.set_rms_lds``."""


def rms_norm_ref(x, w, eps, residual=None):
    s = x if residual is None else (x.float() + residual.float()).to(x.dtype)
    sf = s.float()
    rstd = torch.rsqrt(sf.pow(2).mean(-1, keepdim=True) + eps)
    wf = (w if w.requires_grad else w.detach()).float()  # never save a ZeRO-3 param object
    y = (sf * rstd * wf).to(x.dtype)
    return y, s


class _FusedAddRMSNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, residual, w, eps, ext=0):
        C = native()
        _occupancy_cap(C)
        x = x.contiguous()
        if ext and x.dim() == 2:
            # y as the first H columns of a [rows, H + ext] buffer (row-strided kernel output)
            y = torch.empty(x.shape[0], x.shape[1] + ext, dtype=x.dtype,
                            device=x.device)[:, :x.shape[1]]
        else:
            y = torch.empty_like(x)
        rows = x.numel() // x.shape[-1]
        rstd = torch.empty(rows, dtype=torch.float32, device=x.device)
        if residual is not None:
            s = torch.empty_like(x)
            C.rmsnorm_fwd(x, residual.contiguous(), w, y, s, rstd, eps)
        else:
            s = x
            C.rmsnorm_fwd(x, None, w, y, None, rstd, eps)
        ctx.save_for_backward(s, w, rstd)
        ctx.has_res = residual is not None
        ctx.w_grad = w.requires_grad
        if residual is not None:
            return y, s
        # no residual: s is x itself; hand back a view so autograd tracks it as an output
        return y, s.view_as(s)

    @staticmethod
    def backward(ctx, dy, ds):
        C = native()
        _occupancy_cap(C)
        s, w, rstd = ctx.saved_tensors
        dx = torch.empty_like(s)
        dw = torch.zeros(w.shape, dtype=torch.float32, device=w.device) if ctx.w_grad else None
        C.rmsnorm_bwd(dy.contiguous(), s, w, rstd,
                      ds.contiguous() if ds is not None else None, dx, dw)
        dres = dx if ctx.has_res else None
        return dx, dres, (dw.to(w.dtype) if dw is not None else None), None, None


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float,
             residual: Optional[torch.Tensor] = None,
             ext: int = 0) -> Tuple[torch.Tensor, torch.Tensor]:
    if use_native(x):
        return _FusedAddRMSNorm.apply(x, residual, w, eps, ext)
    return rms_norm_ref(x, w, eps, residual)


def layer_norm(x, w, b, eps):
    """OPT LayerNorm (torch op); frozen params enter autograd as detached aliases."""
    fz = lambda t: t if (t is None or t.requires_grad) else t.detach()  # noqa: E731
    return torch.nn.functional.layer_norm(x, (x.shape[-1],), fz(w), fz(b), eps)


# ---- Dynamic Tanh (DyT): tanh(alpha * x) * w + b, no mean or variance ------------------------
# A DyT norm is the triple (w [W], b [W], alpha [] ) of fp32 tensors; alpha stays on the device
# (the kernels read it there, so a captured graph never bakes a value in).  Everything is
# computed in fp32; only the result is rounded to ``out_dtype``.
def dyt_ref(x, norm, out_dtype=None):
    w, b, alpha = norm
    y = torch.tanh(alpha.float() * x.float()) * w.float() + b.float()
    return y.to(out_dtype or x.dtype)


def dyt(x: torch.Tensor, norm, out_dtype=None) -> torch.Tensor:
    """DyT of the rows of ``x`` [rows, W] (fp32 or 16-bit) in ``out_dtype``."""
    from ._seqmix import DT, call, use_seqmix

    out_dtype = out_dtype or x.dtype
    if not use_seqmix(x):
        return dyt_ref(x, norm, out_dtype)
    x = x.contiguous()
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    call("sm_dyt", DT[x.dtype], DT[out_dtype], x, norm[0], norm[1], norm[2], out,
         x.numel() // x.shape[-1], x.shape[-1])
    return out


def dyt_residual_ref(x, y, post, pre=None, out_dtype=None):
    x.add_(dyt_ref(y, post, torch.float32))
    return x, (dyt_ref(x, pre, out_dtype or y.dtype) if pre is not None else None)


def dyt_residual(x: torch.Tensor, y: torch.Tensor, post, pre=None, out_dtype=None):
    """The fp32 residual stream ``x`` [T, W] takes a sublayer's output in place,
    x += DyT_post(y), and -- fused -- the next sublayer's input h = DyT_pre(x) is produced in
    ``out_dtype``.  Returns (x, h or None)."""
    from ._seqmix import DT, call, use_seqmix

    out_dtype = out_dtype or y.dtype
    if not use_seqmix(x):
        return dyt_residual_ref(x, y, post, pre, out_dtype)
    assert x.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous()
    h = torch.empty(x.shape, dtype=out_dtype, device=x.device) if pre is not None else None
    p = pre or (None, None, None)
    call("sm_dyt_residual", DT[y.dtype], DT[out_dtype], x, y, post[0], post[1], post[2], h,
         p[0], p[1], p[2], x.shape[0], x.shape[1])
    return x, h


# ---- RMS norm in groups ------------------------------------------------------------------------
# The row is split into ``groups`` equal consecutive parts and each part is divided by its own
# sqrt(mean(part^2) + eps); the whole row is then multiplied by w (groups = 1: the ordinary RMS
# norm with a plain weight).  fp32 throughout; only a stored result is rounded.
# (HIP: ``csrc/seqmix/rms_group.hip``.)
def group_rms_norm_ref(x, w, groups, eps, out_dtype=None):
    shp = x.shape
    g = x.float().reshape(*shp[:-1], groups, shp[-1] // groups)
    y = (g / torch.sqrt((g * g).mean(-1, keepdim=True) + eps)).reshape(shp) * w.float()
    return y.to(out_dtype or x.dtype)


def group_rms_norm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float,
                   out_dtype=None) -> torch.Tensor:
    """Group RMS norm of the rows of ``x`` [rows, W] (fp32 or 16-bit; the rows may be a column
    slice of a wider buffer) with the fp32 weight ``w`` [W], stored in ``out_dtype``."""
    from ._seqmix import DT, call, use_seqmix

    out_dtype = out_dtype or x.dtype
    if x.shape[-1] % groups:
        raise ValueError(f"width {x.shape[-1]} is not a multiple of {groups} groups")
    if not use_seqmix(x):
        return group_rms_norm_ref(x, w, groups, eps, out_dtype)
    assert x.dim() == 2 and x.stride(1) == 1 and w.dtype == torch.float32
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    call("sm_group_rms", DT[x.dtype], DT[out_dtype], x, x.stride(0), w, None, out, out.stride(0),
         x.shape[0], x.shape[1], groups, eps)
    return out


def group_rms_residual_ref(x, y, w, groups, eps, cast=None):
    x.add_(group_rms_norm_ref(y, w, groups, eps, torch.float32))
    return x, (x.to(cast) if cast is not None and cast != x.dtype else None)


def group_rms_residual(x: torch.Tensor, y: torch.Tensor, w: torch.Tensor, groups: int,
                       eps: float, cast=None):
    """The fp32 residual stream ``x`` [T, W] takes a sublayer's normed output in place,
    x += group_rms_norm(y) * w, and -- fused, when ``cast`` is a 16-bit dtype -- the new stream is
    also returned rounded to ``cast`` (what the next sublayer's GEMMs read).  Returns
    (x, x in ``cast`` or None)."""
    from ._seqmix import DT, call, use_seqmix

    if x.shape[-1] % groups:
        raise ValueError(f"width {x.shape[-1]} is not a multiple of {groups} groups")
    if not use_seqmix(x):
        return group_rms_residual_ref(x, y, w, groups, eps, cast)
    assert x.dtype == torch.float32 and x.is_contiguous() and y.stride(1) == 1
    xb = None
    if cast is not None and cast != torch.float32:
        xb = torch.empty(x.shape, dtype=cast, device=x.device)
    call("sm_group_rms", DT[y.dtype], DT[cast if xb is not None else torch.float32], y,
         y.stride(0), w, x, xb, x.shape[1], x.shape[0], x.shape[1], groups, eps)
    return x, xb


# ---- layer norm with a weight and no shift, fused with a scaled residual add -------------------
# LN(x) = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w.  The fp32 residual stream takes a
# sublayer's output multiplied by a constant, x += mult * y, and the same pass produces the next
# sublayer's input LN(x) in the model dtype.  fp32 throughout; only a stored result is rounded.
# (HIP: ``csrc/seqmix/layer_norm.hip``.)
def weight_layer_norm_ref(x, w, eps, out_dtype=None):
    xf = x.float()
    d = xf - xf.mean(-1, keepdim=True)
    y = d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w.float()
    return y.to(out_dtype or x.dtype)


def scaled_residual_layer_norm_ref(x, y, mult, w, eps, out_dtype=None):
    if y is not None:
        x.add_(y.float(), alpha=mult)
    return x, (weight_layer_norm_ref(x, w, eps, out_dtype or x.dtype) if w is not None else None)


def scaled_residual_layer_norm(x: torch.Tensor, y: Optional[torch.Tensor], mult: float,
                               w: Optional[torch.Tensor], eps: float, out_dtype=None):
    """The fp32 residual stream ``x`` [T, W] takes ``mult * y`` in place (``y`` None: nothing is
    added) and -- fused, when ``w`` [W] (fp32) is given -- h = LN(x) * w is produced in
    ``out_dtype``.  Returns (x, h or None)."""
    from ._seqmix import DT, call, use_seqmix

    if not use_seqmix(x):
        return scaled_residual_layer_norm_ref(x, y, mult, w, eps, out_dtype)
    assert x.dtype == torch.float32 and x.is_contiguous()
    assert y is None or (y.is_contiguous() and y.shape == x.shape)
    assert w is None or (w.dtype == torch.float32 and w.is_contiguous())
    if y is None and w is None:
        return x, None
    out_dtype = out_dtype or (y.dtype if y is not None else x.dtype)
    h = torch.empty(x.shape, dtype=out_dtype, device=x.device) if w is not None else None
    call("sm_layer_norm", DT[y.dtype] if y is not None else 0, DT[out_dtype], x, y, float(mult), w,
         h, x.shape[0], x.shape[1], eps)
    return x, h


def weight_layer_norm(x: torch.Tensor, w: torch.Tensor, eps: float, out_dtype=None) -> torch.Tensor:
    """LN(x) * w of the fp32 rows ``x`` [T, W] in ``out_dtype``."""
    return scaled_residual_layer_norm(x, None, 0.0, w, eps, out_dtype or x.dtype)[1]


# ---- depth-weighted layer inputs: layer scale, history, weighted average, next norm ---------------
# A stack whose layer i reads a weighted average of everything before it keeps every layer's
# result X_0 .. X_L of the step's rows in ``hist`` [L + 1, T, W] (fp32).  One pass per layer:
#     X_n = x + sum_k scale_k * y_k          (the sublayers' outputs with per-channel scales)
#     x  <- sum_{j <= n} mix[j] * X_j         (what the next layer reads)
#     h   = x / sqrt(mean(x^2) + eps) * w     (its norm, in the compute dtype)
# fp32 throughout; only h is rounded.  (HIP: ``csrc/seqmix/foderax.hip``.)
def depth_mix_norm_ref(hist, n, x, ys, scales, mix, w, eps, out_dtype):
    new = x.float().clone()
    for y, sc in zip(ys, scales):
        new += y.float() * sc.float()
    hist[n] = new
    xn = (hist[:n + 1] * mix.float().view(n + 1, 1, 1)).sum(0)
    h = None
    if w is not None:
        h = (xn / torch.sqrt((xn * xn).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)
    return xn, h


def depth_mix_norm(hist: torch.Tensor, n: int, x: torch.Tensor, ys, scales, mix: torch.Tensor,
                   w: Optional[torch.Tensor], eps: float, out_dtype=None):
    """``hist`` [L + 1, T, W] fp32 holds X_0 .. X_(n-1); ``x`` [T, W] fp32 is the stream layer
    n - 1 read; ``ys`` (up to three [T, W] sublayer outputs in the compute dtype) join it with the
    per-channel fp32 ``scales`` [W] and the sum is stored as X_n; the new stream is
    sum_j ``mix``[j] X_j over j = 0 .. n (``mix`` [n + 1] fp32) and, with ``w`` [W] (fp32, the
    weight the normed row is multiplied by), h = rms_norm(stream) * w in ``out_dtype``.  Returns
    (stream fp32 [T, W], h or None)."""
    from ._seqmix import DT, call, use_seqmix

    if not 1 <= len(ys) <= 3 or len(ys) != len(scales):
        raise ValueError("one to three sublayer outputs, each with its scale")
    if not 1 <= n < hist.shape[0] or mix.numel() != n + 1:
        raise ValueError(f"history of {hist.shape[0]} entries, entry {n}, {mix.numel()} weights")
    out_dtype = out_dtype or ys[0].dtype
    if not use_seqmix(x):
        return depth_mix_norm_ref(hist, n, x, ys, scales, mix, w, eps, out_dtype)
    T, W = x.shape
    assert hist.dtype == torch.float32 and hist.is_contiguous() and tuple(hist.shape[1:]) == (T, W)
    assert x.dtype == torch.float32 and x.is_contiguous() and mix.dtype == torch.float32
    for y, sc in zip(ys, scales):
        assert y.is_contiguous() and y.shape == x.shape and y.dtype == ys[0].dtype
        assert sc.dtype == torch.float32 and sc.is_contiguous() and sc.numel() == W
    assert w is None or (w.dtype == torch.float32 and w.is_contiguous())
    xn = torch.empty_like(x)
    h = torch.empty(T, W, dtype=out_dtype, device=x.device) if w is not None else None
    yp = list(ys) + [None] * (3 - len(ys))
    sp = list(scales) + [None] * (3 - len(ys))
    call("sm_depth_mix", DT[ys[0].dtype], DT[out_dtype], hist, n, x, yp[0], sp[0], yp[1], sp[1],
         yp[2], sp[2], mix, w, xn, h, T, W, eps)
    return xn, h
