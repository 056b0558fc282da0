"""A plain, slow implementation of the Fanopel design in float64: whole sequences, dense masks,
one function per mechanism.  It shares no code with ``lumen``; the tests compare the framework's
kernels and engine with it.

Weights are a dict {checkpoint tensor name: tensor}; the configuration is the checkpoint's
``config.json`` as a dict.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def weight_layer_norm(x, w, eps):
    """(x - mean) / sqrt(var + eps) * w over the last axis (population variance, no shift)."""
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def head_slopes(H):
    """Distance-bias slope of head h (0-based) among H: 2^(-8 (h + 1) / H)."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=F64)


def visible(T, window, keep_first):
    """mask[i, j]: row i sees key j when j <= i and (i - j < window or j < keep_first)."""
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    return (j <= i) & ((i - j < window) | (j < keep_first))


def gated_window_attention(h, w, p, m, eps):
    """Grouped-query attention whose values are the un-normalised keys; q and k are RMS-normed
    over their WHOLE projection (all heads at once) with a weight of that size; soft-capped scores
    minus slope_h * distance; sliding window plus the sequence's first tokens; each head's output
    scaled by the sigmoid of its own gate logit."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = h @ w[p + "q"].T
    k = h @ w[p + "k"].T
    v = k.view(T, G, D)
    q = (rms_unit(q, eps) * w[p + "q.norm"]).view(T, H, D)
    kn = (rms_unit(k, eps) * w[p + "k.norm"]).view(T, G, D)
    rep = H // G
    kn = kn.repeat_interleave(rep, 1)
    v = v.repeat_interleave(rep, 1)
    s = torch.einsum("ihd,jhd->hij", q, kn) * m["scale"]
    cap = m.get("softcap")
    if cap:
        s = cap * torch.tanh(s / cap)
    pos = torch.arange(T)
    dist = (pos.view(T, 1) - pos.view(1, T)).to(F64)
    s = s - head_slopes(H).view(H, 1, 1) * dist
    mask = visible(T, int(m["mask"]["size"]), int(m["mask"].get("keep_first", 0)))
    s = s.masked_fill(~mask, -math.inf)
    a = torch.softmax(s, -1)
    o = torch.einsum("hij,jhd->ihd", a, v)
    gate = torch.sigmoid(h @ w[p + "g"].T)                   # [T, H]
    o = (o * gate.view(T, H, 1)).reshape(T, H * D)
    return o @ w[p + "o"].T


def route(h, w, p, r):
    """Dense routing weights [T, E]: sigmoid scores; the choice adds a per-expert correction and is
    limited to the best groups (a group's rank: the sum of its two largest corrected scores); the
    chosen experts' uncorrected scores are normalised to sum 1 and scaled."""
    T = h.shape[0]
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(h @ w[p + "router"].T)
    c = s + w[p + "correction"]
    gr = r.get("groups") or {}
    n, keep = int(gr.get("count", 1)), int(gr.get("keep", 1))
    if n > 1 and keep < n:
        per = E // n
        cg = c.view(T, n, per)
        rank = cg.topk(min(2, per), -1).values.sum(-1)        # [T, n]
        best = rank.topk(keep, -1).indices
        allow = torch.zeros(T, n, dtype=torch.bool).scatter_(1, best, True)
        c = cg.masked_fill(~allow.view(T, n, 1), -math.inf).reshape(T, E)
    idx = c.topk(top, -1).indices
    chosen = torch.gather(s, 1, idx)
    wt = chosen / (chosen.sum(-1, keepdim=True) + 1e-20) * r.get("scale", 1.0)
    return torch.zeros(T, E, dtype=F64).scatter_(1, idx, wt)


def expert(h, w, p):
    return torch.relu(h @ w[p + "up"].T) ** 2 @ w[p + "down"].T


def moe_ff(h, w, p, f):
    wt = route(h, w, p, f["router"])
    out = torch.zeros_like(h)
    for e in range(f["router"]["experts"]):
        out = out + wt[:, e:e + 1] * expert(h, w, p + f"e{e}.")
    return out


def forward(cfg: dict, weights: dict, tokens, layers_out=None):
    """Logits [T, vocab] of one whole sequence from position 0."""
    w = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in weights.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.shape[0]
    eps = cfg["norm"]["eps"]
    mult = cfg.get("residual_mult", 1.0)
    x = w["embed"][tokens] + w["pos"][:T]
    for i, L in enumerate(cfg["layers"]):
        if L["type"] != "attention":
            raise ValueError(L["type"])
        h = weight_layer_norm(x, w[f"l{i}.norm1"], eps)
        x = x + mult * gated_window_attention(h, w, f"l{i}.mix.", L["mixer"], eps)
        f = L.get("mlp")
        if f:
            if f["kind"] != "moe":
                raise ValueError(f["kind"])
            x = x + mult * moe_ff(weight_layer_norm(x, w[f"l{i}.norm2"], eps), w, f"l{i}.mlp.", f)
        if layers_out is not None:
            layers_out.append(x.clone())
    return weight_layer_norm(x, w["final.norm"], eps) @ w["head"].T
