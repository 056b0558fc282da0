"""A plain, slow implementation of the Foderax design in float64: whole sequences, dense masks,
one function per mechanism.  It shares no code with ``lumen``; the tests compare the framework's
kernels and engine with it.

Weights are a dict {checkpoint tensor name: tensor}; the configuration is the checkpoint's
``config.json`` as a dict.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_rms_norm(x, w, eps):
    """RMS norm whose stored weight is an offset from one."""
    return rms_unit(x, eps) * (1.0 + w)


def angles(T, dims, base):
    """[T, dims / 2]: position * base^(-2 i / dims)."""
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    return torch.arange(T, dtype=F64).view(T, 1) * f.view(1, -1)


def rotate_half_layout(x, dims, base):
    """x [T, n, D]: entry i pairs with entry i + dims / 2 (i < dims / 2); the rest passes."""
    T = x.shape[0]
    a = angles(T, dims, base).view(T, 1, -1)
    c, s = torch.cos(a), torch.sin(a)
    half = dims // 2
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def rotate_pair_layout(x, dims, base):
    """x [T, n, D]: entry 2 i pairs with entry 2 i + 1 (i < dims / 2); the rest passes."""
    T = x.shape[0]
    a = angles(T, dims, base).view(T, 1, -1)
    c, s = torch.cos(a), torch.sin(a)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def causal(T):
    return torch.tril(torch.ones(T, T, dtype=torch.bool))


# ---- the left half of a parallel mixer: attention whose weights are sigmoids ------------------
def sigmoid_attention(h, w, p, m):
    """Grouped-query attention, half-layout rotation, weight of a visible key = sigmoid(score +
    a per-head bias), each weight on its own (no softmax)."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m["rot"]
    q = rotate_half_layout((h @ w[p + "q"].T).view(T, H, D), rot["dims"], rot["base"])
    k = rotate_half_layout((h @ w[p + "k"].T).view(T, G, D), rot["dims"], rot["base"])
    v = (h @ w[p + "v"].T).view(T, G, Dv)
    rep = H // G
    s = torch.einsum("ihd,jhd->hij", q, k.repeat_interleave(rep, 1)) * m["scale"]
    a = torch.sigmoid(s + w[p + "pb"].view(H, 1, 1)) * causal(T)
    o = torch.einsum("hij,jhd->ihd", a, v.repeat_interleave(rep, 1)).reshape(T, H * Dv)
    return o @ w[p + "o"].T


# ---- the right half: minGRU, gate and candidate computed from one token alone ------------------
def min_gru(h, w, p, state=None):
    """S_t = (1 - z_t) S_(t-1) + z_t c_t element by element, z = sigmoid(W_z h + b_z),
    c = g(W_x h + b_x) with g(u) = u + 1/2 for u >= 0 and sigmoid(u) below; the output is
    W_o (S_t * silu(W_g h)).  Returns (output, last state)."""
    T = h.shape[0]
    z = torch.sigmoid(h @ w[p + "z"].T + w[p + "z.b"])
    u = h @ w[p + "x"].T + w[p + "x.b"]
    c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    S = torch.zeros(z.shape[1], dtype=F64) if state is None else state
    rows = []
    for t in range(T):
        S = (1.0 - z[t]) * S + z[t] * c[t]
        rows.append(S)
    S_all = torch.stack(rows)
    g = h @ w[p + "g"].T
    return (S_all * (g * torch.sigmoid(g))) @ w[p + "o"].T, S


def parallel_mixer(h, w, p, m):
    left = sigmoid_attention(h, w, p + "left.", m["left"])
    right, _ = min_gru(h, w, p + "right.")
    return m["left_scale"] * left + m["right_scale"] * right


# ---- latent attention with a sink and a per-head output gate -----------------------------------
def latent_sink_attention(h, w, p, m, eps):
    """Queries and keys/values through normed low-rank latents, no positions; softmax whose
    denominator gains exp(sink_h); head h's output times sigmoid of its own gate logit."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    cq = rms_unit(h @ w[p + "dq"].T, eps) * w[p + "dq.norm"]
    q = (cq @ w[p + "uq"].T).view(T, H, D)
    c = rms_unit(h @ w[p + "dkv"].T, eps) * w[p + "dkv.norm"]
    k = (c @ w[p + "uk"].T).view(T, H, D)
    v = (c @ w[p + "uv"].T).view(T, H, Dv)
    s = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    s = s.masked_fill(~causal(T), -math.inf)
    sink = w[p + "sink"].view(H, 1, 1)
    mx = torch.maximum(s.max(-1, keepdim=True).values, sink)
    e = torch.exp(s - mx)
    a = e / (e.sum(-1, keepdim=True) + torch.exp(sink - mx))
    o = torch.einsum("hij,jhd->ihd", a, v)
    gate = torch.sigmoid(h @ w[p + "g"].T)                    # [T, H]
    return (o * gate.view(T, H, 1)).reshape(T, H * Dv) @ w[p + "o"].T


# ---- differential attention ----------------------------------------------------------------------
def diff_keys_values(h, w, p, m):
    """(k [T, G, 2, D] rotated, v [T, G, Dv]) of a differential-attention layer."""
    T = h.shape[0]
    G, D, Dv = m["kv_heads"], m["dim"], m["vdim"]
    rot = m["rot"]
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, G * 2, D)
    k = rotate_pair_layout(k, rot["dims"], rot["base"]).view(T, G, 2, D)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, Dv)
    return k, v


def diff_lambda(w, p, m):
    return (torch.exp((w[p + "lq1"] * w[p + "lk1"]).sum())
            - torch.exp((w[p + "lq2"] * w[p + "lk2"]).sum()) + m["diff"])


def differential_attention(h, w, p, m, eps, kv=None):
    """Two softmax maps per head over the same values, o = a1 - lambda a2, unit RMS per head,
    times (1 - diff); an element-wise sigmoid gate before the output projection.  ``kv``: the keys
    and values of the layer this one borrows them from."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m["rot"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, H * 2, D)
    q = rotate_pair_layout(q, rot["dims"], rot["base"]).view(T, H, 2, D)
    k, v = kv if kv is not None else diff_keys_values(h, w, p, m)
    rep = H // G
    kk = k.repeat_interleave(rep, 1)                           # [T, H, 2, D]
    s = torch.einsum("ihmd,jhmd->hmij", q, kk) * m["scale"]
    s = s.masked_fill(~causal(T), -math.inf)
    a = torch.softmax(s, -1)
    o = torch.einsum("hmij,jhd->ihmd", a, v.repeat_interleave(rep, 1))   # [T, H, 2, Dv]
    o = o[:, :, 0] - diff_lambda(w, p, m) * o[:, :, 1]
    o = rms_unit(o, eps) * (1.0 - m["diff"])
    gate = torch.sigmoid(h @ w[p + "g"].T)
    return (o.reshape(T, H * Dv) * gate) @ w[p + "o"].T


# ---- experts ---------------------------------------------------------------------------------------
def route(h, w, p, r):
    """Dense routing weights [T, E]: softmax scores over all experts; a group of neighbouring
    experts scores as its best member and only the best groups' experts can be chosen; the ``top``
    chosen experts weigh in with their scores as they are."""
    T = h.shape[0]
    E, top = r["experts"], r["top"]
    s = torch.softmax(h @ w[p + "router"].T, -1)
    c = s
    gr = r.get("groups") or {}
    n = int(gr.get("count", 1))
    keep = int(gr.get("keep", n))
    if n > 1 and keep < n:
        sg = s.view(T, n, E // n)
        best = sg.max(-1).values.topk(keep, -1).indices
        allow = torch.zeros(T, n, dtype=torch.bool).scatter_(1, best, True)
        c = sg.masked_fill(~allow.view(T, n, 1), -math.inf).reshape(T, E)
    idx = c.topk(top, -1).indices
    return torch.zeros(T, E, dtype=F64).scatter_(1, idx, torch.gather(s, 1, idx))


def expert(h, w, p):
    return torch.relu(h @ w[p + "up"].T) ** 2 @ w[p + "down"].T


def moe_ff(h, w, p, f):
    wt = route(h, w, p, f["router"])
    out = torch.zeros_like(h)
    for e in range(f["router"]["experts"]):
        out = out + wt[:, e:e + 1] * expert(h, w, p + f"e{e}.")
    return out


def soft_cap(z, cap):
    return cap * torch.tanh(z / cap)


def forward(cfg: dict, weights: dict, tokens, layers_out=None):
    """Logits [T, vocab] of one whole sequence from position 0."""
    w = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in weights.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = cfg["norm"]["eps"]
    x = w["embed"][tokens] * cfg["embedding"]["scale"]
    results = [x]                                               # X_0, then every layer's result
    kv = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        h = offset_rms_norm(x, w[p + "norm1"], eps)
        if L["type"] == "parallel":
            y = parallel_mixer(h, w, p + "mix.", m)
        elif L["type"] == "latent_attention":
            y = latent_sink_attention(h, w, p + "mix.", m, eps)
        elif L["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kv[i] = diff_keys_values(h, w, p + "mix.", m)
            y = differential_attention(h, w, p + "mix.", m, eps, kv[i if src is None else src])
        else:
            raise ValueError(L["type"])
        new = x + w[p + "ls1"] * y
        f = L.get("mlp")
        if f:
            if f["kind"] != "moe":
                raise ValueError(f["kind"])
            new = new + w[p + "ls2"] * moe_ff(h, w, p + "mlp.", f)
        results.append(new)
        a = w[p + "dwa"]
        x = sum(a[j] * results[j] for j in range(i + 2))
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = offset_rms_norm(x, w["final.norm"], eps) @ w["embed"].T
    cap = cfg.get("logit_softcap")
    return soft_cap(logits, cap) if cap else logits
