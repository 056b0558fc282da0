"""Foderax: a decoder-only stack of parallel layers whose inputs are depth-weighted averages.

The stream starts as X_0 = embed[token] * embedding_scale and is kept in fp32.  Layer i reads the
current stream x (for layer 0: X_0), norms it ONCE, and both sublayers read that:

    h       = x / sqrt(mean(x^2) + eps) * (1 + w_norm1)
    X_(i+1) = x + ls1 * mixer(h) + ls2 * experts(h)          (ls1, ls2: per-channel layer scales)
    x      <- sum_{j = 0 .. i+1} dwa_i[j] * X_j               (what layer i + 1 and the head read)

Mixers (``layers[i].type``):

``parallel``  two token mixers run on the same h: ``left_scale * left + right_scale * right``.
    left: grouped-query attention, half-layout rotary (entry i pairs with i + dims / 2) on the
    first ``rot.dims`` entries of q and k; a visible key weighs sigmoid(score * scale + pb_h) --
    no softmax; each weight stands on its own.
    right: minGRU, an element-wise linear recurrence with token-local gate and candidate:
    z = sigmoid(W_z h + b_z), u = W_x h + b_x, c = u + 1/2 (u >= 0) or sigmoid(u) (u < 0),
    S_t = (1 - z) S_(t-1) + z c element-wise from S = 0, output W_o (S_t * silu(W_g h)).

``latent_attention``  no positions.  c_q = rms(W_dq h) * w, q = W_uq c_q; the cached latent
    c = rms(W_dkv h) * w; per head k = W_uk c, v = W_uv c; softmax with an extra denominator term
    exp(sink_h); head h's output times sigmoid((W_g h)_h).  The serving path never expands the
    cache: q is projected into the latent space (W_uk^T q) and W_uv is applied to the
    attention-weighted latent.

``attention``  differential attention: every head has two score maps (q and k carry
    [map 1 | map 2] per head, biased projections, pair-layout rotary on each map) over the same
    values; o = a_1 - lambda a_2 with lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, then
    o / rms(o) * (1 - diff) per head, an element-wise sigmoid gate, the output projection.  A
    layer with ``kv_from: j`` has no key / value projections and reads layer j's caches.

Feed-forward ``moe``: experts W_down relu(W_up h)^2; router scores softmax(W_r h) over all
experts; experts form ``groups.count`` groups of neighbours, a group scores as its best member
and only the ``groups.keep`` best groups' experts can be chosen; the ``top`` chosen experts weigh
in with their scores as they are.

Output: the same offset-weight RMS norm with ``final.norm``, logits through the embedding table
(unscaled), then cap * tanh(logits / cap).

The checkpoint names tensors ``embed`` / ``l<i>.<part>`` / ``final.norm``; this module keeps
exactly those names.  The serving step function is
``lumen.serve.hybrid_runner.FoderaxWeights.run_layers``; ``forward`` runs it on fresh caches.
"""
from __future__ import annotations

import math
from typing import Dict

import torch

from .config import ModelConfig
from .named import NamedTensorModel

MIXERS = ("parallel", "latent_attention", "attention")
# the candidate of the recurrence is u + CANDIDATE_SHIFT for u >= 0 (and sigmoid(u) below, which
# meets it at u = 0): the design fixes it
CANDIDATE_SHIFT = 0.5


def router_groups(f: dict) -> tuple:
    """(count, keep) of a feed-forward's expert groups; a router without groups is one group."""
    g = f["router"].get("groups") or {}
    return int(g.get("count", 1)), int(g.get("keep", g.get("count", 1)))


def tensor_shapes(cfg: ModelConfig) -> Dict[str, tuple]:
    """{checkpoint tensor name: shape} of a configuration."""
    W, V = cfg.hidden_size, cfg.vocab_size
    out: Dict[str, tuple] = {"embed": (V, W)}
    for i, L in enumerate(cfg.layer_specs):
        p, m = f"l{i}.", L["mixer"]
        x = p + "mix."
        out[p + "norm1"] = (W,)
        if L["type"] == "parallel":
            a, Wd = m["left"], m["right"]["width"]
            H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            y = x + "left."
            out[y + "q"], out[y + "k"], out[y + "v"] = (H * D, W), (G * D, W), (G * Dv, W)
            out[y + "pb"] = (H,)
            out[y + "o"] = (W, H * Dv)
            y = x + "right."
            for n in ("z", "x"):
                out[y + n], out[y + n + ".b"] = (Wd, W), (Wd,)
            out[y + "g"] = (Wd, W)
            out[y + "o"] = (W, Wd)
        elif L["type"] == "latent_attention":
            H, D, Dv, R, Q = m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            out[x + "dq"], out[x + "dq.norm"] = (Q, W), (Q,)
            out[x + "uq"] = (H * D, Q)
            out[x + "dkv"], out[x + "dkv.norm"] = (R, W), (R,)
            out[x + "uk"], out[x + "uv"] = (H * D, R), (H * Dv, R)
            out[x + "sink"] = (H,)
            out[x + "g"] = (H, W)
            out[x + "o"] = (W, H * Dv)
        else:
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out[x + "q"], out[x + "q.b"] = (2 * H * D, W), (2 * H * D,)
            if m.get("kv_from") is None:
                out[x + "k"], out[x + "k.b"] = (2 * G * D, W), (2 * G * D,)
                out[x + "v"], out[x + "v.b"] = (G * Dv, W), (G * Dv,)
            for n in ("lq1", "lk1", "lq2", "lk2"):
                out[x + n] = (D,)
            out[x + "g"] = (H * Dv, W)
            out[x + "o"] = (W, H * Dv)
        f = L.get("mlp")
        if f:
            y = p + "mlp."
            E, ff = f["router"]["experts"], f["expert"]["ff"]
            for e in range(E):
                out[y + f"e{e}.up"] = (ff, W)
                out[y + f"e{e}.down"] = (W, ff)
            out[y + "router"] = (E, W)
            out[p + "ls2"] = (W,)
        out[p + "ls1"] = (W,)
        out[p + "dwa"] = (i + 2,)
    out["final.norm"] = (W,)
    return out


def _check_heads(i, m, what=""):
    if m["heads"] % m["kv_heads"]:
        raise ValueError(f"layer {i}{what}: heads {m['heads']} not a multiple of kv_heads "
                         f"{m['kv_heads']}")
    rot = m["rot"]
    if rot["dims"] % 2 or not 0 <= rot["dims"] <= m["dim"]:
        raise ValueError(f"layer {i}{what}: rot.dims {rot['dims']} must be even and at most dim "
                         f"{m['dim']}")
    if max(m["dim"], m["vdim"]) > 512:
        raise ValueError(f"layer {i}{what}: head sizes above 512 are not supported")


def validate(cfg: ModelConfig) -> None:
    """Reject configurations the step function or its kernels cannot run, with the reason."""
    for i, L in enumerate(cfg.layer_specs):
        if L["type"] not in MIXERS:
            raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
        m = L["mixer"]
        if L["type"] == "parallel":
            _check_heads(i, m["left"], " (left)")
            if int(m["right"]["width"]) < 1:
                raise ValueError(f"layer {i}: the recurrence needs a positive width")
        elif L["type"] == "latent_attention":
            if m["kv_rank"] > 512:
                raise ValueError(f"layer {i}: kv_rank {m['kv_rank']} > 512 is not supported")
        else:
            _check_heads(i, m)
            src = m.get("kv_from")
            if src is not None:
                if not 0 <= int(src) < i:
                    raise ValueError(f"layer {i}: kv_from {src} must name an earlier layer")
                o = cfg.layer_specs[int(src)]
                om = o["mixer"]
                if o["type"] != "attention" or om.get("kv_from") is not None:
                    raise ValueError(f"layer {i}: kv_from {src} must name an attention layer with "
                                     "key / value projections of its own")
                if any(om[k] != m[k] for k in ("kv_heads", "dim", "vdim", "rot")):
                    raise ValueError(f"layer {i}: its key heads, head sizes and rotation must "
                                     f"equal those of layer {src}, whose caches it reads")
        f = L.get("mlp")
        if not f:
            continue
        if f.get("kind") != "moe":
            raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")
        E, top = f["router"]["experts"], f["router"]["top"]
        n, keep = router_groups(f)
        if n < 1 or E % n or not 1 <= keep <= n:
            raise ValueError(f"layer {i}: {E} experts do not form {n} equal groups of which "
                             f"{keep} are kept")
        if not 1 <= top <= keep * (E // n):
            raise ValueError(f"layer {i}: top {top} must be in [1, {keep * (E // n)}] (the "
                             "experts of the kept groups)")
        if E > 1024:
            raise ValueError(f"layer {i}: more than 1024 experts are not supported")


class FoderaxForCausalLM(NamedTensorModel):
    supports_packing = False

    def __init__(self, config: ModelConfig, dtype=torch.bfloat16, device=None):
        validate(config)
        super().__init__(config, tensor_shapes(config), dtype, device)

    @torch.no_grad()
    def init_weights(self, std: float = 0.02, seed: int = 0):
        """Random weights for synthetic runs: projections Normal(0, 1 / sqrt(fan_in)), norm
        offsets small around 0, latent norm weights near 1, layer scales near 1/2, depth weights
        that favour the newest result, gate biases, sinks and score biases of order one."""
        g = torch.Generator(device="cpu").manual_seed(seed)
        for name in self.tensor_names():
            p = self.tensor(name)
            leaf = name.rsplit(".", 1)[-1]
            if name == "embed":
                v = torch.randn(p.shape, generator=g) / math.sqrt(p.shape[1])
            elif p.dim() == 2:
                v = torch.randn(p.shape, generator=g) / math.sqrt(p.shape[1])
            elif leaf == "dwa":
                v = 0.2 * torch.randn(p.shape, generator=g) / p.shape[0]
                v[-1] += 1.0
            elif leaf in ("ls1", "ls2"):
                v = 0.5 + 0.1 * torch.randn(p.shape, generator=g)
            elif leaf == "norm" and name != "final.norm":        # dq.norm / dkv.norm: plain
                v = 1.0 + 0.1 * torch.randn(p.shape, generator=g)
            elif leaf in ("lq1", "lk1", "lq2", "lk2"):
                v = 0.3 * torch.randn(p.shape, generator=g)
            elif leaf in ("pb", "sink", "b"):
                v = 0.5 * torch.randn(p.shape, generator=g)
            else:                                                  # norm1 / final.norm offsets
                v = 0.1 * torch.randn(p.shape, generator=g)
            p.copy_(v.to(p.dtype))

    @torch.no_grad()
    def forward(self, input_ids: torch.Tensor) -> torch.Tensor:
        """Logits [B, S, V] of whole sequences starting at position 0: the serving step function
        on a private cache, every row's logits kept."""
        from ..serve.hybrid_runner import forward_fresh

        if input_ids.dim() == 1:
            input_ids = input_ids.view(1, -1)
        return forward_fresh(self, input_ids)


@torch.no_grad()
def load_foderax_weights(model: FoderaxForCausalLM, handles: dict, path: str) -> None:
    """Every tensor the configuration implies must be in the checkpoint with its shape; tensors
    the configuration has no use for are listed in ``model.ignored_tensors`` and not read."""
    names = set(model.tensor_names())
    missing = sorted(names - set(handles))
    if missing:
        raise KeyError(f"{path}: missing tensors {missing[:8]}")
    model.ignored_tensors = sorted(set(handles) - names)
    for name in model.tensor_names():
        t = handles[name].get_tensor(name)
        dst = model.tensor(name)
        if tuple(t.shape) != tuple(dst.shape):
            raise ValueError(f"{name}: checkpoint {tuple(t.shape)} != model {tuple(dst.shape)}")
        if not t.is_floating_point():
            raise ValueError(f"{name}: expected a floating-point tensor, got {t.dtype}")
        dst.copy_(t.to(dst.dtype))
