"""Fanopel: a decoder-only stack of gated sliding-window attention layers with routed experts.

The stream starts as x = embed[token] + pos[position] (a learned table, positions from 0) and
is kept in fp32.  Per layer, with LN(z) = (z - mean) / sqrt(var + eps) * w (no shift) and the
configuration's ``residual_mult`` c:

    x <- x + c * mixer(LN_1(x))
    x <- x + c * experts(LN_2(x))                       (layers with a feed-forward)

Mixer ``attention`` (h is its input row):

    q = W_q h, k = W_k h;  the VALUES are k as projected (no value projection)
    q <- q / rms(q) * w_q,  k' = k / rms(k) * w_k        rms over the WHOLE projection, all heads
    s_h(i, j) = cap * tanh((q_h(i) . k'_g(j)) * scale / cap) - slope_h * (i - j)
                with g = h // (H / G) and slope_h = 2^(-8 (h + 1) / H)
    row i sees key j when j <= i and (i - j < mask.size or j < mask.keep_first)
    o_h(i) = sigmoid(W_g h(i))_h * sum_j softmax_j(s_h(i, j)) k_g(j);   y = W_o [o_0 .. o_{H-1}]

Feed-forward ``moe``: experts W_down relu(W_up h)^2.  The router scores s = sigmoid(W_r h); the
CHOICE looks at s + correction and only at the experts of the ``groups.keep`` best of
``groups.count`` equal groups of neighbours (a group ranks by the sum of its two largest
corrected scores); the ``top`` chosen experts weigh in with s_e / (sum of the chosen s + 1e-20)
* router.scale.

Output: LN with ``final.norm``, logits through ``head``.

The checkpoint names tensors ``embed`` / ``pos`` / ``l<i>.<part>`` / ``final.norm`` / ``head``;
this module keeps exactly those names.  The serving step function is
``lumen.serve.hybrid_runner.FanopelWeights.run_layers``; ``forward`` runs it on fresh caches.
"""
from __future__ import annotations

import math
from typing import Dict

import torch

from .config import ModelConfig
from .named import NamedTensorModel

MIXERS = ("attention",)
# the routing weights divide by (sum of the chosen scores + ROUTE_SUM_EPS): the design fixes it
ROUTE_SUM_EPS = 1e-20
# a group of experts ranks by the sum of this many of its largest corrected scores
GROUP_RANK_TOP = 2


def head_slopes(H: int) -> torch.Tensor:
    """Per-head rate of the linear distance bias: 2^(-8 (h + 1) / H), h = 0 .. H - 1 (fp32)."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=torch.float32)


def router_groups(f: dict) -> tuple:
    """(count, keep) of a feed-forward's expert groups; a router without groups is one group."""
    g = f["router"].get("groups") or {}
    return int(g.get("count", 1)), int(g.get("keep", g.get("count", 1)))


def tensor_shapes(cfg: ModelConfig) -> Dict[str, tuple]:
    """{checkpoint tensor name: shape} of a configuration."""
    W, V = cfg.hidden_size, cfg.vocab_size
    out: Dict[str, tuple] = {"embed": (V, W), "pos": (cfg.max_position_embeddings, W)}
    for i, L in enumerate(cfg.layer_specs):
        p, m = f"l{i}.", L["mixer"]
        x = p + "mix."
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m.get("vdim", m["dim"])
        out[p + "norm1"] = (W,)
        out[x + "q"], out[x + "k"] = (H * D, W), (G * D, W)
        out[x + "q.norm"], out[x + "k.norm"] = (H * D,), (G * D,)
        out[x + "g"] = (H, W)
        out[x + "o"] = (W, H * Dv)
        f = L.get("mlp")
        if f:
            out[p + "norm2"] = (W,)
            y = p + "mlp."
            E, ff = f["router"]["experts"], f["expert"]["ff"]
            for e in range(E):
                out[y + f"e{e}.up"] = (ff, W)
                out[y + f"e{e}.down"] = (W, ff)
            out[y + "router"] = (E, W)
            out[y + "correction"] = (E,)
    out["final.norm"] = (W,)
    out["head"] = (V, W)
    return out


def validate(cfg: ModelConfig) -> None:
    """Reject configurations the step function or its kernels cannot run, with the reason."""
    if cfg.max_position_embeddings < 1:
        raise ValueError("max_positions must be at least 1")
    for i, L in enumerate(cfg.layer_specs):
        if L["type"] not in MIXERS:
            raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
        m = L["mixer"]
        if m["heads"] % m["kv_heads"]:
            raise ValueError(f"layer {i}: heads {m['heads']} not a multiple of kv_heads "
                             f"{m['kv_heads']}")
        if m.get("vdim", m["dim"]) != m["dim"]:
            raise ValueError(f"layer {i}: the values are the keys, so vdim must equal dim")
        if m["dim"] > 512:
            raise ValueError(f"layer {i}: head size {m['dim']} > 512 is not supported")
        mask = m["mask"]
        if int(mask["size"]) < 1 or int(mask.get("keep_first", 0)) < 0:
            raise ValueError(f"layer {i}: mask.size must be >= 1 and mask.keep_first >= 0")
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


class FanopelForCausalLM(NamedTensorModel):
    supports_packing = False

    def __init__(self, config: ModelConfig, dtype=torch.bfloat16, device=None):
        validate(config)
        super().__init__(config, tensor_shapes(config), dtype, device)

    @torch.no_grad()
    def init_weights(self, std: float = 0.02, seed: int = 0):
        """Random weights for synthetic runs: projections Normal(0, 1 / sqrt(fan_in)), norm
        weights near 1, embeddings of unit and positions of a third of unit spread, router
        corrections small around 0."""
        g = torch.Generator(device="cpu").manual_seed(seed)
        for name in self.tensor_names():
            p = self.tensor(name)
            leaf = name.rsplit(".", 1)[-1]
            if name == "embed":
                v = torch.randn(p.shape, generator=g)
            elif name == "pos":
                v = 0.3 * torch.randn(p.shape, generator=g)
            elif p.dim() == 2:
                v = torch.randn(p.shape, generator=g) / math.sqrt(p.shape[1])
            elif leaf == "correction":
                v = 0.1 * torch.randn(p.shape, generator=g)
            else:                                              # norm weights
                v = 1.0 + 0.1 * torch.randn(p.shape, generator=g)
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
def load_fanopel_weights(model: FanopelForCausalLM, handles: dict, path: str) -> None:
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
