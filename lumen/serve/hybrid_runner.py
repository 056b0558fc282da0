"""Serving runner for stacks whose layers each name their own mixer (Gedatar, Dalavik,
Fanopel, Foderax): paged caches + per-sequence recurrent state.

Four families share the runner, the segments, the block manager and the hipGraph decode; each
has its weights class (stacked projections, fp32 constants), its caches and its step function:
Gedatar (``HybridWeights`` / ``HybridState`` / ``run_layers``, described next), Dalavik
(``DalavikWeights`` / ``DalavikState``), Fanopel (``FanopelWeights`` / ``FanopelState``) and
Foderax (``FoderaxWeights`` / ``FoderaxState``), further down.

One step function for prefill chunks, decode rows and mixtures of both.  The rows of a step are
cut into segments (``ops.segments.SegBatch``: one per chunk, one per decode row); per layer

    h  = DyT + causal depthwise conv (HIP, one pass; conv tails per state slot)
    y  = mixer(h):  attention      q|k GEMM -> keys into the paged cache -> chunk/sink attention
                    wkv            token shift -> r,k,v,g GEMMs + decay GEMMs -> scan (HIP)
                    general_delta  one fused r|k|v|g|a|w1 GEMM + decay GEMM -> scan (HIP)
         -> output GEMM
    x += DyT(y); h2 = DyT(x)           (HIP, fused)
    y2 = feed-forward(h2): gate|up GEMM -> gated activation (x routing weight) -> down GEMM
    x += DyT(y2)
The residual stream x, every norm, the router, the scores and the recurrences are fp32; GEMMs and
their activations run in the model dtype (bf16 with fp32 accumulation, or true fp32).

State (``HybridState``) is indexed by the slot ``serve.state_manager.StateSlots`` gives a sequence
while it runs: conv tails [slots, taps - 1, W] for every layer, the previous row [slots, W] and
the matrix state [slots, H, D, D] of the recurrent mixers.  Nothing is cleared when a slot is
handed to a new sequence: a segment that starts at position 0 reads zeros instead of the slot.
Attention layers keep un-normalised keys only (the values are the keys) in a cache paged by the
engine's BlockManager, [blocks, block_size, kv_heads, dim] per layer.

Pure decode steps replay a hipGraph per batch bucket (ModelRunner.decode), the segment tensors
being static buffers; padding rows use the spare state slot and write no keys.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn.functional as F

from ..models.config import ModelConfig
from ..models.gedatar import DELTA_DECAY, DELTA_KEY_EPS
from ..ops.attention import (chunk_sink_attention, diff_head_combine, head_norm_write,
                             latent_write, row_attention, row_norm_write, transposed_values_ok,
                             write_key_cache)
from ..ops.conv import dyt_canon
from ..ops.embedding import embed_positions, embed_scaled, gated_token_slice, soft_cap
from ..ops.moe import gated_act, moe, route_groups, route_topk, router_logits
from ..ops.norm import (depth_mix_norm, dyt, dyt_residual, group_rms_norm, group_rms_residual,
                        scaled_residual_layer_norm, weight_layer_norm)
from ..ops.recurrent import delta_scan, min_gru_scan, token_shift, wkv_scan
from ..ops.rope import rotary_write, rotate_interleaved_
from ..ops.segments import SegBatch, whole_sequences
from .model_runner import ModelRunner, StepInput


@dataclass
class HybridLayerW:
    kind: str                       # attention | wkv | general_delta
    m: dict                         # the mixer's sizes and constants
    norms: Dict[str, tuple]         # norm1 / norm1b / norm2 / norm2b -> (w, b, alpha) fp32
    canon: torch.Tensor             # [W, taps] fp32
    w: Dict[str, torch.Tensor] = field(default_factory=dict)
    ff: Optional[dict] = None       # feed-forward: E, top, ff, ffs, gu, down, router, router_b


class HybridWeights:
    """Inference weights of a GedatarForCausalLM: projections that share an input are stacked
    into one GEMM; norm weights, biases, decay offsets and the router are kept in fp32."""

    def __init__(self, model, tp_rank: int = 0, tp_size: int = 1):
        if tp_size != 1:
            raise NotImplementedError("hybrid models are served at tensor-parallel size 1")
        cfg: ModelConfig = model.config
        self.cfg = cfg
        t = model.tensor
        f32 = lambda n: t(n).detach().float().contiguous()  # noqa: E731
        norm = lambda n: (f32(n), f32(n + ".b"), f32(n + ".alpha"))  # noqa: E731
        self.dtype = t("embed").dtype
        self.embed = t("embed").detach()
        self.final = norm("final.norm")
        self.lm_head = t("head").detach()
        self.vocab_shard = cfg.vocab_size
        self.layers: List[HybridLayerW] = []
        with torch.no_grad():
            for i, spec in enumerate(cfg.layer_specs):
                p = f"l{i}."
                x = p + "mix."
                m = spec["mixer"]
                names = ("norm1", "norm1b") + (("norm2", "norm2b") if spec.get("mlp") else ())
                L = HybridLayerW(spec["type"], m, {n: norm(p + n) for n in names},
                                 f32(p + "canon1"))
                if L.kind == "attention":
                    L.w["qk"] = torch.cat([t(x + "q"), t(x + "k")], 0).contiguous()
                elif L.kind == "wkv":
                    L.w["mu"] = torch.stack([f32(x + "mu." + s) for s in "rkvgw"]).contiguous()
                    L.w["rkvg"] = torch.stack([t(x + s).t() for s in "rkvg"]).contiguous()
                    L.w["w1"], L.w["w2"] = t(x + "w1").detach(), t(x + "w2").detach()
                    L.w["u"] = f32(x + "u")
                else:
                    L.w["in"] = torch.cat([t(x + s) for s in ("r", "k", "v", "g", "a", "w1")],
                                          0).contiguous()
                    L.w["w2"] = t(x + "w2").detach()
                    L.w["a_b"] = f32(x + "a.b")
                if L.kind != "attention":
                    L.w["w0"], L.w["norm"] = f32(x + "w0"), f32(x + "norm")
                L.w["o"] = t(x + "o").detach()
                f = spec.get("mlp")
                if f:
                    y = p + "mlp."
                    if f["kind"] == "dense":
                        L.ff = dict(E=0, top=0, ff=0, ffs=f["ff"],
                                    gu=torch.cat([t(y + "gate"), t(y + "up")], 0).contiguous(),
                                    down=t(y + "down").detach())
                    else:
                        E, top = f["router"]["experts"], f["router"]["top"]
                        ffe = f["expert"]["ff"]
                        ffs = f["shared"]["ff"] if f.get("shared") else 0
                        gu = [w for e in range(E) for w in (t(y + f"e{e}.gate"), t(y + f"e{e}.up"))]
                        dn = [t(y + f"e{e}.down") for e in range(E)]
                        if ffs:
                            gu += [t(y + "shared.gate"), t(y + "shared.up")]
                            dn.append(t(y + "shared.down"))
                        L.ff = dict(E=E, top=top, ff=ffe, ffs=ffs, gu=torch.cat(gu, 0).contiguous(),
                                    down=torch.cat(dn, 1).contiguous(), router=f32(y + "router"),
                                    router_b=f32(y + "router.b"))
                self.layers.append(L)


    # ---- what HybridRunner asks of a family's weights ----------------------------------------
    def new_state(self, slots: int, num_blocks: int, block_size: int, device):
        return HybridState(self, slots, num_blocks, block_size, device)

    def run_layers(self, st, tokens, seg, observe=None) -> torch.Tensor:
        return run_layers(self, st, tokens, seg, observe)

    def head(self, x: torch.Tensor) -> torch.Tensor:
        return F.linear(dyt(x, self.final, self.dtype), self.lm_head)


class HybridState:
    """Per-layer caches of a hybrid model: ``slots`` sequences of recurrent state (+ one spare
    slot for graph padding rows) and ``num_blocks`` pages of keys for the attention layers."""

    def __init__(self, w: HybridWeights, slots: int, num_blocks: int, block_size: int, device):
        cfg = w.cfg
        W, K = cfg.hidden_size, max(cfg.canon_taps - 1, 0)
        f32 = dict(dtype=torch.float32, device=device)
        self.slots = slots
        self.spare = slots
        self.tail = [torch.zeros(slots + 1, K, W, **f32) for _ in w.layers]
        self.prev: List[Optional[torch.Tensor]] = []
        self.S: List[Optional[torch.Tensor]] = []
        self.keys: List[Optional[torch.Tensor]] = []
        for L in w.layers:
            m = L.m
            rec = L.kind != "attention"
            self.prev.append(torch.zeros(slots + 1, W, **f32) if L.kind == "wkv" else None)
            self.S.append(torch.zeros(slots + 1, m["heads"], m["dim"], m["dim"], **f32)
                          if rec else None)
            self.keys.append(None if rec else torch.zeros(
                num_blocks, block_size, m["kv_heads"], m["dim"], dtype=w.dtype, device=device))


def key_bytes_per_token(cfg: ModelConfig, dtype_bytes: int = 2) -> int:
    """Bytes of paged cache one token takes over all layers."""
    if cfg.arch == "fanopel":                  # normed keys + the keys as projected (the values)
        return max(1, sum(2 * L["mixer"]["kv_heads"] * L["mixer"]["dim"]
                          for L in cfg.layer_specs) * dtype_bytes)
    if cfg.arch == "foderax":
        n = 0
        for L in cfg.layer_specs:
            m = L["mixer"]
            if L["type"] == "parallel":
                n += m["left"]["kv_heads"] * (m["left"]["dim"] + m["left"]["vdim"])
            elif L["type"] == "latent_attention":
                n += 2 * m["kv_rank"]                      # the latent twice: rows and transposed
            elif m.get("kv_from") is None:
                n += m["kv_heads"] * (2 * m["dim"] + m["vdim"])
        return max(1, n * dtype_bytes)
    if cfg.arch == "dalavik":
        n = 0
        for L in cfg.layer_specs:
            m = L["mixer"]
            if L["type"] == "attention":
                n += m["kv_heads"] * (m["dim"] + m["vdim"])
            elif m.get("kv_from") is None:
                n += 2 * m["kv_rank"] + m["rot_dim"]     # the latent twice: rows and transposed
        return max(1, n * dtype_bytes)
    return max(1, sum(L["mixer"]["kv_heads"] * L["mixer"]["dim"] for L in cfg.layer_specs
                      if L["type"] == "attention") * dtype_bytes)


def state_bytes_per_slot(cfg: ModelConfig) -> int:
    if cfg.arch in ("dalavik", "fanopel"):
        return 0
    if cfg.arch == "foderax":
        return 4 * sum(L["mixer"]["right"]["width"] for L in cfg.layer_specs
                       if L["type"] == "parallel")
    n = 0
    for L in cfg.layer_specs:
        n += max(cfg.canon_taps - 1, 0) * cfg.hidden_size
        if L["type"] != "attention":
            n += L["mixer"]["heads"] * L["mixer"]["dim"] ** 2
        if L["type"] == "wkv":
            n += cfg.hidden_size
    return 4 * n


def run_layers(w: HybridWeights, st: HybridState, tokens: torch.Tensor, seg: SegBatch,
               observe=None) -> torch.Tensor:
    """The step function: token ids [T] + their segments -> the fp32 residual stream [T, W]
    after the last layer.  State and key cache in ``st`` move on by the step's rows."""
    cfg = w.cfg
    dt = w.dtype
    eps = cfg.rms_norm_eps
    x = F.embedding(tokens, w.embed).float()
    for i, L in enumerate(w.layers):
        m = L.m
        h = dyt_canon(x, L.norms["norm1"], L.canon, st.tail[i], seg, dt)
        if L.kind == "attention":
            H, G, D = m["heads"], m["kv_heads"], m["dim"]
            qk = F.linear(h, L.w["qk"])
            write_key_cache(qk[:, H * D:], st.keys[i], seg.cache_slots)
            o = chunk_sink_attention(qk[:, :H * D], st.keys[i], seg, H, G, D, float(m["scale"]),
                                     int(m["mask"]["size"]), eps, sink=True)
        elif L.kind == "wkv":
            H, D = m["heads"], m["dim"]
            mix = token_shift(h, L.w["mu"], st.prev[i], seg)
            rkvg = torch.bmm(mix[:4], L.w["rkvg"])
            wl = F.linear(torch.tanh(F.linear(mix[4], L.w["w1"])), L.w["w2"])
            o = wkv_scan(rkvg[0], rkvg[1], rkvg[2], wl, rkvg[3], L.w["w0"], L.w["u"], L.w["norm"],
                         st.S[i], seg, H, D, eps)
        else:
            H, D = m["heads"], m["dim"]
            HD = H * D
            z = F.linear(h, L.w["in"])
            wl = F.linear(torch.tanh(z[:, 5 * HD:]), L.w["w2"])
            o = delta_scan(z[:, :HD], z[:, HD:2 * HD], z[:, 2 * HD:3 * HD], wl,
                           z[:, 4 * HD:5 * HD], z[:, 3 * HD:4 * HD], L.w["w0"], L.w["a_b"],
                           L.w["norm"], st.S[i], seg, H, D, eps, DELTA_DECAY, DELTA_KEY_EPS)
        y = F.linear(o, L.w["o"])
        f = L.ff
        if f is None:
            x, _ = dyt_residual(x, y, L.norms["norm1b"], None, dt)
        else:
            x, h2 = dyt_residual(x, y, L.norms["norm1b"], L.norms["norm2"], dt)
            if f["E"]:
                # the router in fp32, on the (possibly 16-bit rounded) normed row
                z = torch.addmm(f["router_b"], h2.float(), f["router"].t())
                y2 = moe(h2, route_topk(z, f["top"]), f["gu"], f["down"], f["E"], f["top"],
                         f["ff"], f["ffs"])
            else:
                y2 = F.linear(gated_act(F.linear(h2, f["gu"]), None, 0, 0, f["ffs"]), f["down"])
            x, _ = dyt_residual(x, y2, L.norms["norm2b"], None, dt)
        if observe is not None:
            observe(i, x)
    return x


# ---- Dalavik: latent attention + grouped-query attention with score shaping ----------------------
#
#   x, xb   the fp32 residual stream and (16-bit serving) its rounded copy that the GEMMs read;
#           every residual kernel hands both on, so no separate cast pass exists
#   latent_attention
#       z  = [W_dq ; W_dkv] xb               one GEMM; a layer that borrows a cache has W_dq only
#       cache row <- [rms(z_kv[:R]) * w | rotate(z_kv[R:])]                     (latent_write)
#       q  = W_uq (rms(z_q) * w), its rotated part turned in place               (rotate_interleaved_)
#       qa = per-head W_uk^T q_plain         the query in the latent space (batched GEMM)
#       ol = row_attention([qa | q_rot] against the cached row, value = its first R columns)
#       y  = W_o (per-head W_uv ol)          (batched GEMM into the token-major layout, then GEMM)
#   attention
#       qkv = [W_q ; W_k ; W_v] xb + b       one GEMM
#       q normed in place, normed k and v into their caches                      (head_norm_write)
#       o  = row_attention(temperature, soft cap, distance bias, head mixing, sink);  y = W_o o
#   x += gnorm_1(y)                          (group_rms_residual, also the next xb)
#   x += gnorm_2(W_down (relu(gate) * up))   one [gate ; up] GEMM, fused activation
#   x += rms(W_proj (gelu_tanh(W_sgate xb) * E[token, slice])) * w               (token side input)
#
# fp32: the stream, every norm, angles, scores, softmax; model dtype: GEMMs and what they store.
# Nothing here is per-sequence state: a sequence's whole memory is its cache blocks.
@dataclass
class DalavikLayerW:
    kind: str                       # latent_attention | attention
    m: dict                         # the mixer's sizes and constants
    norm1: torch.Tensor
    w: Dict[str, torch.Tensor] = field(default_factory=dict)
    ff: Optional[dict] = None       # gu [2 ff, W], down [W, ff], ff, norm
    side: Optional[dict] = None     # gate [d, W], proj [W, d], norm [W], col0
    kv_layer: int = -1              # latent attention: the layer whose cache rows it reads


class DalavikWeights:
    """Inference weights of a DalavikForCausalLM: projections that share an input are stacked
    into one GEMM, the per-head up projections are laid out for batched GEMMs, norm weights and
    the attention's per-head constants are fp32."""

    def __init__(self, model, tp_rank: int = 0, tp_size: int = 1):
        if tp_size != 1:
            raise NotImplementedError("Dalavik models are served at tensor-parallel size 1")
        from ..ops.rope import interleaved_inv_freq

        cfg: ModelConfig = model.config
        self.cfg = cfg
        t = model.tensor
        f32 = lambda n: t(n).detach().float().contiguous()  # noqa: E731
        self.dtype = t("embed").dtype
        dev = t("embed").device
        self.embed = t("embed").detach()
        self.lm_head = self.embed                           # tied
        self.final = f32("final.norm")
        self.vocab_shard = cfg.vocab_size
        sd = cfg.token_side_dim
        self.side_embed = t("side.embed").detach() if sd else None
        self.layers: List[DalavikLayerW] = []
        with torch.no_grad():
            for i, spec in enumerate(cfg.layer_specs):
                p, m = f"l{i}.", spec["mixer"]
                x = p + "mix."
                L = DalavikLayerW(spec["type"], m, f32(p + "norm1"))
                if L.kind == "latent_attention":
                    H, D, Dv, R = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
                    own = m.get("kv_from") is None
                    L.kv_layer = i if own else int(m["kv_from"])
                    L.w["down"] = (torch.cat([t(x + "dq"), t(x + "dkv")], 0).contiguous()
                                   if own else t(x + "dq").detach())
                    L.w["dq_norm"] = f32(x + "dq.norm")
                    if own:
                        L.w["dkv_norm"] = f32(x + "dkv.norm")
                    L.w["uq"] = t(x + "uq").detach()
                    L.w["uk"] = t(x + "uk").detach().view(H, D, R)                   # q_h @ uk[h]
                    L.w["uvT"] = t(x + "uv").detach().view(H, Dv, R).transpose(1, 2).contiguous()
                    L.w["inv_freq"] = interleaved_inv_freq(m["rot"]["dims"], m["rot"]["base"], dev)
                else:
                    L.w["qkv"] = torch.cat([t(x + n) for n in "qkv"], 0).contiguous()
                    L.w["qkv_b"] = torch.cat([t(x + n + ".b") for n in "qkv"], 0).contiguous()
                    for n in ("q.norm", "k.norm", "r1", "r2", "talk", "sink"):
                        L.w[n] = f32(x + n)
                L.w["o"] = t(x + "o").detach()
                f = spec.get("mlp")
                if f:
                    L.ff = dict(ff=f["ff"], norm=f32(p + "norm2"), down=t(p + "mlp.down").detach(),
                                gu=torch.cat([t(p + "mlp.gate"), t(p + "mlp.up")], 0).contiguous())
                if sd:
                    L.side = dict(gate=t(p + "side.gate").detach(), proj=t(p + "side.proj").detach(),
                                  norm=f32(p + "side.norm"), col0=i * sd)
                self.layers.append(L)

    def new_state(self, slots: int, num_blocks: int, block_size: int, device):
        return DalavikState(self, slots, num_blocks, block_size, device)

    def run_layers(self, st, tokens, seg, observe=None) -> torch.Tensor:
        return run_dalavik_layers(self, st, tokens, seg, observe)

    def head(self, x: torch.Tensor) -> torch.Tensor:
        h = group_rms_norm(x, self.final, self.cfg.norm_groups, self.cfg.rms_norm_eps, self.dtype)
        return F.linear(h, self.lm_head)


class DalavikState:
    """Paged caches of a Dalavik model: one row [latent | rotated key part] per token for every
    latent-attention layer that projects its own (a borrowing layer reads the lender's) plus,
    where the matrix-core value product can use it, the latents transposed within each block
    [blocks, R, block]; normed keys and values for every grouped-query layer.  No per-sequence state: ``spare`` only names
    the slot number graph padding rows carry."""

    def __init__(self, w: DalavikWeights, slots: int, num_blocks: int, block_size: int, device):
        self.slots = slots
        self.spare = slots
        kw = dict(dtype=w.dtype, device=device)
        self.lat: List[Optional[torch.Tensor]] = []
        self.latT: List[Optional[torch.Tensor]] = []
        self.k: List[Optional[torch.Tensor]] = []
        self.v: List[Optional[torch.Tensor]] = []
        for i, L in enumerate(w.layers):
            m = L.m
            own = L.kind == "latent_attention" and L.kv_layer == i
            self.lat.append(torch.zeros(num_blocks, block_size, m["kv_rank"] + m["rot_dim"], **kw)
                            if own else None)
            self.latT.append(torch.zeros(num_blocks, m["kv_rank"], block_size, **kw)
                             if own and transposed_values_ok(w.dtype, m["kv_rank"], m["rot_dim"],
                                                             block_size, device) else None)
            att = L.kind == "attention"
            self.k.append(torch.zeros(num_blocks, block_size, m["kv_heads"], m["dim"], **kw)
                          if att else None)
            self.v.append(torch.zeros(num_blocks, block_size, m["kv_heads"], m["vdim"], **kw)
                          if att else None)


def run_dalavik_layers(w: DalavikWeights, st: DalavikState, tokens: torch.Tensor, seg: SegBatch,
                       observe=None) -> torch.Tensor:
    """The step function: token ids [T] + their segments -> the fp32 residual stream [T, W]
    after the last layer; the caches in ``st`` take the step's rows."""
    cfg = w.cfg
    dt = w.dtype
    eps, groups = cfg.rms_norm_eps, cfg.norm_groups
    T = tokens.shape[0]
    x = F.embedding(tokens, w.embed).float()
    cast = dt if dt != torch.float32 else None
    xb = x.to(dt) if cast is not None else x
    for i, L in enumerate(w.layers):
        m = L.m
        if L.kind == "latent_attention":
            H, D, Dr, Dv, R, Q = (m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"],
                                  m["q_rank"])
            z = F.linear(xb, L.w["down"])
            if L.kv_layer == i:
                latent_write(z[:, Q:], L.w["dkv_norm"], L.w["inv_freq"], seg.positions,
                             seg.cache_slots, st.lat[i], R, m["rot"]["dims"], eps, st.latT[i])
            cache = st.lat[L.kv_layer]
            q = F.linear(group_rms_norm(z[:, :Q], L.w["dq_norm"], 1, eps, dt), L.w["uq"])
            rotate_interleaved_(q, seg.positions, H, D + Dr, D, m["rot"]["dims"], L.w["inv_freq"])
            q3 = q.view(T, H, D + Dr)
            qa = torch.bmm(q3[:, :, :D].transpose(0, 1), L.w["uk"])              # [H, T, R]
            ol = torch.empty(H, T, R, dtype=dt, device=x.device)
            row_attention(qa.transpose(0, 1), q3[:, :, D:], cache, cache, R, ol.transpose(0, 1),
                          seg, H, 1, float(m["scale"]), vt=st.latT[L.kv_layer])
            o = torch.empty(T, H, Dv, dtype=dt, device=x.device)
            torch.bmm(ol, L.w["uvT"], out=o.transpose(0, 1))
        else:
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            qkv = F.linear(xb, L.w["qkv"], L.w["qkv_b"])
            head_norm_write(qkv, L.w["q.norm"], L.w["k.norm"], seg.cache_slots, st.k[i], st.v[i],
                            H, G, D, Dv, eps)
            qt = m.get("q_temp")
            o = torch.empty(T, H, Dv, dtype=dt, device=x.device)
            row_attention(qkv[:, :H * D].view(T, H, D), None, st.k[i], st.v[i], Dv, o, seg, H, G,
                          float(m["scale"]), float(m.get("softcap") or 0.0),
                          (float(qt["coef"]), int(qt["every"])) if qt else None,
                          L.w["r1"], L.w["r2"], L.w["talk"], L.w["sink"])
        y = F.linear(o.view(T, H * Dv), L.w["o"])
        x, xc = group_rms_residual(x, y, L.norm1, groups, eps, cast)
        xb = xc if cast is not None else x
        f = L.ff
        if f is not None:
            y = F.linear(gated_act(F.linear(xb, f["gu"]), None, 0, 0, f["ff"], "relu"), f["down"])
            x, xc = group_rms_residual(x, y, f["norm"], groups, eps, cast)
            xb = xc if cast is not None else x
        sd = L.side
        if sd is not None:
            g = gated_token_slice(F.linear(xb, sd["gate"]), w.side_embed, tokens, sd["col0"])
            x, xc = group_rms_residual(x, F.linear(g, sd["proj"]), sd["norm"], 1, eps, cast)
            xb = xc if cast is not None else x
        if observe is not None:
            observe(i, x)
    return x


# ---- Fanopel: gated window attention over keys-as-values + group-limited sigmoid routing ---------
#
#   x = embed[token] + pos[position]           fp32 stream (embed_positions); h = LN_1(x)
#   attention
#       z  = [W_q ; W_k ; W_g ; 0] h            one GEMM (rows padded to a multiple of 8 columns)
#       q normed over the whole projection in place; k normed the same way into the key cache, k as
#       projected into the value cache                                            (row_norm_write)
#       o  = row_attention(soft cap, linear distance bias, window + kept first keys, sigmoid gate
#            of z's gate columns on every head's output);  y = W_o o
#   x += c y; h = LN_2(x)                       (scaled_residual_layer_norm, one pass)
#   experts
#       r  = route_groups(W_r h in fp32)        dense weights [T, E], zero off the chosen experts
#            (router_logits: exact 16-bit products, fp32 accumulation and result)
#       y  = [W_down_0 .. W_down_E-1] (relu(W_up h)^2 * r)     two stacked GEMMs, or per expert on
#            its own rows for prefill-sized steps (ops.moe)
#   x += c y; h = LN_1 of the next layer (or the final norm's weight after the last layer)
#
# fp32: the stream, every norm, the router, scores, softmax, the gate's sigmoid; model dtype: GEMMs
# and what they store.  A sequence's whole memory is its cache blocks.
@dataclass
class FanopelLayerW:
    m: dict                         # the mixer's sizes and constants
    norm1: torch.Tensor
    w: Dict[str, torch.Tensor] = field(default_factory=dict)
    ff: Optional[dict] = None       # E, top, ff, up [E ff, W], down [W, E ff], router, correction...


class FanopelWeights:
    """Inference weights of a FanopelForCausalLM: q | k | gate stacked into one GEMM, the experts'
    up projections stacked row-wise and their down projections side by side; norm weights, the
    router's correction and the distance-bias slopes in fp32 (the router's weight stays in the
    model dtype: its logits are formed in fp32 from the exact products, ``ops.moe.router_logits``)."""

    def __init__(self, model, tp_rank: int = 0, tp_size: int = 1):
        if tp_size != 1:
            raise NotImplementedError("Fanopel models are served at tensor-parallel size 1")
        from ..models.fanopel import GROUP_RANK_TOP, ROUTE_SUM_EPS, head_slopes, router_groups

        cfg: ModelConfig = model.config
        self.cfg = cfg
        t = model.tensor
        f32 = lambda n: t(n).detach().float().contiguous()  # noqa: E731
        self.dtype = t("embed").dtype
        dev = t("embed").device
        self.embed = t("embed").detach()
        self.pos = t("pos").detach()
        self.lm_head = t("head").detach()
        self.final = f32("final.norm")
        self.vocab_shard = cfg.vocab_size
        self.max_positions = int(self.pos.shape[0])
        self.mult = float(cfg.residual_mult)
        self.layers: List[FanopelLayerW] = []
        with torch.no_grad():
            for i, spec in enumerate(cfg.layer_specs):
                p, m = f"l{i}.", spec["mixer"]
                x = p + "mix."
                L = FanopelLayerW(m, f32(p + "norm1"))
                H, G, D = m["heads"], m["kv_heads"], m["dim"]
                W = cfg.hidden_size
                rows = (H + G) * D + H
                pad = -rows % 8                # the q / k / gate views keep 16-byte row strides
                parts = [t(x + "q"), t(x + "k"), t(x + "g")]
                if pad:
                    parts.append(torch.zeros(pad, W, dtype=self.dtype, device=dev))
                L.w["qkg"] = torch.cat(parts, 0).contiguous()
                L.w["q.norm"], L.w["k.norm"] = f32(x + "q.norm"), f32(x + "k.norm")
                L.w["slopes"] = head_slopes(H).to(dev)
                L.w["o"] = t(x + "o").detach()
                f = spec.get("mlp")
                if f:
                    y = p + "mlp."
                    r = f["router"]
                    E = r["experts"]
                    n, keep = router_groups(f)
                    L.ff = dict(E=E, top=int(r["top"]), ff=int(f["expert"]["ff"]), groups=n, keep=keep,
                                scale=float(r.get("scale", 1.0)), sum_eps=ROUTE_SUM_EPS,
                                rank_top=GROUP_RANK_TOP, norm=f32(p + "norm2"),
                                up=torch.cat([t(y + f"e{e}.up") for e in range(E)], 0).contiguous(),
                                down=torch.cat([t(y + f"e{e}.down") for e in range(E)], 1).contiguous(),
                                router=t(y + "router").detach(), correction=f32(y + "correction"))
                self.layers.append(L)

    def new_state(self, slots: int, num_blocks: int, block_size: int, device):
        return FanopelState(self, slots, num_blocks, block_size, device)

    def run_layers(self, st, tokens, seg, observe=None) -> torch.Tensor:
        return run_fanopel_layers(self, st, tokens, seg, observe)

    def head(self, x: torch.Tensor) -> torch.Tensor:
        return F.linear(weight_layer_norm(x, self.final, self.cfg.rms_norm_eps, self.dtype),
                        self.lm_head)


class FanopelState:
    """Paged caches of a Fanopel model: per layer the normed keys (what the scores read) and the
    keys as projected (the values), [blocks, block, kv_heads, dim] each.  No per-sequence state:
    ``spare`` only names the slot number graph padding rows carry."""

    def __init__(self, w: FanopelWeights, slots: int, num_blocks: int, block_size: int, device):
        self.slots = slots
        self.spare = slots
        kw = dict(dtype=w.dtype, device=device)
        shape = lambda m: (num_blocks, block_size, m["kv_heads"], m["dim"])  # noqa: E731
        self.k = [torch.zeros(shape(L.m), **kw) for L in w.layers]
        self.v = [torch.zeros(shape(L.m), **kw) for L in w.layers]


def run_fanopel_layers(w: FanopelWeights, st: FanopelState, tokens: torch.Tensor, seg: SegBatch,
                       observe=None) -> torch.Tensor:
    """The step function: token ids [T] + their segments -> the fp32 residual stream [T, W]
    after the last layer; the caches in ``st`` take the step's rows."""
    cfg = w.cfg
    dt = w.dtype
    eps, c = cfg.rms_norm_eps, w.mult
    T = tokens.shape[0]
    x = embed_positions(tokens, seg.positions, w.embed, w.pos)
    h = weight_layer_norm(x, w.layers[0].norm1, eps, dt)
    n_layers = len(w.layers)
    for i, L in enumerate(w.layers):
        m = L.m
        H, G, D = m["heads"], m["kv_heads"], m["dim"]
        z = F.linear(h, L.w["qkg"])
        row_norm_write(z, L.w["q.norm"], L.w["k.norm"], seg.cache_slots, st.k[i], st.v[i],
                       H * D, G * D, eps)
        o = torch.empty(T, H, D, dtype=dt, device=x.device)
        mask = m["mask"]
        row_attention(z[:, :H * D].view(T, H, D), None, st.k[i], st.v[i], D, o, seg, H, G,
                      float(m["scale"]), float(m.get("softcap") or 0.0), slopes=L.w["slopes"],
                      window=int(mask["size"]), keep_first=int(mask.get("keep_first", 0)),
                      gate=z[:, (H + G) * D:(H + G) * D + H])
        y = F.linear(o.view(T, H * D), L.w["o"])
        nxt = w.layers[i + 1].norm1 if i + 1 < n_layers else None
        f = L.ff
        if f is None:
            x, h = scaled_residual_layer_norm(x, y, c, nxt, eps, dt)
        else:
            x, h2 = scaled_residual_layer_norm(x, y, c, f["norm"], eps, dt)
            # the router in fp32, on the (possibly 16-bit rounded) normed row
            r = route_groups(router_logits(h2, f["router"]), f["correction"], f["top"], f["groups"],
                             f["keep"], f["scale"], f["sum_eps"], f["rank_top"])
            y2 = moe(h2, r, f["up"], f["down"], f["E"], f["top"], f["ff"], 0, "relu2", gated=False)
            x, h = scaled_residual_layer_norm(x, y2, c, nxt, eps, dt)
        if observe is not None:
            observe(i, x)
    return x


# ---- Foderax: parallel layers on depth-weighted inputs ---------------------------------------------
#
#   hist[0] = embed[token] * scale (fp32);  x = hist[0];  h = rms(x) * (1 + w)   (model dtype)
#   per layer i, every sublayer reading the same h:
#   parallel
#       z  = [W_q ; W_k ; W_v ; W_z ; W_x ; W_g] h     one GEMM (left attention | right recurrence)
#       q, k turned in the half layout, k and v into their caches                 (rotary_write)
#       o  = row_attention(sigmoid weights: sigmoid(score + pb_h), not normalised);  y_l = W_ol o
#       r  = min_gru_scan(z's last three blocks, the slot's fp32 state);          y_r = W_or r
#   latent_attention
#       z  = [W_dq ; W_dkv ; W_g] h                    one GEMM
#       cache row <- rms(z_kv) * w                      (latent_write, + the per-block transpose)
#       q  = W_uq (rms(z_q) * w);  qa = per-head W_uk^T q   (the query in the latent space)
#       ol = row_attention(qa against the cached rows, value = the row, sink, per-head gate)
#       y  = W_o (per-head W_uv ol)
#   attention (differential)
#       z  = [W_q' ; W_k ; W_v ; W_g] h + b            one GEMM; q' = q's rows reordered to
#            [key head][map][query head of the group], so that the two maps are 2 H heads on 2 G
#            key heads sharing G value heads
#       q', k turned in the pair layout, k and v into their caches (a borrowing layer: q' only)
#       a  = row_attention(2 H heads, v_div = 2);  o = diff_head_combine(a, lambda, 1 - diff, gate)
#       y  = W_o o
#   experts: r = route_groups(softmax scores, groups ranked by their best member, weights as they
#            are);  y_f = [W_down_e] (relu(W_up h)^2 * r)
#   hist[i + 1] = x + ls1 * y (+ ls2 * y_f);  x = sum_j dwa[j] hist[j];  h = rms(x) * (1 + w_next)
#                                                                          (depth_mix_norm, one pass)
#   logits = cap * tanh((embed h_final) / cap)         fp32 product of the 16-bit operands
#
# fp32: the stream and its history, norms, angles, scores, sigmoid / softmax weights, sinks, the
# map combination and its norm, gates' sigmoids, the recurrence (gates, candidate, state), the
# router; model dtype: GEMMs and what they store.
@dataclass
class FoderaxLayerW:
    kind: str                       # parallel | latent_attention | attention
    m: dict                         # the mixer's sizes and constants
    norm1: torch.Tensor             # 1 + the stored offset, fp32
    w: Dict[str, torch.Tensor] = field(default_factory=dict)
    c: dict = field(default_factory=dict)      # host constants
    ff: Optional[dict] = None
    kv_layer: int = -1              # attention: the layer whose caches it reads


def _pad_rows(parts, dtype, dev):
    """Stack projection weights row-wise, zero rows added up to a multiple of 8 output columns (so
    that every view of the GEMM's output keeps 16-byte row strides)."""
    rows = sum(p.shape[0] for p in parts)
    pad = -rows % 8
    if pad:
        parts = list(parts) + [torch.zeros(pad, parts[0].shape[1], dtype=dtype, device=dev)]
    return torch.cat(parts, 0).contiguous()


class FoderaxWeights:
    """Inference weights of a FoderaxForCausalLM: projections that share the layer's one normed
    input are stacked into one GEMM, differential queries are reordered by key head and map, the
    per-head up projections of latent attention are laid out for batched GEMMs, the experts' up
    projections are stacked row-wise and their down projections side by side; norm weights (with
    the 1 added), layer scales (with the mixers' constant scales folded in), depth weights and
    per-head constants are fp32."""

    def __init__(self, model, tp_rank: int = 0, tp_size: int = 1):
        if tp_size != 1:
            raise NotImplementedError("Foderax models are served at tensor-parallel size 1")
        from ..models.foderax import CANDIDATE_SHIFT, router_groups
        from ..ops.rope import interleaved_inv_freq

        cfg: ModelConfig = model.config
        self.cfg = cfg
        t = model.tensor
        f32 = lambda n: t(n).detach().float().contiguous()  # noqa: E731
        f64 = lambda n: t(n).detach().double()  # noqa: E731
        self.dtype = dt = t("embed").dtype
        dev = t("embed").device
        self.embed = t("embed").detach()
        self.lm_head = self.embed                           # tied, unscaled
        self.final = (1.0 + f32("final.norm")).contiguous()
        self.vocab_shard = cfg.vocab_size
        self.shift = float(CANDIDATE_SHIFT)
        self.layers: List[FoderaxLayerW] = []
        with torch.no_grad():
            for i, spec in enumerate(cfg.layer_specs):
                p, m = f"l{i}.", spec["mixer"]
                x = p + "mix."
                L = FoderaxLayerW(spec["type"], m, (1.0 + f32(p + "norm1")).contiguous())
                ls1 = f32(p + "ls1")
                if L.kind == "parallel":
                    a = m["left"]
                    lt, rt = x + "left.", x + "right."
                    L.w["in"] = _pad_rows([t(lt + "q"), t(lt + "k"), t(lt + "v"), t(rt + "z"),
                                           t(rt + "x"), t(rt + "g")], dt, dev)
                    L.w["pb"] = f32(lt + "pb")
                    L.w["b_z"], L.w["b_x"] = f32(rt + "z.b"), f32(rt + "x.b")
                    L.w["o_l"], L.w["o_r"] = t(lt + "o").detach(), t(rt + "o").detach()
                    L.w["inv_freq"] = interleaved_inv_freq(a["rot"]["dims"], a["rot"]["base"], dev)
                    L.w["scales"] = [(ls1 * float(m["left_scale"])).contiguous(),
                                     (ls1 * float(m["right_scale"])).contiguous()]
                elif L.kind == "latent_attention":
                    H, D, Dv, R = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
                    L.w["in"] = _pad_rows([t(x + "dq"), t(x + "dkv"), t(x + "g")], dt, dev)
                    L.w["dq_norm"], L.w["dkv_norm"] = f32(x + "dq.norm"), f32(x + "dkv.norm")
                    L.w["uq"] = t(x + "uq").detach()
                    L.w["uk"] = t(x + "uk").detach().view(H, D, R)                   # q_h @ uk[h]
                    L.w["uvT"] = t(x + "uv").detach().view(H, Dv, R).transpose(1, 2).contiguous()
                    L.w["sink"] = f32(x + "sink")
                    L.w["o"] = t(x + "o").detach()
                    L.w["scales"] = [ls1]
                else:
                    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
                    rep = H // G
                    own = m.get("kv_from") is None
                    L.kv_layer = i if own else int(m["kv_from"])
                    # query rows [head][map][D] -> [key head][map][head of the group][D]
                    perm = (torch.arange(2 * H * D, device=dev).view(G, rep, 2, D)
                            .permute(0, 2, 1, 3).reshape(-1))
                    parts = [t(x + "q").detach()[perm]]
                    bias = [t(x + "q.b").detach()[perm]]
                    if own:
                        parts += [t(x + "k"), t(x + "v")]
                        bias += [t(x + "k.b"), t(x + "v.b")]
                    parts.append(t(x + "g"))
                    bias.append(torch.zeros(H * Dv, dtype=dt, device=dev))
                    L.w["in"] = _pad_rows(parts, dt, dev)
                    b = torch.cat(bias, 0)
                    L.w["in_b"] = torch.cat([b, b.new_zeros(L.w["in"].shape[0] - b.shape[0])])
                    L.c["lam"] = float(torch.exp((f64(x + "lq1") * f64(x + "lk1")).sum())
                                       - torch.exp((f64(x + "lq2") * f64(x + "lk2")).sum())
                                       + float(m["diff"]))
                    L.w["inv_freq"] = interleaved_inv_freq(m["rot"]["dims"], m["rot"]["base"], dev)
                    L.w["o"] = t(x + "o").detach()
                    L.w["scales"] = [ls1]
                L.w["dwa"] = f32(p + "dwa")
                f = spec.get("mlp")
                if f:
                    y = p + "mlp."
                    r = f["router"]
                    E = r["experts"]
                    n, keep = router_groups(f)
                    L.ff = dict(E=E, top=int(r["top"]), ff=int(f["expert"]["ff"]), groups=n, keep=keep,
                                up=torch.cat([t(y + f"e{e}.up") for e in range(E)], 0).contiguous(),
                                down=torch.cat([t(y + f"e{e}.down") for e in range(E)], 1).contiguous(),
                                router=t(y + "router").detach(), ls2=f32(p + "ls2"))
                self.layers.append(L)

    def new_state(self, slots: int, num_blocks: int, block_size: int, device):
        return FoderaxState(self, slots, num_blocks, block_size, device)

    def run_layers(self, st, tokens, seg, observe=None) -> torch.Tensor:
        return run_foderax_layers(self, st, tokens, seg, observe)

    def head(self, x: torch.Tensor) -> torch.Tensor:
        h = group_rms_norm(x, self.final, 1, self.cfg.rms_norm_eps, self.dtype)
        z = router_logits(h, self.lm_head)       # fp32 logits from the 16-bit (or fp32) operands
        cap = self.cfg.logit_softcap
        return soft_cap(z, cap) if cap > 0 else z


class FoderaxState:
    """Caches and state of a Foderax model.  Paged through the engine's block manager: rotated keys
    and values of every parallel layer's attention half, the normed latent of every
    latent-attention layer (+ its per-block transpose where the matrix-core value product can use
    it), both maps' rotated keys and the values of every differential layer that projects its own
    (a borrowing layer reads the lender's).  Per state slot (+ one spare for graph padding rows):
    the fp32 recurrent state [slots + 1, width] of every parallel layer's recurrence."""

    def __init__(self, w: FoderaxWeights, slots: int, num_blocks: int, block_size: int, device):
        self.slots = slots
        self.spare = slots
        kw = dict(dtype=w.dtype, device=device)
        n = len(w.layers)
        self.k: List[Optional[torch.Tensor]] = [None] * n
        self.v: List[Optional[torch.Tensor]] = [None] * n
        self.lat: List[Optional[torch.Tensor]] = [None] * n
        self.latT: List[Optional[torch.Tensor]] = [None] * n
        self.S: List[Optional[torch.Tensor]] = [None] * n
        for i, L in enumerate(w.layers):
            m = L.m
            if L.kind == "parallel":
                a = m["left"]
                self.k[i] = torch.zeros(num_blocks, block_size, a["kv_heads"], a["dim"], **kw)
                self.v[i] = torch.zeros(num_blocks, block_size, a["kv_heads"], a["vdim"], **kw)
                self.S[i] = torch.zeros(slots + 1, m["right"]["width"], dtype=torch.float32,
                                        device=device)
            elif L.kind == "latent_attention":
                R = m["kv_rank"]
                self.lat[i] = torch.zeros(num_blocks, block_size, R, **kw)
                if transposed_values_ok(w.dtype, R, 0, block_size, device):
                    self.latT[i] = torch.zeros(num_blocks, R, block_size, **kw)
            elif L.kv_layer == i:
                self.k[i] = torch.zeros(num_blocks, block_size, 2 * m["kv_heads"], m["dim"], **kw)
                self.v[i] = torch.zeros(num_blocks, block_size, m["kv_heads"], m["vdim"], **kw)


def run_foderax_layers(w: FoderaxWeights, st: FoderaxState, tokens: torch.Tensor, seg: SegBatch,
                       observe=None) -> torch.Tensor:
    """The step function: token ids [T] + their segments -> the fp32 stream [T, W] the head
    reads; caches and recurrent state in ``st`` move on by the step's rows."""
    cfg = w.cfg
    dt = w.dtype
    eps = cfg.rms_norm_eps
    T = tokens.shape[0]
    dev = tokens.device
    n_layers = len(w.layers)
    hist = torch.empty(n_layers + 1, T, cfg.hidden_size, dtype=torch.float32, device=dev)
    x = embed_scaled(tokens, w.embed, cfg.embedding_scale, hist[0])
    h = group_rms_norm(x, w.layers[0].norm1, 1, eps, dt)
    for i, L in enumerate(w.layers):
        m = L.m
        if L.kind == "parallel":
            a = m["left"]
            H, G, D, Dv, Wd = a["heads"], a["kv_heads"], a["dim"], a["vdim"], m["right"]["width"]
            z = F.linear(h, L.w["in"])
            rotary_write(z, seg.positions, seg.cache_slots, st.k[i], st.v[i], H, G, D,
                         int(a["rot"]["dims"]), L.w["inv_freq"], True)
            o = torch.empty(T, H, Dv, dtype=dt, device=dev)
            row_attention(z[:, :H * D].view(T, H, D), None, st.k[i], st.v[i], Dv, o, seg, H, G,
                          float(a["scale"]), sigmoid_bias=L.w["pb"])
            c0 = (H + G) * D + G * Dv
            r = min_gru_scan(z[:, c0:c0 + 3 * Wd], L.w["b_z"], L.w["b_x"], st.S[i], seg, Wd,
                             w.shift)
            ys = [F.linear(o.view(T, H * Dv), L.w["o_l"]), F.linear(r, L.w["o_r"])]
        elif L.kind == "latent_attention":
            H, D, Dv, R, Q = m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            z = F.linear(h, L.w["in"])
            latent_write(z[:, Q:Q + R], L.w["dkv_norm"], None, seg.positions, seg.cache_slots,
                         st.lat[i], R, 0, eps, st.latT[i])
            q = F.linear(group_rms_norm(z[:, :Q], L.w["dq_norm"], 1, eps, dt), L.w["uq"])
            qa = torch.bmm(q.view(T, H, D).transpose(0, 1), L.w["uk"])          # [H, T, R]
            ol = torch.empty(H, T, R, dtype=dt, device=dev)
            row_attention(qa.transpose(0, 1), None, st.lat[i], st.lat[i], R, ol.transpose(0, 1),
                          seg, H, 1, float(m["scale"]), sink=L.w["sink"], vt=st.latT[i],
                          gate=z[:, Q + R:Q + R + H])
            o = torch.empty(T, H, Dv, dtype=dt, device=dev)
            torch.bmm(ol, L.w["uvT"], out=o.transpose(0, 1))
            ys = [F.linear(o.view(T, H * Dv), L.w["o"])]
        else:
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            own = L.kv_layer == i
            z = F.linear(h, L.w["in"], L.w["in_b"])
            rotary_write(z, seg.positions, seg.cache_slots, st.k[i], st.v[i], 2 * H,
                         2 * G if own else 0, D, int(m["rot"]["dims"]), L.w["inv_freq"], False)
            av = torch.empty(T, 2 * H, Dv, dtype=dt, device=dev)
            row_attention(z[:, :2 * H * D].view(T, 2 * H, D), None, st.k[L.kv_layer],
                          st.v[L.kv_layer], Dv, av, seg, 2 * H, 2 * G, float(m["scale"]), v_div=2)
            g0 = 2 * H * D + ((2 * G * D + G * Dv) if own else 0)
            o = diff_head_combine(av.view(T, 2 * H * Dv), L.c["lam"], 1.0 - float(m["diff"]), eps,
                                  z[:, g0:g0 + H * Dv], G, H // G, Dv)
            ys = [F.linear(o, L.w["o"])]
        scales = list(L.w["scales"])
        f = L.ff
        if f is not None:
            # the router in fp32, on the (possibly 16-bit rounded) normed row
            r = route_groups(router_logits(h, f["router"]), None, f["top"], f["groups"], f["keep"],
                             1.0, rank_top=1, score="softmax", normalize=False)
            ys.append(moe(h, r, f["up"], f["down"], f["E"], f["top"], f["ff"], 0, "relu2",
                          gated=False))
            scales.append(f["ls2"])
        nxt = w.layers[i + 1].norm1 if i + 1 < n_layers else None
        x, h = depth_mix_norm(hist, i + 1, x, ys, scales, L.w["dwa"], nxt, eps, dt)
        if observe is not None:
            observe(i, x)
    return x


WEIGHTS = {"gedatar": HybridWeights, "dalavik": DalavikWeights, "fanopel": FanopelWeights,
           "foderax": FoderaxWeights}


class HybridRunner(ModelRunner):
    """ModelRunner for hybrid stacks: the same step interface (execute / decode / sample, the
    hipGraph decode buckets), its own weights, caches and step function."""

    def __init__(self, weights: HybridWeights, num_blocks: int, block_size: int,
                 device: torch.device, max_model_len: int = 4096, state_slots: int = 256,
                 use_graphs: bool = True, max_graph_batch: int = 256):
        self.w = weights
        self.cfg = weights.cfg
        self.device = device
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.max_model_len = max_model_len
        self.tp_group, self.tp, self.car, self.lora = None, 1, None, None
        self.max_blocks = (max_model_len + block_size - 1) // block_size
        self.kv_dtype = weights.dtype
        self.state = weights.new_state(state_slots, num_blocks, block_size, device)
        self.use_graphs = use_graphs and device.type == "cuda"
        self.graph_buckets = [b for b in (1, 2, 4, 8, 16, 32, 64, 96, 128, 160, 192, 224, 256)
                              if b <= max(1, max_graph_batch)]
        self._graph_gathers = True
        self._graphs: Dict[int, tuple] = {}
        self._graph_pool = None
        self.observe = None   # callable(layer, x) after every layer (debugging / layer dumps)

    def _logits_rows(self, x: torch.Tensor, rows: Optional[torch.Tensor]) -> torch.Tensor:
        if rows is not None:
            if rows.numel() == 0:
                return torch.empty(0, self.cfg.vocab_size, device=x.device, dtype=self.w.dtype)
            x = x[rows]
        return self.w.head(x)

    @torch.no_grad()
    def execute(self, inp: StepInput) -> torch.Tensor:
        x = self.w.run_layers(self.state, inp.tokens, inp.seg, self.observe)
        if inp.extra_rows is not None and inp.extra_rows.numel():
            self.extra_logits = self._logits_rows(x, inp.extra_rows)
        return self._logits_rows(x, inp.sample_rows)

    prefill = execute

    # ---- decode: one row per sequence (graph hooks of ModelRunner.decode) --------------------
    def _decode_input(self, inp: StepInput) -> torch.Tensor:
        return self._logits_rows(self.w.run_layers(self.state, inp.tokens, inp.seg,
                                                   self.observe), None)

    def _static_inputs(self, bucket: int) -> dict:
        dev = self.device
        i32 = dict(dtype=torch.int32, device=dev)
        ar = torch.arange(bucket + 1, **i32)
        return {"tokens": torch.zeros(bucket, dtype=torch.long, device=dev),
                "seg": SegBatch(ar, torch.full((bucket,), self.state.spare, **i32),
                                torch.zeros(bucket, **i32), ar[:bucket].clone(),
                                torch.zeros(bucket, **i32),
                                torch.zeros(bucket, self.max_blocks, **i32),
                                torch.full((bucket,), -1, dtype=torch.long, device=dev))}

    def _fill_static(self, st: dict, inp: StepInput, N: int, bucket: int) -> None:
        sg, src = st["seg"], inp.seg
        st["tokens"][:N].copy_(inp.tokens)
        sg.slot[:N].copy_(src.slot)
        sg.start[:N].copy_(src.start)
        sg.positions[:N].copy_(src.positions)
        sg.tables[:N, :src.tables.shape[1]].copy_(src.tables)
        sg.cache_slots[:N].copy_(src.cache_slots)
        if N < bucket:  # padding rows: position 0 of the spare state slot, no key written
            sg.slot[N:].fill_(self.state.spare)
            sg.start[N:].zero_()
            sg.positions[N:].zero_()
            sg.cache_slots[N:].fill_(-1)

    def _decode_static(self, st: dict) -> torch.Tensor:
        return self._logits_rows(self.w.run_layers(self.state, st["tokens"], st["seg"]), None)


@torch.no_grad()
def forward_fresh(model, input_ids: torch.Tensor, block_size: int = 16) -> torch.Tensor:
    """Logits [B, S, V] of whole sequences on a private, fresh cache (the models' ``forward``)."""
    B, S = input_ids.shape
    dev = input_ids.device
    w = WEIGHTS[model.config.arch](model)
    nb = B * ((S + block_size - 1) // block_size)
    st = w.new_state(B, nb, block_size, dev)
    seg = whole_sequences([S] * B, dev, block_size=block_size)
    x = w.run_layers(st, input_ids.reshape(-1), seg)
    return w.head(x).view(B, S, -1)
