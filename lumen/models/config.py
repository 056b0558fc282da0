"""Model configurations.

The reference fine-tunes ``meta-llama/Llama-2-7b-hf`` loaded through HF transformers
(``training/train_baseline.py:122-126``) and the north-star adds Llama-2-70B and OPT-125m
(``/root/repo/BASELINE.json`` configs).  There is no network on the build or GPU boxes, so
every architecture is described here by its published hyper-parameters and instantiated with
random weights unless a local HF checkpoint directory (``config.json`` + ``*.safetensors``) is
given.
"""
from __future__ import annotations

import json
import os
from dataclasses import asdict, dataclass, field, fields
from typing import Optional


@dataclass
class ModelConfig:
    arch: str = "llama"  # "llama" | "opt" | "gedatar" | "dalavik" | "fanopel" | "foderax"
    vocab_size: int = 32000
    hidden_size: int = 4096
    intermediate_size: int = 11008
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    num_key_value_heads: int = 32
    max_position_embeddings: int = 4096
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = False
    # OPT specifics
    ffn_dim: int = 0
    word_embed_proj_dim: int = 0
    do_layer_norm_before: bool = True
    layer_norm_eps: float = 1e-5
    pad_token_id: int = 0
    bos_token_id: int = 1
    eos_token_id: int = 2
    name: str = "custom"
    # Gedatar (hybrid stack: every layer names its own mixer and feed-forward):
    # layer_specs[i] = {"type": "attention" | "wkv" | "general_delta", "mixer": {...},
    # "mlp": {...} | None}, exactly as the checkpoint's config.json lists them
    layer_specs: Optional[list] = None
    canon_taps: int = 0          # taps of the causal depthwise convolution on the mixer input
    # Dalavik (layer_specs with "latent_attention" | "attention" mixers): groups of the RMS norms
    # and the per-layer width of the second, per-token embedding (0: the design's side input is off)
    norm_groups: int = 1
    token_side_dim: int = 0
    # Fanopel (layer_specs of gated window attention + routed experts; learned positions, so
    # max_position_embeddings is the position table's row count): every sublayer's output is
    # multiplied by this before it joins the residual stream
    residual_mult: float = 1.0
    # Foderax (layer_specs of "parallel" | "latent_attention" | "attention" mixers + routed
    # experts, depth-weighted layer inputs): the embedding rows are multiplied by
    # ``embedding_scale``; logits pass through cap * tanh(. / cap) when ``logit_softcap`` > 0
    embedding_scale: float = 1.0
    logit_softcap: float = 0.0

    @property
    def is_hybrid(self) -> bool:
        """Every layer names its own mixer and keeps its own kind of cache or state; such a stack
        is served by ``serve.hybrid_runner`` on the step's row segments."""
        return self.arch in ("gedatar", "dalavik", "fanopel", "foderax")

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    def num_params(self) -> int:
        """Total parameter count (base model, no adapters)."""
        h, v, L = self.hidden_size, self.vocab_size, self.num_hidden_layers
        if self.is_hybrid:
            if self.arch == "gedatar":
                from .gedatar import tensor_shapes
            elif self.arch == "fanopel":
                from .fanopel import tensor_shapes
            elif self.arch == "foderax":
                from .foderax import tensor_shapes
            else:
                from .dalavik import tensor_shapes

            n = 0
            for shape in tensor_shapes(self).values():
                k = 1
                for d in shape:
                    k *= d
                n += k
            return n
        if self.arch == "llama":
            attn = h * (self.q_size + 2 * self.kv_size) + self.q_size * h
            mlp = 3 * h * self.intermediate_size
            norms = 2 * h
            emb = v * h * (1 if self.tie_word_embeddings else 2)
            return L * (attn + mlp + norms) + emb + h
        # OPT: biases + learned positions + layernorms
        f = self.ffn_dim
        attn = 4 * h * h + 4 * h
        mlp = 2 * h * f + f + h
        norms = 4 * h
        return L * (attn + mlp + norms) + v * h + (self.max_position_embeddings + 2) * h + 2 * h

    def to_dict(self):
        return asdict(self)

    def save(self, path: str):
        with open(path, "w") as f:
            json.dump(self.to_dict(), f, indent=2)

    @classmethod
    def from_dict(cls, d: dict) -> "ModelConfig":
        names = {f.name for f in fields(cls)}
        return cls(**{k: v for k, v in d.items() if k in names})


def _gedatar_to_config(d: dict) -> ModelConfig:
    """config.json of a Gedatar checkpoint: {"architecture": "Gedatar", "vocab", "width",
    "norm": {"eps"}, "canon": {"taps"}, "layers": [{"type", "mixer", "mlp"}, ...]}."""
    layers = d["layers"]
    if not layers:
        raise ValueError("a Gedatar config needs at least one layer")
    for i, L in enumerate(layers):
        if L.get("type") not in ("attention", "wkv", "general_delta"):
            raise ValueError(f"layer {i}: unknown mixer type {L.get('type')!r}")
        kind = (L.get("mlp") or {}).get("kind", None)
        if L.get("mlp") is not None and kind not in ("dense", "moe"):
            raise ValueError(f"layer {i}: unknown feed-forward kind {kind!r}")
    return ModelConfig(
        arch="gedatar", vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
        num_hidden_layers=len(layers), rms_norm_eps=float(d["norm"]["eps"]),
        canon_taps=int(d["canon"]["taps"]), layer_specs=layers, intermediate_size=0,
        num_attention_heads=0, num_key_value_heads=0, max_position_embeddings=1 << 20,
        bos_token_id=int(d.get("bos_token_id", 0)), eos_token_id=int(d.get("eos_token_id", -1)),
        pad_token_id=int(d.get("pad_token_id", 0)), name=d.get("_name_or_path", "gedatar"))


def gedatar_to_dict(cfg: ModelConfig) -> dict:
    """The checkpoint form of a Gedatar configuration (inverse of ``_gedatar_to_config``)."""
    return {"architecture": "Gedatar", "vocab": cfg.vocab_size, "width": cfg.hidden_size,
            "norm": {"eps": cfg.rms_norm_eps}, "canon": {"taps": cfg.canon_taps},
            "layers": cfg.layer_specs, "eos_token_id": cfg.eos_token_id}


def _dalavik_to_config(d: dict) -> ModelConfig:
    """config.json of a Dalavik checkpoint: {"architecture": "Dalavik", "vocab", "width",
    "norm": {"eps", "groups"}, "token_side": {"dim"}, "layers": [{"type", "mixer", "mlp"}, ...]}."""
    layers = d["layers"]
    if not layers:
        raise ValueError("a Dalavik config needs at least one layer")
    for i, L in enumerate(layers):
        if L.get("type") not in ("latent_attention", "attention"):
            raise ValueError(f"layer {i}: unknown mixer type {L.get('type')!r}")
    side = d.get("token_side") or {}
    return ModelConfig(
        arch="dalavik", vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
        num_hidden_layers=len(layers), rms_norm_eps=float(d["norm"]["eps"]),
        norm_groups=int(d["norm"].get("groups", 1)), token_side_dim=int(side.get("dim", 0)),
        layer_specs=layers, intermediate_size=0, num_attention_heads=0, num_key_value_heads=0,
        max_position_embeddings=1 << 20, tie_word_embeddings=True,
        bos_token_id=int(d.get("bos_token_id", 0)), eos_token_id=int(d.get("eos_token_id", -1)),
        pad_token_id=int(d.get("pad_token_id", 0)), name=d.get("_name_or_path", "dalavik"))


def dalavik_to_dict(cfg: ModelConfig) -> dict:
    """The checkpoint form of a Dalavik configuration (inverse of ``_dalavik_to_config``)."""
    d = {"architecture": "Dalavik", "vocab": cfg.vocab_size, "width": cfg.hidden_size,
         "norm": {"eps": cfg.rms_norm_eps, "groups": cfg.norm_groups},
         "layers": cfg.layer_specs, "eos_token_id": cfg.eos_token_id}
    if cfg.token_side_dim:
        d["token_side"] = {"dim": cfg.token_side_dim}
    return d


def _fanopel_to_config(d: dict) -> ModelConfig:
    """config.json of a Fanopel checkpoint: {"architecture": "Fanopel", "vocab", "width",
    "max_positions", "residual_mult", "norm": {"eps"}, "layers": [{"type", "mixer", "mlp"}, ...]}."""
    layers = d["layers"]
    if not layers:
        raise ValueError("a Fanopel config needs at least one layer")
    for i, L in enumerate(layers):
        if L.get("type") != "attention":
            raise ValueError(f"layer {i}: unknown mixer type {L.get('type')!r}")
        kind = (L.get("mlp") or {}).get("kind", None)
        if L.get("mlp") is not None and kind != "moe":
            raise ValueError(f"layer {i}: unknown feed-forward kind {kind!r}")
    return ModelConfig(
        arch="fanopel", vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
        num_hidden_layers=len(layers), rms_norm_eps=float(d["norm"]["eps"]),
        residual_mult=float(d.get("residual_mult", 1.0)), layer_specs=layers,
        intermediate_size=0, num_attention_heads=0, num_key_value_heads=0,
        max_position_embeddings=int(d["max_positions"]),
        bos_token_id=int(d.get("bos_token_id", 0)), eos_token_id=int(d.get("eos_token_id", -1)),
        pad_token_id=int(d.get("pad_token_id", 0)), name=d.get("_name_or_path", "fanopel"))


def fanopel_to_dict(cfg: ModelConfig) -> dict:
    """The checkpoint form of a Fanopel configuration (inverse of ``_fanopel_to_config``)."""
    return {"architecture": "Fanopel", "vocab": cfg.vocab_size, "width": cfg.hidden_size,
            "max_positions": cfg.max_position_embeddings, "residual_mult": cfg.residual_mult,
            "norm": {"eps": cfg.rms_norm_eps}, "layers": cfg.layer_specs,
            "eos_token_id": cfg.eos_token_id}


def _foderax_to_config(d: dict) -> ModelConfig:
    """config.json of a Foderax checkpoint: {"architecture": "Foderax", "vocab", "width",
    "embedding": {"scale"}, "logit_softcap", "norm": {"eps"}, "layers": [{"type", "mixer",
    "mlp"}, ...]}."""
    layers = d["layers"]
    if not layers:
        raise ValueError("a Foderax config needs at least one layer")
    for i, L in enumerate(layers):
        if L.get("type") not in ("parallel", "latent_attention", "attention"):
            raise ValueError(f"layer {i}: unknown mixer type {L.get('type')!r}")
        kind = (L.get("mlp") or {}).get("kind", None)
        if L.get("mlp") is not None and kind != "moe":
            raise ValueError(f"layer {i}: unknown feed-forward kind {kind!r}")
    return ModelConfig(
        arch="foderax", vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
        num_hidden_layers=len(layers), rms_norm_eps=float(d["norm"]["eps"]),
        embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
        logit_softcap=float(d.get("logit_softcap") or 0.0), layer_specs=layers,
        intermediate_size=0, num_attention_heads=0, num_key_value_heads=0,
        max_position_embeddings=1 << 20, tie_word_embeddings=True,
        bos_token_id=int(d.get("bos_token_id", 0)), eos_token_id=int(d.get("eos_token_id", -1)),
        pad_token_id=int(d.get("pad_token_id", 0)), name=d.get("_name_or_path", "foderax"))


def foderax_to_dict(cfg: ModelConfig) -> dict:
    """The checkpoint form of a Foderax configuration (inverse of ``_foderax_to_config``)."""
    return {"architecture": "Foderax", "vocab": cfg.vocab_size, "width": cfg.hidden_size,
            "embedding": {"scale": cfg.embedding_scale}, "logit_softcap": cfg.logit_softcap,
            "norm": {"eps": cfg.rms_norm_eps}, "layers": cfg.layer_specs,
            "eos_token_id": cfg.eos_token_id}


def _hf_to_config(d: dict) -> ModelConfig:
    if d.get("architecture") == "Foderax":
        return _foderax_to_config(d)
    if d.get("architecture") == "Fanopel":
        return _fanopel_to_config(d)
    if d.get("architecture") == "Gedatar":
        return _gedatar_to_config(d)
    if d.get("architecture") == "Dalavik":
        return _dalavik_to_config(d)
    mt = d.get("model_type", "llama")
    if mt == "opt":
        return ModelConfig(
            arch="opt", vocab_size=d["vocab_size"], hidden_size=d["hidden_size"],
            intermediate_size=d["ffn_dim"], ffn_dim=d["ffn_dim"],
            num_hidden_layers=d["num_hidden_layers"], num_attention_heads=d["num_attention_heads"],
            num_key_value_heads=d["num_attention_heads"],
            max_position_embeddings=d.get("max_position_embeddings", 2048),
            word_embed_proj_dim=d.get("word_embed_proj_dim", d["hidden_size"]),
            do_layer_norm_before=d.get("do_layer_norm_before", True),
            tie_word_embeddings=True, pad_token_id=d.get("pad_token_id", 1),
            bos_token_id=d.get("bos_token_id", 2), eos_token_id=d.get("eos_token_id", 2),
            name=d.get("_name_or_path", "opt"))
    return ModelConfig(
        arch="llama", vocab_size=d["vocab_size"], hidden_size=d["hidden_size"],
        intermediate_size=d["intermediate_size"], num_hidden_layers=d["num_hidden_layers"],
        num_attention_heads=d["num_attention_heads"],
        num_key_value_heads=d.get("num_key_value_heads", d["num_attention_heads"]),
        max_position_embeddings=d.get("max_position_embeddings", 4096),
        rms_norm_eps=d.get("rms_norm_eps", 1e-5), rope_theta=d.get("rope_theta", 10000.0),
        tie_word_embeddings=d.get("tie_word_embeddings", False),
        bos_token_id=d.get("bos_token_id", 1), eos_token_id=d.get("eos_token_id", 2),
        pad_token_id=d.get("pad_token_id", 0) or 0, name=d.get("_name_or_path", "llama"))


PRESETS = {
    # meta-llama/Llama-2-7b-hf: 6,738,415,616 params
    "llama2-7b": dict(arch="llama", vocab_size=32000, hidden_size=4096, intermediate_size=11008,
                      num_hidden_layers=32, num_attention_heads=32, num_key_value_heads=32,
                      max_position_embeddings=4096, name="meta-llama/Llama-2-7b-hf"),
    "llama2-13b": dict(arch="llama", vocab_size=32000, hidden_size=5120, intermediate_size=13824,
                       num_hidden_layers=40, num_attention_heads=40, num_key_value_heads=40,
                       max_position_embeddings=4096, name="meta-llama/Llama-2-13b-hf"),
    # meta-llama/Llama-2-70b-hf (GQA, 8 kv heads)
    "llama2-70b": dict(arch="llama", vocab_size=32000, hidden_size=8192, intermediate_size=28672,
                       num_hidden_layers=80, num_attention_heads=64, num_key_value_heads=8,
                       max_position_embeddings=4096, name="meta-llama/Llama-2-70b-hf"),
    # Llama-2-7B layer shapes (H, F, heads, vocab) at reduced depth: multi-rank rehearsals with
    # every rank on one shared GPU (8 full 7B ranks would not fit its HBM)
    "llama2-7b-2l": dict(arch="llama", vocab_size=32000, hidden_size=4096, intermediate_size=11008,
                         num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=32,
                         max_position_embeddings=4096, name="llama2-7b-2l"),
    # Llama-2-70B layer shapes (H 8192, GQA 64 / 8 heads, F 28672, vocab 32000) at depth 2:
    # world-8 rehearsals of BASELINE config 5's per-layer shapes on one shared GPU
    "llama2-70b-2l": dict(arch="llama", vocab_size=32000, hidden_size=8192,
                          intermediate_size=28672, num_hidden_layers=2, num_attention_heads=64,
                          num_key_value_heads=8, max_position_embeddings=4096,
                          name="llama2-70b-2l"),
    # facebook/opt-125m
    "opt-125m": dict(arch="opt", vocab_size=50272, hidden_size=768, intermediate_size=3072,
                     ffn_dim=3072, num_hidden_layers=12, num_attention_heads=12,
                     num_key_value_heads=12, max_position_embeddings=2048,
                     word_embed_proj_dim=768, tie_word_embeddings=True, pad_token_id=1,
                     bos_token_id=2, eos_token_id=2, name="facebook/opt-125m"),
    # small test models (CPU unit tests, smoke)
    "tiny-llama": dict(arch="llama", vocab_size=512, hidden_size=256, intermediate_size=688,
                       num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=4,
                       max_position_embeddings=512, name="tiny-llama"),
    # deeper toy model: 8 ZeRO-3 units, so the release ring / prefetch / turn-reuse logic has room
    "tiny-llama-deep": dict(arch="llama", vocab_size=512, hidden_size=128, intermediate_size=344,
                            num_hidden_layers=6, num_attention_heads=4, num_key_value_heads=2,
                            max_position_embeddings=512, name="tiny-llama-deep"),
    # head_dim 128 like Llama-2: exercises the HIP flash-attention / fused-RoPE path at toy size
    "small-llama": dict(arch="llama", vocab_size=1024, hidden_size=512, intermediate_size=1376,
                        num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
                        max_position_embeddings=1024, name="small-llama"),
    "tiny-llama-gqa": dict(arch="llama", vocab_size=512, hidden_size=256, intermediate_size=688,
                           num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
                           max_position_embeddings=512, name="tiny-llama-gqa"),
    # 8 heads / 8 kv heads / FFN and vocab divisible by 8 x 8: tensor parallelism up to 8
    "tiny-llama-tp8": dict(arch="llama", vocab_size=1024, hidden_size=512, intermediate_size=2048,
                           num_hidden_layers=2, num_attention_heads=8, num_key_value_heads=8,
                           max_position_embeddings=512, name="tiny-llama-tp8"),
    # hybrid stack at toy size: chunked sink attention (GQA), RWKV-style and generalized-delta
    # recurrences, dense and mixture-of-experts feed-forwards, one layer without a feed-forward
    "tiny-gedatar": dict(
        arch="gedatar", vocab_size=320, hidden_size=128, num_hidden_layers=4,
        rms_norm_eps=1e-5, canon_taps=4, intermediate_size=0, num_attention_heads=0,
        num_key_value_heads=0, max_position_embeddings=1 << 20, eos_token_id=-1,
        name="tiny-gedatar", layer_specs=[
            {"type": "wkv", "mixer": {"heads": 2, "dim": 32},
             "mlp": {"kind": "dense", "ff": 192}},
            {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 32,
                                            "scale": 0.2, "mask": {"size": 24}},
             "mlp": {"kind": "moe", "router": {"experts": 6, "top": 3}, "expert": {"ff": 64},
                     "shared": {"ff": 96}}},
            {"type": "general_delta", "mixer": {"heads": 2, "dim": 48}, "mlp": None},
            {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 64, "vdim": 64,
                                            "scale": 0.1, "mask": {"size": 40}},
             "mlp": {"kind": "dense", "ff": 160}}]),
    # latent attention (one layer borrowing another's cache) + grouped-query attention with
    # temperature, soft cap, distance bias, head mixing and sink; grouped norms; token side input
    "tiny-dalavik": dict(
        arch="dalavik", vocab_size=288, hidden_size=96, num_hidden_layers=4, rms_norm_eps=1e-5,
        norm_groups=3, token_side_dim=8, intermediate_size=0, num_attention_heads=0,
        num_key_value_heads=0, max_position_embeddings=1 << 20, eos_token_id=-1,
        tie_word_embeddings=True, name="tiny-dalavik", layer_specs=[
            {"type": "attention", "mixer": {"heads": 6, "kv_heads": 2, "dim": 24, "vdim": 16,
                                            "scale": 0.2, "softcap": 12.0,
                                            "q_temp": {"coef": 0.25, "every": 20}},
             "mlp": {"kind": "dense", "ff": 160}},
            {"type": "latent_attention", "mixer": {"heads": 3, "dim": 24, "rot_dim": 8,
                                                   "vdim": 40, "kv_rank": 32, "q_rank": 48,
                                                   "scale": 0.15,
                                                   "rot": {"base": 5000.0, "dims": 8}},
             "mlp": None},
            {"type": "latent_attention", "mixer": {"heads": 5, "dim": 16, "rot_dim": 8,
                                                   "vdim": 24, "kv_rank": 32, "q_rank": 40,
                                                   "scale": 0.2, "kv_from": 1,
                                                   "rot": {"base": 5000.0, "dims": 8}},
             "mlp": {"kind": "dense", "ff": 128}},
            {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 32, "vdim": 48,
                                            "scale": 0.18, "softcap": 30.0,
                                            "q_temp": {"coef": 0.1, "every": 7}},
             "mlp": {"kind": "dense", "ff": 96}}]),
    # gated window attention (whole-projection q / k norms, keys as values, soft cap, linear
    # distance bias, kept first tokens) + sigmoid-routed experts chosen within the best groups;
    # learned positions; one layer without a feed-forward
    "tiny-fanopel": dict(
        arch="fanopel", vocab_size=272, hidden_size=112, num_hidden_layers=3, rms_norm_eps=1e-5,
        residual_mult=0.7, intermediate_size=0, num_attention_heads=0, num_key_value_heads=0,
        max_position_embeddings=384, eos_token_id=-1, name="tiny-fanopel", layer_specs=[
            {"type": "attention", "mixer": {"heads": 6, "kv_heads": 3, "dim": 24, "vdim": 24,
                                            "scale": 0.2, "softcap": 20.0,
                                            "mask": {"size": 21, "keep_first": 3}},
             "mlp": {"kind": "moe", "expert": {"ff": 40},
                     "router": {"experts": 12, "top": 4, "scale": 1.5,
                                "groups": {"count": 4, "keep": 2}}}},
            {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 32, "vdim": 32,
                                            "scale": 0.18, "softcap": 8.0,
                                            "mask": {"size": 70, "keep_first": 1}},
             "mlp": None},
            {"type": "attention", "mixer": {"heads": 4, "kv_heads": 4, "dim": 16, "vdim": 16,
                                            "scale": 0.25, "softcap": 50.0,
                                            "mask": {"size": 9, "keep_first": 5}},
             "mlp": {"kind": "moe", "expert": {"ff": 56},
                     "router": {"experts": 5, "top": 2, "scale": 1.0,
                                "groups": {"count": 1, "keep": 1}}}}]),
    # parallel layer (sigmoid-weight attention beside a minGRU), latent attention with a sink and
    # a per-head gate, differential attention (one layer borrowing the other's caches), softmax
    # routed experts within the best groups, one layer without a feed-forward; depth-weighted
    # layer inputs, scaled embedding, soft-capped logits
    "tiny-foderax": dict(
        arch="foderax", vocab_size=304, hidden_size=80, num_hidden_layers=4, rms_norm_eps=1e-5,
        embedding_scale=8.0, logit_softcap=20.0, intermediate_size=0, num_attention_heads=0,
        num_key_value_heads=0, max_position_embeddings=1 << 20, eos_token_id=-1,
        tie_word_embeddings=True, name="tiny-foderax", layer_specs=[
            {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24,
                                            "scale": 0.25, "diff": 0.2,
                                            "rot": {"base": 5000.0, "dims": 8}},
             "mlp": {"kind": "moe", "expert": {"ff": 40},
                     "router": {"experts": 8, "top": 3, "groups": {"count": 4, "keep": 2}}}},
            {"type": "parallel", "mixer": {
                "left": {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 16, "scale": 0.2,
                         "rot": {"base": 20000.0, "dims": 16}},
                "right": {"width": 72}, "left_scale": 0.7, "right_scale": 0.4},
             "mlp": None},
            {"type": "latent_attention", "mixer": {"heads": 3, "dim": 24, "vdim": 32,
                                                   "kv_rank": 32, "q_rank": 40, "scale": 0.2},
             "mlp": {"kind": "moe", "expert": {"ff": 48},
                     "router": {"experts": 5, "top": 2, "groups": {"count": 1, "keep": 1}}}},
            {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24,
                                            "scale": 0.3, "diff": 0.35, "kv_from": 0,
                                            "rot": {"base": 5000.0, "dims": 8}},
             "mlp": {"kind": "moe", "expert": {"ff": 40},
                     "router": {"experts": 6, "top": 3, "groups": {"count": 3, "keep": 2}}}}]),
    "tiny-opt": dict(arch="opt", vocab_size=512, hidden_size=64, intermediate_size=256,
                     ffn_dim=256, num_hidden_layers=2, num_attention_heads=4,
                     num_key_value_heads=4, max_position_embeddings=256, word_embed_proj_dim=64,
                     tie_word_embeddings=True, pad_token_id=1, bos_token_id=2, eos_token_id=2,
                     name="tiny-opt"),
}

# HF hub ids accepted by --model_name, mapped to presets (offline: random init).
HUB_ALIASES = {
    "meta-llama/Llama-2-7b-hf": "llama2-7b",
    "meta-llama/Llama-2-7b-chat-hf": "llama2-7b",
    "meta-llama/Llama-2-13b-hf": "llama2-13b",
    "meta-llama/Llama-2-70b-hf": "llama2-70b",
    "facebook/opt-125m": "opt-125m",
}


def get_config(name_or_path: str) -> ModelConfig:
    """Resolve a preset name, an HF hub id (offline alias) or a local HF checkpoint dir."""
    if name_or_path in HUB_ALIASES:
        name_or_path = HUB_ALIASES[name_or_path]
    if name_or_path in PRESETS:
        import copy

        return ModelConfig(**copy.deepcopy(PRESETS[name_or_path]))   # layer lists are the caller's
    if os.path.isdir(name_or_path):
        cfg_path = os.path.join(name_or_path, "config.json")
        with open(cfg_path) as f:
            d = json.load(f)
        if "arch" in d and "model_type" not in d and "architecture" not in d:
            return ModelConfig.from_dict(d)
        return _hf_to_config(d)
    raise ValueError(f"unknown model '{name_or_path}' (presets: {sorted(PRESETS)})")


def checkpoint_dir(name_or_path: str) -> Optional[str]:
    """Local directory holding weights for this model, if any."""
    if os.path.isdir(name_or_path):
        return name_or_path
    return None
