"""Prefill / decode throughput of a per-layer-mixer design (Gedatar, Dalavik, Fanopel, Foderax)
beside Llama at equal size.

``python bench.py --hybrid [--hybrid_family dalavik|fanopel|foderax]`` (one GPU).  Fanopel also
runs beside the closest design the framework already had: a Gedatar stack of attention layers
(keys as values) with routed experts of the same shapes; Foderax beside Dalavik (latent and
grouped-query attention through the same row kernels) and Fanopel (experts of the same shapes).
All models get random
weights of layer shapes that resemble real models (width 2048 / 4096, head size 128 / 64, FFN 2.75 x width, vocab 32000), the
same depth, and run the same forced-token workload through the serving engine
(``lumen.serve.trace.TraceReplay``: the engine's input builder, block manager, state slots,
runner, hipGraph decode):

* prefill: ``--hybrid_batch`` prompts of ``--hybrid_prompt`` tokens in ONE step (tokens / s);
* decode: one token for each of the sequences per step, ``--hybrid_decode_steps`` steps at that
  context (tokens / s; the steps replay a decode graph).

Prints one JSON line per (size, model) and a closing summary line.  Random weights, synthetic
tokens; dtype bf16.
"""
from __future__ import annotations

import json
import time

import torch


def gedatar_config(width: int, depth_groups: int = 1):
    from ..models.config import ModelConfig

    W = width
    ff = int(2.75 * W)
    att = lambda mlp: {"type": "attention", "mlp": mlp,  # noqa: E731
                       "mixer": {"heads": W // 128, "kv_heads": max(1, W // 512), "dim": 128,
                                 "vdim": 128, "scale": 0.09, "mask": {"size": 1024}}}
    dense = {"kind": "dense", "ff": ff}
    moe = {"kind": "moe", "router": {"experts": 8, "top": 2}, "expert": {"ff": ff // 4},
           "shared": {"ff": ff // 4}}
    layers = [att(dense), {"type": "wkv", "mixer": {"heads": W // 64, "dim": 64}, "mlp": moe},
              {"type": "general_delta", "mixer": {"heads": W // 128, "dim": 128}, "mlp": dense},
              att(moe)] * depth_groups
    return ModelConfig(arch="gedatar", vocab_size=32000, hidden_size=W,
                       num_hidden_layers=len(layers), rms_norm_eps=1e-6, canon_taps=4,
                       intermediate_size=0, num_attention_heads=0, num_key_value_heads=0,
                       max_position_embeddings=1 << 20, eos_token_id=-1,
                       name=f"gedatar-w{W}", layer_specs=layers)


def dalavik_config(width: int, depth_groups: int = 1):
    """Latent attention at the published shapes of compressed-KV models (heads of 128 + 64
    rotated, latent 512, query latent 3/4 of the width), one grouped-query layer with every score
    shaping on, one latent layer that borrows a cache; FFN 2.75 x width; token side input 128."""
    from ..models.config import ModelConfig

    W = width
    ff = {"kind": "dense", "ff": int(2.75 * W)}
    H = W // 128

    def lat(src=None):
        m = {"heads": H, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512,
             "q_rank": 3 * W // 4, "scale": 192 ** -0.5, "rot": {"base": 10000.0, "dims": 64}}
        if src is not None:
            m["kv_from"] = src
        return {"type": "latent_attention", "mixer": m, "mlp": ff}

    att = {"type": "attention", "mlp": ff,
           "mixer": {"heads": H, "kv_heads": max(1, W // 512), "dim": 128, "vdim": 128,
                     "scale": 128 ** -0.5, "softcap": 30.0, "q_temp": {"coef": 0.1, "every": 1024}}}
    layers = []
    for g in range(depth_groups):
        layers += [lat(), lat(), att, lat(4 * g + 1)]
    return ModelConfig(arch="dalavik", vocab_size=32000, hidden_size=W,
                       num_hidden_layers=len(layers), rms_norm_eps=1e-6, norm_groups=4,
                       token_side_dim=128, intermediate_size=0, num_attention_heads=0,
                       num_key_value_heads=0, max_position_embeddings=1 << 20, eos_token_id=-1,
                       tie_word_embeddings=True, name=f"dalavik-w{W}", layer_specs=layers)


def fanopel_config(width: int, depth: int = 4):
    """Gated window attention (heads of 128, one key head per four query heads, window 1024 + 4
    kept tokens, soft cap 30) and 16 routed experts of FFN width 2.75 / 4 x model width in 4 groups
    of which 2 are kept, top 4: the active FFN width equals the dense 2.75 x width."""
    from ..models.config import ModelConfig

    W = width
    layer = {"type": "attention",
             "mixer": {"heads": W // 128, "kv_heads": max(1, W // 512), "dim": 128, "vdim": 128,
                       "scale": 128 ** -0.5, "softcap": 30.0,
                       "mask": {"size": 1024, "keep_first": 4}},
             "mlp": {"kind": "moe", "expert": {"ff": int(2.75 * W) // 4},
                     "router": {"experts": 16, "top": 4, "scale": 2.0,
                                "groups": {"count": 4, "keep": 2}}}}
    return ModelConfig(arch="fanopel", vocab_size=32000, hidden_size=W, num_hidden_layers=depth,
                       rms_norm_eps=1e-6, residual_mult=0.5, intermediate_size=0,
                       num_attention_heads=0, num_key_value_heads=0, max_position_embeddings=4096,
                       eos_token_id=-1, name=f"fanopel-w{W}", layer_specs=[layer] * depth)


def foderax_config(width: int, depth_groups: int = 1):
    """One of each layer kind per group of four: a parallel layer (sigmoid-weight attention with
    heads of 128 beside a minGRU of the model's width), latent attention at Dalavik's shapes
    (latent 512, query latent 3/4 of the width), differential attention (two maps of 128 per head
    over values of 256) and a second one that borrows the first one's caches; 16 experts of FFN
    width 2.75 / 4 x model width in 4 groups of which 2 are kept, top 4 (Fanopel's shapes)."""
    from ..models.config import ModelConfig

    W = width
    H = W // 128
    mlp = {"kind": "moe", "expert": {"ff": int(2.75 * W) // 4},
           "router": {"experts": 16, "top": 4, "groups": {"count": 4, "keep": 2}}}
    layers = []
    for g in range(depth_groups):
        dif = {"heads": H // 2, "kv_heads": max(1, H // 8), "dim": 128, "vdim": 256,
               "scale": 128 ** -0.5, "diff": 0.25, "rot": {"base": 500000.0, "dims": 128}}
        layers += [
            {"type": "parallel", "mlp": mlp, "mixer": {
                "left": {"heads": H, "kv_heads": max(1, H // 4), "dim": 128, "vdim": 128,
                         "scale": 128 ** -0.5, "rot": {"base": 20000.0, "dims": 64}},
                "right": {"width": W}, "left_scale": 0.7, "right_scale": 0.4}},
            {"type": "latent_attention", "mlp": mlp,
             "mixer": {"heads": H, "dim": 128, "vdim": 128, "kv_rank": 512, "q_rank": 3 * W // 4,
                       "scale": 128 ** -0.5}},
            {"type": "attention", "mlp": mlp, "mixer": dict(dif)},
            {"type": "attention", "mlp": mlp, "mixer": dict(dif, kv_from=4 * g + 2)}]
    return ModelConfig(arch="foderax", vocab_size=32000, hidden_size=W,
                       num_hidden_layers=len(layers), rms_norm_eps=1e-6,
                       embedding_scale=float(W) ** 0.5, logit_softcap=30.0, intermediate_size=0,
                       num_attention_heads=0, num_key_value_heads=0,
                       max_position_embeddings=1 << 20, eos_token_id=-1, tie_word_embeddings=True,
                       name=f"foderax-w{W}", layer_specs=layers)


def gedatar_attention_moe_config(width: int, depth: int = 4):
    """The closest older design at Fanopel's shapes: Gedatar attention layers (keys as values,
    chunk mask of 1024) with 16 gated experts of the same FFN width, top 4, no shared expert."""
    from ..models.config import ModelConfig

    W = width
    layer = {"type": "attention",
             "mixer": {"heads": W // 128, "kv_heads": max(1, W // 512), "dim": 128, "vdim": 128,
                       "scale": 0.09, "mask": {"size": 1024}},
             "mlp": {"kind": "moe", "router": {"experts": 16, "top": 4},
                     "expert": {"ff": int(2.75 * W) // 4}}}
    return ModelConfig(arch="gedatar", vocab_size=32000, hidden_size=W, num_hidden_layers=depth,
                       rms_norm_eps=1e-6, canon_taps=4, intermediate_size=0,
                       num_attention_heads=0, num_key_value_heads=0,
                       max_position_embeddings=1 << 20, eos_token_id=-1,
                       name=f"gedatar-attnmoe-w{W}", layer_specs=[layer] * depth)


def llama_config(width: int, layers: int):
    from ..models.config import ModelConfig

    return ModelConfig(arch="llama", vocab_size=32000, hidden_size=width,
                       intermediate_size=int(2.75 * width), num_hidden_layers=layers,
                       num_attention_heads=width // 128, num_key_value_heads=max(1, width // 512),
                       max_position_embeddings=4096, name=f"llama-w{width}")


def _timed(fn, dev) -> float:
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    fn()
    torch.cuda.synchronize(dev)
    return time.perf_counter() - t0


def run_one(cfg, batch: int, prompt: int, decode_steps: int, warmup: int, dev) -> dict:
    from ..models import build_model
    from ..serve.engine import EngineConfig, LLMEngine
    from ..serve.trace import TraceReplay

    model = build_model(cfg, dtype=torch.bfloat16, device=dev, init="random", seed=0)
    bs = 16
    total = prompt + decode_steps + warmup + 2
    blocks = batch * ((total + bs - 1) // bs) + 8

    class _Tok:
        eos_token_id = None

    eng = LLMEngine(EngineConfig(model=cfg.name, dtype="bf16", max_model_len=total + bs,
                                 block_size=bs, num_blocks=blocks, max_num_seqs=batch,
                                 max_num_batched_tokens=batch * prompt, async_scheduling=False),
                    model=model, tokenizer=_Tok())
    rp = TraceReplay(eng)
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(3, cfg.vocab_size, (batch, total), generator=g).tolist()
    names = [f"s{i}" for i in range(batch)]

    def prefill(tag):
        return rp.step([{"id": tag + n, "tokens": ids[i][:prompt], "want": [prompt - 1]}
                        for i, n in enumerate(names)], [])

    # warm-up prefill on throw-away requests (GEMM heuristics, allocator), then the timed one
    prefill("w")
    for n in names:
        rp._retire("w" + n)
    t_pre = _timed(lambda: prefill(""), dev)

    def decode(j):
        return rp.step([{"id": n, "tokens": [ids[i][prompt + j]], "want": [0]}
                        for i, n in enumerate(names)], [])

    for j in range(warmup):
        decode(j)
    t_dec = _timed(lambda: [decode(warmup + j) for j in range(decode_steps)], dev)
    out = {"model": cfg.name, "params_m": round(cfg.num_params() / 1e6, 1), "batch": batch,
           "prompt": prompt, "prefill_tok_s": round(batch * prompt / t_pre, 1),
           "prefill_ms": round(t_pre * 1e3, 3), "decode_steps": decode_steps,
           "decode_tok_s": round(batch * decode_steps / t_dec, 1),
           "decode_ms_per_step": round(t_dec / decode_steps * 1e3, 3)}
    del rp, eng, model
    torch.cuda.empty_cache()
    return out


def run_hybrid_bench(args) -> list:
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    from ..ops._native import native, native_error

    assert native() is not None, native_error()
    rows = []
    family = getattr(args, "hybrid_family", "gedatar")
    make = {"gedatar": gedatar_config, "dalavik": dalavik_config, "fanopel": fanopel_config,
            "foderax": foderax_config}[family]
    for width in [int(w) for w in str(args.hybrid_widths).split(",")]:
        gcfg = make(width)
        beside = [llama_config(width, gcfg.num_hidden_layers)]
        if family == "fanopel":
            beside.insert(0, gedatar_attention_moe_config(width, gcfg.num_hidden_layers))
        if family == "foderax":
            beside = [dalavik_config(width), fanopel_config(width, gcfg.num_hidden_layers)] + beside
        if getattr(args, "hybrid_only", False):
            beside = []
        for cfg in [gcfg] + beside:
            for batch in [int(b) for b in str(args.hybrid_batch).split(",")]:
                r = run_one(cfg, batch, args.hybrid_prompt, args.hybrid_decode_steps, 3, dev)
                r["width"] = width
                rows.append(r)
                print(json.dumps(r), flush=True)
    by = {(r["width"], r["batch"], r["model"].split("-")[0]): r for r in rows}
    summ = []
    if getattr(args, "hybrid_only", False):
        return rows
    for (w, b, kind), r in list(by.items()):
        if kind != family:
            continue
        ll = by[(w, b, "llama")]
        row = {"width": w, "batch": b,
               "prefill_vs_llama": round(r["prefill_tok_s"] / ll["prefill_tok_s"], 3),
               "decode_vs_llama": round(r["decode_tok_s"] / ll["decode_tok_s"], 3)}
        if family == "fanopel":
            gd = by[(w, b, "gedatar")]
            row["prefill_vs_gedatar"] = round(r["prefill_tok_s"] / gd["prefill_tok_s"], 3)
            row["decode_vs_gedatar"] = round(r["decode_tok_s"] / gd["decode_tok_s"], 3)
        if family == "foderax":
            for other in ("dalavik", "fanopel"):
                o = by[(w, b, other)]
                row[f"prefill_vs_{other}"] = round(r["prefill_tok_s"] / o["prefill_tok_s"], 3)
                row[f"decode_vs_{other}"] = round(r["decode_tok_s"] / o["decode_tok_s"], 3)
        summ.append(row)
    metric = "hybrid" if family == "gedatar" else family
    print(json.dumps({"metric": f"{metric}_vs_llama_tokens_per_s", "dtype": "bf16",
                      "data": "synthetic", "rows": summ}), flush=True)
    return rows
