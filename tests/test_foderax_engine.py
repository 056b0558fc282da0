"""Foderax through the serving engine (model registry, loader, block manager, state slots,
scheduler, hybrid runner, trace replay) against the float64 whole-sequence oracle of
tests/_ref_foderax.py.

Every test runs on the CPU (the ops' torch path) and, marked ``gpu``, on the HIP kernels.  The
configurations are small and unlike each other: head sizes that are and are not multiples of the
vector and matrix-core widths, grouped, multi-query and full-head attention, rotary on a part of
the head and on all of it, latents that do and do not fit the matrix-core kernel, routers with one
group, with every group kept, with groups of one expert and with one expert in all, layers
without a feed-forward, borrowed key / value caches, scales of 1 and unlike 1, stacks that begin
with each kind of layer."""
import copy
import os

import pytest
import torch

import _ref_foderax as ref

from lumen.models import build_model
from lumen.models.config import ModelConfig, foderax_to_dict, get_config
from lumen.models.foderax import FoderaxForCausalLM
from lumen.serve.engine import EngineConfig, LLMEngine
from lumen.serve.sequence import SamplingParams
from lumen.serve.trace import TraceReplay

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def _cfg(name, vocab, width, emb, cap, eps, layers):
    return ModelConfig(arch="foderax", vocab_size=vocab, hidden_size=width,
                       num_hidden_layers=len(layers), rms_norm_eps=eps, embedding_scale=emb,
                       logit_softcap=cap, intermediate_size=0, num_attention_heads=0,
                       num_key_value_heads=0, max_position_embeddings=1 << 20, eos_token_id=-1,
                       tie_word_embeddings=True, name=name, layer_specs=layers)


def _par(H, G, D, Dv, rot, scale, width, ls, rs, mlp, base=20000.0):
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv, "scale": scale,
                               "rot": {"base": base, "dims": rot}},
                      "right": {"width": width}, "left_scale": ls, "right_scale": rs}}


def _lat(H, D, Dv, R, Q, scale, mlp):
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": H, "dim": D, "vdim": Dv, "kv_rank": R, "q_rank": Q, "scale": scale}}


def _dif(H, G, D, Dv, rot, scale, diff, mlp, kv_from=None, base=5000.0):
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv, "scale": scale, "diff": diff,
         "rot": {"base": base, "dims": rot}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mlp": mlp, "mixer": m}


def _moe(E, top, ff, n=1, keep=1):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": E, "top": top, "groups": {"count": n, "keep": keep}}}


CONFIGS = {
    "tiny": lambda: copy.deepcopy(get_config("tiny-foderax")),
    # nothing a multiple of 8: scalar key and value paths; full-head and multi-query attention;
    # rotary on a part of the head; groups of one expert each; every group kept; a latent the
    # matrix-core kernel has no shape for; two borrowers of one cache; a stack that starts with
    # latent attention
    "odd": lambda: _cfg("odd", 131, 60, 3.7, 9.0, 3e-6, [
        _lat(5, 6, 10, 20, 12, 0.3, _moe(6, 2, 28, 6, 3)),
        _dif(3, 1, 6, 10, 2, 0.4, 0.45, None),
        _par(3, 3, 10, 14, 6, 0.31, 30, 1.3, 0.2, _moe(9, 4, 15, 3, 3)),
        _dif(3, 1, 6, 10, 2, 0.25, 0.1, _moe(7, 7, 9), kv_from=1),
        _dif(3, 1, 6, 10, 2, 0.5, 0.15, None, kv_from=1)]),
    # one of everything: one head, one key head, one expert, scales of 1, rotary over the whole
    # head, equal key and value sizes, no soft cap, an embedding scale of 1
    "one": lambda: _cfg("one", 64, 48, 1.0, 0.0, 1e-4, [
        _par(1, 1, 16, 16, 16, 0.25, 48, 1.0, 1.0, _moe(1, 1, 40)),
        _dif(1, 1, 16, 16, 16, 0.25, 0.5, _moe(2, 1, 24, 2, 1)),
        _lat(1, 16, 16, 16, 16, 0.25, None)]),
    # head sizes 64 and 128 and a latent of 128 (the matrix-core kernels' shapes), 8 query heads
    # on 2 key heads, many experts in many groups, a recurrence wider than the stream
    "wide": lambda: _cfg("wide", 200, 128, 11.3, 30.0, 1e-5, [
        _par(4, 2, 128, 64, 64, 0.09, 320, 0.8, 0.35, _moe(32, 4, 16, 8, 3)),
        _lat(4, 32, 48, 128, 64, 0.17, None),
        _dif(8, 2, 64, 64, 32, 0.12, 0.4, _moe(16, 2, 48, 4, 1)),
        _dif(8, 2, 64, 64, 32, 0.12, 0.2, None, kv_from=2)]),
}


def make(name, device, dtype=torch.float32, seed=0):
    m = FoderaxForCausalLM(CONFIGS[name](), dtype=dtype, device=device)
    m.init_weights(seed=seed)
    return m


class Oracle:
    def __init__(self, model):
        self.cfg = foderax_to_dict(model.config)
        self.w = {n: model.tensor(n).detach().cpu() for n in model.tensor_names()}

    def forward(self, toks, cfg=None, w=None):
        return ref.forward(cfg or self.cfg, w or self.w, toks)


oracle = Oracle


class _NoTokenizer:
    eos_token_id = None


def engine(model, device, blocks=64, bs=16, seqs=4, budget=4096, graphs=True, **kw):
    return LLMEngine(EngineConfig(model=model.config.name, device=device, dtype="fp32" if
                                  model.dtype == torch.float32 else "bf16", num_blocks=blocks,
                                  block_size=bs, max_num_seqs=seqs, max_num_batched_tokens=budget,
                                  max_model_len=blocks * bs, use_graphs=graphs, **kw),
                     model=model, tokenizer=_NoTokenizer())


def tokens(model, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, model.config.vocab_size, (n,), generator=g).tolist()


def check(got, want, rtol=2e-4):
    got, want = got.to(ref.F64), want.to(ref.F64)
    scale = float(want.std())
    err = float((got - want).abs().max())
    assert err <= rtol * max(scale, 1.0), f"max error {err:.3e} at logit scale {scale:.3f}"


def check_rounding(got, want, typical=2e-2, stray=0.1):
    """16-bit activations: per position, the root mean square of the logits' error as a fraction
    of the logits' spread.  Rounding alone keeps it below ``typical``.  A router's choice between
    two experts with nearly equal scores may fall the other way in 16 bits; that moves the position
    (and those that attend to it) by far more, so up to ``stray`` of the positions may exceed
    ``typical`` -- a fault in a kernel moves them all."""
    got, want = got.to(ref.F64), want.to(ref.F64)
    scale = max(float(want.std()), 1.0)
    per = (got - want).pow(2).mean(-1).sqrt() / scale
    assert float(per.median()) <= typical / 2, f"median {float(per.median()):.3e}"
    over = int((per > typical).sum())
    assert over <= stray * per.numel(), f"{over} of {per.numel()} positions over {typical}"


def replay_alone(model, device, toks, pieces, **kw):
    """One request fed in ``pieces`` (cycled); logits of every position."""
    rp = TraceReplay(engine(model, device, **kw))
    out, at, k = [], 0, 0
    while at < len(toks):
        c = min(pieces[k % len(pieces)], len(toks) - at)
        k += 1
        out.append(rp.step([{"id": "a", "tokens": toks[at:at + c], "want": list(range(c))}],
                           ["a"] if at + c == len(toks) else []))
        at += c
    return torch.cat(out, 0)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_matches_oracle(device, name):
    m = make(name, device)
    toks = tokens(m, 150, 1)
    want = oracle(m).forward(toks)
    check(replay_alone(m, device, toks, [1000]), want)
    # the model's own forward (fresh caches, every row) is the same step function
    check(m(torch.tensor(toks, device=device))[0].cpu(), want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["tiny", "odd"])
def test_stream_after_every_layer(device, name):
    """The runner's per-layer hook against the oracle's stream (after the depth average): a fault
    shows at its layer."""
    m = make(name, device, seed=13)
    toks = tokens(m, 29, 14)
    layers = []
    o = oracle(m)
    ref.forward(o.cfg, o.w, toks, layers)
    eng = engine(m, device)
    seen = {}
    eng.runner.observe = lambda i, x: seen.__setitem__(i, x.detach().float().cpu().clone())
    TraceReplay(eng).step([{"id": "a", "tokens": toks, "want": []}], ["a"])
    assert sorted(seen) == list(range(len(layers)))
    for i, want in enumerate(layers):
        err = float((seen[i].to(ref.F64) - want).abs().max())
        assert err <= 1e-4 * max(1.0, float(want.abs().max())), f"layer {i}: {err:.3e}"


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_prefill_then_long_decode(device, name):
    """A short prompt, then token by token across block and tile borders: the recurrent state and
    every cache carried from step to step."""
    m = make(name, device, seed=1)
    toks = tokens(m, 210, 2)
    want = oracle(m).forward(toks)
    check(replay_alone(m, device, toks, [5] + [1] * 300), want)
    # from the very first token on, one at a time (the first token is a one-row prefill)
    check(replay_alone(m, device, toks[:40], [1]), want[:40])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("pieces", [[2], [3, 1, 2, 17, 2, 1, 1, 30], [16], [15, 1, 17], [64, 2, 63],
                                    [129, 2]])
def test_portions_of_several_sizes(device, pieces):
    m = make("tiny", device, seed=2)
    toks = tokens(m, 137, 3)
    check(replay_alone(m, device, toks, pieces, bs=8), oracle(m).forward(toks))


@pytest.mark.parametrize("device", DEVICES)
def test_long_portions_carry_the_recurrence(device):
    """Portions longer than the scan's chunks, cut off the chunk grid: the state a portion leaves
    is what the next one starts from."""
    m = make("odd", device, seed=12)
    toks = tokens(m, 420, 4)
    want = oracle(m).forward(toks)
    check(replay_alone(m, device, toks, [1000]), want)
    check(replay_alone(m, device, toks, [257, 1, 130, 2]), want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["tiny", "odd"])
def test_first_tokens(device, name):
    m = make(name, device, seed=3)
    orc = oracle(m)
    for n in (1, 2, 3, 6):
        toks = tokens(m, n, 10 + n)
        check(replay_alone(m, device, toks, [1000]), orc.forward(toks))
        check(replay_alone(m, device, toks, [1]), orc.forward(toks))


def _sharpen(m, factor=4.0):
    """Scale the query projections up: sharp scores, so that a few keys -- wherever they lie --
    carry a row's weight."""
    with torch.no_grad():
        for i, L in enumerate(m.config.layer_specs):
            for n in {"parallel": ["left.q"], "latent_attention": ["uq"],
                      "attention": ["q"]}[L["type"]]:
                m.tensor(f"l{i}.mix.{n}").mul_(factor)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["tiny", "wide"])
def test_every_constant_counts(device, name):
    """Sharp scores.  The oracle itself says that leaving out a sink, a score bias, the lambda
    offset, the map norm's constant, a mixer's scale, a layer scale, the depth weights, the
    embedding scale, the soft cap or the group limit would move the logits far beyond the
    tolerance -- and the engine matches the true model whole, in ragged portions and decoded token
    by token."""
    m = make(name, device, seed=21)
    _sharpen(m)
    toks = tokens(m, 200, 22)
    orc = oracle(m)
    want = orc.forward(toks)
    scale = max(float(want.std()), 1.0)
    kinds = [L["type"] for L in orc.cfg["layers"]]
    ip, il, ia = kinds.index("parallel"), kinds.index("latent_attention"), kinds.index("attention")
    ie = next(i for i, L in enumerate(orc.cfg["layers"])
              if L["mlp"] and L["mlp"]["router"]["groups"]["keep"] < L["mlp"]["router"]["groups"]["count"])

    def cfg_with(fn):
        c = copy.deepcopy(orc.cfg)
        fn(c)
        return c, None

    def w_with(name_, fn):
        w = dict(orc.w)
        w[name_] = fn(w[name_].float()).to(w[name_].dtype)
        return None, w

    def set_(d, k, v):
        d[k] = v

    changes = {
        "sink": w_with(f"l{il}.mix.sink", lambda t: t - 30.0),
        "score bias": w_with(f"l{ip}.mix.left.pb", lambda t: t * 0.0 + 1.0),
        "diff": cfg_with(lambda c: set_(c["layers"][ia]["mixer"], "diff",
                                        c["layers"][ia]["mixer"]["diff"] * 0.5)),
        "left scale": cfg_with(lambda c: set_(c["layers"][ip]["mixer"], "left_scale", 1.0)),
        "right scale": cfg_with(lambda c: set_(c["layers"][ip]["mixer"], "right_scale", 1.0)),
        "layer scale": w_with(f"l{ia}.ls1", lambda t: t * 0.0 + 1.0),
        "depth weights": w_with(f"l{il}.dwa", lambda t: torch.flip(t, [0])),
        "embedding scale": cfg_with(lambda c: set_(c["embedding"], "scale", 1.0)),
        "soft cap": cfg_with(lambda c: set_(c, "logit_softcap", 0.0)),
        "group limit": cfg_with(lambda c: set_(c["layers"][ie]["mlp"]["router"]["groups"], "keep",
                                               c["layers"][ie]["mlp"]["router"]["groups"]["count"])),
        "gate": w_with(f"l{il}.mix.g", lambda t: t * 0.0),
        "recurrence bias": w_with(f"l{ip}.mix.right.z.b", lambda t: t + 2.0),
    }
    for what, (c, w) in changes.items():
        moved = float((orc.forward(toks, c, w) - want).abs().max())
        assert moved > 20 * 5e-4 * scale, f"{what}: moves the logits by {moved:.2e} only"
    check(replay_alone(m, device, toks, [1000]), want, rtol=5e-4)
    check(replay_alone(m, device, toks, [37, 2, 50, 1, 64, 3], bs=8), want, rtol=5e-4)
    check(replay_alone(m, device, toks, [100] + [1] * 200), want, rtol=5e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_far_token_is_seen(device):
    """Changing the FIRST token of a long prompt changes the last logits (every mixer sees all of
    the past); the engine agrees with the oracle on both prompts, the far token's keys lying in
    the first cache block and many tiles away from the row that asks."""
    m = make("tiny", device, seed=23)
    _sharpen(m, 3.0)
    orc = oracle(m)
    a = tokens(m, 330, 24)
    b = list(a)
    b[0] = (a[0] + 1) % m.config.vocab_size
    wa, wb = orc.forward(a)[-1], orc.forward(b)[-1]
    assert float((wa - wb).abs().max()) > 1e-3
    for toks, want in ((a, wa), (b, wb)):
        check(replay_alone(m, device, toks, [300, 7, 1], bs=8)[-1:], want[None], rtol=5e-4)
        check(replay_alone(m, device, toks, [250] + [1] * 80, bs=8)[-1:], want[None], rtol=5e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["tiny", "odd"])
def test_mixed_batches_reuse_blocks_and_slots(device, name):
    """Seven unequal requests through three sequence slots and a pool of 20 blocks of 8: portions
    of some beside single tokens of others; finished requests hand their blocks and their state
    slot (with the recurrent state still in it) to new ones.  Every request must come out as if it
    had run alone."""
    m = make(name, device, seed=4)
    orc = oracle(m)
    lens = [41, 9, 66, 2, 30, 17, 50]
    reqs = {f"r{i}": tokens(m, n, 20 + i) for i, n in enumerate(lens)}
    eng = engine(m, device, blocks=20, bs=8, seqs=3)
    rp = TraceReplay(eng)
    g = torch.Generator().manual_seed(5)
    waiting = list(reqs)
    live, at, got = [], {}, {r: [] for r in reqs}
    sizes = [2, 1, 1, 13, 1, 5, 1, 1, 24, 3]
    k = 0
    seen_blocks, seen_slots = [], []
    while waiting or live:
        while waiting and len(live) < 3:
            need = sum((len(reqs[r]) + 7) // 8 for r in live + [waiting[0]])
            if need > 20:
                break
            r = waiting.pop(0)
            live.append(r)
            at[r] = 0
        entries, end = [], []
        for r in list(live):
            if len(live) > 1 and torch.rand((), generator=g) < 0.3:
                continue                                   # left out of this step
            c = min(sizes[k % len(sizes)], len(reqs[r]) - at[r])
            k += 1
            entries.append({"id": r, "tokens": reqs[r][at[r]:at[r] + c], "want": list(range(c))})
            at[r] += c
            if at[r] == len(reqs[r]):
                end.append(r)
                live.remove(r)
        if not entries:
            continue
        seen_slots += list(eng.states.owner.values())
        out = rp.step(entries, end)
        seen_blocks += [b for t in eng.blocks.tables.values() for b in t]
        o = 0
        for e in entries:
            got[e["id"]].append(out[o:o + len(e["tokens"])])
            o += len(e["tokens"])
    assert eng.blocks.num_free == 20 and len(set(seen_blocks)) <= 20
    assert eng.states.num_free == 3 and set(seen_slots) <= {0, 1, 2}
    for r, toks in reqs.items():
        check(torch.cat(got[r], 0), orc.forward(toks))


@pytest.mark.parametrize("device", DEVICES)
def test_blocks_and_slot_reused_after_finish(device):
    """The second request gets the first one's blocks and state slot (stale keys, values, latents
    and recurrent state)."""
    m = make("tiny", device, seed=6)
    orc = oracle(m)
    eng = engine(m, device, blocks=8, bs=16, seqs=1)
    rp = TraceReplay(eng)
    a, b = tokens(m, 100, 30), tokens(m, 60, 31)
    rp.step([{"id": "a", "tokens": a, "want": []}], ["a"])
    got = torch.cat([rp.step([{"id": "b", "tokens": b[:33], "want": list(range(33))}], []),
                     rp.step([{"id": "b", "tokens": b[33:], "want": list(range(27))}], ["b"])], 0)
    check(got, orc.forward(b))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["tiny", "one"])
def test_greedy_generation_through_scheduler(device, name):
    """LLMEngine.generate: chunked prefill under a small token budget, more prompts than
    sequence slots, async scheduling, greedy sampling -- every generated token is the oracle's
    arg-max (up to a tie within the tolerance) given the tokens before it."""
    m = make(name, device, seed=7)
    orc = oracle(m)
    eng = engine(m, device, blocks=48, bs=8, seqs=3, budget=24)
    prompts = [tokens(m, n, 40 + n) for n in (5, 37, 1, 20, 52)]
    seqs = eng.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True))
    assert eng.blocks.num_free == 48 and eng.states.num_free == 3
    for p, s in zip(prompts, seqs):
        assert len(s.output_ids) == 10
        want = orc.forward(p + s.output_ids[:-1])
        for j, tok in enumerate(s.output_ids):
            row = want[len(p) - 1 + j]
            assert float(row.max() - row[tok]) <= 1e-3 * max(float(row.std()), 1.0)


@pytest.mark.parametrize("device", DEVICES)
def test_preemption_recomputes_caches_and_state(device):
    """A pool too small for all running sequences: the scheduler preempts and later recomputes a
    sequence from its first token in whatever blocks and slot it then gets; outputs stay the
    oracle's."""
    m = make("odd", device, seed=8)
    orc = oracle(m)
    eng = engine(m, device, blocks=12, bs=4, seqs=3, budget=64, async_scheduling=False)
    prompts = [tokens(m, n, 60 + n) for n in (9, 11, 10)]
    seqs = eng.generate(prompts, SamplingParams(max_tokens=14, temperature=0.0, ignore_eos=True))
    assert eng.scheduler.num_preemptions > 0
    for p, s in zip(prompts, seqs):
        want = orc.forward(p + s.output_ids[:-1])
        for j, tok in enumerate(s.output_ids):
            row = want[len(p) - 1 + j]
            assert float(row.max() - row[tok]) <= 1e-3 * max(float(row.std()), 1.0)


def _random_config(seed):
    """A random stack: 2 - 6 layers in random order, sizes that are and are not multiples of the
    vector and matrix-core widths, borrowed caches where an earlier layer can lend."""
    import random

    rng = random.Random(seed)
    W = rng.choice([64, 96, 160, 192])
    layers = []
    lenders = {}
    for i in range(rng.randint(2, 6)):
        mlp = None
        if rng.random() < 0.8:
            n = rng.choice([1, 2, 3, 4])
            per = rng.choice([1, 2, 3, 5])
            keep = rng.randint(1, n)
            mlp = _moe(n * per, rng.randint(1, keep * per), rng.choice([8, 20, 48]), n, keep)
        H = rng.choice([1, 2, 3, 4, 6, 8, 12])
        G = rng.choice([g for g in (1, 2, 3, 4, H) if H % g == 0])
        D = rng.choice([8, 12, 16, 20, 32, 64])
        Dv = rng.choice([8, 12, 24, 32, 64, 72])
        rot = rng.choice([2, D // 2 // 2 * 2, D])
        kind = rng.choice(["parallel", "latent_attention", "attention", "attention"])
        if kind == "parallel":
            layers.append(_par(H, G, D, Dv, rot, rng.uniform(0.05, 0.3), rng.choice([8, 50, 64, 200]),
                               rng.uniform(0.3, 1.2), rng.uniform(0.3, 1.2), mlp))
        elif kind == "latent_attention":
            layers.append(_lat(H, D, Dv, rng.choice([16, 24, 64, 128]), rng.choice([8, 20, 64]),
                               rng.uniform(0.05, 0.3), mlp))
        elif lenders and rng.random() < 0.5:
            j = rng.choice(list(lenders))
            g, d, dv, r, b = lenders[j]
            h = g * rng.choice([1, 2, 3])
            layers.append(_dif(h, g, d, dv, r, rng.uniform(0.05, 0.3), rng.uniform(0.05, 0.6), mlp,
                               kv_from=j, base=b))
        else:
            base = rng.choice([100.0, 5000.0, 300000.0])
            lenders[i] = (G, D, Dv, rot, base)
            layers.append(_dif(H, G, D, Dv, rot, rng.uniform(0.05, 0.3), rng.uniform(0.05, 0.6), mlp,
                               base=base))
    return _cfg(f"random{seed}", rng.randint(50, 400), W, rng.choice([1.0, 4.0, 12.5]),
                rng.choice([0.0, 8.0, 30.0]), rng.choice([1e-6, 1e-5]), layers)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("seed", [0, 1, 2, 3, 4, 5, 6, 7])
def test_random_configurations(device, seed):
    """Whole, in ragged portions, and decoded across a 128-key border: the oracle's logits (fp32)
    and, on the GPU in 16 bits, the same logits however the prompt was cut."""
    cfg = _random_config(seed)
    m = FoderaxForCausalLM(cfg, dtype=torch.float32, device=device)
    m.init_weights(seed=seed)
    toks = tokens(m, 150, seed)
    want = oracle(m).forward(toks)
    for pieces in ([1000], [37, 2, 1, 50, 1, 1, 1, 3], [120] + [1] * 30):
        check(replay_alone(m, device, toks, pieces), want, rtol=5e-4)
    if device == "cuda":
        m16 = FoderaxForCausalLM(cfg, dtype=torch.bfloat16, device=device)
        m16.init_weights(seed=seed)
        whole = replay_alone(m16, device, toks, [1000])
        check_rounding(replay_alone(m16, device, toks, [37, 2, 1, 50, 1, 1, 1, 3]), whole)
        check_rounding(replay_alone(m16, device, toks, [120] + [1] * 30), whole)


def test_configuration_is_validated():
    bad = CONFIGS["odd"]()
    bad.layer_specs[2]["mixer"]["left"]["kv_heads"] = 2   # 3 heads on 2 key heads
    with pytest.raises(ValueError):
        FoderaxForCausalLM(bad, dtype=torch.float32, device="cpu")
    bad = CONFIGS["odd"]()
    bad.layer_specs[3]["mixer"]["kv_from"] = 2            # the lender is not an attention layer
    with pytest.raises(ValueError):
        FoderaxForCausalLM(bad, dtype=torch.float32, device="cpu")
    bad = CONFIGS["odd"]()
    bad.layer_specs[4]["mixer"]["kv_from"] = 3            # the lender borrows itself
    with pytest.raises(ValueError):
        FoderaxForCausalLM(bad, dtype=torch.float32, device="cpu")
    bad = CONFIGS["odd"]()
    bad.layer_specs[3]["mixer"]["dim"] = 8                # not the lender's head size
    with pytest.raises(ValueError):
        FoderaxForCausalLM(bad, dtype=torch.float32, device="cpu")
    bad = CONFIGS["tiny"]()
    bad.layer_specs[0]["mlp"]["router"]["top"] = 5        # only 2 groups of 2 experts are eligible
    with pytest.raises(ValueError):
        FoderaxForCausalLM(bad, dtype=torch.float32, device="cpu")
    bad = CONFIGS["tiny"]()
    bad.layer_specs[0]["mixer"]["rot"]["dims"] = 7
    with pytest.raises(ValueError):
        FoderaxForCausalLM(bad, dtype=torch.float32, device="cpu")
    bad = CONFIGS["tiny"]()
    bad.layer_specs[1]["type"] = "window"
    with pytest.raises(ValueError):
        FoderaxForCausalLM(bad, dtype=torch.float32, device="cpu")


def test_checkpoint_roundtrip(tmp_path):
    """save -> config.json + model.safetensors under the design's tensor names -> load by
    directory (the class is picked by config.json); a missing tensor or a wrong shape is an
    error."""
    from safetensors.torch import load_file, save_file

    from lumen.models.loading import save_hf_weights

    for name in ("tiny", "odd"):
        m = make(name, "cpu", dtype=torch.bfloat16)
        d = str(tmp_path / name)
        save_hf_weights(m, d)
        m2 = build_model(d, dtype=torch.bfloat16, device="cpu")
        assert m2.config.arch == "foderax" and type(m2) is FoderaxForCausalLM
        assert m2.config.embedding_scale == m.config.embedding_scale
        assert m2.config.logit_softcap == m.config.logit_softcap
        assert m2.config.layer_specs == m.config.layer_specs
        for n in m.tensor_names():
            assert torch.equal(m.tensor(n), m2.tensor(n)), n
    f = os.path.join(d, "model.safetensors")
    sd = load_file(f)
    assert "l3.mix.k" not in sd and "l1.mix.k" in sd       # a borrower has no key projection
    short = dict(sd)
    short.pop("l2.mix.left.pb")
    save_file(short, f)
    with pytest.raises(KeyError):
        build_model(d, dtype=torch.bfloat16, device="cpu")
    sd["l0.dwa"] = torch.zeros(3, dtype=torch.bfloat16)
    save_file(sd, f)
    with pytest.raises(ValueError):
        build_model(d, dtype=torch.bfloat16, device="cpu")


def test_trace_run_command_line(tmp_path):
    """bin/trace_run as a user runs it: a checkpoint directory, JSON steps on stdin, one logits
    file per step that wants any, `done <step>` after every step, exit code 0 at end of input."""
    import json
    import subprocess
    import sys

    import numpy as np

    from lumen.models.loading import save_hf_weights

    m = make("odd", "cpu", dtype=torch.bfloat16)
    d = str(tmp_path / "ckpt")
    out = str(tmp_path / "out")
    save_hf_weights(m, d)
    a, b = tokens(m, 21, 70), tokens(m, 12, 71)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:9], "want": [0, 8]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[9:10], "want": []},
                                     {"id": "b", "tokens": b[:11], "want": [10]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[11:], "want": [0]},
                                     {"id": "a", "tokens": a[10:], "want": [10]}],
              "end": ["a", "b"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d,
                        "--dtype", "float32", "--out", out, "--max-tokens", "128", "--device", "cpu"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True,
                       text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
    orc = oracle(m)
    ra, rb = orc.forward(a), orc.forward(b)
    V = m.config.vocab_size
    got = {i: torch.from_numpy(np.fromfile(os.path.join(out, f"{i}.f32"), dtype="<f4")).view(-1, V)
           for i in range(3)}
    check(got[0], ra[[0, 8]])
    check(got[1], rb[[10]])
    check(got[2], torch.stack([rb[11], ra[20]]))


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["tiny", "odd", "wide"])
def test_bf16_close_to_oracle_and_cut_invariant(name):
    """bf16 serving: within rounding of the float64 oracle, and the same logits (to rounding)
    however the prompt is cut and whether rows decode through the hipGraph path or eagerly."""
    m = make(name, "cuda", dtype=torch.bfloat16, seed=9)
    toks = tokens(m, 170, 50)
    want = oracle(m).forward(toks)
    whole = replay_alone(m, "cuda", toks, [1000])
    cut = replay_alone(m, "cuda", toks, [7, 1, 2, 1, 1, 16])
    eager = replay_alone(m, "cuda", toks, [30] + [1] * 150, graphs=False)
    for got in (whole, cut, eager):
        check_rounding(got, want)
    check_rounding(cut, whole)


@pytest.mark.gpu
def test_graph_replayed_decode_matches_eager():
    """Decode steps replay a captured hipGraph per batch bucket; several replays, with eager
    prefill steps of other requests between them, give what eager decoding gives."""
    m = make("tiny", "cuda", seed=10)
    a, b = tokens(m, 50, 51), tokens(m, 33, 52)
    wa, wb = oracle(m).forward(a), oracle(m).forward(b)
    rp = TraceReplay(engine(m, "cuda", graphs=True))
    got_a = [rp.step([{"id": "a", "tokens": a[:20], "want": list(range(20))}], [])]
    for i in range(20, 35):                                # graph bucket 1
        got_a.append(rp.step([{"id": "a", "tokens": a[i:i + 1], "want": [0]}], []))
    got_b = [rp.step([{"id": "b", "tokens": b[:10], "want": list(range(10))}], [])]
    for i in range(15):                                    # graph bucket 2, both decoding
        o = rp.step([{"id": "a", "tokens": a[35 + i:36 + i], "want": [0]},
                     {"id": "b", "tokens": b[10 + i:11 + i], "want": [0]}], [])
        got_a.append(o[0:1])
        got_b.append(o[1:2])
    check(torch.cat(got_a, 0), wa)
    check(torch.cat(got_b, 0), wb[:25])
