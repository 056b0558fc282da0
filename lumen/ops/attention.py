"""Attention ops for training and serving.

* Training (head_dim 128): the HIP flash-attention kernels (``kernels/flash_attn.hip``) read q/k/v
  straight from the fused token-major QKV buffer (``flash_attention_qkv``); other head dims use
  torch SDPA over head-major q/k/v (``causal_attention``).
* Serving decode: the paged-KV HIP kernel (``kernels/paged_attention.hip``, ``paged_decode``).
* Serving prefill -- whole prompts, chunks of long prompts and the prefill part of mixed
  prefill+decode steps: ``flash_attention_paged``, the 32x32x16 flash forward reading keys /
  values from the paged cache through block tables, queries offset by the cached context.
"""
from __future__ import annotations

import math
import os
from typing import Optional

import torch
import torch.nn.functional as F

from ._native import native, use_native


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                     scale: Optional[float] = None) -> torch.Tensor:
    """q [B,nh,S,D], k/v [B,nkv,S,D] -> [B*S, nh*D] (token-major)."""
    B, nh, S, D = q.shape
    nkv = k.shape[1]
    if nkv != nh:
        if q.is_cuda:
            o = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=scale,
                                               enable_gqa=True)
        else:
            rep = nh // nkv
            o = F.scaled_dot_product_attention(q, k.repeat_interleave(rep, 1),
                                               v.repeat_interleave(rep, 1), is_causal=True,
                                               scale=scale)
    else:
        o = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=scale)
    return o.transpose(1, 2).reshape(B * S, nh * D)


_merge_counters: dict = {}
# Fused split-context merge (two-pass kernel only): measured neutral in decode steps (batch 1:
# 3.857 vs 3.865 ms ITL, profiles/r02_serve); callers may still ask for it (``fused_merge``).
# decode kernel: 0 = two-pass; 1 = single-pass (K and V streamed together, online softmax per
# row group); 2 = single-pass with workgroup-uniform block ids and non-temporal K / V loads
# (used where the block size equals the kernel's rows per step, else 1); 3 = 2 software-pipelined
# (two register sets, the next iteration's K / V loads in flight while one is consumed; default,
# profiles/r5_decode)
PA_ONE_PASS = int(os.environ.get("LUMEN_PA_1PASS", "3"))


def _pa_counters(device: torch.device, n: int) -> torch.Tensor:
    """Zeroed int32 arrival counters for the fused split-context merge.  The kernel leaves them
    zeroed, so one buffer per device serves every layer and step; it is allocated before any
    HIP-graph capture (the runner's eager warm-up steps reach here first) and only grows."""
    key = (device.type, device.index)
    c = _merge_counters.get(key)
    if c is None or c.numel() < n:
        c = torch.zeros(max(n, 1 << 16), device=device, dtype=torch.int32)
        _merge_counters[key] = c
    return c


def paged_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                 block_tables: torch.Tensor, context_lens: torch.Tensor, max_context: int,
                 scale: float, partition_size: int = 512,
                 fused_merge: Optional[bool] = None, one_pass: Optional[bool] = None) -> torch.Tensor:
    """Single-token attention over a paged KV cache.

    q [num_seqs, nh, D]; caches [num_blocks, nkv, block_size, D]; block_tables [num_seqs,
    max_blocks] int32; context_lens [num_seqs] int32 (number of cached tokens incl. current).
    Contexts longer than ``partition_size`` are split over workgroups; with ``fused_merge`` the
    last partition to finish merges the partials (one launch), else a second kernel does.
    """
    num_seqs, nh, D = q.shape
    nb, nkv, bs, _ = k_cache.shape
    if use_native(q):
        max_parts = max(1, math.ceil(max_context / partition_size))
        out = torch.empty(num_seqs, nh, D, device=q.device, dtype=q.dtype)
        if max_parts > 1:
            tm = torch.empty(num_seqs, nh, max_parts, device=q.device, dtype=torch.float32)
            tl = torch.empty_like(tm)
            to = torch.empty(num_seqs, nh, max_parts, D, device=q.device, dtype=torch.float32)
        else:
            tm = torch.empty(1, 1, 1, device=q.device, dtype=torch.float32)
            tl, to = tm, tm
        one = PA_ONE_PASS if one_pass is None else int(one_pass)
        fused = bool(fused_merge) and not one
        cnt = (_pa_counters(q.device, num_seqs * nkv) if fused and max_parts > 1
               else None)
        # q read in place when its heads are contiguous (a view into the fused qkv rows):
        # no per-layer copy of the decode rows' q
        qk = q if (q.stride(2) == 1 and q.stride(1) == D and q.stride(0) % D == 0
                   and q.data_ptr() % 16 == 0) else q.contiguous()
        native().paged_attention_decode(out, qk, k_cache, v_cache, block_tables,
                                        context_lens, nkv, bs, block_tables.shape[1], scale, tm,
                                        tl, to, partition_size, cnt, one)
        return out
    return paged_decode_ref(q, k_cache, v_cache, block_tables, context_lens, scale)


def paged_decode_ref(q, k_cache, v_cache, block_tables, context_lens, scale):
    num_seqs, nh, D = q.shape
    nkv, bs = k_cache.shape[1], k_cache.shape[2]
    g = nh // nkv
    out = torch.empty_like(q)
    for i in range(num_seqs):
        L = int(context_lens[i])
        nblk = (L + bs - 1) // bs
        blks = block_tables[i, :nblk].long()
        kk = k_cache[blks].permute(1, 0, 2, 3).reshape(nkv, nblk * bs, D)[:, :L].float()
        vv = v_cache[blks].permute(1, 0, 2, 3).reshape(nkv, nblk * bs, D)[:, :L].float()
        qq = q[i].float().view(nkv, g, D)
        s = torch.einsum("hgd,hld->hgl", qq, kk) * scale
        p = torch.softmax(s, -1)
        out[i] = torch.einsum("hgl,hld->hgd", p, vv).reshape(nh, D).to(q.dtype)
    return out


def flash_attention_paged(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                          cu_q, kv_lens, block_tables: torch.Tensor, nh: int, nkv: int,
                          D: int, scale: Optional[float] = None,
                          out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of prefill chunks over the paged KV cache.

    q: token-major rows [T, >= nh*D] (e.g. the q part of the fused qkv buffer, already rotated);
    sequence s owns rows cu_q[s]..cu_q[s+1] and sees kv_lens[s] keys (its cached context plus
    this chunk, whose K/V are already in the cache); query row j of s sits at key position
    kv_lens[s] - (cu_q[s+1]-cu_q[s]) + j.  cu_q / kv_lens: int sequences (host) or int32 device
    tensors; block_tables [nseq, max_blocks] int32.  Returns / fills out [T, nh*D]."""
    T = q.shape[0]
    scale = scale if scale is not None else 1.0 / math.sqrt(D)
    if out is None:
        out = torch.empty(T, nh * D, device=q.device, dtype=q.dtype)
    if use_native(q) and D == 128 and k_cache.shape[-1] == 128:
        cu = tuple(int(c) for c in cu_q)
        dev = q.device
        cut = _cu_tensor(cu, dev)
        kl = (kv_lens if isinstance(kv_lens, torch.Tensor)
              else torch.tensor(list(kv_lens), dtype=torch.int32, device=dev))
        kl = kl.to(torch.int32)
        bt = block_tables.to(torch.int32)
        if k_cache.dtype == FP8_KV:
            k_cache, v_cache, bt = _dequant_blocks(k_cache, v_cache, bt, kl, q.dtype)
        native().flash_attn_paged(True, q, k_cache, v_cache, out, cut, kl,
                                  _tiles(cu, 128, dev), bt, nh, nkv, scale)
        return out
    out.copy_(flash_attention_paged_ref(q, k_cache, v_cache, cu_q, kv_lens, block_tables, nh,
                                        nkv, D, scale))
    return out


FP8_KV = torch.float8_e4m3fn  # fp8 KV-cache element type (OCP e4m3fn: gfx950's fp8 converts)
_SCRATCH: dict = {}


def _dequant_blocks(k_cache, v_cache, bt, kv_lens, dtype):
    """fp8 cache -> 16-bit scratch holding only the prefill sequences' blocks (block b of
    sequence s at s * maxb + b), plus the identity block table into it: the prefill kernel's
    LDS-DMA staging moves raw 16-bit rows.  The scratch is reused by every layer and grows."""
    P, maxb = bt.shape
    nb, nkv, bs, D = k_cache.shape
    need = P * maxb
    key = (k_cache.device, dtype, nkv, bs, D)
    scr = _SCRATCH.get(key)
    if scr is None or scr[0].shape[0] < need:
        n = max(need, 256)
        scr = (torch.empty(n, nkv, bs, D, device=k_cache.device, dtype=dtype),
               torch.empty(n, nkv, bs, D, device=k_cache.device, dtype=dtype),
               torch.arange(n, device=k_cache.device, dtype=torch.int32))
        _SCRATCH[key] = scr
    ks, vs, ident = scr
    native().kv_dequant(k_cache, v_cache, ks, vs, bt, kv_lens, maxb)
    return ks, vs, ident[:need].view(P, maxb)


def flash_attention_paged_ref(q, k_cache, v_cache, cu_q, kv_lens, block_tables, nh, nkv, D,
                              scale=None):
    scale = scale if scale is not None else 1.0 / math.sqrt(D)
    cu = [int(c) for c in cu_q]
    kl = [int(x) for x in kv_lens]
    bs = k_cache.shape[2]
    g = nh // nkv
    outs = []
    for s in range(len(kl)):
        a, b = cu[s], cu[s + 1]
        n, L = b - a, kl[s]
        nblk = (L + bs - 1) // bs
        blks = block_tables[s, :nblk].long()
        kk = k_cache[blks].permute(1, 0, 2, 3).reshape(nkv, nblk * bs, D)[:, :L].float()
        vv = v_cache[blks].permute(1, 0, 2, 3).reshape(nkv, nblk * bs, D)[:, :L].float()
        qq = q[a:b, :nh * D].float().view(n, nkv, g, D)
        sc = torch.einsum("nhgd,hld->hgnl", qq, kk) * scale
        qpos = torch.arange(L - n, L, device=q.device)[:, None]
        kpos = torch.arange(L, device=q.device)[None, :]
        sc = sc.masked_fill(kpos > qpos, float("-inf"))
        p = torch.softmax(sc, -1)
        o = torch.einsum("hgnl,hld->nhgd", p, vv).reshape(n, nh * D)
        outs.append(o.to(q.dtype))
    return torch.cat(outs, 0) if outs else q.new_zeros(0, nh * D)


def write_kv_cache(k: torch.Tensor, v: torch.Tensor, k_cache: torch.Tensor,
                   v_cache: torch.Tensor, slot_mapping: torch.Tensor) -> None:
    """k, v: [T, nkv, D] views (row stride may exceed nkv*D); slot_mapping [T] int64."""
    T = slot_mapping.numel()
    if T == 0:
        return
    nb, nkv, bs, D = k_cache.shape
    if use_native(k_cache):
        native().reshape_and_cache(k, v, k_cache, v_cache, slot_mapping, nkv, D, bs,
                                   k.stride(0), v.stride(0))
        return
    sm = slot_mapping.long()
    valid = sm >= 0
    sm = sm[valid]
    blk, off = sm // bs, sm % bs
    k_cache[blk, :, off] = k[valid].to(k_cache.dtype)
    v_cache[blk, :, off] = v[valid].to(v_cache.dtype)


def rope_write_kv(qkv: torch.Tensor, positions: torch.Tensor, nh: int, nkv: int, D: int,
                  cos_t: torch.Tensor, sin_t: torch.Tensor, k_cache: torch.Tensor,
                  v_cache: torch.Tensor, slot_mapping: torch.Tensor) -> None:
    """RoPE on the q and k heads of the fused token-major qkv [T, (nh + 2 nkv) D] in place, then
    the rotated k and v into the paged cache at ``slot_mapping`` (-1 = skip): one HIP kernel
    (``rope_cache_kernel``) on GPU, rope_inplace + write_kv_cache elsewhere."""
    T = qkv.shape[0]
    if T == 0:
        return
    nb, nkv_c, bs, Dc = k_cache.shape
    if use_native(qkv) and D % 16 == 0 and nkv_c == nkv and Dc == D:
        native().rope_cache_write(qkv, positions.to(torch.int32), cos_t, sin_t, k_cache, v_cache,
                                  slot_mapping.to(torch.int64), nh, nkv, D, bs)
        return
    from .rope import rope_inplace

    rope_inplace(qkv, positions, nh + nkv, D, cos_t, sin_t)
    qs, ks = nh * D, nkv * D
    write_kv_cache(qkv[:, qs:qs + ks].view(T, nkv, D), qkv[:, qs + ks:qs + 2 * ks].view(T, nkv, D),
                   k_cache, v_cache, slot_mapping)


# ------------------------------------------------------------------------------------------------
# HIP flash attention over the fused token-major QKV buffer (kernels/flash_attn.hip)
# ------------------------------------------------------------------------------------------------

_TILE_CACHE = {}


def _upload_i32(vals, device) -> torch.Tensor:
    """Small int32 host list -> device without a stream synchronise: a blocking
    ``torch.tensor(..., device=gpu)`` copy waits for every kernel queued before it, which would
    serialise the serving engine's host work (a new chunk layout every step) with the GPU.  The
    pinned staging block is recycled by torch's caching host allocator once the copy is done."""
    h = torch.tensor(vals, dtype=torch.int32)
    if torch.device(device).type != "cuda":
        return h
    return h.pin_memory().to(device, non_blocking=True)


def _tiles(cu: tuple, rows: int, device, heavy_first: bool = True,
           heavy_low: bool = False) -> torch.Tensor:
    """(seq, row start) pairs; heavy_first: causal query tiles (last rows = most keys) first;
    heavy_low: key tiles of the dK/dV kernels (first rows = most queries) first."""
    key = (cu, rows, str(device), heavy_first, heavy_low)
    t = _TILE_CACHE.get(key)
    if t is None:
        lst = []
        for s in range(len(cu) - 1):
            L = cu[s + 1] - cu[s]
            lst += [(s, r) for r in range(0, L, rows)]
        if heavy_low:
            lst.sort(key=lambda x: (x[1], -(cu[x[0] + 1] - cu[x[0]])))
        elif heavy_first:  # causal: the last tiles of a sequence carry the most keys
            lst.sort(key=lambda x: -x[1])
        t = _upload_i32(lst if lst else [(0, 0)], device).reshape(-1)
        if not lst:
            t = t[:0]
        if len(_TILE_CACHE) > 256:
            _TILE_CACHE.clear()
        _TILE_CACHE[key] = t
    return t


def _cu_tensor(cu: tuple, device) -> torch.Tensor:
    key = ("cu", cu, str(device))
    t = _TILE_CACHE.get(key)
    if t is None:
        t = _upload_i32(list(cu), device)
        _TILE_CACHE[key] = t
    return t


def prepare_varlen(cu: tuple, device) -> None:
    """Seed the tile / offset caches for a packed batch's ``cu`` with ONE pinned, non-blocking
    host-to-device copy, before the layer loop: every layer's forward and backward then hits
    the cache instead of building (and synchronously uploading) its tile lists."""
    rows_set = (FA_FWD_ROWS, 64, 128)
    keys = ([("cu", cu, str(device))] + [(cu, r, str(device), True, False) for r in rows_set]
            + [(cu, 64, str(device), True, True)])
    if all(k in _TILE_CACHE for k in keys):
        return
    parts = [list(cu)]
    for rows, low in [(r, False) for r in rows_set] + [(64, True)]:
        lst = []
        for s in range(len(cu) - 1):
            lst += [(s, r) for r in range(0, cu[s + 1] - cu[s], rows)]
        if low:  # dK/dV key tiles, heaviest (lowest) first
            lst.sort(key=lambda x: (x[1], -(cu[x[0] + 1] - cu[x[0]])))
        else:
            lst.sort(key=lambda x: -x[1])
        parts.append([v for t in lst for v in t])
    flat = torch.tensor([v for p in parts for v in p], dtype=torch.int32)
    if torch.cuda.is_available():
        flat = flat.pin_memory()
    dev = flat.to(device, non_blocking=True)
    if len(_TILE_CACHE) > 256:
        _TILE_CACHE.clear()
    o = 0
    for k, p in zip(keys, parts):
        _TILE_CACHE[k] = dev[o:o + len(p)]
        o += len(p)
    _TILE_CACHE[("pin", cu, str(device))] = flat  # host buffer outlives the async copy


import os as _os
# forward: the 32x32x16 MFMA kernel, 32 queries per wave, 128-row tiles (56 vs 71 us for the
# 16x16x32 forms at B8 S512, profiles/r02_fa; those variants were removed)
FA_FWD_MT, FA_FWD_ROWS = 20, 128
# (a 256-query-tile forward, mt 21, measured slower and was removed: profiles/r5_fa)
# backward: 16x16x32 dK/dV (64-key tiles) + 32x32x16 dQ (128-query tiles), or -- while the buffer
# fits -- the dS hand-off pair below
# dS hand-off: the dK/dV kernel stores dS per 64x64 tile and the dQ kernel forms
# dQ = dS K from it, instead of recomputing S = Q K^T and dP = dO V^T (2 of its 3 products).
# Used while the [nh, tiles, 64, 64] 16-bit buffer stays under LUMEN_FA_DS_MB (0 = off).
FA_DS_MB = float(_os.environ.get("LUMEN_FA_DS_MB", "2048"))
# (Measured and removed: an 8-wave 128-key dK/dV kernel, 117.6 vs 108.0 us at B=8 S=512; XCD-
# grouped 1-D tile orders, neutral; the 32x32 dQ kernel forming delta itself, neutral.)


def _ds_offsets(cu: tuple, causal: bool, device):
    """Per-sequence first tile of the dS hand-off buffer and the total tile count."""
    key = ("ds", cu, causal, str(device))
    hit = _TILE_CACHE.get(key)
    if hit is None:
        offs, tot = [], 0
        for s in range(len(cu) - 1):
            n = (cu[s + 1] - cu[s] + 63) // 64
            offs.append(tot)
            tot += n * (n + 1) // 2 if causal else n * n
        hit = (torch.tensor(offs if offs else [0], dtype=torch.int32, device=device), tot)
        _TILE_CACHE[key] = hit
    return hit


DELTA_HANDOFFS = [0]  # backward calls that used a delta handed over by the o_proj backward


class _FlashAttn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, qkv, cu, nh, nkv, D, causal, rope=None, scale=None, out_ext=0):
        C = native()
        T = qkv.shape[0]
        q = qkv[:, :nh * D]
        k = qkv[:, nh * D:(nh + nkv) * D]
        v = qkv[:, (nh + nkv) * D:]
        # out_ext > 0: O is the first nh*D columns of a [T, nh*D + out_ext] buffer (the operand
        # of the o_proj's K-extended LoRA GEMM); the kernels take the row stride
        o = torch.empty(T, nh * D + out_ext, device=qkv.device, dtype=qkv.dtype)[:, :nh * D]
        lse = torch.empty(nh, T, device=qkv.device, dtype=torch.float32)
        cut = _cu_tensor(cu, qkv.device)
        scale = 1.0 / math.sqrt(D) if scale is None else scale
        tl = _tiles(cu, FA_FWD_ROWS, qkv.device)
        C.flash_attn(0, causal, FA_FWD_MT, q, k, v, o, lse, cut, tl, nh, nkv, scale, None, None,
                     None, None, None, None, None, None)
        ctx.save_for_backward(qkv, o, lse)
        ctx.meta = (cu, nh, nkv, D, causal, scale)
        ctx.rope = rope
        # delta hand-off: the o_proj backward (lumen.ops.lora, fused dA + dx kernel) may leave
        # delta = rowsum(dO * O) here for exactly the dO this backward receives
        ctx.delta_slot = {}
        o._lumen_delta_slot = ctx.delta_slot
        return o

    @staticmethod
    def backward(ctx, do):
        C = native()
        qkv, o, lse = ctx.saved_tensors
        cu, nh, nkv, D, causal, scale = ctx.meta
        do = do.contiguous()
        T = qkv.shape[0]
        q = qkv[:, :nh * D]
        k = qkv[:, nh * D:(nh + nkv) * D]
        v = qkv[:, (nh + nkv) * D:]
        dqkv = torch.empty_like(qkv)
        dqkv._lumen_scratch = True  # fresh buffer: consumers may transform it in place
        dq = dqkv[:, :nh * D]
        dk = dqkv[:, nh * D:(nh + nkv) * D]
        dv = dqkv[:, (nh + nkv) * D:]
        slot = ctx.delta_slot
        handed = (slot.get("key") == (do.data_ptr(), do._version)
                  and tuple(slot["delta"].shape) == (nh, T))
        delta = (slot.pop("delta") if handed
                 else torch.empty(nh, T, device=qkv.device, dtype=torch.float32))
        DELTA_HANDOFFS[0] += int(handed)
        slot.clear()
        cut = _cu_tensor(cu, qkv.device)
        # dK/dV (which 2, 64-key tiles) and dQ (which 5, 128-query tiles); both undo the
        # forward's RoPE in their dQ / dK epilogues (d(pre-rotation) written directly): the
        # producer of q|k then skips its own inverse-rotation pass
        wkv, rkv, wq, rq = 2, 64, 5, 128
        rp = ctx.rope
        pos, cos, sin = rp if rp is not None else (None, None, None)
        qtiles = _tiles(cu, rq, qkv.device)
        ds_off, ds_total = (_ds_offsets(cu, causal, qkv.device) if FA_DS_MB > 0
                            else (None, 0))
        if ds_off is not None and nh * ds_total * 8192 <= FA_DS_MB * 2 ** 20:
            ds = torch.empty(nh, ds_total, 4096, device=qkv.device, dtype=qkv.dtype)
            if not handed:
                C.flash_attn(1, causal, 1, q, k, v, o, lse, cut, _tiles(cu, 64, qkv.device), nh,
                             nkv, scale, do, None, None, None, delta, None, None, None)
            # dK/dV: low key tiles carry the most (causal) query steps -> launched first
            t7 = _tiles(cu, 64, qkv.device, heavy_low=causal)
            t8 = _tiles(cu, 64, qkv.device)
            C.flash_attn_ds(7, causal, q, k, v, lse, cut, t7, nh, nkv,
                            scale, do, dq, dk, dv, delta, ds, ds_off, ds_total, pos, cos, sin)
            C.flash_attn_ds(8, causal, q, k, v, lse, cut, t8, nh, nkv,
                            scale, do, dq, dk, dv, delta, ds, ds_off, ds_total, pos, cos, sin)
        else:
            if not handed:
                C.flash_attn(1, causal, 1, q, k, v, o, lse, cut, _tiles(cu, 64, qkv.device), nh,
                             nkv, scale, do, None, None, None, delta, None, None, None)
            C.flash_attn(wkv, causal, 1, q, k, v, o, lse, cut, _tiles(cu, rkv, qkv.device), nh,
                         nkv, scale, do, dq, dk, dv, delta, pos, cos, sin)
            C.flash_attn(wq, causal, 1, q, k, v, o, lse, cut, qtiles, nh, nkv,
                         scale, do, dq, dk, dv, delta, pos, cos, sin)
        if rp is not None:
            dqkv._lumen_rope_undone = True
        return dqkv, None, None, None, None, None, None, None, None


KERNEL_D = 128  # head dim of the HIP flash-attention kernels


def _flash_padded(qkv, cu, nh, nkv, D, causal):
    """Head dims below the kernels' 128 (OPT-125m: 64): every head is zero-padded to 128
    columns -- q.k over the padded heads is the same score, P.V leaves the pad columns of O
    zero -- and the kernel runs with the true 1/sqrt(D) scale.  The pad / slice copies are
    differentiated by autograd (their backward is the slice / pad of the gradient)."""
    T = qkv.shape[0]
    H3 = nh + 2 * nkv
    qkvp = F.pad(qkv.view(T, H3, D), (0, KERNEL_D - D)).view(T, H3 * KERNEL_D)
    o = _FlashAttn.apply(qkvp, cu, nh, nkv, KERNEL_D, causal, None, 1.0 / math.sqrt(D))
    return o.view(T, nh, KERNEL_D)[:, :, :D].reshape(T, nh * D)


def flash_attention_qkv(qkv: torch.Tensor, cu_seqlens, nh: int, nkv: int, D: int,
                        causal: bool = True, rope=None, out_ext: int = 0) -> torch.Tensor:
    """Causal attention straight from the fused token-major QKV buffer [T, (nh+2nkv)*D]
    (q/k already rotated); returns O token-major [T, nh*D].  ``cu_seqlens``: sequence offsets.

    ``rope`` = (pos int32 [T], cos, sin) of the rotation the q/k producer applied: the backward
    then returns the gradient w.r.t. the PRE-rotation q/k (marked ``_lumen_rope_undone`` on the
    dQKV tensor so the producer's backward skips its inverse pass)."""
    cu = tuple(int(c) for c in cu_seqlens)
    if use_native(qkv) and D == KERNEL_D:
        return _FlashAttn.apply(qkv, cu, nh, nkv, D, causal, rope, None, out_ext)
    if use_native(qkv) and D < KERNEL_D and D % 8 == 0 and rope is None:
        return _flash_padded(qkv.contiguous(), cu, nh, nkv, D, causal)
    return flash_attention_ref(qkv, cu, nh, nkv, D, causal)


def flash_attention_fresh(qkv: torch.Tensor, cu, nh: int, nkv: int, D: int, scale: float,
                          out: torch.Tensor) -> torch.Tensor:
    """Inference causal attention of whole fresh prompts straight from the rotated fused qkv rows
    [T, (nh + 2 nkv) D] (the training forward kernel, no autograd), into ``out`` [T, nh D]
    (row-strided views allowed)."""
    cu = tuple(int(c) for c in cu)
    T = qkv.shape[0]
    q = qkv[:, :nh * D]
    k = qkv[:, nh * D:(nh + nkv) * D]
    v = qkv[:, (nh + nkv) * D:(nh + 2 * nkv) * D]
    lse = torch.empty(nh, T, device=qkv.device, dtype=torch.float32)
    native().flash_attn(0, True, FA_FWD_MT, q, k, v, out, lse, _cu_tensor(cu, qkv.device),
                        _tiles(cu, FA_FWD_ROWS, qkv.device), nh, nkv, scale, None, None, None,
                        None, None, None, None, None)
    return out


def flash_attention_ref(qkv, cu, nh, nkv, D, causal=True):
    outs = []
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        n = b - a
        q = qkv[a:b, :nh * D].view(n, nh, D).transpose(0, 1)[None]
        k = qkv[a:b, nh * D:(nh + nkv) * D].view(n, nkv, D).transpose(0, 1)[None]
        v = qkv[a:b, (nh + nkv) * D:].view(n, nkv, D).transpose(0, 1)[None]
        if nkv != nh:
            rep = nh // nkv
            k, v = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
        o = F.scaled_dot_product_attention(q, k, v, is_causal=causal)
        outs.append(o[0].transpose(0, 1).reshape(n, nh * D))
    return torch.cat(outs, 0)


# ---- keys-as-values attention over a paged key cache, block-diagonal mask, optional sink ------
# The cache holds ONE tensor per layer, the un-normalised keys [blocks, block_size, G, D]
# (token-major: a token's keys of all heads are one row), because the values ARE those keys;
# the unit-RMS key the scores use is recomputed from the row the kernel loads anyway, so the
# cache costs half the bytes of a K + V cache.  Row i of a sequence sees key j when j <= i and
# (chunk == 0 or j // chunk == i // chunk); chunks count from position 0 of the sequence.  With
# ``sink`` the softmax denominator gains exp(0): a key of score 0 that carries no value.
# (HIP: ``csrc/seqmix/attention.hip``; scores, softmax and the q / k norms in fp32.)
def write_key_cache(k: torch.Tensor, cache: torch.Tensor, slots: torch.Tensor) -> None:
    """Rows of k [T, G * D] (any row stride) into cache rows ``slots`` (int64; -1 skips)."""
    from ._seqmix import DT, call, use_seqmix

    GD = cache.shape[2] * cache.shape[3]
    if not use_seqmix(k):
        ok = slots >= 0
        cache.view(-1, GD)[slots[ok]] = k[ok].to(cache.dtype)
        return
    assert k.stride(1) == 1 and cache.is_contiguous() and cache.dtype == k.dtype
    call("sm_write_k", DT[k.dtype], k, k.stride(0), cache, slots, k.shape[0], GD)


def chunk_sink_attention_ref(q, cache, seg, H, G, D, scale, chunk, eps, sink=True):
    T = q.shape[0]
    bs = cache.shape[1]
    out = torch.zeros(T, H, D, dtype=torch.float32, device=q.device)
    qf = q.float().reshape(T, H, D)
    qf = qf / torch.sqrt((qf * qf).mean(-1, keepdim=True) + eps)
    row_seg, pos = seg.row_seg.tolist(), seg.positions.tolist()
    rows = cache.view(-1, G, D)
    for t in range(T):
        i = pos[t]
        lo = (i // chunk) * chunk if chunk else 0
        js = torch.arange(lo, i + 1, device=q.device)
        tbl = seg.tables[row_seg[t]].long()
        kr = rows[tbl[js // bs] * bs + js % bs].float()            # [n, G, D] raw keys = values
        kn = kr / torch.sqrt((kr * kr).mean(-1, keepdim=True) + eps)
        for h in range(H):
            g = h // (H // G)
            s = (kn[:, g] @ qf[t, h]) * scale
            m = torch.clamp(s.max(), min=0.0) if sink else s.max()
            e = torch.exp(s - m)
            den = e.sum() + (torch.exp(-m) if sink else 0.0)
            out[t, h] = (e / den) @ kr[:, g]
    return out.reshape(T, H * D).to(q.dtype)


def chunk_sink_attention(q: torch.Tensor, cache: torch.Tensor, seg, H: int, G: int, D: int,
                         scale: float, chunk: int, eps: float, sink: bool = True) -> torch.Tensor:
    """q [T, H * D] (rows may be strided) against the paged raw-key cache; the step's own keys
    must already be in the cache (``write_key_cache``).  Returns [T, H * D] in q's dtype."""
    from ._seqmix import DT, call, tiles_ok, use_seqmix

    if not use_seqmix(q):
        return chunk_sink_attention_ref(q, cache, seg, H, G, D, scale, chunk, eps, sink)
    assert q.stride(1) == 1 and cache.is_contiguous() and cache.dtype == q.dtype
    assert cache.shape[2] == G and cache.shape[3] == D and H % G == 0
    if D > 256:
        raise ValueError(f"attention head size {D} > 256 is not supported")
    T = q.shape[0]
    out = torch.empty(T, H * D, dtype=q.dtype, device=q.device)
    maxb, bs = seg.tables.shape[1], cache.shape[1]
    # prefill chunks: 64-row tiles on the matrix cores (16-bit dtypes, head sizes it is built
    # for); decode rows, fp32 and other head sizes: one wave per (row, head)
    Tp = 0
    if (seg.q_tiles is not None and seg.tile_rows > 0 and q.stride(0) % 8 == 0
            and q.data_ptr() % 16 == 0 and tiles_ok(DT[q.dtype], D)):
        Tp = seg.tile_rows
        call("sm_chunk_attn_tiles", DT[q.dtype], q, q.stride(0), cache, out, seg.tables, maxb,
             seg.q_tiles, seg.q_tiles.shape[0], seg.cu, seg.start, H, G, D, bs, scale, eps, chunk,
             int(sink), seg.tile_size)
    if T > Tp:
        call("sm_chunk_attn", DT[q.dtype], q[Tp:], q.stride(0), cache, out[Tp:], seg.tables, maxb,
             seg.row_seg[Tp:], seg.positions[Tp:], T - Tp, H, G, D, bs, scale, eps, chunk,
             int(sink))
    return out


# ---- row attention over paged caches: latent (shared compressed row) and grouped-query ----------
# One kernel (``csrc/seqmix/row_attention.hip``) serves prompts' portions and decoded rows: a
# row's position and its segment's block table say which keys it sees.  What stands between the
# dot product and the softmax is a parameter: a position-dependent query temperature, a tanh soft
# cap, a logarithmic distance bias per head, a mixing of the heads' scores, a per-head sink in
# the softmax denominator.  Scores and weights are fp32.
def latent_write_ref(z, w_norm, inv_freq, positions, slots, cache, R, dims, eps, vt=None):
    zf = z.float()
    c = zf[:, :R]
    c = c / torch.sqrt((c * c).mean(-1, keepdim=True) + eps) * w_norm.float()
    kr = zf[:, R:].clone()
    if dims:
        a = positions.float().view(-1, 1) * inv_freq.float().view(1, -1)
        u, v = kr[:, 0:dims:2].clone(), kr[:, 1:dims:2].clone()
        kr[:, 0:dims:2] = u * torch.cos(a) - v * torch.sin(a)
        kr[:, 1:dims:2] = v * torch.cos(a) + u * torch.sin(a)
    ok = slots >= 0
    cache.view(-1, cache.shape[-1])[slots[ok]] = torch.cat([c, kr], 1)[ok].to(cache.dtype)
    if vt is not None:
        bs = vt.shape[2]
        vt[slots[ok] // bs, :, slots[ok] % bs] = c[ok].to(vt.dtype)


def transposed_values_ok(dtype, R: int, Dr: int, block_size: int, device) -> bool:
    """Can latent attention over rows [R | Dr] run its value product on the matrix cores, i.e.
    is a per-block transposed copy of the latents [blocks, R, block] worth keeping?"""
    from ._seqmix import DT, latent_attn_ok

    if torch.device(device).type != "cuda" or dtype not in (torch.bfloat16, torch.float16):
        return False
    return latent_attn_ok(DT[dtype], R, R + Dr, R, block_size)


def latent_write(z: torch.Tensor, w_norm: torch.Tensor, inv_freq: torch.Tensor,
                 positions: torch.Tensor, slots: torch.Tensor, cache: torch.Tensor, R: int,
                 dims: int, eps: float, vt: Optional[torch.Tensor] = None) -> None:
    """Rows of a latent-attention layer's down projection z [T, R + Dr] into the paged cache
    [blocks, block, R + Dr] at ``slots`` (int64; -1 skips): the first R columns RMS-normed with
    ``w_norm``, the rest (the key part all heads share) rotated on its first ``dims`` columns.
    ``vt`` [blocks, R, block] (optional) takes the normed latents once more, transposed within
    each cache block: the layout the matrix-core value product reads (keys contiguous)."""
    from ._seqmix import DT, call, use_seqmix

    Dr = z.shape[1] - R
    if cache.shape[-1] != R + Dr or dims > Dr or dims % 2:
        raise ValueError(f"latent row {R}+{Dr} (rotary {dims}) does not fit cache rows of "
                         f"{cache.shape[-1]}")
    if vt is not None and (tuple(vt.shape) != (cache.shape[0], R, cache.shape[1])
                           or vt.dtype != cache.dtype or not vt.is_contiguous()):
        raise ValueError(f"transposed copy {tuple(vt.shape)} does not match cache "
                         f"{tuple(cache.shape)} with latent size {R}")
    if not use_seqmix(z):
        return latent_write_ref(z, w_norm, inv_freq, positions, slots, cache, R, dims, eps, vt)
    assert z.stride(1) == 1 and cache.is_contiguous() and cache.dtype == z.dtype
    call("sm_latent_write", DT[z.dtype], z, z.stride(0), w_norm, inv_freq, positions, slots, cache,
         vt, cache.shape[1], z.shape[0], R, Dr, dims, eps)


def head_norm_write_ref(qkv, wq, wk, slots, kcache, vcache, H, G, D, Dv, eps):
    T = qkv.shape[0]

    def unit(x):
        x = x.float()
        return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)

    q = unit(qkv[:, :H * D].reshape(T, H, D)) * wq.float()
    k = unit(qkv[:, H * D:(H + G) * D].reshape(T, G, D)) * wk.float()
    qkv[:, :H * D] = q.reshape(T, H * D).to(qkv.dtype)
    ok = slots >= 0
    kcache.view(-1, G, D)[slots[ok]] = k[ok].to(kcache.dtype)
    vcache.view(-1, G, Dv)[slots[ok]] = qkv[:, (H + G) * D:].reshape(T, G, Dv)[ok].to(vcache.dtype)


def head_norm_write(qkv: torch.Tensor, wq: torch.Tensor, wk: torch.Tensor, slots: torch.Tensor,
                    kcache: torch.Tensor, vcache: torch.Tensor, H: int, G: int, D: int, Dv: int,
                    eps: float) -> None:
    """qkv [T, H * D + G * D + G * Dv] (a fused projection's output): every query head and key
    head is RMS-normed over its D entries with the weight ``wq`` / ``wk`` [D] shared by the heads;
    q is replaced in place, the normed keys and the values go to their paged caches
    [blocks, block, G, D] / [blocks, block, G, Dv] at ``slots`` (int64; -1 skips)."""
    from ._seqmix import DT, call, use_seqmix

    if qkv.shape[1] != (H + G) * D + G * Dv:
        raise ValueError(f"qkv has {qkv.shape[1]} columns, expected {(H + G) * D + G * Dv}")
    if not use_seqmix(qkv):
        return head_norm_write_ref(qkv, wq, wk, slots, kcache, vcache, H, G, D, Dv, eps)
    assert qkv.stride(1) == 1 and kcache.is_contiguous() and vcache.is_contiguous()
    assert kcache.dtype == qkv.dtype and vcache.dtype == qkv.dtype
    assert tuple(kcache.shape[2:]) == (G, D) and tuple(vcache.shape[2:]) == (G, Dv)
    call("sm_head_norm_write", DT[qkv.dtype], qkv, qkv.stride(0), wq, wk, slots, kcache, vcache,
         qkv.shape[0], H, G, D, Dv, eps)


def row_norm_write_ref(qk, wq, wk, slots, kcache, vcache, HD, GD, eps):
    def unit(x):
        x = x.float()
        return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)

    k = qk[:, HD:HD + GD]
    ok = slots >= 0
    vcache.view(-1, GD)[slots[ok]] = k[ok].to(vcache.dtype)
    kcache.view(-1, GD)[slots[ok]] = (unit(k) * wk.float())[ok].to(kcache.dtype)
    qk[:, :HD] = (unit(qk[:, :HD]) * wq.float()).to(qk.dtype)


def row_norm_write(qk: torch.Tensor, wq: torch.Tensor, wk: torch.Tensor, slots: torch.Tensor,
                   kcache: torch.Tensor, vcache: torch.Tensor, HD: int, GD: int,
                   eps: float) -> None:
    """qk [T, >= HD + GD] (a fused projection's output; further columns are left alone): the
    query part [0, HD) is RMS-normed over ALL its HD entries at once (every head together) with
    the weight ``wq`` [HD] and replaced in place; the key part [HD, HD + GD) goes to the paged
    caches at ``slots`` (int64; -1 skips) twice: normed the same way with ``wk`` [GD] into
    ``kcache``, and as projected into ``vcache`` (the values are the un-normalised keys).  Both
    caches are [blocks, block, G, D] with G * D = GD."""
    from ._seqmix import DT, call, use_seqmix

    if qk.shape[1] < HD + GD:
        raise ValueError(f"qk has {qk.shape[1]} columns, expected at least {HD + GD}")
    if kcache.shape[2:].numel() != GD or vcache.shape[2:].numel() != GD:
        raise ValueError(f"cache rows of {kcache.shape[2:].numel()} / {vcache.shape[2:].numel()} "
                         f"do not hold keys of {GD}")
    if not use_seqmix(qk):
        return row_norm_write_ref(qk, wq, wk, slots, kcache, vcache, HD, GD, eps)
    assert qk.stride(1) == 1 and kcache.is_contiguous() and vcache.is_contiguous()
    assert kcache.dtype == qk.dtype and vcache.dtype == qk.dtype
    assert wq.dtype == torch.float32 and wk.dtype == torch.float32
    assert tuple(wq.shape) == (HD,) and tuple(wk.shape) == (GD,)
    call("sm_row_norm_write", DT[qk.dtype], qk, qk.stride(0), wq, wk, slots, kcache, vcache,
         qk.shape[0], HD, GD, eps)


def row_attention_ref(q1, q2, kcache, vcache, Dv, out, seg, H, G, scale, softcap=0.0,
                      q_temp=None, r1=None, r2=None, talk=None, sink=None, slopes=None,
                      window=0, keep_first=0, gate=None, sigmoid_bias=None, v_div=1):
    T = q1.shape[0]
    D1 = q1.shape[2]
    D2 = q2.shape[2] if q2 is not None else 0
    Dk = D1 + D2
    bs = kcache.shape[1]
    krows = kcache.reshape(kcache.shape[0] * bs, -1)
    vrows = vcache.reshape(vcache.shape[0] * bs, -1)
    q = q1.float() if q2 is None else torch.cat([q1.float(), q2.float()], -1)    # [T, H, Dk]
    row_seg, pos = seg.row_seg.tolist(), seg.positions.tolist()
    hg = torch.arange(H, device=q.device) // (H // G)
    for t in range(T):
        p = pos[t]
        js = torch.arange(0, p + 1, device=q.device)
        if window and window > 0:
            js = js[(p - js < window) | (js < keep_first)]
        tbl = seg.tables[row_seg[t]].long()
        rows = tbl[js // bs] * bs + js % bs
        k = krows[rows][:, :G * Dk].float().view(-1, G, Dk)[:, hg]              # [n, H, Dk]
        v = vrows[rows].float()
        Gv = G // v_div
        v = (v[:, :Gv * Dv].view(-1, Gv, Dv) if G > 1 or vrows.shape[1] == Dv
             else v[:, :Dv].view(-1, 1, Dv))[:, hg // v_div]                    # [n, H, Dv]
        temp = 1.0
        if q_temp is not None and q_temp[0] != 0.0 and q_temp[1] > 0:
            temp = 1.0 + q_temp[0] * math.log((p + 1) // q_temp[1] + 1.0)
        s = torch.einsum("hd,nhd->hn", q[t], k) * (scale * temp)
        if softcap and softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        if r1 is not None:
            d = (p - js).float()
            s = s - r1.float().view(H, 1) * torch.log(1.0 + r2.float().view(H, 1) * d)
        if slopes is not None:
            s = s - slopes.float().view(H, 1) * (p - js).float()
        if talk is not None:
            s = talk.float() @ s
        if sigmoid_bias is not None:
            o = torch.einsum("hn,nhd->hd", torch.sigmoid(s + sigmoid_bias.float().view(H, 1)), v)
            if gate is not None:
                o = o * torch.sigmoid(gate[t].float()).view(H, 1)
            out[t] = o.to(out.dtype)
            continue
        m = s.max(-1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink.float().view(H, 1))
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink.float().view(H, 1) - m)
        o = torch.einsum("hn,nhd->hd", e / den, v)
        if gate is not None:
            o = o * torch.sigmoid(gate[t].float()).view(H, 1)
        out[t] = o.to(out.dtype)
    return out


def _heads_per_block(H: int, Dk: int, need_all: bool) -> int:
    """Heads one workgroup of the row kernel takes: as many as its LDS (64 KB) holds, at most 32;
    a power of two unless all H are needed (head mixing)."""
    from ._seqmix import row_attn_lds

    if need_all:
        if H > 32 or row_attn_lds(H, Dk) > 65536:
            raise ValueError(f"head mixing over {H} heads of key size {Dk} does not fit the "
                             "attention kernel (at most 32 heads, 64 KB of LDS)")
        return H
    hb = 1
    while hb * 2 <= min(H, 16) and row_attn_lds(hb * 2, Dk) <= 65536:
        hb *= 2
    return hb


def row_attention(q1: torch.Tensor, q2: Optional[torch.Tensor], kcache: torch.Tensor,
                  vcache: torch.Tensor, Dv: int, out: torch.Tensor, seg, H: int, G: int,
                  scale: float, softcap: float = 0.0, q_temp=None, r1=None, r2=None, talk=None,
                  sink=None, vt: Optional[torch.Tensor] = None, slopes=None, window: int = 0,
                  keep_first: int = 0, gate: Optional[torch.Tensor] = None,
                  sigmoid_bias: Optional[torch.Tensor] = None, v_div: int = 1) -> torch.Tensor:
    """Causal attention of every row of a step against paged caches.

    q1 [T, H, D1] and (optionally) q2 [T, H, D2] are views with arbitrary row / head strides;
    a key row is ``kcache[block, i, g * Dk : (g + 1) * Dk]`` with Dk = D1 + D2 (q1 faces its
    first D1 entries, q2 the rest); a value row is ``vcache[block, i, g * Dv : (g + 1) * Dv]``
    -- ``vcache`` may be ``kcache`` itself (G = 1: the value is a prefix of the key row).
    ``out`` [T, H, Dv] is a view with arbitrary row / head strides.  The step's own keys must
    already be in the cache.  ``q_temp`` = (coef, every): the score of a row at position p is
    multiplied by 1 + coef * ln(floor((p + 1) / every) + 1).  ``softcap`` > 0: s <- cap *
    tanh(s / cap).  ``r1``, ``r2`` [H]: s <- s - r1 * ln(1 + r2 * distance).  ``talk`` [H, H]:
    the heads' scores are mixed, s_h <- sum_g talk[h, g] s_g.  ``sink`` [H]: exp(sink_h) joins
    the softmax denominator.  ``slopes`` [H]: s <- s - slopes_h * distance (a linear distance
    bias).  ``window`` > 0: a row at position p only sees the keys j with p - j < window and,
    besides them, the sequence's first ``keep_first`` keys (at their true distances); tiles of
    keys between the two ranges are never loaded.  ``gate`` [T, H] (a view, any row stride):
    head h's output is multiplied by sigmoid(gate[t, h]).  ``sigmoid_bias`` [H]: no softmax -- a
    seen key weighs sigmoid(s + sigmoid_bias_h), each weight on its own (nothing sums to one)
    (a sink is meaningless then and refused).  ``v_div`` > 1: ``v_div`` consecutive key heads
    share one value head (key head g reads value head g // v_div; ``vcache`` rows hold G / v_div
    heads) -- several score maps over the same values.  ``vt`` [blocks, Dv, block]: a per-block
    transposed copy of the values (``latent_write`` keeps one); with it, one key/value head,
    values that are a prefix of the key rows and a 16-bit dtype, the whole kernel runs on the
    matrix cores.

    Three kernels serve it.  The prompt portions of a step (``seg.q_tiles``) go to the tiled
    matrix-core kernel of ``csrc/seqmix/window_attention.hip`` when the keys and values have caches
    of their own, one query part, head sizes it is built for (values as wide as the keys or twice
    as wide), a 16-bit dtype and none of temperature, logarithmic bias, head mixing or sink; the latent layout with ``vt`` goes to the
    latent kernel; every other row (decoded rows, fp32, other shapes) to the row kernel.  A row's
    result does not depend on which of them computed it beyond rounding."""
    from ._seqmix import DT, call, latent_attn_ok, use_seqmix, win_tiles_ok

    T, _, D1 = q1.shape
    D2 = q2.shape[2] if q2 is not None else 0
    Dk = D1 + D2
    if H % G:
        raise ValueError(f"{H} heads are not a multiple of {G} key/value heads")
    v_div = int(v_div or 1)
    if v_div < 1 or G % v_div:
        raise ValueError(f"{G} key heads do not share values in groups of {v_div}")
    if sigmoid_bias is not None and sink is not None:
        raise ValueError("sigmoid weights are not normalised: a sink has no meaning")
    if not use_seqmix(q1):
        return row_attention_ref(q1, q2, kcache, vcache, Dv, out, seg, H, G, scale, softcap,
                                 q_temp, r1, r2, talk, sink, slopes, window, keep_first, gate,
                                 sigmoid_bias, v_div)
    if Dv > 512:
        raise ValueError(f"value size {Dv} > 512 is not supported")
    assert kcache.is_contiguous() and vcache.is_contiguous() and kcache.dtype == q1.dtype
    assert q1.stride(2) == 1 and out.stride(2) == 1 and (q2 is None or q2.stride(2) == 1)
    krow = kcache.shape[2:].numel()
    vrow = vcache.shape[2:].numel()
    assert krow >= G * Dk and vrow >= (G // v_div) * Dv
    for f in (r1, r2, talk, sink, slopes, sigmoid_bias):
        assert f is None or (f.dtype == torch.float32 and f.is_contiguous())
    window, keep_first = max(0, int(window or 0)), max(0, int(keep_first or 0))
    if gate is not None:
        assert gate.dtype == q1.dtype and gate.stride(1) == 1 and tuple(gate.shape) == (T, H)
    coef, every = (float(q_temp[0]), int(q_temp[1])) if q_temp is not None else (0.0, 0)
    bs = kcache.shape[1]
    al8 = lambda x: x.data_ptr() % 16 == 0 and x.stride(0) % 8 == 0 and x.stride(1) % 8 == 0  # noqa: E731
    if (vt is not None and G == 1 and talk is None and vcache is kcache and D1 >= Dv
            and slopes is None and window == 0 and sigmoid_bias is None
            and (gate is None or gate.stride(1) == 1)
            and q1.dtype in (torch.bfloat16, torch.float16) and latent_attn_ok(DT[q1.dtype], Dv, Dk, D1, bs)
            and krow % 8 == 0 and al8(q1) and (q2 is None or al8(q2)) and out.data_ptr() % 8 == 0
            and out.stride(0) % 4 == 0 and out.stride(1) % 4 == 0):
        assert tuple(vt.shape) == (kcache.shape[0], Dv, bs) and vt.is_contiguous()
        blocks = T * ((H + 15) // 16)
        tiles = (seg.tables.shape[1] * bs + 127) // 128
        nsplit = max(1, min(tiles, 32, 512 // max(blocks, 1)))
        ws_ml = ws_o = None
        if nsplit > 1:
            ws_ml = torch.empty(T * H * nsplit * 2, dtype=torch.float32, device=q1.device)
            ws_o = torch.empty(T * H * nsplit * Dv, dtype=torch.float32, device=q1.device)
        call("sm_latent_attn", DT[q1.dtype], q1, q1.stride(0), q1.stride(1), D1,
             q2, q2.stride(0) if q2 is not None else 0, q2.stride(1) if q2 is not None else 0, D2,
             kcache, krow, vt, Dv, out, out.stride(0), out.stride(1),
             seg.tables, seg.tables.shape[1], seg.row_seg, seg.positions, T, H, bs,
             scale, float(softcap or 0.0), coef, every, r1, r2, sink,
             gate, gate.stride(0) if gate is not None else 0, nsplit, ws_ml, ws_o)
        return out
    # a step's prompt portions: tiles of consecutive rows of one segment on the matrix cores, when
    # nothing needs all heads of a (row, key) pair at once and the kernel has the head size; the
    # decoded rows after them (and every other case) take the row kernel below
    Tp = 0
    if (seg.q_tiles is not None and seg.tile_rows > 0 and q2 is None and talk is None
            and sink is None and r1 is None and q_temp is None and vcache is not kcache
            and krow == G * D1 and vrow == (G // v_div) * Dv and win_tiles_ok(DT[q1.dtype], D1, Dv)
            and q1.stride(1) == D1 and q1.stride(0) % 8 == 0 and q1.data_ptr() % 16 == 0
            and out.stride(1) == Dv and out.stride(0) == H * Dv and out.data_ptr() % 8 == 0):
        Tp = seg.tile_rows
        call("sm_win_attn_tiles", DT[q1.dtype], q1, q1.stride(0), kcache, vcache, out, gate,
             gate.stride(0) if gate is not None else 0, seg.tables, seg.tables.shape[1],
             seg.q_tiles, seg.q_tiles.shape[0], seg.cu, seg.start, H, G, D1, bs, scale,
             float(softcap or 0.0), slopes, window, keep_first, seg.tile_size, Dv, sigmoid_bias,
             v_div)
        if Tp >= T:
            return out
        q1, out, T = q1[Tp:], out[Tp:], T - Tp
        gate = gate[Tp:] if gate is not None else None
    row_seg, positions = seg.row_seg[Tp:], seg.positions[Tp:]
    HB = _heads_per_block(H, Dk, talk is not None)
    # few rows (decoding): deal a row's 64-key tiles out to several workgroups so that ~2 per CU
    # run; the count depends on the step's size only, never on device data (graph capture)
    tiles = (seg.tables.shape[1] * kcache.shape[1] + 63) // 64
    if window > 0:                     # a row visits the window's tiles and the kept first ones
        tiles = min(tiles, (window + 63) // 64 + 1 + (keep_first + 63) // 64)
    while talk is None and HB > 4 and T * ((H + HB - 1) // HB) * tiles < 512:
        HB //= 2                       # fewer heads per workgroup: more workgroups
    blocks = T * ((H + HB - 1) // HB)
    nsplit = max(1, min(tiles, 32, 512 // max(blocks, 1)))
    ws_ml = ws_o = None
    if nsplit > 1:
        ws_ml = torch.empty(T * H * nsplit * 2, dtype=torch.float32, device=q1.device)
        ws_o = torch.empty(T * H * nsplit * Dv, dtype=torch.float32, device=q1.device)
    call("sm_row_attn", DT[q1.dtype], q1, q1.stride(0), q1.stride(1), D1,
         q2, q2.stride(0) if q2 is not None else 0, q2.stride(1) if q2 is not None else 0, D2,
         kcache, krow, vcache, vrow, Dv, out, out.stride(0), out.stride(1),
         seg.tables, seg.tables.shape[1], row_seg, positions, T, H, G, HB,
         kcache.shape[1], scale, float(softcap or 0.0), coef, every, r1, r2, talk, sink,
         slopes, window, keep_first, gate, gate.stride(0) if gate is not None else 0,
         sigmoid_bias, v_div, nsplit, ws_ml, ws_o)
    return out


# ---- differential attention: two score maps per head combined, normed and gated -------------------
# ``a`` holds both maps' outputs over the same values, laid out [T, G, 2, rep, Dv] (key head, map,
# query head within the key head).  Head h = g * rep + r becomes
#     o = a[g, 0, r] - lam * a[g, 1, r];   o <- o / sqrt(mean(o^2) + eps) * out_scale
# and the concatenated heads are multiplied element-wise by sigmoid(gate).  fp32 throughout; only
# the stored result is rounded.  (HIP: ``csrc/seqmix/foderax.hip``.)
def diff_head_combine_ref(a, lam, out_scale, eps, gate, G, rep, Dv):
    T = a.shape[0]
    af = a.float().reshape(T, G, 2, rep, Dv)
    o = af[:, :, 0] - lam * af[:, :, 1]                          # [T, G, rep, Dv]
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * out_scale
    o = o.reshape(T, G * rep * Dv)
    if gate is not None:
        o = o * torch.sigmoid(gate.float())
    return o.to(a.dtype)


def diff_head_combine(a: torch.Tensor, lam: float, out_scale: float, eps: float,
                      gate: Optional[torch.Tensor], G: int, rep: int, Dv: int) -> torch.Tensor:
    """a [T, G * 2 * rep * Dv] (contiguous) -> [T, G * rep * Dv] in a's dtype; ``gate``
    [T, G * rep * Dv] (logits; a view with any row stride) or None."""
    from ._seqmix import DT, call, use_seqmix

    T = a.shape[0]
    if a.shape[1:].numel() != G * 2 * rep * Dv:
        raise ValueError(f"a has {a.shape[1:].numel()} columns, expected {G * 2 * rep * Dv}")
    if not use_seqmix(a):
        return diff_head_combine_ref(a, lam, out_scale, eps, gate, G, rep, Dv)
    assert a.is_contiguous() and (gate is None or (gate.stride(1) == 1 and gate.dtype == a.dtype))
    if Dv > 512:
        raise ValueError(f"value size {Dv} > 512 is not supported")
    out = torch.empty(T, G * rep * Dv, dtype=a.dtype, device=a.device)
    call("sm_diff_combine", DT[a.dtype], a, gate, gate.stride(0) if gate is not None else 0, out,
         T, G, rep, Dv, float(lam), float(out_scale), float(eps))
    return out
