"""Token-embedding lookup: HIP row gather (``kernels/embedding.hip``) for frozen
16-bit tables on the GPU; ``F.embedding`` otherwise (CPU, f32 tables, trainable tables)."""
from __future__ import annotations

import torch
import torch.nn.functional as F

from ._native import native, use_native


def embedding(ids: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """[..] int ids -> [.., H] rows of ``weight`` (no gradient w.r.t. a frozen table)."""
    if (use_native(weight) and not (weight.requires_grad and torch.is_grad_enabled())
            and weight.dtype in (torch.bfloat16, torch.float16) and weight.is_contiguous()
            and weight.shape[1] % 8 == 0 and ids.is_cuda):
        flat = ids.reshape(-1)
        if flat.dtype != torch.int64 or not flat.is_contiguous():
            flat = flat.to(torch.int64).contiguous()
        out = torch.empty(flat.numel(), weight.shape[1], device=weight.device, dtype=weight.dtype)
        native().embedding(weight, flat, out)
        return out.view(*ids.shape, weight.shape[1])
    return F.embedding(ids, weight)


def gated_token_slice_ref(z, table, tokens, col0):
    dim = z.shape[1]
    e = table[tokens][:, col0:col0 + dim].float()
    return (F.gelu(z.float(), approximate="tanh") * e).to(z.dtype)


def gated_token_slice(z: torch.Tensor, table: torch.Tensor, tokens: torch.Tensor,
                      col0: int) -> torch.Tensor:
    """gelu_tanh(z) * table[tokens, col0 : col0 + dim] for z [T, dim]: a column slice of a second
    per-token embedding, gated by a projection of the residual stream (gather and activation in
    one pass; HIP ``csrc/seqmix/rms_group.hip``)."""
    from ._seqmix import DT, call, use_seqmix

    T, dim = z.shape
    if col0 < 0 or col0 + dim > table.shape[1]:
        raise ValueError(f"columns [{col0}, {col0 + dim}) outside a table of {table.shape[1]}")
    if not use_seqmix(z):
        return gated_token_slice_ref(z, table, tokens, col0)
    assert z.stride(1) == 1 and table.stride(1) == 1 and table.dtype == z.dtype
    assert tokens.dtype == torch.int64 and tokens.is_contiguous()
    out = torch.empty(T, dim, dtype=z.dtype, device=z.device)
    call("sm_gate_rows", DT[z.dtype], z, z.stride(0), table, table.stride(0), tokens, col0, dim,
         out, T)
    return out


def embed_positions_ref(tokens, positions, table, pos_table):
    return table[tokens].float() + pos_table[positions.long()].float()


def embed_positions(tokens: torch.Tensor, positions: torch.Tensor, table: torch.Tensor,
                    pos_table: torch.Tensor) -> torch.Tensor:
    """table[token] + pos_table[position] per row, summed in fp32: the start of a residual stream
    with learned positions, [T, W] fp32.  ``positions`` must be below the position table's row
    count (the caller's length limit guarantees it).  (HIP ``csrc/seqmix/layer_norm.hip``.)"""
    from ._seqmix import DT, call, use_seqmix

    if not use_seqmix(table):
        return embed_positions_ref(tokens, positions, table, pos_table)
    assert table.is_contiguous() and pos_table.is_contiguous() and table.dtype == pos_table.dtype
    assert tokens.dtype == torch.int64 and tokens.is_contiguous()
    assert positions.dtype == torch.int32 and positions.is_contiguous()
    T, W = tokens.shape[0], table.shape[1]
    out = torch.empty(T, W, dtype=torch.float32, device=table.device)
    call("sm_embed_pos", DT[table.dtype], table, pos_table, tokens, positions, out, T, W,
         table.shape[0], pos_table.shape[0])
    return out


def embed_scaled_ref(tokens, table, scale, out):
    out.copy_(table[tokens].float() * scale)
    return out


def embed_scaled(tokens: torch.Tensor, table: torch.Tensor, scale: float,
                 out: torch.Tensor) -> torch.Tensor:
    """table[token] * scale per row in fp32 into ``out`` [T, W] (fp32, contiguous): the start of a
    residual stream whose embedding is multiplied by a constant.  (HIP
    ``csrc/seqmix/foderax.hip``.)"""
    from ._seqmix import DT, call, use_seqmix

    if not use_seqmix(table):
        return embed_scaled_ref(tokens, table, scale, out)
    assert table.is_contiguous() and out.is_contiguous() and out.dtype == torch.float32
    assert tokens.dtype == torch.int64 and tokens.is_contiguous()
    T, W = tokens.shape[0], table.shape[1]
    assert tuple(out.shape) == (T, W)
    call("sm_embed_scaled", DT[table.dtype], table, tokens, out, T, W, table.shape[0], float(scale))
    return out


def soft_cap_ref(z, cap):
    return cap * torch.tanh(z.float() / cap)


def soft_cap(z: torch.Tensor, cap: float) -> torch.Tensor:
    """cap * tanh(z / cap) element-wise in fp32 (z fp32 or 16-bit, contiguous) -> fp32."""
    from ._seqmix import DT, call, use_seqmix

    if not use_seqmix(z):
        return soft_cap_ref(z, cap)
    z = z.contiguous()
    out = torch.empty(z.shape, dtype=torch.float32, device=z.device)
    call("sm_soft_cap", DT[z.dtype], z, out, z.numel(), float(cap))
    return out
