"""Loader for the sequence-mixing kernel library ``lumen/_C_seqmix.so`` (``lumen/csrc/seqmix``).

The library is plain ``extern "C"`` launchers (raw pointers, sizes, a HIP stream) bound through
ctypes, so it builds in seconds without the torch headers and a model that needs only these
kernels does not wait for the full extension.  Policy as for ``lumen._C``: on a GPU tensor the
HIP kernel is THE implementation; when the library is missing it is built once (hipcc, gfx950),
and if that is impossible every op raises.  CPU tensors take the torch reference path.
"""
from __future__ import annotations

import ctypes
import os

import torch

_lib = None
_err = None

_T = {"p": ctypes.c_void_p, "i": ctypes.c_int, "l": ctypes.c_longlong, "f": ctypes.c_float}

# launcher name -> argument kinds (p pointer, i int32, l int64, f float); a hipStream_t follows
SIGNATURES = {
    "sm_dyt": "iipppppii",
    "sm_dyt_residual": "iipppppppppii",
    "sm_dyt_canon": "ipppppppppppiii",
    "sm_canon_tail": "ppppppppiii",
    "sm_token_shift": "ippppppppiii",
    "sm_shift_tail": "ippppii",
    "sm_wkv": "iplplplplplppppplpppiiif",
    "sm_gdelta": "iplplplplplplppppplpppiiifff",
    "sm_write_k": "iplppii",
    "sm_chunk_attn": "iplpppippiiiiiffii",
    "sm_chunk_attn_tiles": "iplpppipippiiiiffiii",
    "sm_route_topk": "ppiii",
    "sm_gated_act": "ipppiiiii",
    "sm_group_rms": "iiplpppliiif",
    "sm_gate_rows": "iplplpiipi",
    "sm_rotate_heads": "iplliiippi",
    "sm_latent_write": "iplppppppiiiiif",
    "sm_head_norm_write": "iplpppppiiiiif",
    "sm_latent_attn": "i" "plli" "plli" "pl" "pi" "pll" "pi" "pp" "iii" "fffi" "ppp" "pl" "ipp",
    "sm_row_attn": "i" "plli" "plli" "pl" "pli" "pll" "pi" "pp" "iiiii" "fffi" "pppp" "piipl"
                   "pi" "ipp",
    "sm_win_attn_tiles": "iplppppl" "pi" "pi" "pp" "iiii" "ff" "p" "iii" "ipi",
    "sm_row_norm_write": "iplpppppiiif",
    "sm_layer_norm": "iippfppiif",
    "sm_embed_pos": "ipppppiiii",
    "sm_route_groups": "pppiiiiiiffii",
    "sm_rotary_write": "iplppppiiiiipii",
    "sm_min_gru": "iplpppppppiifppii",
    "sm_diff_combine": "ipplpiiiifff",
    "sm_depth_mix": "iipipppppppppppiif",
    "sm_embed_scaled": "ipppiiif",
    "sm_soft_cap": "ipplf",
    "sm_scaled_act": "ipppiiiii",
}


def _load():
    global _lib, _err
    if _lib is not None or _err is not None:
        return _lib
    try:
        from ..csrc.build import build_seqmix, seqmix_path, seqmix_stale

        path = seqmix_path()
        if not os.path.exists(path) or seqmix_stale():
            build_seqmix(verbose=False)
        lib = ctypes.CDLL(path)
        for name, sig in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = [_T[c] for c in sig] + [ctypes.c_void_p]
            fn.restype = ctypes.c_int
        lib.sm_chunk_attn_tiles_ok.argtypes = [ctypes.c_int, ctypes.c_int]
        lib.sm_chunk_attn_tiles_ok.restype = ctypes.c_int
        lib.sm_win_attn_tiles_ok.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int]
        lib.sm_win_attn_tiles_ok.restype = ctypes.c_int
        lib.sm_row_attn_lds.argtypes = [ctypes.c_int, ctypes.c_int]
        lib.sm_row_attn_lds.restype = ctypes.c_int
        lib.sm_latent_attn_ok.argtypes = [ctypes.c_int] * 5
        lib.sm_latent_attn_ok.restype = ctypes.c_int
        lib.sm_min_gru_sub.argtypes = []
        lib.sm_min_gru_sub.restype = ctypes.c_int
        _lib = lib
    except Exception as e:  # pragma: no cover - depends on build state
        _err = e
    return _lib


def seqmix_error():
    _load()
    return _err


def use_seqmix(t: torch.Tensor) -> bool:
    """True when ``t`` lives on the GPU (the HIP path must run, or this raises)."""
    if not t.is_cuda:
        return False
    if _load() is None:
        raise RuntimeError(f"lumen sequence-mixing kernels are not available ({_err!r}); build "
                           "them with `python -m lumen.csrc.build --seqmix`")
    return True


DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def tiles_ok(dt: int, D: int) -> bool:
    """Does the matrix-core prefill attention have a kernel for this dtype code / head size?"""
    return bool(_load().sm_chunk_attn_tiles_ok(dt, D))


def win_tiles_ok(dt: int, D: int, Dv: int = 0) -> bool:
    """Does the matrix-core prefill attention over paged key and value caches have a kernel for
    this dtype code / key size / value size (0: the key size)?"""
    return bool(_load().sm_win_attn_tiles_ok(dt, D, Dv or D))


def row_attn_lds(HB: int, Dk: int) -> int:
    """LDS bytes the row-attention kernel needs for a block of HB heads with key size Dk."""
    return int(_load().sm_row_attn_lds(HB, Dk))


def latent_attn_ok(dt: int, Dv: int, Dk: int, D1: int, bs: int) -> bool:
    """Does the matrix-core latent attention have a kernel for these sizes?"""
    return bool(_load().sm_latent_attn_ok(dt, Dv, Dk, D1, bs))


def min_gru_sub() -> int:
    """Sub-chunks the minGRU scan cuts a tile of prompt rows into (sizes its scratch)."""
    return int(_load().sm_min_gru_sub())


def _arg(kind, v):
    if kind == "p":
        if v is None:
            return None
        if torch.is_tensor(v):
            return v.data_ptr()
        return v
    if kind == "f":
        return float(v)
    return int(v)


def call(name: str, *args) -> None:
    """Launch ``name`` on the current stream; tensors are passed by their data pointers."""
    lib = _load()
    sig = SIGNATURES[name]
    if len(args) != len(sig):
        raise TypeError(f"{name}: {len(args)} arguments for signature {sig!r}")
    dev_t = next(a for a in args if torch.is_tensor(a))
    stream = torch.cuda.current_stream(dev_t.device).cuda_stream
    rc = getattr(lib, name)(*[_arg(k, a) for k, a in zip(sig, args)], stream)
    if rc != 0:
        raise RuntimeError(f"{name}: HIP error {rc}")
