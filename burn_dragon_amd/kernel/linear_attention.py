"""linear_attention::fused_state_aligned and default_alibi_slopes
(reference: src/kernel/linear_attention.rs:11-163) on the HIP library."""
from __future__ import annotations

import ctypes
from typing import List, Optional

import numpy as np
import torch

from .. import ffi
from ..positional import RotaryEmbedding
from .block_sparse import BlockPattern2d


def default_alibi_slopes(n_head: int) -> List[float]:
    lib = ffi.load_library()
    out = np.zeros(max(n_head, 0), np.float32)
    rc = lib.bdh_default_alibi_slopes(n_head, out.ctypes.data if n_head > 0 else None)
    if rc != ffi.OK:
        raise ffi.BdhError(rc, "bdh_default_alibi_slopes")
    return out.tolist()


def build_freqs(latent: int, theta: float, rotary_embedding: RotaryEmbedding, device=None) -> torch.Tensor:
    """Attention::build_freqs (src/model/attention.rs:351-373) -> [1,1,1,latent]."""
    lib = ffi.load_library()
    out = np.zeros(latent, np.float32)
    rc = lib.bdh_build_freqs(latent, float(theta), int(rotary_embedding), out.ctypes.data)
    if rc != ffi.OK:
        raise ffi.BdhError(rc, "bdh_build_freqs")
    t = torch.from_numpy(out).reshape(1, 1, 1, latent)
    return t.to(device) if device is not None else t


def fused_state_aligned(query: torch.Tensor, value: torch.Tensor, freqs: torch.Tensor,
                        alibi_slopes: Optional[torch.Tensor], layout: BlockPattern2d,
                        rotary_embedding: RotaryEmbedding, row_normalize: bool = True,
                        ctx: Optional[ffi.Context] = None) -> torch.Tensor:
    """query [B,h,T,N], value [B,1,T,dv], freqs [1,1,1,N] -> [B,h,T,dv]."""
    ctx = ctx or ffi.default_context(query.device.index or 0)
    B, h, T, N = query.shape
    dv = value.shape[-1]
    query = query.contiguous().float()
    value = value.reshape(B, T, dv).contiguous().float()
    freqs = freqs.reshape(-1).contiguous().float().to(query.device)
    slopes = None if alibi_slopes is None else np.ascontiguousarray(alibi_slopes.detach().cpu().numpy(), np.float32)
    pairs, n_pairs = None, 0
    if layout.is_sparse():
        arr = np.ascontiguousarray(np.array(sorted(layout.active_pairs), np.int32).reshape(-1, 2))
        pairs, n_pairs = arr, arr.shape[0]
    out = torch.empty((B, h, T, dv), device=query.device, dtype=torch.float32)
    ctx.check(ctx.lib.bdh_fused_state_aligned(ctx.handle, B, h, T, N, dv, ffi.ptr(query), ffi.ptr(value),
                                              ffi.ptr(freqs), ffi.ptr(slopes), max(layout.block_size, 1),
                                              ffi.ptr(pairs), n_pairs, int(rotary_embedding), int(row_normalize),
                                              ffi.ptr(out)))
    return out
