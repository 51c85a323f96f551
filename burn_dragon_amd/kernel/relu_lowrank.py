"""relu_lowrank::fused_forward (reference: src/kernel/relu_lowrank.rs:7-37) on the HIP library."""
from __future__ import annotations

from typing import Optional

import torch

from .. import ffi
from .block_sparse import BlockPattern1d


def fused_forward(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], threshold: float,
                  layout: BlockPattern1d, gate: Optional[torch.Tensor] = None,
                  ctx: Optional[ffi.Context] = None) -> torch.Tensor:
    """input [B,1|h,T,d], weight [1,h,d,N] or [h,d,N], bias [h,1,N]|None -> [B,h,T,N]."""
    ctx = ctx or ffi.default_context(input.device.index or 0)
    if weight.dim() == 4:
        assert weight.shape[0] == 1
        weight = weight[0]
    B, h_in, T, d = input.shape
    h, d_w, N = weight.shape
    if d != d_w:
        raise ValueError(f"inner dimensions differ: {d} vs {d_w}")
    input, weight = input.contiguous().float(), weight.contiguous().float()
    bias_c = None if bias is None else bias.reshape(h, N).contiguous().float()
    gate_c = None if gate is None else gate.contiguous().float()
    out = torch.empty((B, h, T, N), device=input.device, dtype=torch.float32)
    blocks = layout.block_bytes(N) if layout.is_sparse() else None
    ctx.check(ctx.lib.bdh_relu_lowrank(ctx.handle, B, h_in, T, d, h, N, ffi.ptr(input), ffi.ptr(weight),
                                       ffi.ptr(bias_c), float(threshold), max(layout.block_size, 1),
                                       blocks, 0 if blocks is None else len(blocks), ffi.ptr(gate_c), ffi.ptr(out)))
    return out
