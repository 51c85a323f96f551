"""Attention (reference: src/model/attention.rs:102-349): rotation of the sparse activations and the
all-tokens-at-once normalised causal linear attention, over the C ABI."""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from .. import ffi
from ..kernel import BlockPattern2d
from ..kernel.linear_attention import build_freqs, default_alibi_slopes, fused_state_aligned
from ..positional import RotaryEmbedding
from .config import FusedKernelConfig


class Attention:
    """src/model/attention.rs:102-140.  Holds the frequency table, the ALiBi slopes and the time-block
    pattern of one model; `forward` is the stateless form (training path), `rotate_positions` the
    rotation the cached step applies at `state.position`."""

    def __init__(self, latent: int, n_head: int, device, kernel: FusedKernelConfig):
        self.device = torch.device(device)
        self.n_head = n_head
        self.latent = latent
        self.rotary_embedding = RotaryEmbedding.parse(kernel.rotary_embedding)
        self.freqs = build_freqs(latent, kernel.rope_theta, self.rotary_embedding, device=self.device)  # [1,1,1,N]
        self.use_alibi = self.rotary_embedding == RotaryEmbedding.ALIBI
        slopes = kernel.alibi_slopes if (self.use_alibi and kernel.alibi_slopes is not None) else None
        if self.use_alibi and slopes is None:
            slopes = default_alibi_slopes(n_head)
        # zeros when ALiBi is off, as the reference stores them (:128-130)
        self.alibi_slopes = torch.tensor(slopes if slopes is not None else [0.0] * n_head, dtype=torch.float32)
        self.fused = bool(kernel.enabled)
        self.block_pattern = kernel.block_sparse.time

    def forward(self, query: torch.Tensor, value: torch.Tensor, ctx: Optional[ffi.Context] = None) -> torch.Tensor:
        """src/model/attention.rs:142-175: query [B,h,T,N], value [B,1,T,dv] -> [B,h,T,dv].  The fused
        branch is fused_state_aligned with the model's time-block pattern; the plain branch masks with
        tril(-1) element-wise, which is the same computation with blocks of one token."""
        layout = self.block_pattern if self.fused else BlockPattern2d.dense(1)
        return fused_state_aligned(query, value, self.freqs, self.alibi_slopes if self.use_alibi else None, layout,
                                   self.rotary_embedding, True, ctx)

    def rotate_positions(self, values: torch.Tensor, start: int, positions: Optional[torch.Tensor] = None,
                         ctx: Optional[ffi.Context] = None) -> torch.Tensor:
        """src/model/attention.rs:177-179,332-349: values [B,h,T,N] at positions start..start+T (or
        positions[b] + t, device int32 [B]) -> [B,h,T,N] (PoPE: [B,h,T,2N]; ALiBi: a copy)."""
        ctx = ctx or ffi.default_context(values.device.index or 0)
        values = values.contiguous().float()
        B, h, T, N = values.shape
        Nq = 2 * N if self.rotary_embedding == RotaryEmbedding.POPE else N
        out = torch.empty((B, h, T, Nq), device=values.device, dtype=torch.float32)
        freqs = self.freqs.reshape(-1).to(values.device)
        ctx.check(ctx.lib.bdh_rotate(ctx.handle, B, h, T, N, int(self.rotary_embedding), ffi.ptr(values), ffi.ptr(freqs),
                                     int(start), ffi.ptr(positions), ffi.ptr(out)))
        return out

    def alibi_decay(self) -> Optional[np.ndarray]:
        """src/model/attention.rs:181-186: exp(-slopes), or None without ALiBi."""
        if not self.use_alibi:
            return None
        return np.exp(-self.alibi_slopes.numpy().astype(np.float32)).astype(np.float32)
