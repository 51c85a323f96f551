"""BDH (reference: src/model/bdh.rs) — inference surface over the HIP library.

Parameters are torch tensors on the GPU in the reference's record order and shapes
(embed [V,d], encoder [h,d,N], encoder_v [h,d,N], decoder [h*N,d], lm_head [d,V]);
forward_with_state is one call of bdh_model_forward.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import numpy as np
import torch

from .. import ffi
from ..positional import RotaryEmbedding
from .config import BDHConfig
from .state import LayerState, ModelState

UINT63_MAX = (1 << 63) - 1


class BDH:
    def __init__(self, config: BDHConfig, device="cuda:0", seed: Optional[int] = None, weights: Optional[dict] = None,
                 rho_dtype: int = ffi.F32):
        """BDH::new (src/model/bdh.rs:37-84).  `weights` (numpy/torch, the reference's shapes) or a
        seed for Normal(0, 0.02) projections and a Normal(0, 1) embedding."""
        self.config = config
        self.device = torch.device(device)
        self.n_layer, self.n_embd, self.n_head = config.n_layer, config.n_embd, config.n_head
        self.vocab_size = config.vocab_size
        self.latent = config.latent_per_head()
        self.kernel = config.fused_kernels
        self.rho_dtype = rho_dtype
        h, d, N, V = self.n_head, self.n_embd, self.latent, self.vocab_size
        shapes = {"embed": (V, d), "encoder": (h, d, N), "encoder_v": (h, d, N), "decoder": (h * N, d),
                  "lm_head": (d, V)}
        if weights is None:
            rng = np.random.default_rng(0 if seed is None else seed)
            weights = {"embed": rng.standard_normal(shapes["embed"]).astype(np.float32)}
            for name in ("encoder", "encoder_v", "decoder", "lm_head"):
                weights[name] = (0.02 * rng.standard_normal(shapes[name])).astype(np.float32)
        self.params = {}
        for name, shape in shapes.items():
            t = torch.as_tensor(np.asarray(weights[name]) if not torch.is_tensor(weights[name]) else weights[name])
            if tuple(t.shape) != shape:
                raise ValueError(f"{name}: expected shape {shape}, got {tuple(t.shape)}")
            self.params[name] = t.to(self.device, torch.float32).contiguous()
        self.ctx = ffi.default_context(self.device.index or 0)
        rot = RotaryEmbedding.parse(self.kernel.rotary_embedding)
        slopes = None
        if rot == RotaryEmbedding.ALIBI and self.kernel.alibi_slopes is not None:
            slopes = np.ascontiguousarray(self.kernel.alibi_slopes, np.float32)
            assert slopes.size == h
        cfg = ffi.ModelConfigC(self.n_layer, d, h, N, V, int(rot), float(self.kernel.rope_theta),
                               float(self.kernel.relu_threshold), None if slopes is None else slopes.ctypes.data)
        wts = ffi.ModelWeightsC(*[self.params[n].data_ptr() for n in ("embed", "encoder", "encoder_v", "decoder",
                                                                     "lm_head")])
        handle = ctypes.c_void_p()
        self.ctx.check(self.ctx.lib.bdh_model_create(self.ctx.handle, ctypes.byref(cfg), ctypes.byref(wts),
                                                     ctypes.byref(handle)))
        self.handle = handle
        self.latent_q = 2 * N if rot == RotaryEmbedding.POPE else N

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                self.ctx.lib.bdh_model_destroy(self.handle)
                self.handle = None
        except Exception:
            pass

    def init_state(self) -> ModelState:
        """src/model/bdh.rs:254-256."""
        return ModelState.new(self.n_layer)

    def _ensure_state(self, state: ModelState, batch: int) -> torch.Tensor:
        """Zero state on first use or on a shape change (src/model/bdh.rs:274-284)."""
        shape = (self.n_layer, batch, self.n_head, self.latent_q, self.n_embd)
        dt = torch.float32 if self.rho_dtype == ffi.F32 else torch.bfloat16
        if state.storage is None or tuple(state.storage.shape) != shape or state.storage.dtype != dt:
            state.storage = torch.zeros(shape, device=self.device, dtype=dt)
            for i, layer in enumerate(state.layers):
                layer.rho = state.storage[i]
        return state.storage

    def forward_with_state(self, tokens: torch.Tensor, state: ModelState, want_next: bool = False,
                           x_tap: Optional[torch.Tensor] = None):
        """src/model/bdh.rs:309-450.  tokens [B,T] int64 -> logits [B,T,V] (and the greedy next
        token per sequence, kept on the device, when want_next)."""
        assert len(state.layers) == self.n_layer, "model state layers mismatch"  # :314-318
        tokens = tokens.to(self.device, torch.int64).contiguous()
        B, T = tokens.shape
        rho = self._ensure_state(state, B)
        logits = torch.empty((B, T, self.vocab_size), device=self.device, dtype=torch.float32)
        nxt = torch.empty((B,), device=self.device, dtype=torch.int64) if want_next else None
        self.ctx.check(self.ctx.lib.bdh_model_forward(self.handle, tokens.data_ptr(), B, T, rho.data_ptr(),
                                                      self.rho_dtype, state.position, logits.data_ptr(),
                                                      ffi.ptr(nxt), ffi.ptr(x_tap)))
        state.position = min(state.position + T, UINT63_MAX)  # saturating_add, :445
        return (logits, nxt) if want_next else logits

    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        """src/model/bdh.rs:91-94."""
        return self.forward_with_state(tokens, self.init_state())

    def generate(self, indices: torch.Tensor, max_new_tokens: int) -> torch.Tensor:
        """Greedy form (top_k = 1) of src/model/bdh.rs:170-252; the argmax stays on the device."""
        assert indices.shape[0] == 1, "generation currently supports batch size 1"  # :178
        state = self.init_state()
        indices = indices.to(self.device, torch.int64)
        _, nxt = self.forward_with_state(indices, state, want_next=True)
        out = [indices]
        for _ in range(max_new_tokens):
            tok = nxt.reshape(1, 1)
            out.append(tok)
            _, nxt = self.forward_with_state(tok, state, want_next=True)
        return torch.cat(out, dim=1)
