"""The recurrent state step through the C ABI (reference: BDH::recurrent_attention,
src/model/bdh.rs:258-307, including the rotate at :265)."""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from . import ffi
from .positional import RotaryEmbedding


def recurrent_attention(query: torch.Tensor, value: torch.Tensor, rho: torch.Tensor, freqs: torch.Tensor,
                        position: int, rotary_embedding: RotaryEmbedding = RotaryEmbedding.ROPE,
                        alibi_slopes=None, positions: Optional[torch.Tensor] = None, want_bitmask: bool = False,
                        want_rows: bool = False, ctx: Optional[ffi.Context] = None):
    """query [B,h,T,N] (un-rotated), value [B,1,T,d] or [B,T,d], rho [B,h,Nq,d] (updated in
    place, f32 or bf16).  Returns out [B,h,T,d] (+ bitmask [B,h,T,ceil(N/64)] int64 view of the
    uint64 words, + rows_touched [B,h,T] int32 when asked)."""
    ctx = ctx or ffi.default_context(query.device.index or 0)
    B, h, T, N = query.shape
    d = value.shape[-1]
    rot = RotaryEmbedding.parse(rotary_embedding)
    Nq = 2 * N if rot == RotaryEmbedding.POPE else N
    assert query.dtype == torch.float32 and query.is_contiguous()
    value = value.reshape(B, T, d)
    assert value.dtype == torch.float32 and value.is_contiguous()
    assert rho.is_contiguous() and tuple(rho.shape) == (B, h, Nq, d), "rho must be [B,h,Nq,d]"
    dt = {torch.float32: ffi.F32, torch.bfloat16: ffi.BF16}[rho.dtype]
    freqs = freqs.reshape(-1)
    out = torch.empty((B, h, T, d), device=query.device, dtype=torch.float32)
    bm = torch.zeros((B, h, T, (N + 63) // 64), device=query.device, dtype=torch.int64) if want_bitmask else None
    rows = torch.zeros((B, h, T), device=query.device, dtype=torch.int32) if want_rows else None
    slopes = None if alibi_slopes is None else np.ascontiguousarray(alibi_slopes, np.float32)
    ctx.check(ctx.lib.bdh_recurrent_attention(ctx.handle, B, h, T, N, d, int(rot), ffi.ptr(query), ffi.ptr(value),
                                              ffi.ptr(freqs), int(position), ffi.ptr(positions), ffi.ptr(slopes),
                                              ffi.ptr(rho), dt, ffi.ptr(out), ffi.ptr(bm), ffi.ptr(rows)))
    res = [out]
    if want_bitmask:
        res.append(bm)
    if want_rows:
        res.append(rows)
    return res[0] if len(res) == 1 else tuple(res)


def recurrent_attention_lazy_alibi(query: torch.Tensor, value: torch.Tensor, rho: torch.Tensor,
                                   stamps: torch.Tensor, clock: int, alibi_slopes=None,
                                   clocks: Optional[torch.Tensor] = None, want_bitmask: bool = False,
                                   want_rows: bool = False, ctx: Optional[ffi.Context] = None):
    """BDH::recurrent_attention for ALiBi (src/model/bdh.rs:258-307 with the decay of :299-301) on a
    state kept lazily decayed: rho [B,h,N,d] and stamps [B,h,N] int32 are updated in place, only the
    rows with a non-zero activation are touched.  `clock` = tokens absorbed before this call."""
    ctx = ctx or ffi.default_context(query.device.index or 0)
    B, h, T, N = query.shape
    d = value.shape[-1]
    assert query.dtype == torch.float32 and query.is_contiguous()
    value = value.reshape(B, T, d)
    assert value.dtype == torch.float32 and value.is_contiguous()
    assert rho.is_contiguous() and tuple(rho.shape) == (B, h, N, d), "rho must be [B,h,N,d]"
    assert stamps.dtype == torch.int32 and stamps.is_contiguous() and tuple(stamps.shape) == (B, h, N)
    dt = {torch.float32: ffi.F32, torch.bfloat16: ffi.BF16}[rho.dtype]
    out = torch.empty((B, h, T, d), device=query.device, dtype=torch.float32)
    bm = torch.zeros((B, h, T, (N + 63) // 64), device=query.device, dtype=torch.int64) if want_bitmask else None
    rows = torch.zeros((B, h, T), device=query.device, dtype=torch.int32) if want_rows else None
    slopes = None if alibi_slopes is None else np.ascontiguousarray(alibi_slopes, np.float32)
    ctx.check(ctx.lib.bdh_recurrent_attention_lazy_alibi(ctx.handle, B, h, T, N, d, ffi.ptr(query), ffi.ptr(value),
                                                         int(clock), ffi.ptr(clocks), ffi.ptr(slopes), ffi.ptr(rho), dt,
                                                         ffi.ptr(stamps), ffi.ptr(out), ffi.ptr(bm), ffi.ptr(rows)))
    res = [out]
    if want_bitmask:
        res.append(bm)
    if want_rows:
        res.append(rows)
    return res[0] if len(res) == 1 else tuple(res)


def alibi_materialize(rho: torch.Tensor, stamps: torch.Tensor, clock: int, alibi_slopes=None,
                      clocks: Optional[torch.Tensor] = None, ctx: Optional[ffi.Context] = None) -> None:
    """Brings a lazily decayed ALiBi state up to date in place (rho [..., B,h,N,d] with stamps [..., B,h,N];
    leading dimensions, e.g. layers, are folded into the batch): afterwards rho is what the reference holds."""
    ctx = ctx or ffi.default_context(rho.device.index or 0)
    assert rho.is_contiguous() and stamps.is_contiguous() and stamps.dtype == torch.int32
    h, N, d = rho.shape[-3:]
    B = rho.numel() // (h * N * d) if rho.numel() else 0
    assert stamps.numel() == B * h * N
    assert clocks is None or B == rho.shape[-4], "per-sequence clocks need a plain [B,h,N,d] state"
    dt = {torch.float32: ffi.F32, torch.bfloat16: ffi.BF16}[rho.dtype]
    slopes = None if alibi_slopes is None else np.ascontiguousarray(alibi_slopes, np.float32)
    ctx.check(ctx.lib.bdh_alibi_materialize(ctx.handle, B, h, N, d, int(clock), ffi.ptr(clocks), ffi.ptr(slopes),
                                            ffi.ptr(rho), dt, ffi.ptr(stamps)))


def rho_energy(rho: torch.Tensor, stamps: Optional[torch.Tensor] = None, clock: int = 0, alibi_slopes=None,
               clocks: Optional[torch.Tensor] = None, ctx: Optional[ffi.Context] = None) -> torch.Tensor:
    """The energy map of a state, `rho_last` of LayerVizState (src/model/bdh.rs:411-419): rho [B,h,N,d]
    -> [h,N], the batch mean of each row's mean |rho|.  With stamps [B,h,N] a lazily decayed ALiBi state is
    read through its pending decay at `clock` (or the per-sequence device `clocks`)."""
    ctx = ctx or ffi.default_context(rho.device.index or 0)
    assert rho.dim() == 4 and rho.is_contiguous()
    B, h, N, d = rho.shape
    assert stamps is None or (stamps.is_contiguous() and stamps.dtype == torch.int32 and stamps.numel() == B * h * N)
    dt = {torch.float32: ffi.F32, torch.bfloat16: ffi.BF16}[rho.dtype]
    slopes = None if alibi_slopes is None else np.ascontiguousarray(alibi_slopes, np.float32)
    out = torch.empty((h, N), device=rho.device, dtype=torch.float32)
    ctx.check(ctx.lib.bdh_rho_energy(ctx.handle, B, h, N, d, ffi.ptr(rho), dt, ffi.ptr(stamps), int(clock),
                                     ffi.ptr(clocks), ffi.ptr(slopes), ffi.ptr(out)))
    return out


def layer_norm(x: torch.Tensor, ctx: Optional[ffi.Context] = None) -> torch.Tensor:
    """BDH::layer_norm (src/model/bdh.rs:86-89)."""
    ctx = ctx or ffi.default_context(x.device.index or 0)
    x = x.contiguous().float()
    out = torch.empty_like(x)
    d = x.shape[-1]
    ctx.check(ctx.lib.bdh_layer_norm(ctx.handle, x.numel() // max(d, 1), d, ffi.ptr(x), ffi.ptr(out)))
    return out


def prefill_chunked(x_bf16: torch.Tensor, v_bf16: torch.Tensor, rho: torch.Tensor, freqs: torch.Tensor,
                    position: int, state_is_zero: bool = False, chunk: int = 0, hilo: bool = False,
                    all_scores: bool = False, ctx: Optional[ffi.Context] = None) -> torch.Tensor:
    """The recurrent path (src/model/bdh.rs:258-307, RoPE) for T tokens at once on the bf16 matrix
    cores.  x_bf16 [B,h,T,N] bfloat16 un-rotated, v_bf16 [B,T,d] bfloat16, rho [B,h,N,d] float32
    (updated in place).  chunk = tokens per internal pass (0 = 2048; the workspace grows with it, not
    with T); hilo = the state carried into the call enters its product as a bf16 pair; all_scores = never the
    chunk-recurrent form.  Returns out [B,h,T,d] float32."""
    ctx = ctx or ffi.default_context(x_bf16.device.index or 0)
    B, h, T, N = x_bf16.shape
    d = v_bf16.shape[-1]
    assert x_bf16.dtype == torch.bfloat16 and x_bf16.is_contiguous()
    v_bf16 = v_bf16.reshape(B, T, d)
    assert v_bf16.dtype == torch.bfloat16 and v_bf16.is_contiguous()
    assert rho.dtype == torch.float32 and rho.is_contiguous() and tuple(rho.shape) == (B, h, N, d)
    out = torch.empty((B, h, T, d), device=x_bf16.device, dtype=torch.float32)
    freqs = freqs.reshape(-1)
    flags = ((ffi.PREFILL_STATE_IS_ZERO if state_is_zero else 0) | (ffi.PREFILL_STATE_HILO if hilo else 0) |
             (ffi.PREFILL_ALL_SCORES if all_scores else 0))
    ctx.check(ctx.lib.bdh_prefill_chunked(ctx.handle, B, h, T, N, d, ffi.ptr(x_bf16), ffi.ptr(v_bf16),
                                          ffi.ptr(freqs), int(position), int(chunk), flags, ffi.ptr(rho),
                                          ffi.ptr(out)))
    return out


def prefill_chunked_ex(x_bf16: torch.Tensor, v_bf16: torch.Tensor, rho: Optional[torch.Tensor], freqs: torch.Tensor,
                       position: int, rotary: RotaryEmbedding = RotaryEmbedding.ROPE,
                       alibi_slopes=None, row_normalize: bool = False,
                       block_size: int = 1, state_is_zero: bool = False, chunk: int = 0, hilo: bool = False,
                       all_scores: bool = False, ctx: Optional[ffi.Context] = None) -> torch.Tensor:
    """prefill_chunked for all three positional schemes (PoPE: rho [B,h,2N,d]; ALiBi: the state decays by
    exp(-slope) per token, src/model/bdh.rs:299-301), and with row_normalize the bf16 matrix-core form of
    kernel::linear_attention::fused_state_aligned (src/kernel/linear_attention.rs:11-115, dense causal layout with
    time blocks of block_size; stateless: rho is not used and may be None; the additive ALiBi term whenever
    alibi_slopes is given).  Returns out [B,h,T,d] float32."""
    ctx = ctx or ffi.default_context(x_bf16.device.index or 0)
    B, h, T, N = x_bf16.shape
    d = v_bf16.shape[-1]
    rotary = RotaryEmbedding(rotary)
    nq = 2 * N if rotary == RotaryEmbedding.POPE else N
    assert x_bf16.dtype == torch.bfloat16 and x_bf16.is_contiguous()
    v_bf16 = v_bf16.reshape(B, T, d)
    assert v_bf16.dtype == torch.bfloat16 and v_bf16.is_contiguous()
    if rho is not None:
        assert rho.dtype == torch.float32 and rho.is_contiguous() and tuple(rho.shape) == (B, h, nq, d)
    out = torch.empty((B, h, T, d), device=x_bf16.device, dtype=torch.float32)
    freqs_ptr = ffi.ptr(freqs.reshape(-1)) if freqs is not None else None
    slopes = None if alibi_slopes is None else np.ascontiguousarray(alibi_slopes, np.float32)
    flags = ((ffi.PREFILL_STATE_IS_ZERO if state_is_zero else 0) | (ffi.PREFILL_STATE_HILO if hilo else 0) |
             (ffi.PREFILL_ALL_SCORES if all_scores else 0) | (ffi.PREFILL_ROW_NORMALIZE if row_normalize else 0))
    ctx.check(ctx.lib.bdh_prefill_chunked_ex(ctx.handle, B, h, T, N, d, int(rotary), ffi.ptr(x_bf16), ffi.ptr(v_bf16),
                                             freqs_ptr, ffi.ptr(slopes), int(position), int(chunk), flags, int(block_size),
                                             ffi.ptr(rho) if rho is not None else None, ffi.ptr(out)))
    return out


class StateLog:
    """The pending rank-1 updates of ONE state tensor rho [B,h,N,d] (bdh_state_log): the deferred decode step
    reads its active state rows and logs its update; `flush` (called by the step itself when `capacity` steps are
    pending) applies the logged updates in step order, after which rho holds the bits the eager step leaves.
    Flush before anything else reads or writes rho."""

    def __init__(self, B: int, h: int, N: int, d: int, rho_dtype: torch.dtype = torch.float32, capacity: int = 32,
                 ctx: Optional[ffi.Context] = None, device_id: int = 0):
        import ctypes

        self.ctx = ctx or ffi.default_context(device_id)
        self.shape = (B, h, N, d)
        self.rho_dtype = rho_dtype
        self.capacity = capacity
        dt = {torch.float32: ffi.F32, torch.bfloat16: ffi.BF16}[rho_dtype]
        handle = ctypes.c_void_p()
        self.ctx.check(self.ctx.lib.bdh_state_log_create(self.ctx.handle, B, h, N, d, dt, capacity, ctypes.byref(handle)))
        self.handle = handle

    @property
    def pending(self) -> int:
        return int(self.ctx.lib.bdh_state_log_pending(self.handle))

    @property
    def nbytes(self) -> int:
        return int(self.ctx.lib.bdh_state_log_bytes(self.handle))

    def flush(self, rho: torch.Tensor) -> None:
        self.ctx.check(self.ctx.lib.bdh_state_flush(self.ctx.handle, self.handle, ffi.ptr(rho)))

    def close(self) -> None:
        import sys

        if getattr(self, "handle", None) and getattr(self.ctx, "handle", None):
            if not sys.is_finalizing():
                self.ctx.lib.bdh_state_log_destroy(self.ctx.handle, self.handle)
        self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def state_step_deferred(log: StateLog, query: torch.Tensor, value: torch.Tensor, rho: torch.Tensor,
                        freqs: torch.Tensor, position: int, positions: Optional[torch.Tensor] = None,
                        want_bitmask: bool = False, want_rows: bool = False):
    """BDH::recurrent_attention at T = 1 (src/model/bdh.rs:258-307, RoPE) with the update of :298 logged in `log`
    instead of written to rho.  query [B,h,N] or [B,h,1,N] un-rotated, value [B,d]; returns out [B,h,d]
    (+ bitmask [B,h,ceil(N/64)] int64 view, + rows_touched [B,h] int32 when asked)."""
    ctx = log.ctx
    B, h, N, d = log.shape
    query = query.reshape(B, h, N)
    value = value.reshape(B, d)
    assert query.dtype == torch.float32 and query.is_contiguous()
    assert value.dtype == torch.float32 and value.is_contiguous()
    assert rho.is_contiguous() and tuple(rho.shape) == (B, h, N, d) and rho.dtype == log.rho_dtype
    freqs = freqs.reshape(-1)
    out = torch.empty((B, h, d), device=query.device, dtype=torch.float32)
    bm = torch.zeros((B, h, (N + 63) // 64), device=query.device, dtype=torch.int64) if want_bitmask else None
    rows = torch.zeros((B, h), device=query.device, dtype=torch.int32) if want_rows else None
    ctx.check(ctx.lib.bdh_state_step_deferred(ctx.handle, log.handle, ffi.ptr(query), ffi.ptr(value), ffi.ptr(freqs),
                                              int(position), ffi.ptr(positions), ffi.ptr(rho), ffi.ptr(out), ffi.ptr(bm),
                                              ffi.ptr(rows)))
    res = [out]
    if want_bitmask:
        res.append(bm)
    if want_rows:
        res.append(rows)
    return res[0] if len(res) == 1 else tuple(res)
