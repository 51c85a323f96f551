"""BDH (reference: src/model/bdh.rs) — inference surface over the HIP library.

Parameters are torch tensors on the GPU in the reference's record order and shapes
(embed [V,d], encoder [h,d,N], encoder_v [h,d,N], decoder [h*N,d], lm_head [d,V]);
forward_with_state is one call of bdh_model_forward.
"""
from __future__ import annotations

import ctypes
import sys
from typing import Optional

import numpy as np
import torch

from .. import ffi
from ..positional import RotaryEmbedding
from .config import BDHConfig
from .state import LayerState, LayerVizState, ModelState

UINT63_MAX = (1 << 63) - 1


class BDH:
    def __init__(self, config: BDHConfig, device="cuda:0", seed: Optional[int] = None, weights: Optional[dict] = None,
                 rho_dtype: int = ffi.F32, alibi_lazy: bool = False, defer_updates: int = 0):
        """BDH::new (src/model/bdh.rs:37-84).  `weights` (numpy/torch, the reference's shapes) or a
        seed for Normal(0, 0.02) projections and a Normal(0, 1) embedding.  alibi_lazy (ALiBi models
        only): keep the state lazily decayed, so a step touches only the rows of the active neurons
        instead of multiplying the whole state by exp(-slope) (src/model/bdh.rs:299-301);
        materialize_state() turns it back into the reference's state.  defer_updates = K > 0 (RoPE models with
        n_embd in {256, 512}): single-token calls log their state updates (src/model/bdh.rs:298) instead of
        writing them and the state is rewritten once per K tokens; any other call, and materialize_state(),
        applies what is pending first, after which the state holds the bits of the eager steps."""
        self.config = config
        self.defer_updates = int(defer_updates)
        self.alibi_lazy = bool(alibi_lazy)
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
        if self.alibi_lazy and rot != RotaryEmbedding.ALIBI:
            raise ValueError("alibi_lazy needs rotary_embedding = alibi")
        self._slopes = slopes
        if self.defer_updates and (rot != RotaryEmbedding.ROPE or d not in (256, 512)):
            raise ValueError("defer_updates needs a RoPE model with n_embd in {256, 512}")

    @classmethod
    def from_checkpoint_dir(cls, directory: str, device="cuda:0", rho_dtype: int = ffi.F32, alibi_lazy: bool = False):
        """A trained model from a directory holding the reference's model.bin (Burn BinFileRecorder
        record), config.json and optionally vocab.json — the loading steps of src/bin/infer.rs:170-186.
        Returns (model, tokenizer or None, block_size)."""
        from ..record import load_checkpoint_dir
        from ..tokenizer import CharVocab

        config, weights, vocab_json, block_size = load_checkpoint_dir(directory)
        tokenizer = CharVocab.from_json_str(vocab_json) if vocab_json is not None else None
        model = cls(config, device, weights=weights, rho_dtype=rho_dtype, alibi_lazy=alibi_lazy)
        return model, tokenizer, block_size

    def __del__(self):
        try:
            # at interpreter exit the HIP runtime may already be gone: the process is about to release everything
            if getattr(self, "handle", None) and not sys.is_finalizing():
                self.ctx._lib.bdh_model_destroy(self.handle)  # not .lib: no stream lookup while tearing down
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
            state.stamps = None
            state.logs = None  # updates logged against the old storage go with it
        if self.alibi_lazy and state.stamps is None:
            # a state that arrives without stamps is up to date as of its position
            state.stamps = torch.full(shape[:-1], min(state.position, 0x7FFFFFFF), device=self.device,
                                      dtype=torch.int32)
        return state.storage

    def flush_state(self, state: ModelState) -> None:
        """Applies the logged updates of a model built with defer_updates: afterwards state.storage holds what
        the eager steps would have left.  No-op when nothing is pending."""
        logs = getattr(state, "logs", None)
        if logs is not None and state.storage is not None and logs.pending:
            self.ctx.check(self.ctx.lib.bdh_model_flush(self.handle, logs.handle, state.storage.data_ptr()))

    def materialize_state(self, state: ModelState) -> None:
        """Applies the pending decay of a lazily decayed ALiBi state, or the logged updates of a deferred one:
        afterwards state.storage is the state the reference holds after state.position tokens.  No-op for an
        eager state."""
        self.flush_state(state)
        if state.storage is None or state.stamps is None:
            return
        from ..recurrent import alibi_materialize

        # layers are folded into the batch: the head index, which selects the slope, is unaffected
        alibi_materialize(state.storage, state.stamps, state.position, self._slopes, None, self.ctx)

    def forward_with_state(self, tokens: torch.Tensor, state: ModelState, want_next: bool = False,
                           x_tap: Optional[torch.Tensor] = None, viz: bool = False):
        """src/model/bdh.rs:309-450.  tokens [B,T] int64 -> logits [B,T,V] (and the greedy next
        token per sequence, kept on the device, when want_next).  viz=True also fills every
        layer's LayerVizState as the reference does when built with its "viz" feature (:386-434)."""
        assert len(state.layers) == self.n_layer, "model state layers mismatch"  # :314-318
        tokens = tokens.to(self.device, torch.int64).contiguous()
        B, T = tokens.shape
        rho = self._ensure_state(state, B)
        logits = torch.empty((B, T, self.vocab_size), device=self.device, dtype=torch.float32)
        nxt = torch.empty((B,), device=self.device, dtype=torch.int64) if want_next else None
        if self.defer_updates and T == 1 and x_tap is None and not viz:
            if state.logs is None or state.logs.batch != B:
                state.logs = ModelLogs(self, B, self.defer_updates)
            self.ctx.check(self.ctx.lib.bdh_model_forward_deferred(self.handle, state.logs.handle, tokens.data_ptr(), B,
                                                                   rho.data_ptr(), self.rho_dtype, state.position, None,
                                                                   logits.data_ptr(), ffi.ptr(nxt)))
            state.position = min(state.position + T, UINT63_MAX)
            return (logits, nxt) if want_next else logits
        self.flush_state(state)  # a call that writes the state itself: the logged updates go first
        maps = None
        if viz and T > 0:
            maps = torch.empty((self.n_layer, 4, self.n_head, self.latent), device=self.device, dtype=torch.float32)
        self.ctx.check(self.ctx.lib.bdh_model_forward_viz(self.handle, tokens.data_ptr(), B, T, rho.data_ptr(),
                                                          self.rho_dtype, ffi.ptr(state.stamps), state.position,
                                                          None, logits.data_ptr(), ffi.ptr(nxt), ffi.ptr(x_tap),
                                                          ffi.ptr(maps)))
        if maps is not None:
            for layer, m in zip(state.layers, maps):
                layer.viz = LayerVizState(x_last=m[0], y_last=m[1], xy_last=m[2], rho_last=m[3])
        state.position = min(state.position + T, UINT63_MAX)  # saturating_add, :445
        return (logits, nxt) if want_next else logits

    def capture_decode_step(self, state: ModelState, tokens: torch.Tensor) -> "DecodeGraph":
        """Captures ONE greedy decode step (forward_with_state on the last sampled token, argmax kept on
        the device, position advanced on the device) in a HIP graph.  Every replay is one token for
        every sequence of the batch; nothing crosses to the host between tokens (the reference syncs
        and copies the logits every token, src/generation.rs:114-124)."""
        return DecodeGraph(self, state, tokens)

    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        """src/model/bdh.rs:91-94."""
        return self.forward_with_state(tokens, self.init_state())

    def forward_fast(self, tokens: torch.Tensor) -> torch.Tensor:
        """src/model/bdh.rs:96-168: the stateless forward over all tokens at once (the form the reference
        trains with): Attention::forward in place of the recurrent state.  tokens [B,T] -> logits [B,T,V]."""
        tokens = tokens.to(self.device, torch.int64).contiguous()
        B, T = tokens.shape
        logits = torch.empty((B, T, self.vocab_size), device=self.device, dtype=torch.float32)
        sparse = self.kernel.block_sparse
        if not self.kernel.enabled:  # plain branch: the patterns are not consulted (src/model/bdh.rs:114-151)
            self.ctx.check(self.ctx.lib.bdh_model_forward_fast(self.handle, tokens.data_ptr(), B, T, 0, logits.data_ptr()))
            return logits
        block = max(sparse.time.block_size, 1)
        pairs, n_pairs = None, 0
        if sparse.time.is_sparse():
            flat = np.array(sorted(sparse.time.active_pairs), dtype=np.int32).reshape(-1, 2)
            pairs, n_pairs = np.ascontiguousarray(flat), flat.shape[0]
            if n_pairs == 0:
                pairs = np.zeros((1, 2), np.int32)  # a valid pointer: an empty pattern is still a sparse one
        blocks = sparse.latent.block_bytes(self.latent) if sparse.latent.is_sparse() else None
        self.ctx.check(self.ctx.lib.bdh_model_forward_fast_ex(
            self.handle, tokens.data_ptr(), B, T, block, ffi.ptr(pairs), n_pairs, max(sparse.latent.block_size, 1),
            blocks, 0 if blocks is None else len(blocks), logits.data_ptr()))
        return logits

    def generate(self, indices: torch.Tensor, max_new_tokens: int, temperature: float = 1.0,
                 top_k: Optional[int] = 1, generator: Optional[torch.Generator] = None) -> torch.Tensor:
        """src/model/bdh.rs:170-252: prompt through forward_with_state, then max_new_tokens draws from
        softmax(logits / temperature) restricted to the top_k values (None or 0 = all).  The draw runs on the
        device (bdh_sample_top_k) with uniform variates from `generator` standing for the reference's
        thread_rng; top_k = 1 is greedy decoding and takes the argmax the lm_head kernel already wrote."""
        assert indices.shape[0] == 1, "generation currently supports batch size 1"  # :178
        state = self.init_state()
        indices = indices.to(self.device, torch.int64)
        greedy = top_k == 1
        logits, nxt = self.forward_with_state(indices, state, want_next=True)
        out = [indices]
        if not greedy:  # the variates come a block at a time: no host work per token
            from ..generation import VariateStream, sample_from_logits

            variates = VariateStream(self.device, generator)
        for _ in range(max_new_tokens):
            if not greedy:
                nxt = sample_from_logits(self, logits[:, -1], temperature, top_k, variates.next())
            tok = nxt.reshape(1, 1)
            out.append(tok)
            logits, nxt = self.forward_with_state(tok, state, want_next=True)
        return torch.cat(out, dim=1)


class ModelLogs:
    """bdh_model_logs: the update logs of a model's layers for a batch of `batch` sequences."""

    def __init__(self, model: BDH, batch: int, capacity: int):
        self.model, self.batch, self.capacity = model, batch, capacity
        handle = ctypes.c_void_p()
        model.ctx.check(model.ctx.lib.bdh_model_logs_create(model.handle, batch, model.rho_dtype, capacity,
                                                            ctypes.byref(handle)))
        self.handle = handle

    @property
    def pending(self) -> int:
        return int(self.model.ctx._lib.bdh_model_logs_pending(self.handle))

    def __del__(self):
        try:
            if getattr(self, "handle", None) and getattr(self.model, "handle", None) and not sys.is_finalizing():
                self.model.ctx._lib.bdh_model_logs_destroy(self.model.handle, self.handle)
                self.handle = None
        except Exception:
            pass


class DecodeGraph:
    """One captured decode step.  `tokens` [B] int64 are the tokens to feed first (e.g. the argmax of the
    prefill); after each replay() the buffer holds the newly generated tokens and `logits` [B,1,V] the
    logits they were taken from.  The state must already hold its rho tensors (run the prefill first)."""

    def __init__(self, model: BDH, state: ModelState, tokens: torch.Tensor):
        assert state.storage is not None, "run the prefill before capturing the decode step"
        model.flush_state(state)  # the captured step writes the state itself (the pending count of a log lives on the host)
        self.model, self.state = model, state
        B = state.storage.shape[1]
        dev = model.device
        self.tokens = tokens.to(dev, torch.int64).reshape(B).clone()
        self.positions = torch.full((B,), state.position, device=dev, dtype=torch.int32)
        self.logits = torch.empty((B, 1, model.vocab_size), device=dev, dtype=torch.float32)
        ctx, lib = model.ctx, model.ctx.lib

        def step():
            ctx.check(lib.bdh_model_forward_lazy(model.handle, self.tokens.data_ptr(), B, 1,
                                                 state.storage.data_ptr(), model.rho_dtype, ffi.ptr(state.stamps), 0,
                                                 self.positions.data_ptr(), self.logits.data_ptr(),
                                                 self.tokens.data_ptr(), None))
            ctx.check(lib.bdh_advance_positions(ctx.handle, self.positions.data_ptr(), B, 1))

        # one eager step on a side stream sizes every scratch buffer (no allocation may happen under capture)
        keep = (self.tokens.clone(), self.positions.clone(), state.storage.clone(),
                None if state.stamps is None else state.stamps.clone())
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            ctx.set_stream(side.cuda_stream)
            step()
        side.synchronize()
        self.tokens.copy_(keep[0]); self.positions.copy_(keep[1]); state.storage.copy_(keep[2])
        if keep[3] is not None:
            state.stamps.copy_(keep[3])
        torch.cuda.synchronize(dev)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=side):
            ctx.set_stream(torch.cuda.current_stream(dev).cuda_stream)
            step()
        ctx.set_stream(torch.cuda.current_stream(dev).cuda_stream)

    def replay(self, n: int = 1) -> None:
        for _ in range(n):
            self.graph.replay()
        self.state.position = min(self.state.position + n, UINT63_MAX)
