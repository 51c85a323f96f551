"""ctypes binding of libbdh_mi355x.so (declared in include/bdh_mi355x.h).

PyTorch appears here only as the owner of device memory and of the HIP stream; every
computation is a call into the C ABI.  There is no fallback: if the library has not been
built, or no HIP device is present, loading or context creation raises.
"""
from __future__ import annotations

import ctypes
import os
import sys
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p
from typing import Optional

PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG, "libbdh_mi355x.so")

OK, E_INVAL, E_SHAPE, E_ALIGN, E_HIP, E_NOMEM, E_UNSUPPORTED = 0, -1, -2, -3, -4, -5, -6
ROPE, ALIBI, POPE = 0, 1, 2
F32, BF16 = 0, 1
PREFILL_STATE_IS_ZERO, PREFILL_STATE_HILO, PREFILL_ALL_SCORES, PREFILL_ROW_NORMALIZE = 1, 2, 4, 8

# every symbol include/bdh_mi355x.h declares
EXPORTS = [
    "bdh_version", "bdh_status_string", "bdh_ctx_create", "bdh_ctx_destroy", "bdh_ctx_set_stream",
    "bdh_ctx_synchronize", "bdh_last_error", "bdh_ctx_set_option", "bdh_build_freqs", "bdh_default_alibi_slopes",
    "bdh_recurrent_attention", "bdh_state_step", "bdh_relu_lowrank", "bdh_layer_norm",
    "bdh_fused_state_aligned", "bdh_prefill_chunked", "bdh_prefill_chunked_ex", "bdh_model_create", "bdh_model_destroy",
    "bdh_model_state_bytes", "bdh_model_forward", "bdh_model_forward_ex", "bdh_advance_positions",
    "bdh_sample_top_k", "bdh_recurrent_attention_lazy_alibi", "bdh_alibi_materialize", "bdh_model_forward_lazy",
    "bdh_rho_energy", "bdh_model_forward_viz", "bdh_rotate",
    "bdh_model_forward_fast", "bdh_model_forward_fast_ex", "bdh_state_step_noalloc", "bdh_probe_chunks",
    "bdh_state_log_create", "bdh_state_log_destroy", "bdh_state_log_pending", "bdh_state_log_bytes",
    "bdh_state_step_deferred", "bdh_state_flush", "bdh_model_forward_layers",
    "bdh_model_logs_create", "bdh_model_logs_destroy", "bdh_model_logs_pending", "bdh_model_forward_deferred",
    "bdh_model_flush", "bdh_model_forward_deferred_layers", "bdh_model_flush_layers",
]


class BdhError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"bdh status {status}: {message}")
        self.status = status


class ModelConfigC(ctypes.Structure):
    _fields_ = [
        ("n_layer", c_int32), ("n_embd", c_int32), ("n_head", c_int32), ("latent", c_int32),
        ("vocab", c_int32), ("rotary", c_int32), ("rope_theta", c_float), ("relu_threshold", c_float),
        ("alibi_slopes_host", c_void_p),
    ]


class ModelWeightsC(ctypes.Structure):
    _fields_ = [("embed", c_void_p), ("encoder", c_void_p), ("encoder_v", c_void_p), ("decoder", c_void_p),
                ("lm_head", c_void_p)]


_lib = None


def load_library(path: Optional[str] = None) -> ctypes.CDLL:
    """Loads the built library.  Import torch first so both share one HIP runtime."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    path = path or LIB_PATH
    if not os.path.exists(path):
        raise RuntimeError(
            f"{path} is missing: the HIP library is the only compute path. "
            "Build it with `python -m burn_dragon_amd.build`.")
    try:
        import torch  # noqa: F401  (loads torch's libamdhip64.so.7 so the SONAME resolves to it)
    except Exception:  # pragma: no cover - torch is optional for pure C callers
        pass
    lib = ctypes.CDLL(path)
    P = c_void_p
    lib.bdh_version.restype = c_char_p
    lib.bdh_status_string.restype = c_char_p
    lib.bdh_status_string.argtypes = [c_int]
    lib.bdh_ctx_create.argtypes = [c_int, P, POINTER(P)]
    lib.bdh_ctx_destroy.argtypes = [P]
    lib.bdh_ctx_set_stream.argtypes = [P, P]
    lib.bdh_ctx_synchronize.argtypes = [P]
    lib.bdh_last_error.restype = c_char_p
    lib.bdh_last_error.argtypes = [P]
    lib.bdh_ctx_set_option.argtypes = [P, c_char_p, c_int]
    lib.bdh_build_freqs.argtypes = [c_int, c_float, c_int, P]
    lib.bdh_default_alibi_slopes.argtypes = [c_int, P]
    lib.bdh_recurrent_attention.argtypes = [P, c_int, c_int, c_int, c_int, c_int, c_int, P, P, P, c_int64, P, P, P,
                                            c_int, P, P, P]
    lib.bdh_state_step.argtypes = [P, c_int, c_int, c_int, c_int, c_int, P, P, P, c_int64, P, P, P, c_int, P, P, P]
    lib.bdh_state_step_noalloc.argtypes = lib.bdh_state_step.argtypes
    lib.bdh_probe_chunks.argtypes = [P, P, c_size_t, P, c_int, c_int, c_int, c_int]
    lib.bdh_state_log_create.argtypes = [P, c_int, c_int, c_int, c_int, c_int, c_int, POINTER(P)]
    lib.bdh_state_log_destroy.argtypes = [P, P]
    lib.bdh_state_log_pending.argtypes = [P]
    lib.bdh_state_log_bytes.restype = c_size_t
    lib.bdh_state_log_bytes.argtypes = [P]
    lib.bdh_state_step_deferred.argtypes = [P, P, P, P, P, c_int64, P, P, P, P, P]
    lib.bdh_state_flush.argtypes = [P, P, P]
    lib.bdh_model_forward_layers.argtypes = [P, P, c_int, c_int, P, c_int, P, c_int64, P, P, P, P]
    lib.bdh_model_logs_create.argtypes = [P, c_int, c_int, c_int, POINTER(P)]
    lib.bdh_model_logs_destroy.argtypes = [P, P]
    lib.bdh_model_logs_pending.argtypes = [P]
    lib.bdh_model_forward_deferred.argtypes = [P, P, P, c_int, P, c_int, c_int64, P, P, P]
    lib.bdh_model_flush.argtypes = [P, P, P]
    lib.bdh_model_forward_deferred_layers.argtypes = [P, P, P, c_int, P, c_int, c_int64, P, P, P]
    lib.bdh_model_flush_layers.argtypes = [P, P, P]
    lib.bdh_relu_lowrank.argtypes = [P, c_int, c_int, c_int, c_int, c_int, c_int, P, P, P, c_float, c_int, P, c_int,
                                     P, P]
    lib.bdh_layer_norm.argtypes = [P, c_int64, c_int, P, P]
    lib.bdh_fused_state_aligned.argtypes = [P, c_int, c_int, c_int, c_int, c_int, P, P, P, P, c_int, P, c_int, c_int,
                                            c_int, P]
    lib.bdh_prefill_chunked.argtypes = [P, c_int, c_int, c_int, c_int, c_int, P, P, P, c_int64, c_int, c_int, P, P]
    lib.bdh_prefill_chunked_ex.argtypes = [P, c_int, c_int, c_int, c_int, c_int, c_int, P, P, P, P, c_int64, c_int,
                                           c_int, c_int, P, P]
    lib.bdh_model_create.argtypes = [P, POINTER(ModelConfigC), POINTER(ModelWeightsC), POINTER(P)]
    lib.bdh_model_destroy.argtypes = [P]
    lib.bdh_model_state_bytes.restype = c_size_t
    lib.bdh_model_state_bytes.argtypes = [P, c_int, c_int]
    lib.bdh_model_forward.argtypes = [P, P, c_int, c_int, P, c_int, c_int64, P, P, P]
    lib.bdh_model_forward_ex.argtypes = [P, P, c_int, c_int, P, c_int, c_int64, P, P, P, P]
    lib.bdh_advance_positions.argtypes = [P, P, c_int, c_int]
    lib.bdh_sample_top_k.argtypes = [P, c_int, c_int, P, c_int64, c_float, c_int, P, P]
    lib.bdh_recurrent_attention_lazy_alibi.argtypes = [P, c_int, c_int, c_int, c_int, c_int, P, P, c_int64, P, P, P,
                                                       c_int, P, P, P, P]
    lib.bdh_alibi_materialize.argtypes = [P, c_int, c_int, c_int, c_int, c_int64, P, P, P, c_int, P]
    lib.bdh_model_forward_lazy.argtypes = [P, P, c_int, c_int, P, c_int, P, c_int64, P, P, P, P]
    lib.bdh_model_forward_fast.argtypes = [P, P, c_int, c_int, c_int, P]
    lib.bdh_model_forward_fast_ex.argtypes = [P, P, c_int, c_int, c_int, P, c_int, c_int, P, c_int, P]
    lib.bdh_rotate.argtypes = [P, c_int, c_int, c_int, c_int, c_int, P, P, c_int64, P, P]
    lib.bdh_rho_energy.argtypes = [P, c_int, c_int, c_int, c_int, P, c_int, P, c_int64, P, P, P]
    lib.bdh_model_forward_viz.argtypes = [P, P, c_int, c_int, P, c_int, P, c_int64, P, P, P, P, P]
    for name in EXPORTS:
        fn = getattr(lib, name)
        if fn.restype is c_int and name not in ("bdh_version",):
            fn.restype = c_int
    if path == LIB_PATH:
        _lib = lib
    return lib


def ptr(t) -> Optional[int]:
    """Device (or host) address of a torch tensor / numpy array / None."""
    if t is None:
        return None
    if hasattr(t, "data_ptr"):
        return t.data_ptr()
    return t.ctypes.data


class Context:
    """bdh_ctx bound to a device and a HIP stream.  Without an explicit stream the context follows torch's
    current stream: every access to `.lib` (each wrapper fetches it right before its call) re-binds the context
    when the current stream has changed, so tensors torch allocates or fills on that stream and the library's
    kernels stay ordered, also inside `with torch.cuda.stream(s)` and under graph capture; on such a re-bind the
    new stream first waits for what the old one still has queued (the context's workspace is shared by all calls).
    A context created with a stream, or given one through set_stream(..., pin=True), keeps it.  Work that should
    overlap on two streams needs two contexts."""

    def __init__(self, device_id: int = 0, stream: Optional[int] = None):
        self._lib = load_library()
        self.device_id = device_id
        self._follow = stream is None
        if stream is None:
            import torch

            stream = torch.cuda.current_stream(device_id).cuda_stream
        handle = c_void_p()
        rc = self._lib.bdh_ctx_create(device_id, stream or None, ctypes.byref(handle))
        if rc != OK:
            raise BdhError(rc, self._lib.bdh_status_string(rc).decode() + " (bdh_ctx_create; is a HIP device present?)")
        self.handle = handle
        self._stream = stream or 0

    @property
    def lib(self):
        if self._follow and getattr(self, "handle", None) and not sys.is_finalizing():
            import torch

            cur = torch.cuda.current_stream(self.device_id)
            current = cur.cuda_stream
            if current != self._stream:
                # The context's workspace and the model's activation scratch are shared by every call: work queued on
                # the old stream may still use them, so the new stream waits for it (not under graph capture, where
                # an event recorded outside the capture must not be waited on; a capture orders its own work).
                if not torch.cuda.is_current_stream_capturing():
                    old = (torch.cuda.ExternalStream(self._stream, device=self.device_id) if self._stream
                           else torch.cuda.default_stream(self.device_id))
                    done = torch.cuda.Event()
                    done.record(old)
                    cur.wait_event(done)
                self._lib.bdh_ctx_set_stream(self.handle, current or None)
                self._stream = current
        return self._lib

    def check(self, rc: int):
        if rc != OK:
            raise BdhError(rc, self._lib.bdh_last_error(self.handle).decode())

    def set_stream(self, stream: int, pin: bool = False):
        """Binds the context to `stream`; with pin=True it stops following torch's current stream."""
        self.check(self._lib.bdh_ctx_set_stream(self.handle, stream or None))
        self._stream = stream or 0
        if pin:
            self._follow = False

    def set_option(self, name: str, value: int):
        self.check(self._lib.bdh_ctx_set_option(self.handle, name.encode(), int(value)))

    def synchronize(self):
        self.check(self._lib.bdh_ctx_synchronize(self.handle))

    def close(self):
        if getattr(self, "handle", None):
            if not sys.is_finalizing():  # at interpreter exit the HIP runtime may already be gone
                self._lib.bdh_ctx_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


_default_ctx = {}


def default_context(device_id: int = 0) -> Context:
    if device_id not in _default_ctx:
        _default_ctx[device_id] = Context(device_id)
    return _default_ctx[device_id]
