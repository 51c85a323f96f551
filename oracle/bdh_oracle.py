"""CPU oracle for the BDH cached-inference path (TEST INFRASTRUCTURE ONLY).

Two restatements of the reference's algorithm live under ``oracle/``:

* ``bdh_oracle.c``  -- plain C, binary32, the reference's op order; loaded here
  through ctypes as :class:`COracle`.  It is the checker for config-sized inputs
  and the CPU baseline the benchmark times.
* this module     -- an independent, vectorised numpy statement of the same
  functions with a selectable dtype (float32 to compare with the C one, float64
  for the invariants that pin both).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package.  The product (``burn_dragon_amd``) never
does: it fails loudly when its HIP library is missing.

Every function cites the reference lines (paths relative to the reference tree)
that it restates.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple

import numpy as np

ROPE, ALIBI, POPE = 0, 1, 2
ROTARY_NAMES = {"rope": ROPE, "alibi": ALIBI, "pope": POPE}

LAYER_NORM_EPS = 1e-5  # src/model/bdh.rs:17
ROW_NORM_EPS = 1e-6  # src/model/attention.rs:11
ROPE_THETA = 65536.0  # src/model/config.rs:25

_HERE = os.path.dirname(os.path.abspath(__file__))


# --------------------------------------------------------------------------
# numpy restatement
# --------------------------------------------------------------------------
def build_freqs(latent: int, theta: float = ROPE_THETA, rotary: int = ROPE, dtype=np.float32):
    """src/model/attention.rs:351-373 (second statement: tests/fused_kernel_tests.rs:172-196)."""
    dt = np.dtype(dtype).type
    idx = np.arange(latent).astype(dtype)
    if rotary == ROPE:
        exponent = (np.floor(idx / dt(2.0)) * dt(2.0)) / dt(latent)
    elif rotary == POPE:
        exponent = idx / dt(latent)
    else:
        return np.zeros(latent, dtype=dtype)
    two_pi = dt(2.0) * dt(np.float32(np.pi)) if dtype == np.float32 else dt(2.0 * np.pi)
    return (dt(1.0) / np.power(dt(theta), exponent) / two_pi).astype(dtype)


def default_alibi_slopes(n_head: int, dtype=np.float32):
    """src/kernel/linear_attention.rs:152-163."""
    dt = np.dtype(dtype).type
    ratio = np.arange(n_head).astype(dtype) / dt(n_head)
    return (dt(1.0) / np.power(dt(2.0), ratio)).astype(dtype)


def alibi_decay(slopes):
    """src/model/attention.rs:181-186."""
    return np.exp(-np.asarray(slopes))


def softplus(x):
    """burn activation::softplus(x, 1.0) as called at src/model/attention.rs:324."""
    one = x.dtype.type(1.0)
    return np.log(np.exp(x * one) + one) / one


def phases(freqs, start: int, time: int):
    """src/model/attention.rs:338-343: raw = f32(pos)*freq; (raw - floor(raw)) * 2*pi."""
    dtype = freqs.dtype
    dt = dtype.type
    pos = np.arange(start, start + time, dtype=np.int64).astype(dtype).reshape(time, 1)
    raw = pos * freqs.reshape(1, -1)
    two_pi = dt(2.0) * dt(np.float32(np.pi)) if dtype == np.float32 else dt(2.0 * np.pi)
    return (raw - np.floor(raw)) * two_pi  # [T, N]


def rope(ph, values):
    """src/model/attention.rs:305-321 (also src/kernel/linear_attention.rs:117-137)."""
    cos, sin = np.cos(ph), np.sin(ph)
    b, h, t, n = values.shape
    pairs = values.reshape(b, h, t, n // 2, 2)
    even, odd = pairs[..., 0], pairs[..., 1]
    rotated = np.stack([-odd, even], axis=4).reshape(b, h, t, n)
    return values * cos + rotated * sin


def pope(ph, values):
    """src/model/attention.rs:323-330."""
    mag = softplus(values)
    return np.concatenate([mag * np.cos(ph), mag * np.sin(ph)], axis=3)


def rotate(values, freqs, rotary: int, start: int = 0):
    """src/model/attention.rs:332-349. values [B,h,T,N] -> [B,h,T,Nq]."""
    if rotary == ALIBI:
        return values
    ph = phases(freqs.astype(values.dtype), start, values.shape[2])
    return rope(ph, values) if rotary == ROPE else pope(ph, values)


def layer_norm(x):
    """src/model/bdh.rs:86-89: biased variance, eps 1e-5, no affine."""
    dt = x.dtype.type
    mean = x.mean(axis=-1, keepdims=True, dtype=x.dtype)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True, dtype=x.dtype)
    return (x - mean) / np.sqrt(var + dt(LAYER_NORM_EPS))


def block_mask_1d(elements: int, block_size: int, active_blocks: Optional[Sequence[int]], dtype=np.float32):
    """src/kernel/block_sparse.rs:48-63 BlockPattern1d::mask."""
    if active_blocks is None:
        return np.ones(elements, dtype=dtype)
    block_size = max(block_size, 1)
    mask = np.zeros(elements, dtype=dtype)
    for blk in range(-(-elements // block_size)):
        if blk in set(active_blocks):
            mask[blk * block_size : min((blk + 1) * block_size, elements)] = 1
    return mask


def relu_lowrank(inp, weight, bias=None, threshold: float = 0.0, block_size: int = 1, active_blocks=None):
    """src/kernel/relu_lowrank.rs:7-37. inp [B,1|h,T,d], weight [h,d,N], bias [h,N]|None."""
    dt = inp.dtype.type
    proj = np.matmul(inp, weight[None])  # broadcast over dim 1 like Burn's matmul
    if bias is not None:
        proj = proj + bias[None, :, None, :]
    if threshold != 0.0:
        proj = proj - dt(threshold)
    act = np.maximum(proj, dt(0))
    if active_blocks is not None:
        act = act * block_mask_1d(weight.shape[-1], block_size, active_blocks, inp.dtype)
    return act


def recurrent_attention(q, v, rho, decay=None):
    """src/model/bdh.rs:286-306 after the rotate. q [B,h,T,Nq] rotated, v [B,T,d],
    rho [B,h,Nq,d] (updated copy returned). Readout uses the OLD rho (:293-295)."""
    B, h, T, Nq = q.shape
    rho = rho.copy()
    outs = []
    for t in range(T):
        x_t = q[:, :, t, :, None]  # [B,h,Nq,1]  (:289,291)
        v_t = v[:, None, t, None, :]  # [B,1,1,d] repeated over heads (:290)
        outs.append((rho * x_t).sum(axis=2))  # (:293-295)
        rho = rho + x_t * v_t  # (:298)
        if decay is not None:
            rho = rho * np.asarray(decay, dtype=rho.dtype).reshape(1, h, 1, 1)  # (:299-301)
    return np.stack(outs, axis=2), rho


def causal_unnormalised(q, v):
    """tril(-1)(q q^T) v  -- the closed form the recurrent path must equal (no ALiBi)."""
    scores = np.tril(np.matmul(q, np.swapaxes(q, 2, 3)), -1)
    return np.matmul(scores, v[:, None])


def attention_forward(query, value, freqs, slopes=None, rotary: int = ROPE, row_normalize: bool = True):
    """src/model/attention.rs:154-174 (unfused). value [B,T,dv]."""
    q = rotate(query, freqs, rotary, 0)
    T = q.shape[2]
    scores = np.tril(np.matmul(q, np.swapaxes(q, 2, 3)), -1)
    if slopes is not None:
        pos = np.arange(T, dtype=q.dtype)
        bias = np.tril(pos[None, :] - pos[:, None], -1)
        scores = scores + np.asarray(slopes, dtype=q.dtype).reshape(1, -1, 1, 1) * bias
    if row_normalize:
        scores = scores / (np.abs(scores).sum(axis=3, keepdims=True) + q.dtype.type(ROW_NORM_EPS))
    return np.matmul(scores, value[:, None])


def fused_state_aligned(query, value, freqs, slopes=None, block_size: int = 64, rotary: int = ROPE, pairs=None):
    """src/kernel/linear_attention.rs:11-115. value [B,T,dv]; pairs: optional set of
    (row, col) active time-block pairs (dense lower-triangular when None)."""
    q = rotate(query, freqs, rotary, 0)
    B, h, T, _ = q.shape
    dv = value.shape[-1]
    dt = q.dtype.type
    block_size = max(block_size, 1)
    total = -(-T // block_size)
    pos = np.arange(T, dtype=q.dtype)
    sl = None if slopes is None else np.asarray(slopes, dtype=q.dtype).reshape(1, h, 1, 1)
    outs = []
    for row in range(total):
        rs = slice(row * block_size, min((row + 1) * block_size, T))
        qb = q[:, :, rs]
        acc = np.zeros((B, h, qb.shape[2], dv), dtype=q.dtype)
        norm = np.zeros((B, h, qb.shape[2], 1), dtype=q.dtype)
        cols = [c for c in range(total) if ((c <= row) if pairs is None else ((row, c) in pairs))]
        if not cols:
            outs.append(acc)
            continue
        for col in cols:
            cs = slice(col * block_size, min((col + 1) * block_size, T))
            scores = np.matmul(qb, np.swapaxes(q[:, :, cs], 2, 3))
            if row == col:
                scores = np.tril(scores, -1)
            if sl is not None:
                scores = scores + sl * (pos[cs][None, :] - pos[rs][:, None])  # (:97-100) whole block
            norm = norm + np.abs(scores).sum(axis=3, keepdims=True)
            acc = acc + np.matmul(scores, value[:, None, cs])
        outs.append(acc / (norm + dt(ROW_NORM_EPS)))
    return np.concatenate(outs, axis=2)


@dataclass
class BDHWeights:
    """Parameters in the reference module's record order (src/model/bdh.rs:27-33)."""

    embed: np.ndarray  # [V, d]
    encoder: np.ndarray  # [h, d, N]   D_x
    encoder_v: np.ndarray  # [h, d, N]   D_y
    decoder: np.ndarray  # [h*N, d]    E
    lm_head: np.ndarray  # [d, V]


@dataclass
class BDHShape:
    """src/model/config.rs:113-164 (latent_per_head = mult*d/h)."""

    n_layer: int = 6
    n_embd: int = 256
    n_head: int = 4
    mlp_internal_dim_multiplier: int = 4
    vocab_size: int = 256
    rotary: int = ALIBI  # src/positional.rs:12-13 default
    rope_theta: float = ROPE_THETA
    relu_threshold: float = 0.0
    alibi_slopes: Optional[Sequence[float]] = None

    @property
    def latent_per_head(self) -> int:
        total = self.mlp_internal_dim_multiplier * self.n_embd
        assert total % self.n_head == 0, "latent size must be divisible by the number of heads"
        return total // self.n_head


def init_weights(shape: BDHShape, seed: int, dtype=np.float32) -> BDHWeights:
    """Seeded stand-in for src/model/bdh.rs:37-84: Normal(0, 0.02) for the four
    projection matrices (:50-67); embedding Normal(0, 1).  Burn's own RNG stream
    cannot be reproduced without the Rust crates, so 'same seed' means this
    generator feeds the oracle and the device path identically."""
    rng = np.random.default_rng(seed)
    h, d, N, V = shape.n_head, shape.n_embd, shape.latent_per_head, shape.vocab_size
    return BDHWeights(
        embed=rng.standard_normal((V, d)).astype(dtype),
        encoder=(0.02 * rng.standard_normal((h, d, N))).astype(dtype),
        encoder_v=(0.02 * rng.standard_normal((h, d, N))).astype(dtype),
        decoder=(0.02 * rng.standard_normal((h * N, d))).astype(dtype),
        lm_head=(0.02 * rng.standard_normal((d, V))).astype(dtype),
    )


@dataclass
class ModelState:
    """src/model/state.rs:5-57."""

    n_layer: int
    rho: List[Optional[np.ndarray]] = field(default_factory=list)
    position: int = 0

    def __post_init__(self):
        if not self.rho:
            self.rho = [None] * self.n_layer

    def reset(self):
        self.rho = [None] * self.n_layer
        self.position = 0


def forward_with_state(shape: BDHShape, w: BDHWeights, tokens, state: ModelState, taps: Optional[dict] = None):
    """src/model/bdh.rs:309-450, numpy statement. tokens [B,T] ints -> logits [B,T,V]."""
    assert len(state.rho) == shape.n_layer, "model state layers mismatch"  # :314-318
    dtype = w.encoder.dtype
    tokens = np.asarray(tokens)
    B, T = tokens.shape
    h, d, N = shape.n_head, shape.n_embd, shape.latent_per_head
    Nq = 2 * N if shape.rotary == POPE else N
    cur = layer_norm(w.embed[tokens].reshape(B, 1, T, d))  # :319-322
    freqs = build_freqs(N, shape.rope_theta, shape.rotary, dtype)
    decay = None
    if shape.rotary == ALIBI:
        slopes = default_alibi_slopes(h, dtype) if shape.alibi_slopes is None else np.asarray(shape.alibi_slopes, dtype)
        decay = alibi_decay(slopes)
    start = state.position  # :334
    for l in range(shape.n_layer):
        x = relu_lowrank(cur, w.encoder, None, shape.relu_threshold)  # :337-351
        q = rotate(x, freqs, shape.rotary, start)  # :265
        rho = state.rho[l]
        if rho is None or rho.shape != (B, h, Nq, d):  # :274-284
            rho = np.zeros((B, h, Nq, d), dtype=dtype)
        attn, rho = recurrent_attention(q, cur[:, 0], rho, decay)
        state.rho[l] = rho
        if taps is not None:
            taps.setdefault("x", []).append(x)
            taps.setdefault("attn", []).append(attn)
        attn = layer_norm(attn)  # :359
        y = relu_lowrank(attn, w.encoder_v, None, shape.relu_threshold)  # :361-375
        xy = x * y  # :380
        if taps is not None and T > 0:  # :386-434, feature "viz"
            taps.setdefault("viz", []).append(dict(
                x_last=x[0, :, T - 1], y_last=y[0, :, T - 1], xy_last=xy[0, :, T - 1],
                rho_last=rho_energy(rho) if Nq == N else np.zeros((h, N), dtype)))
        mixed = np.swapaxes(xy, 1, 2).reshape(B * T, h * N)  # :383, :436
        mlp = layer_norm(np.matmul(mixed, w.decoder).reshape(B, 1, T, d))  # :438-440
        cur = layer_norm(cur + mlp)  # :441
    state.position = state.position + T  # :445
    return np.matmul(cur.reshape(B * T, d), w.lm_head).reshape(B, T, shape.vocab_size)  # :446-449


def forward_fast(shape: BDHShape, w: BDHWeights, tokens, fused: bool = False, time_block: int = 64,
                 time_pairs=None, latent_block: int = 1, latent_active=None):
    """src/model/bdh.rs:96-168, numpy statement: the stateless forward over all tokens at once, a
    composition of relu_lowrank, Attention::forward (plain branch) or fused_state_aligned (fused branch),
    layer_norm and two matmuls.  tokens [B,T] ints -> logits [B,T,V].  The fused branch hands the latent
    block pattern to both projections and the time-block pattern to the attention (:111, :114-151,
    src/model/attention.rs:142-152); the plain branch consults neither.  The parts are pinned (see the C
    file's header); the reference itself checks only the shape of the result (tests/model_paths.rs:48,81),
    so the composition as a whole is "parity unpinned"."""
    dtype = w.encoder.dtype
    tokens = np.asarray(tokens)
    B, T = tokens.shape
    h, d, N = shape.n_head, shape.n_embd, shape.latent_per_head
    cur = layer_norm(w.embed[tokens].reshape(B, 1, T, d))  # :97-100
    freqs = build_freqs(N, shape.rope_theta, shape.rotary, dtype)
    slopes = None
    if shape.rotary == ALIBI:
        slopes = default_alibi_slopes(h, dtype) if shape.alibi_slopes is None else np.asarray(shape.alibi_slopes, dtype)
    for _ in range(shape.n_layer):
        lat = dict(block_size=latent_block, active_blocks=latent_active) if fused else {}
        x = relu_lowrank(cur, w.encoder, None, shape.relu_threshold, **lat)  # :114-129
        if fused:  # :131, src/model/attention.rs:142-152
            attn = fused_state_aligned(x, cur[:, 0], freqs, slopes, time_block, shape.rotary, time_pairs)
        else:  # src/model/attention.rs:154-174
            attn = attention_forward(x, cur[:, 0], freqs, slopes, shape.rotary, True)
        attn = layer_norm(attn.astype(dtype))  # :132
        y = relu_lowrank(attn, w.encoder_v, None, shape.relu_threshold, **lat)  # :134-151
        xy = x * y
        mixed = np.swapaxes(xy, 1, 2).reshape(B * T, h * N)  # :156-160
        mlp = layer_norm(np.matmul(mixed, w.decoder).reshape(B, 1, T, d))  # :162-164
        cur = layer_norm(cur + mlp)  # :165
    return np.matmul(cur.reshape(B * T, d), w.lm_head).reshape(B, T, shape.vocab_size)  # :168-172


def rho_energy(rho):
    """src/model/bdh.rs:411-419: [B,h,N,d] -> [h,N], mean over the batch of the per-row mean |rho|."""
    B, _, _, d = rho.shape
    per_row = np.abs(rho).sum(axis=3, dtype=rho.dtype) / rho.dtype.type(d)
    return per_row.sum(axis=0, dtype=rho.dtype) / rho.dtype.type(B)


def greedy_token(logits_row) -> int:
    """src/generation.rs:26-72 with top_k=Some(1): argmax when the maximum is unique."""
    return int(np.argmax(logits_row))


def sample_from_logits(logits_row, temperature: float, top_k: Optional[int], u: float, dtype=np.float32):
    """src/generation.rs:117 and :26-72 with the uniform variate `u` of WeightedIndex explicit.
    Returns (index, probabilities)."""
    v = (np.asarray(logits_row, dtype) / dtype(temperature)).astype(dtype)
    V = v.size
    if top_k is not None and 0 < top_k < V:
        threshold = np.sort(v)[::-1][top_k - 1]
        v = np.where(v < threshold, dtype(-np.inf), v)
    with np.errstate(invalid="ignore"):
        p = np.exp(v - np.nanmax(v) if not np.all(np.isnan(v)) else v).astype(dtype)
    s = dtype(0)
    for e in p:
        s = dtype(s + e)
    p = np.full(V, dtype(1) / dtype(V), dtype) if (s == 0 or np.isnan(s)) else (p / s).astype(dtype)
    cum = np.zeros(V, dtype)
    acc = dtype(0)
    for i, e in enumerate(p):
        acc = dtype(acc + e)
        cum[i] = acc
    chosen = dtype(min(max(u, 0.0), 0.99999994)) * cum[-1]
    return int(np.searchsorted(cum[:-1], chosen, side="right")), p


# --------------------------------------------------------------------------
# helpers shared by tests: what the compaction must produce
# --------------------------------------------------------------------------
def active_bitmask(x) -> np.ndarray:
    """Bit n%64 of word n//64 is set iff x[..., n] > 0.  x [..., N], N % 64 == 0."""
    N = x.shape[-1]
    bits = (x > 0).reshape(*x.shape[:-1], N // 64, 64).astype(np.uint64)
    weights = np.uint64(1) << np.arange(64, dtype=np.uint64)
    return (bits * weights).sum(axis=-1, dtype=np.uint64)


def pair_closed_rows(x) -> np.ndarray:
    """Number of state rows a RoPE step touches per leading index: both rows of every
    lane pair (2j, 2j+1) with at least one positive element."""
    pairs = (x > 0).reshape(*x.shape[:-1], x.shape[-1] // 2, 2).any(axis=-1)
    return 2 * pairs.sum(axis=-1)


# --------------------------------------------------------------------------
# C oracle through ctypes
# --------------------------------------------------------------------------
class _OrcModel(ctypes.Structure):
    _fields_ = [
        ("n_layer", ctypes.c_int),
        ("n_embd", ctypes.c_int),
        ("n_head", ctypes.c_int),
        ("latent", ctypes.c_int),
        ("vocab", ctypes.c_int),
        ("rotary", ctypes.c_int),
        ("rope_theta", ctypes.c_float),
        ("relu_threshold", ctypes.c_float),
        ("alibi_slopes", ctypes.c_void_p),
        ("embed", ctypes.c_void_p),
        ("encoder", ctypes.c_void_p),
        ("encoder_v", ctypes.c_void_p),
        ("decoder", ctypes.c_void_p),
        ("lm_head", ctypes.c_void_p),
    ]


def build_c_oracle(force: bool = False) -> str:
    """Compile oracle/bdh_oracle.c with the committed Makefile; returns the .so path."""
    so = os.path.join(_HERE, "libbdh_oracle.so")
    if force or not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(os.path.join(_HERE, "bdh_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libbdh_oracle.so"], stdout=subprocess.DEVNULL)
    return so


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


class COracle:
    """ctypes view of oracle/bdh_oracle.c (binary32, reference op order)."""

    def __init__(self, path: Optional[str] = None):
        path = path or os.path.join(_HERE, "libbdh_oracle.so")
        if not os.path.exists(path):
            path = build_c_oracle()
        self.lib = ctypes.CDLL(path)
        self.lib.orc_forward_with_state.restype = ctypes.c_int
        self.lib.orc_forward_with_state_viz.restype = ctypes.c_int
        self.lib.orc_greedy_token.restype = ctypes.c_int
        self.lib.orc_sample_from_logits.restype = ctypes.c_int

    def build_freqs(self, latent, theta=ROPE_THETA, rotary=ROPE):
        out = np.empty(latent, np.float32)
        self.lib.orc_build_freqs(ctypes.c_int(latent), ctypes.c_float(theta), ctypes.c_int(rotary), _p(out))
        return out

    def default_alibi_slopes(self, n_head):
        out = np.empty(n_head, np.float32)
        self.lib.orc_default_alibi_slopes(ctypes.c_int(n_head), _p(out))
        return out

    def alibi_decay(self, slopes):
        slopes = _f32(slopes)
        out = np.empty_like(slopes)
        self.lib.orc_alibi_decay(ctypes.c_int(slopes.size), _p(slopes), _p(out))
        return out

    def rotate(self, x, freqs, rotary=ROPE, start=0):
        x, freqs = _f32(x), _f32(freqs)
        B, h, T, N = x.shape
        Nq = 2 * N if rotary == POPE else N
        q = np.empty((B, h, T, Nq), np.float32)
        self.lib.orc_rotate(_p(x), B, h, T, N, _p(freqs), ctypes.c_int(rotary), ctypes.c_int64(start), _p(q))
        return q

    def layer_norm(self, x):
        x = _f32(x)
        out = np.empty_like(x)
        d = x.shape[-1]
        self.lib.orc_layer_norm(_p(x), ctypes.c_int64(x.size // d), ctypes.c_int(d), _p(out))
        return out

    def relu_lowrank(self, inp, weight, bias=None, threshold=0.0, block_size=1, active_blocks=None):
        inp, weight = _f32(inp), _f32(weight)
        B, hin, T, d = inp.shape
        h, d2, N = weight.shape
        assert d == d2 and hin in (1, h)
        bias_a = None if bias is None else _f32(bias).reshape(h, N)
        act = None
        nblk = 0
        if active_blocks is not None:
            nblk = -(-N // max(block_size, 1))
            act = np.zeros(nblk, np.uint8)
            for blk in active_blocks:
                if blk < nblk:
                    act[blk] = 1
        out = np.empty((B, h, T, N), np.float32)
        self.lib.orc_relu_lowrank(_p(inp), B, hin, T, d, _p(weight), h, N, _p(bias_a), ctypes.c_float(threshold),
                                  ctypes.c_int(block_size), _p(act), ctypes.c_int(nblk), _p(out))
        return out

    def recurrent_attention(self, q, v, rho, decay=None, sparse=False):
        """Returns (out [B,h,T,d], new rho). rho is copied, not modified."""
        q, v = _f32(q), _f32(v)
        rho = np.array(rho, dtype=np.float32, order="C", copy=True)
        B, h, T, Nq = q.shape
        d = v.shape[-1]
        assert rho.shape == (B, h, Nq, d) and v.shape == (B, T, d)
        out = np.empty((B, h, T, d), np.float32)
        if sparse:
            assert decay is None
            self.lib.orc_recurrent_attention_sparse(_p(q), _p(v), _p(rho), B, h, T, Nq, d, _p(out))
        else:
            dec = None if decay is None else _f32(decay)
            self.lib.orc_recurrent_attention(_p(q), _p(v), _p(rho), _p(dec), B, h, T, Nq, d, _p(out))
        return out, rho

    def fused_state_aligned(self, query, value, freqs, slopes=None, block_size=64, rotary=ROPE, pairs=None):
        query, value, freqs = _f32(query), _f32(value), _f32(freqs)
        B, h, T, N = query.shape
        dv = value.shape[-1]
        sl = None if slopes is None else _f32(slopes)
        pr, npairs = None, 0
        if pairs is not None:
            pr = np.ascontiguousarray(np.array(sorted(pairs), dtype=np.int32).reshape(-1, 2))
            npairs = pr.shape[0]
        out = np.empty((B, h, T, dv), np.float32)
        self.lib.orc_fused_state_aligned(_p(query), _p(value), _p(freqs), _p(sl), B, h, T, N, dv,
                                         ctypes.c_int(block_size), _p(pr), ctypes.c_int(npairs),
                                         ctypes.c_int(rotary), _p(out))
        return out

    def attention_forward(self, query, value, freqs, slopes=None, rotary=ROPE, row_normalize=True):
        query, value, freqs = _f32(query), _f32(value), _f32(freqs)
        B, h, T, N = query.shape
        dv = value.shape[-1]
        sl = None if slopes is None else _f32(slopes)
        out = np.empty((B, h, T, dv), np.float32)
        self.lib.orc_attention_forward(_p(query), _p(value), _p(freqs), _p(sl), B, h, T, N, dv,
                                       ctypes.c_int(rotary), ctypes.c_int(int(row_normalize)), _p(out))
        return out

    def forward_with_state(self, shape: BDHShape, w: BDHWeights, tokens, rho: np.ndarray, position: int,
                           taps: bool = False, sparse_state: bool = True):
        """rho [L,B,h,Nq,d] float32 C-contiguous, updated IN PLACE.
        Returns (logits [B,T,V], new position, x_tap|None, attn_tap|None)."""
        tokens = np.ascontiguousarray(tokens, dtype=np.int64)
        B, T = tokens.shape
        h, d, N, V, L = shape.n_head, shape.n_embd, shape.latent_per_head, shape.vocab_size, shape.n_layer
        Nq = 2 * N if shape.rotary == POPE else N
        assert rho.dtype == np.float32 and rho.flags.c_contiguous and rho.shape == (L, B, h, Nq, d)
        keep = [_f32(w.embed), _f32(w.encoder), _f32(w.encoder_v), _f32(w.decoder), _f32(w.lm_head)]
        sl = None if shape.alibi_slopes is None else _f32(shape.alibi_slopes)
        m = _OrcModel(L, d, h, N, V, shape.rotary, shape.rope_theta, shape.relu_threshold,
                      None if sl is None else sl.ctypes.data, *[a.ctypes.data for a in keep])
        logits = np.empty((B, T, V), np.float32)
        x_tap = np.empty((L, B, h, T, N), np.float32) if taps else None
        attn_tap = np.empty((L, B, h, T, d), np.float32) if taps else None
        pos = ctypes.c_int64(position)
        rc = self.lib.orc_forward_with_state(ctypes.byref(m), _p(tokens), B, T, _p(rho), ctypes.byref(pos),
                                             _p(logits), _p(x_tap), _p(attn_tap), ctypes.c_int(int(sparse_state)))
        if rc != 0:
            raise ValueError("token id out of range")
        return logits, pos.value, x_tap, attn_tap

    def rho_energy(self, rho):
        rho = _f32(rho)
        B, h, N, d = rho.shape
        out = np.empty((h, N), np.float32)
        self.lib.orc_rho_energy(_p(rho), B, h, N, d, _p(out))
        return out

    def forward_with_state_viz(self, shape: BDHShape, w: BDHWeights, tokens, rho: np.ndarray, position: int,
                               sparse_state: bool = True):
        """forward_with_state plus the LayerVizState taps: returns (logits, new position, viz [L,4,h,N])
        with viz[l] = (x_last, y_last, xy_last, rho_last).  rho is updated in place."""
        tokens = np.ascontiguousarray(tokens, dtype=np.int64)
        B, T = tokens.shape
        h, d, N, V, L = shape.n_head, shape.n_embd, shape.latent_per_head, shape.vocab_size, shape.n_layer
        Nq = 2 * N if shape.rotary == POPE else N
        assert rho.dtype == np.float32 and rho.flags.c_contiguous and rho.shape == (L, B, h, Nq, d)
        keep = [_f32(w.embed), _f32(w.encoder), _f32(w.encoder_v), _f32(w.decoder), _f32(w.lm_head)]
        sl = None if shape.alibi_slopes is None else _f32(shape.alibi_slopes)
        m = _OrcModel(L, d, h, N, V, shape.rotary, shape.rope_theta, shape.relu_threshold,
                      None if sl is None else sl.ctypes.data, *[a.ctypes.data for a in keep])
        logits = np.empty((B, T, V), np.float32)
        viz = np.zeros((L, 4, h, N), np.float32)
        pos = ctypes.c_int64(position)
        rc = self.lib.orc_forward_with_state_viz(ctypes.byref(m), _p(tokens), B, T, _p(rho), ctypes.byref(pos),
                                                 _p(logits), ctypes.c_int(int(sparse_state)), _p(viz))
        if rc != 0:
            raise ValueError("token id out of range")
        return logits, pos.value, viz

    def greedy_token(self, logits_row) -> int:
        row = _f32(logits_row)
        return int(self.lib.orc_greedy_token(_p(row), ctypes.c_int(row.size)))

    def sample_from_logits(self, logits_row, temperature, top_k, u):
        row = _f32(logits_row)
        probs = np.empty(row.size, np.float32)
        idx = self.lib.orc_sample_from_logits(_p(row), ctypes.c_int(row.size), ctypes.c_float(temperature),
                                              ctypes.c_int(0 if top_k is None else int(top_k)), ctypes.c_float(u),
                                              _p(probs))
        return int(idx), probs

    def state_step_dense(self, x, v, freqs, position, rho):
        """Single-layer decode step (rotate + dense recurrent_attention, T=1); rho IN PLACE."""
        x, v, freqs = _f32(x), _f32(v), _f32(freqs)
        B, h, N = x.shape
        d = v.shape[-1]
        assert rho.dtype == np.float32 and rho.flags.c_contiguous and rho.shape == (B, h, N, d)
        q = np.empty((B, h, N), np.float32)
        out = np.empty((B, h, d), np.float32)
        self.lib.orc_state_step_dense(_p(x), _p(v), _p(freqs), ctypes.c_int64(position), _p(rho), B, h, N, d,
                                      _p(q), _p(out))
        return out
