"""Reader and writer for the checkpoint files of the reference: Burn 0.19 `BinFileRecorder`
records of the BDH module (written by src/bin/train.rs:396 and src/bin/quantize.rs:44-57,
read by src/bin/infer.rs:177-186 and src/web.rs:173-187).

The file is a bincode 2 stream (standard configuration: little endian, variable-length
integers) of `BurnRecord { metadata, item }`:

    metadata   five strings: float type, int type, recorder format, crate version, settings
    item       the fields of the module record in declaration order (src/model/bdh.rs:20-34);
               every field that is not a parameter (numbers, configs, plain tensors, Dropout)
               is a `ConstantRecord`, one 0x00 byte; a parameter is
               { id: string, param: { bytes: byte string, shape: [usize], dtype: enum index } }

A string / byte string / sequence is its length as a varint followed by the elements; a varint
below 251 is one byte, 251 / 252 / 253 announce a little-endian u16 / u32 / u64.

How many constant fields sit between the parameters depends on the version of the struct that
wrote the file (the record shipped under www/assets/model/tiny_shakespeare has 5 and 6 where
the current struct would write 6 and 8), so the reader skips constants wherever they appear and
identifies the five parameters by order and shape: embed.weight [V,d], encoder [h,d,N],
encoder_v [h,d,N], decoder [h*N,d], lm_head [d,V].

Nothing in the file is executed or evaluated: it is parsed as numbers and bytes only.
"""
from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import numpy as np

PARAM_ORDER = ("embed", "encoder", "encoder_v", "decoder", "lm_head")

# burn-tensor 0.19 `DType` variant indices that a float record can hold
_DTYPES = {0: ("f64", np.dtype("<f8")), 1: ("f32", np.dtype("<f4")), 3: ("f16", np.dtype("<f2"))}
_BF16 = 4
_DTYPE_INDEX = {"f64": 0, "f32": 1, "f16": 3}

FULL_PRECISION = "FullPrecisionSettings"
HALF_PRECISION = "HalfPrecisionSettings"
_FORMAT = "burn_core::record::file::BinFileRecorder<burn_core::record::settings::{}>"


class RecordError(ValueError):
    """The bytes are not a BDH record this reader understands."""


@dataclass
class RecordMetadata:
    float: str
    int: str
    format: str
    version: str
    settings: str


@dataclass
class ParamEntry:
    id: str
    shape: Tuple[int, ...]
    dtype: str
    data: np.ndarray  # float32, shaped


class _Reader:
    def __init__(self, buf: bytes):
        self.buf, self.off = memoryview(buf), 0

    def remaining(self) -> int:
        return len(self.buf) - self.off

    def take(self, n: int) -> memoryview:
        if n < 0 or n > self.remaining():
            raise RecordError(f"truncated record: need {n} bytes at offset {self.off}, {self.remaining()} left")
        out = self.buf[self.off:self.off + n]
        self.off += n
        return out

    def peek(self) -> int:
        if not self.remaining():
            raise RecordError("truncated record")
        return self.buf[self.off]

    def varint(self) -> int:
        b = self.take(1)[0]
        if b < 251:
            return b
        if b == 251:
            return struct.unpack("<H", self.take(2))[0]
        if b == 252:
            return struct.unpack("<I", self.take(4))[0]
        if b == 253:
            return struct.unpack("<Q", self.take(8))[0]
        raise RecordError(f"unsupported varint marker {b} at offset {self.off - 1}")

    def string(self, limit: int = 4096) -> str:
        n = self.varint()
        if n > limit:
            raise RecordError(f"string of {n} bytes at offset {self.off} exceeds the limit {limit}")
        try:
            return bytes(self.take(n)).decode("utf-8")
        except UnicodeDecodeError as e:
            raise RecordError(f"string at offset {self.off - n} is not utf-8") from e


def _varint(v: int) -> bytes:
    if v < 251:
        return bytes([v])
    if v < 1 << 16:
        return b"\xfb" + struct.pack("<H", v)
    if v < 1 << 32:
        return b"\xfc" + struct.pack("<I", v)
    return b"\xfd" + struct.pack("<Q", v)


def _string(s: str) -> bytes:
    b = s.encode("utf-8")
    return _varint(len(b)) + b


def parse_record(buf: bytes) -> Tuple[RecordMetadata, List[ParamEntry]]:
    """Metadata and the parameters in file order; constants between them are skipped."""
    r = _Reader(buf)
    meta = RecordMetadata(*(r.string() for _ in range(5)))
    if "BinFileRecorder" not in meta.format and "BinBytesRecorder" not in meta.format:
        raise RecordError(f"not a bincode recorder file: format {meta.format!r}")
    params: List[ParamEntry] = []
    while r.remaining():
        if r.peek() == 0:  # ConstantRecord (serialised as `None`)
            r.take(1)
            continue
        pid = r.string(limit=64)
        nbytes = r.varint()
        raw = r.take(nbytes)
        rank = r.varint()
        if rank > 8:
            raise RecordError(f"parameter {pid!r}: rank {rank}")
        shape = tuple(r.varint() for _ in range(rank))
        dt = r.varint()
        count = int(np.prod(shape, dtype=np.int64)) if shape else 1
        if dt == _BF16:
            if nbytes != 2 * count:
                raise RecordError(f"parameter {pid!r}: {nbytes} bytes for bf16 shape {shape}")
            u = np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16
            data, name = u.view(np.float32), "bf16"
        elif dt in _DTYPES:
            name, npdt = _DTYPES[dt]
            if nbytes != npdt.itemsize * count:
                raise RecordError(f"parameter {pid!r}: {nbytes} bytes for {name} shape {shape}")
            data = np.frombuffer(raw, dtype=npdt).astype(np.float32)
        else:
            raise RecordError(f"parameter {pid!r}: dtype index {dt} is not a float type")
        params.append(ParamEntry(pid, shape, name, np.ascontiguousarray(data.reshape(shape))))
    return meta, params


def weights_from_params(params: List[ParamEntry]) -> Dict[str, np.ndarray]:
    """The five BDH parameters by name, with the shape relations of src/model/bdh.rs:37-84 checked."""
    if len(params) != 5:
        raise RecordError(f"expected 5 parameters (embed, encoder, encoder_v, decoder, lm_head), found {len(params)}")
    w = {name: p.data for name, p in zip(PARAM_ORDER, params)}
    if w["embed"].ndim != 2 or w["encoder"].ndim != 3 or w["decoder"].ndim != 2 or w["lm_head"].ndim != 2:
        raise RecordError("parameter ranks do not match the BDH module")
    V, d = w["embed"].shape
    h, d2, N = w["encoder"].shape
    if d2 != d or w["encoder_v"].shape != (h, d, N) or w["decoder"].shape != (h * N, d) or w["lm_head"].shape != (d, V):
        raise RecordError("parameter shapes do not match the BDH module: "
                          + ", ".join(f"{k}{tuple(v.shape)}" for k, v in w.items()))
    return w


def load_record(path: str) -> Tuple[RecordMetadata, Dict[str, np.ndarray]]:
    """Reads `path` (the recorder appends `.bin` to a base name: both spellings are accepted)."""
    if not os.path.exists(path) and os.path.exists(path + ".bin"):
        path = path + ".bin"
    with open(path, "rb") as f:
        meta, params = parse_record(f.read())
    return meta, weights_from_params(params)


def infer_dimensions(w: Dict[str, np.ndarray]) -> Dict[str, int]:
    """vocab_size, n_embd, n_head and mlp_internal_dim_multiplier implied by the shapes
    (latent_per_head = multiplier * n_embd / n_head, src/model/config.rs:141-155)."""
    V, d = w["embed"].shape
    h, _, N = w["encoder"].shape
    if (N * h) % d:
        raise RecordError(f"latent_total {N * h} is not a multiple of n_embd {d}")
    return {"vocab_size": int(V), "n_embd": int(d), "n_head": int(h), "mlp_internal_dim_multiplier": int(N * h // d)}


def _param_id(index: int) -> str:
    digits = "0123456789abcdefghijklmnopqrstuv"
    v, out = (0x9E3779B97F4A7C15 * (index + 1)) & ((1 << 64) - 1), []
    for _ in range(13):
        out.append(digits[v & 31])
        v >>= 5
    return "".join(out)


def serialize_record(weights: Dict[str, np.ndarray], half: bool = False, version: str = "0.19.1") -> bytes:
    """The bytes BinFileRecorder would write for a BDH module with these parameters
    (FullPrecisionSettings, or HalfPrecisionSettings as src/bin/quantize.rs:44-57), with the constant
    fields of the current module struct: six before the embedding, Dropout and the seven fields of
    Attention (src/model/attention.rs:101-110) after it."""
    settings = HALF_PRECISION if half else FULL_PRECISION
    out = bytearray()
    for s in ("f16" if half else "f32", "i16" if half else "i32", _FORMAT.format(settings), version, settings):
        out += _string(s)
    npdt = np.dtype("<f2") if half else np.dtype("<f4")
    dt_index = _DTYPE_INDEX["f16" if half else "f32"]

    def param(i: int, a: np.ndarray):
        raw = np.ascontiguousarray(a, dtype=npdt).tobytes()
        out.extend(_string(_param_id(i)))
        out.extend(_varint(len(raw)))
        out.extend(raw)
        out.extend(_varint(a.ndim))
        for s in a.shape:
            out.extend(_varint(int(s)))
        out.extend(_varint(dt_index))

    weights_from_params([ParamEntry("", tuple(np.shape(weights[n])), "f32", np.asarray(weights[n])) for n in PARAM_ORDER])
    out += b"\x00" * 6
    param(0, np.asarray(weights["embed"]))
    out += b"\x00" * 8
    for i, name in enumerate(PARAM_ORDER[1:], start=1):
        param(i, np.asarray(weights[name]))
    return bytes(out)


def save_record(path: str, weights: Dict[str, np.ndarray], half: bool = False) -> str:
    if not path.endswith(".bin"):
        path += ".bin"
    with open(path, "wb") as f:
        f.write(serialize_record(weights, half=half))
    return path


def load_checkpoint_dir(directory: str):
    """A directory in the layout of www/assets/model/<name>/: model.bin, config.json
    ({run_name, block_size, overrides{...}}, the overrides being src/inference.rs ModelOverrides) and
    optionally vocab.json.  Returns (BDHConfig, weights, vocab-json text or None, block_size)."""
    from .inference import ModelOverrides, build_model_config

    with open(os.path.join(directory, "config.json"), "r", encoding="utf-8") as f:
        cfg_json = json.load(f)
    block_size = int(cfg_json.get("block_size", 256))
    ov = cfg_json.get("overrides", {}) or {}
    from .positional import RotaryEmbedding

    fields = {k: ov[k] for k in ("n_layer", "n_embd", "n_head", "mlp_internal_dim_multiplier", "relu_threshold",
                                 "dropout", "fused_kernels", "block_size") if ov.get(k) is not None}
    if ov.get("rotary_embedding") is not None:
        fields["rotary_embedding"] = RotaryEmbedding.parse(ov["rotary_embedding"])
    overrides = ModelOverrides(**fields)
    config = build_model_config(overrides, block_size)
    _, weights = load_record(os.path.join(directory, "model.bin"))
    dims = infer_dimensions(weights)
    config.vocab_size = dims["vocab_size"]  # src/bin/infer.rs:175: the tokenizer decides the vocabulary size
    for k in ("n_embd", "n_head", "mlp_internal_dim_multiplier"):
        if getattr(config, k) != dims[k]:
            raise RecordError(f"config.json says {k}={getattr(config, k)}, the record holds {dims[k]}")
    vocab_path = os.path.join(directory, "vocab.json")
    vocab = None
    if os.path.exists(vocab_path):
        with open(vocab_path, "r", encoding="utf-8") as f:
            vocab = f.read()
    return config, weights, vocab, block_size
