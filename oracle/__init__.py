"""ctypes front end of the CPU oracle (test infrastructure, never the product path).

The C library restates the reference's Rust CPU path
(crates/attention/src/{attention,cache,error}.rs, crates/cpu-compute/src/cpu.rs:506-655,
the f16 mirror in crates/wgpu-compute/src/kernels/k1_q4k_gemv.rs:285-329). This module
gives it the names the Rust API uses so the KATs read like the reference's tests.
Only tests, the smoke check and the benchmark's cpu_baseline leg import it.
"""
from __future__ import annotations

import ctypes as C
import math
import os
import subprocess
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libitak_oracle.so")


def build(force: bool = False) -> str:
    """Compile the oracle with the recipe in the Makefile next to this file."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "-B", "-s"])
    else:
        subprocess.check_call(["make", "-C", _HERE, "-s"])
    return _LIB_PATH


class _Err(C.Structure):
    _fields_ = [
        ("code", C.c_int32),
        ("what", C.c_char * 96),
        ("a", C.c_uint64),
        ("b", C.c_uint64),
        ("c", C.c_uint64),
        ("d", C.c_uint64),
        ("message", C.c_char * 512),
    ]


class _Checkpoint(C.Structure):
    _fields_ = [
        ("cache_id", C.c_uint64),
        ("serial", C.c_uint64),
        ("max_round_tokens", C.c_uint64),
        ("saved_bytes", C.c_uint64),
        ("layer_count", C.c_uint64),
        ("bases", C.POINTER(C.c_uint64)),
    ]


class _Stats(C.Structure):
    _fields_ = [
        ("layer", C.c_uint64),
        ("window", C.c_uint64),
        ("appended", C.c_uint64),
        ("stored", C.c_uint64),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        f32p = C.POINTER(C.c_float)
        u64p = C.POINTER(C.c_uint64)
        L.orc_f32_to_f16_bits.restype = C.c_uint16
        L.orc_f32_to_f16_bits.argtypes = [C.c_float]
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_f16_array.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.orc_f16_to_f32_array.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.orc_round_through_f16.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.orc_fnv1a64.restype = C.c_uint64
        L.orc_fnv1a64.argtypes = [C.c_void_p, C.c_size_t]
        L.orc_prefix_hash.restype = C.c_uint64
        L.orc_prefix_hash.argtypes = [C.c_void_p, C.c_size_t]
        L.orc_rope_half_split.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint64, C.c_float]
        L.orc_rope_half_split_partial.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t,
                                                  C.c_uint64, C.c_float]
        L.orc_rope_interleaved.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t,
                                           C.c_uint64, C.c_float]
        L.orc_rms_norm.argtypes = [C.c_void_p, C.c_void_p, C.c_float, C.c_size_t, C.c_void_p]
        L.orc_sigmoid.restype = C.c_float
        L.orc_sigmoid.argtypes = [C.c_float]
        L.orc_logit_softcap.restype = C.c_float
        L.orc_logit_softcap.argtypes = [C.c_float, C.c_float]
        L.orc_cache_new.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64,
                                    C.c_int, C.POINTER(C.c_void_p), C.POINTER(_Err)]
        L.orc_cache_free.argtypes = [C.c_void_p]
        for name in ("orc_cache_layer_count", "orc_cache_num_kv_heads", "orc_cache_head_dim"):
            getattr(L, name).restype = C.c_uint64
            getattr(L, name).argtypes = [C.c_void_p]
        for name in ("orc_cache_layer_window", "orc_cache_stored_len", "orc_cache_next_position",
                     "orc_view_len"):
            getattr(L, name).argtypes = [C.c_void_p, C.c_uint64, u64p, C.POINTER(_Err)]
        L.orc_cache_append.argtypes = [C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint64, C.c_void_p,
                                       C.c_uint64, C.c_uint64, C.POINTER(_Err)]
        L.orc_cache_restore_bulk.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_void_p,
                                             C.c_uint64, C.c_void_p, C.c_uint64, C.POINTER(_Err)]
        L.orc_cache_stats.argtypes = [C.c_void_p, C.POINTER(_Stats)]
        L.orc_cache_checkpoint_active.argtypes = [C.c_void_p]
        L.orc_cache_checkpoint.argtypes = [C.c_void_p, C.c_uint64, C.POINTER(_Checkpoint),
                                           C.POINTER(_Err)]
        L.orc_cache_rewind_to.argtypes = [C.c_void_p, C.POINTER(_Checkpoint), C.c_uint64,
                                          C.POINTER(_Err)]
        L.orc_cache_release.argtypes = [C.c_void_p, C.POINTER(_Checkpoint), C.POINTER(_Err)]
        L.orc_checkpoint_free.argtypes = [C.POINTER(_Checkpoint)]
        L.orc_view_position_at.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, u64p]
        L.orc_view_key.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64,
                                   C.POINTER(f32p)]
        L.orc_view_value.argtypes = L.orc_view_key.argtypes
        L.orc_gqa_attention.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_void_p,
                                        C.c_uint64, C.c_void_p, C.c_uint64, C.c_float, C.c_float,
                                        C.c_int, C.c_void_p, C.POINTER(_Err)]
        L.orc_attention_step.argtypes = [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p,
                                         C.c_uint64, C.c_uint64, C.c_uint64, C.c_float, C.c_float,
                                         C.c_int, C.c_void_p, C.POINTER(_Err)]
        _lib = L
    return _lib


# ---------------------------------------------------------------------------
# Errors: one class, variant name + fields, comparable like the Rust enum.

_VARIANTS = {
    1: ("ZeroDimension", ("what",)),
    2: ("InvalidWindow", ("window",)),
    3: ("SizeOverflow", ("what",)),
    4: ("ShapeMismatch", ("what", "expected", "actual")),
    5: ("InvalidLayer", ("layer", "layer_count")),
    6: ("OutOfOrderPosition", ("layer", "expected", "actual")),
    7: ("NonDivisibleHeads", ("num_q_heads", "num_kv_heads")),
    8: ("NoVisibleKeys", ("position",)),
    9: ("CheckpointBusy", ()),
    10: ("StaleCheckpoint", ("checkpoint",)),
    11: ("CheckpointTooDeep", ("max_round_tokens", "window")),
    12: ("CheckpointRangeExceeded", ("layer", "position", "limit")),
    13: ("BulkRestoreNotFresh", ("layer", "appended")),
    14: ("RewindOutOfRange", ("layer", "base", "appended", "target")),
    15: ("StepFailed", ("what",)),
}


class AttentionError(Exception):
    """Mirror of attention::AttentionError (crates/attention/src/error.rs:9-127)."""

    def __init__(self, variant: str, **fields):
        self.variant = variant
        self.fields = fields
        self.message = fields.pop("_message", "")
        super().__init__(self.message or f"{variant} {fields}")

    def __eq__(self, other):
        return (isinstance(other, AttentionError) and self.variant == other.variant
                and self.fields == other.fields)

    def __hash__(self):
        return hash((self.variant, tuple(sorted(self.fields.items()))))

    def __repr__(self):
        inner = ", ".join(f"{k}={v!r}" for k, v in self.fields.items())
        return f"AttentionError.{self.variant}({inner})"


def error_from_fields(code: int, what: str, nums: Sequence[int], message: str) -> AttentionError:
    variant, names = _VARIANTS[code]
    fields = {}
    it = iter(nums)
    for n in names:
        fields[n] = what if n == "what" else int(next(it))
    return AttentionError(variant, _message=message, **fields)


def _raise(err: _Err):
    raise error_from_fields(err.code, err.what.decode(), (err.a, err.b, err.c, err.d),
                            err.message.decode())


def Err(variant: str, **fields) -> AttentionError:
    """Spell an expected refusal the way the Rust tests do."""
    return AttentionError(variant, **fields)


# ---------------------------------------------------------------------------
# Scalars and arrays.

def f32_to_f16_bits(x) -> int:
    return int(lib().orc_f32_to_f16_bits(C.c_float(float(np.float32(x)))))


def f32_bits_to_f16_bits(bits: int) -> int:
    x = np.array([bits], dtype=np.uint32).view(np.float32)
    out = np.empty(1, dtype=np.uint16)
    lib().orc_f32_to_f16_array(x.ctypes.data, out.ctypes.data, 1)
    return int(out[0])


def f16_to_f32(bits: int) -> np.float32:
    src = np.array([bits], dtype=np.uint16)
    out = np.empty(1, dtype=np.float32)
    lib().orc_f16_to_f32_array(src.ctypes.data, out.ctypes.data, 1)
    return out[0]


def f32_to_f16_array(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_f32_to_f16_array(x.ctypes.data, out.ctypes.data, x.size)
    return out


def f16_to_f32_array(bits: np.ndarray) -> np.ndarray:
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(bits.shape, dtype=np.float32)
    lib().orc_f16_to_f32_array(bits.ctypes.data, out.ctypes.data, bits.size)
    return out


def round_through_f16(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().orc_round_through_f16(x.ctypes.data, out.ctypes.data, x.size)
    return out


def checksum(data: bytes) -> int:
    buf = np.frombuffer(data, dtype=np.uint8)
    return int(lib().orc_fnv1a64(buf.ctypes.data if buf.size else None, buf.size))


def prefix_hash(tokens: Sequence[int]) -> int:
    arr = np.asarray(tokens, dtype=np.uint32)
    return int(lib().orc_prefix_hash(arr.ctypes.data if arr.size else None, arr.size))


def rope_half_split(x: np.ndarray, position: int, base: float) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().orc_rope_half_split(x.ctypes.data, out.ctypes.data, x.size, position, base)
    return out


def rope_rows(x: np.ndarray, first_position: int, base: float) -> np.ndarray:
    """Rotate rows [n][heads][head_dim]; row i sits at position first_position + i."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    n, heads, d = x.shape
    half = d // 2
    pos = (first_position + np.arange(n, dtype=np.float64))[:, None]
    i = np.arange(half, dtype=np.float64)[None, :]
    angle = pos * np.power(np.float64(np.float32(base)), -(2.0 * i) / d)
    s, c = np.sin(angle)[:, None, :], np.cos(angle)[:, None, :]
    a, b = x[..., :half].astype(np.float64), x[..., half:].astype(np.float64)
    out = np.empty_like(x)
    out[..., :half] = (a * c - b * s).astype(np.float32)
    out[..., half:] = (a * s + b * c).astype(np.float32)
    return out


def rope_interleaved(x: np.ndarray, position: int, base: float, rotary_dim: Optional[int] = None) -> np.ndarray:
    """torch_math::rope_interleaved(_partial) (rope_interleaved.rs:65-116) on one head row."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().orc_rope_interleaved(x.ctypes.data, out.ctypes.data, x.size, rotary_dim or x.size,
                               position, base)
    return out


def rope_half_split_partial(x: np.ndarray, position: int, base: float, rotary_dim: Optional[int] = None) -> np.ndarray:
    """torch_math::rope(_partial) (rope.rs:63-116) on one head row."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().orc_rope_half_split_partial(x.ctypes.data, out.ctypes.data, x.size, rotary_dim or x.size,
                                      position, base)
    return out


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """torch_math::rms_norm (norm.rs:21-52) on one row."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(weight, dtype=np.float32)
    assert x.size == w.size and x.size > 0
    out = np.empty_like(x)
    lib().orc_rms_norm(x.ctypes.data, w.ctypes.data, eps, x.size, out.ctypes.data)
    return out


def sigmoid(x: float) -> float:
    """cpu-compute/src/cpu.rs:162-169."""
    return float(lib().orc_sigmoid(C.c_float(x)))


def attn_gate(attn_out: np.ndarray, gate: np.ndarray) -> np.ndarray:
    """CpuCompute::attn_gate (cpu.rs:657-673): a * sigmoid(g), f32."""
    a = np.ascontiguousarray(attn_out, dtype=np.float32).reshape(-1)
    g = np.ascontiguousarray(gate, dtype=np.float32).reshape(-1)
    assert a.size == g.size
    s = np.array([sigmoid(float(v)) for v in g], dtype=np.float32)
    return (a * s).astype(np.float32)


def attention_prep(rows: np.ndarray, heads: int, head_dim: int, first_position: int,
                   norm_weight: Optional[np.ndarray], eps: float, rope_base: float,
                   interleaved: bool = True, rotary_dim: Optional[int] = None) -> np.ndarray:
    """What one of Q or K goes through between its projection and attention: per-head RMSNorm
    (muse-glimmer/src/model.rs:445-451 -> CpuCompute::rms_norm, cpu.rs:445-475) and then RoPE per
    head at the row's position (cpu.rs:598-622, rope_row cpu.rs:398-418). norm_weight None skips
    the norm, rope_base 0 the rotation (a global, NoPE layer). rows: [n][heads*head_dim]."""
    x = np.ascontiguousarray(rows, dtype=np.float32).reshape(-1, heads, head_dim)
    out = np.empty_like(x)
    for r in range(x.shape[0]):
        for h in range(heads):
            row = x[r, h]
            if norm_weight is not None:
                row = rms_norm(row, norm_weight, eps)
            if rope_base > 0:
                fn = rope_interleaved if interleaved else rope_half_split_partial
                row = fn(row, first_position + r, rope_base, rotary_dim)
            out[r, h] = row
    return out.reshape(x.shape[0], heads * head_dim)


def logit_softcap(x: float, cap: float) -> float:
    return float(lib().orc_logit_softcap(C.c_float(x), C.c_float(cap)))


# ---------------------------------------------------------------------------
# LayerKind / AttentionParams.

@dataclass(frozen=True)
class LayerKind:
    """attention::LayerKind (cache.rs:36-66): `window is None` means Global."""

    window_size: Optional[int] = None
    is_windowed: bool = False

    @staticmethod
    def windowed(window: int) -> "LayerKind":
        if window == 0:
            raise AttentionError("InvalidWindow", window=0)
        return LayerKind(window, True)

    @staticmethod
    def Windowed(window: int) -> "LayerKind":
        """The struct literal: no validation, as `LayerKind::Windowed { window }` in Rust."""
        return LayerKind(window, True)

    def window(self) -> Optional[int]:
        return self.window_size if self.is_windowed else None


LayerKind.Global = LayerKind(None, False)


def glimmer_layer_pattern() -> List[LayerKind]:
    """cache.rs:72-84: 52 layers, global at 3, 7, ..., 51, window 2048 elsewhere."""
    return [LayerKind.Global if i % 4 == 3 else LayerKind.Windowed(2048) for i in range(52)]


@dataclass(frozen=True)
class AttentionParams:
    """attention::AttentionParams (attention.rs:17-38) plus the softcap extension."""

    scale: Optional[float] = None
    softcap: float = 0.0

    @staticmethod
    def new() -> "AttentionParams":
        return AttentionParams()

    @staticmethod
    def with_scale(scale: float) -> "AttentionParams":
        return AttentionParams(scale=scale)

    def scale_for(self, head_dim: int) -> np.float32:
        if self.scale is not None:
            return np.float32(self.scale)
        return np.float32(1.0) / np.sqrt(np.float32(head_dim))


def kv_head_for_query_head(q_head: int, num_q_heads: int, num_kv_heads: int) -> int:
    """attention.rs:43-72."""
    if num_kv_heads == 0:
        raise AttentionError("ZeroDimension", what="num_kv_heads")
    if num_q_heads == 0:
        raise AttentionError("ZeroDimension", what="num_q_heads")
    if num_q_heads % num_kv_heads != 0:
        raise AttentionError("NonDivisibleHeads", num_q_heads=num_q_heads,
                             num_kv_heads=num_kv_heads)
    if q_head >= num_q_heads:
        raise AttentionError("ShapeMismatch", what="q_head", expected=num_q_heads, actual=q_head)
    return q_head // (num_q_heads // num_kv_heads)


# ---------------------------------------------------------------------------
# KvCache / CacheView / Checkpoint.

@dataclass
class LayerStats:
    layer: int
    kind: LayerKind
    appended: int
    stored: int


class Checkpoint:
    def __init__(self, raw: _Checkpoint):
        self._raw = raw
        self._bases = [int(raw.bases[i]) for i in range(raw.layer_count)]

    def base(self, layer: int) -> Optional[int]:
        return self._bases[layer] if 0 <= layer < len(self._bases) else None

    def bases(self) -> List[int]:
        return list(self._bases)

    def max_round_tokens(self) -> int:
        return int(self._raw.max_round_tokens)

    def saved_bytes(self) -> int:
        return int(self._raw.saved_bytes)

    def __del__(self):
        try:
            lib().orc_checkpoint_free(C.byref(self._raw))
        except Exception:
            pass


class CacheView:
    def __init__(self, cache: "KvCache", layer: int):
        self._c = cache
        self._layer = layer

    def kind(self) -> LayerKind:
        return self._c.layer_kind(self._layer)

    def window(self) -> Optional[int]:
        return self.kind().window()

    def num_kv_heads(self) -> int:
        return self._c.num_kv_heads()

    def head_dim(self) -> int:
        return self._c.head_dim()

    def len(self) -> int:
        return self._c.stored_len(self._layer)

    def __len__(self) -> int:
        return self.len()

    def is_empty(self) -> bool:
        return self.len() == 0

    def position_at(self, visible_index: int) -> Optional[int]:
        pos = C.c_uint64()
        ok = lib().orc_view_position_at(self._c._h, self._layer, visible_index, C.byref(pos))
        return int(pos.value) if ok else None

    def _row(self, fn, visible_index: int, kv_head: int) -> Optional[np.ndarray]:
        ptr = C.POINTER(C.c_float)()
        if not fn(self._c._h, self._layer, visible_index, kv_head, C.byref(ptr)):
            return None
        return np.ctypeslib.as_array(ptr, shape=(self._c.head_dim(),)).copy()

    def key(self, visible_index: int, kv_head: int) -> Optional[np.ndarray]:
        return self._row(lib().orc_view_key, visible_index, kv_head)

    def value(self, visible_index: int, kv_head: int) -> Optional[np.ndarray]:
        return self._row(lib().orc_view_value, visible_index, kv_head)

    def rows(self):
        """(positions, keys[n][kv_heads][d], values[n][kv_heads][d]) of every visible entry."""
        n, h, d = self.len(), self.num_kv_heads(), self.head_dim()
        pos = np.empty(n, dtype=np.int64)
        keys = np.empty((n, h, d), dtype=np.float32)
        vals = np.empty((n, h, d), dtype=np.float32)
        for vi in range(n):
            pos[vi] = self.position_at(vi)
            for head in range(h):
                keys[vi, head] = self.key(vi, head)
                vals[vi, head] = self.value(vi, head)
        return pos, keys, vals


class KvCache:
    """attention::KvCache (cache.rs:308-834). `store_f16=True` is the f16-KV twin:
    every stored element is rounded through f16 and all math stays f32."""

    def __init__(self, pattern: Sequence[LayerKind], num_kv_heads: int, head_dim: int,
                 store_f16: bool = False):
        kinds = np.array([1 if k.is_windowed else 0 for k in pattern], dtype=np.uint8)
        windows = np.array([(k.window_size or 0) if k.is_windowed else 0 for k in pattern],
                           dtype=np.uint64)
        self._pattern = list(pattern)
        h = C.c_void_p()
        err = _Err()
        rc = lib().orc_cache_new(kinds.ctypes.data if len(kinds) else None,
                                 windows.ctypes.data if len(windows) else None, len(pattern),
                                 num_kv_heads, head_dim, int(store_f16), C.byref(h), C.byref(err))
        if rc != 0:
            _raise(err)
        self._h = h
        # Kept on the object: at interpreter shutdown module globals may be gone before a
        # cache that is still alive is collected.
        self._free = lib().orc_cache_free

    @staticmethod
    def new(pattern, num_kv_heads, head_dim, store_f16=False) -> "KvCache":
        return KvCache(pattern, num_kv_heads, head_dim, store_f16)

    def __del__(self):
        h, free = getattr(self, "_h", None), getattr(self, "_free", None)
        if h and free:
            free(h)
            self._h = None

    def layer_count(self) -> int:
        return int(lib().orc_cache_layer_count(self._h))

    def num_kv_heads(self) -> int:
        return int(lib().orc_cache_num_kv_heads(self._h))

    def head_dim(self) -> int:
        return int(lib().orc_cache_head_dim(self._h))

    def _u64(self, fn, layer: int) -> int:
        out = C.c_uint64()
        err = _Err()
        if fn(self._h, layer, C.byref(out), C.byref(err)) != 0:
            _raise(err)
        return int(out.value)

    def layer_kind(self, layer: int) -> LayerKind:
        self._u64(lib().orc_cache_layer_window, layer)
        return self._pattern[layer]

    def stored_len(self, layer: int) -> int:
        return self._u64(lib().orc_cache_stored_len, layer)

    def next_position(self, layer: int) -> int:
        return self._u64(lib().orc_cache_next_position, layer)

    def append(self, layer: int, k, v, position: int) -> None:
        k = np.ascontiguousarray(k, dtype=np.float32).reshape(-1)
        v = np.ascontiguousarray(v, dtype=np.float32).reshape(-1)
        err = _Err()
        if lib().orc_cache_append(self._h, layer, k.ctypes.data, k.size, v.ctypes.data, v.size,
                                  position, C.byref(err)) != 0:
            _raise(err)

    def restore_bulk(self, layer: int, first_position: int, keys, values) -> None:
        keys = np.ascontiguousarray(keys, dtype=np.float32).reshape(-1)
        values = np.ascontiguousarray(values, dtype=np.float32).reshape(-1)
        err = _Err()
        if lib().orc_cache_restore_bulk(self._h, layer, first_position, keys.ctypes.data, keys.size,
                                        values.ctypes.data, values.size, C.byref(err)) != 0:
            _raise(err)

    def view(self, layer: int) -> CacheView:
        self._u64(lib().orc_cache_stored_len, layer)
        return CacheView(self, layer)

    def stats(self) -> List[LayerStats]:
        n = self.layer_count()
        raw = (_Stats * n)()
        lib().orc_cache_stats(self._h, raw)
        return [LayerStats(int(s.layer), self._pattern[i], int(s.appended), int(s.stored))
                for i, s in enumerate(raw)]

    def checkpoint_active(self) -> bool:
        return bool(lib().orc_cache_checkpoint_active(self._h))

    def checkpoint(self, max_round_tokens: int) -> Checkpoint:
        raw = _Checkpoint()
        err = _Err()
        if lib().orc_cache_checkpoint(self._h, max_round_tokens, C.byref(raw), C.byref(err)) != 0:
            _raise(err)
        return Checkpoint(raw)

    def rewind_to(self, cp: Checkpoint, target: int) -> None:
        err = _Err()
        if lib().orc_cache_rewind_to(self._h, C.byref(cp._raw), target, C.byref(err)) != 0:
            _raise(err)

    def release(self, cp: Checkpoint) -> None:
        err = _Err()
        if lib().orc_cache_release(self._h, C.byref(cp._raw), C.byref(err)) != 0:
            _raise(err)


def gqa_attention(q, num_queries: int, num_q_heads: int, query_positions: Sequence[int],
                  view: CacheView, params: AttentionParams = AttentionParams(),
                  threads: int = 1) -> np.ndarray:
    """attention::gqa_attention (attention.rs:104-215); returns a flat f32 array."""
    q = np.ascontiguousarray(q, dtype=np.float32).reshape(-1)
    pos = np.asarray(query_positions, dtype=np.uint64).reshape(-1)
    out = np.zeros(q.size, dtype=np.float32)
    err = _Err()
    scale = math.nan if params.scale is None else float(params.scale)
    rc = lib().orc_gqa_attention(q.ctypes.data, q.size, num_queries, num_q_heads,
                                 pos.ctypes.data if pos.size else None, pos.size, view._c._h,
                                 view._layer, scale, float(params.softcap), threads,
                                 out.ctypes.data if out.size else None, C.byref(err))
    if rc != 0:
        _raise(err)
    return out[: num_queries * num_q_heads * view.head_dim()] if num_queries else out[:0]


def attention_step(cache: KvCache, layer: int, q, k, v, num_q_heads: int, start_position: int,
                   params: AttentionParams = AttentionParams(), threads: int = 1) -> np.ndarray:
    """The per-row append-then-attend loop of CpuCompute::attention (cpu.rs:558-646)."""
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    q_width = num_q_heads * cache.head_dim()
    rows = q.size // q_width
    out = np.zeros(q.size, dtype=np.float32)
    err = _Err()
    scale = math.nan if params.scale is None else float(params.scale)
    rc = lib().orc_attention_step(cache._h, layer, q.ctypes.data, k.ctypes.data, v.ctypes.data,
                                  rows, num_q_heads, start_position, scale, float(params.softcap),
                                  threads, out.ctypes.data, C.byref(err))
    if rc != 0:
        _raise(err)
    return out


def compute_attention(cache: KvCache, layer: int, q, k, v, num_q_heads: int, start_position: int,
                      rope_freq_base_swa: float, params: AttentionParams = AttentionParams(),
                      threads: int = 1) -> np.ndarray:
    """The body of CpuCompute::attention (cpu.rs:586-646): on a sliding-window layer every
    row's Q and K heads are rotated with the interleaved RoPE at the SWA base and the row's
    own position (rope_row, cpu.rs:398-418); global layers pass through. Then the per-row
    append-then-attend loop."""
    d = cache.head_dim()
    q = np.ascontiguousarray(q, dtype=np.float32).reshape(-1, num_q_heads * d)
    k = np.ascontiguousarray(k, dtype=np.float32).reshape(-1, cache.num_kv_heads() * d)
    if cache.layer_kind(layer).window() is not None:
        q = attention_prep(q, num_q_heads, d, start_position, None, 0.0, rope_freq_base_swa)
        k = attention_prep(k, cache.num_kv_heads(), d, start_position, None, 0.0, rope_freq_base_swa)
    return attention_step(cache, layer, q, k, v, num_q_heads, start_position, params, threads)

