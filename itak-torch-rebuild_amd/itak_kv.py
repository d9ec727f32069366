"""Prefix-KV snapshots: the Python mirror of the reference's `itak-kv` crate for this path
(crates/itak-kv/src/snapshot.rs, hash.rs, error.rs), over the C ABI.

`KvSnapshot.capture(cache, fingerprint)` reads a slot back from the device,
`to_bytes` / `from_bytes` are the ITKV v1 wire format, `restore(pool)` /
`restore_checked(pool, geometry, fingerprint)` gather the rows into a fresh slot of a pool.
Encoded snapshots can also go straight between bytes and a slot without an in-memory
snapshot (`capture_bytes`, `restore_bytes`): at 1.5 GiB per 8192-token prefix that is the
path a session start takes.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import numpy as np

from . import _native as N
from .hip_compute import AttentionError, KvCache, KvPool, LayerKind, _raise_last

SNAPSHOT_FORMAT_VERSION = 1  # snapshot.rs:53


class KvError(Exception):
    """itak_kv::KvError (error.rs:13-124): `variant` names the Rust variant."""

    def __init__(self, variant: str, message: str = "", **fields):
        self.variant = variant
        self.fields = fields
        self.message = message
        super().__init__(message or variant)

    def __repr__(self):
        return f"KvError.{self.variant}({self.message!r})"


def _raise_kv(handle):
    lib = N.load()
    info = N.ErrorInfo()
    lib.itak_last_error_info(handle, C.byref(info))
    if N.KV_ERROR_FIRST <= info.code <= N.KV_ERROR_LAST:
        message = (lib.itak_last_error(handle) or b"").decode()
        name = N.STATUS_NAMES[info.code]
        fields = {}
        if name == "UnsupportedVersion":
            fields = {"what": "snapshot", "version": int(info.a)}
        elif name == "Truncated":
            fields = {"what": "snapshot", "expected": int(info.a), "actual": int(info.b)}
        elif name == "ChecksumMismatch":
            fields = {"stored": int(info.a), "computed": int(info.b)}
        elif name == "BadMagic":
            fields = {"what": "snapshot"}
        raise KvError(name, message, **fields)
    try:
        _raise_last(handle)
    except AttentionError as e:  # KvError::Attention(e): "attention: {e}" (error.rs:145)
        raise KvError("Attention", f"attention: {e.message}", source=e) from e


def _check_kv(handle, status: int):
    if status != N.OK:
        _raise_kv(handle)


def prefix_hash(tokens: Sequence[int]) -> int:  # hash.rs:44-46
    t = np.ascontiguousarray(tokens, dtype=np.uint32)
    return int(N.load().itak_kv_prefix_hash(t.ctypes.data, t.size))


def prefix_discriminator(tokens: Sequence[int]) -> int:  # hash.rs:52-54
    t = np.ascontiguousarray(tokens, dtype=np.uint32)
    return int(N.load().itak_kv_prefix_discriminator(t.ctypes.data, t.size))


def checksum(data: bytes) -> int:  # hash.rs:59-61
    buf = np.frombuffer(data, dtype=np.uint8)
    return int(N.load().itak_kv_checksum(buf.ctypes.data if buf.size else None, buf.size))


def checksum_blocks(data: bytes) -> int:
    """The trailer of snapshot version 2 (this library's own): FNV-1a over the FNV-1a sums of
    consecutive 1 MiB blocks, which host threads share."""
    buf = np.frombuffer(data, dtype=np.uint8)
    return int(N.load().itak_kv_checksum_blocks(buf.ctypes.data if buf.size else None, buf.size))


@dataclass
class KvGeometry:
    """itak_kv::KvGeometry (snapshot.rs:57-138)."""
    layers: List[LayerKind]
    num_kv_heads: int
    head_dim: int

    def row_floats(self) -> int:
        return self.num_kv_heads * self.head_dim

    def bytes_per_token(self) -> int:  # snapshot.rs:99-102, saturating
        return min(min(self.row_floats() * 8, 2**64 - 1) * len(self.layers), 2**64 - 1)

    def stored_bytes_for(self, tokens: int) -> int:  # snapshot.rs:109-120
        rows = sum(tokens if k.window() is None else min(tokens, k.window()) for k in self.layers)
        return min(rows * min(self.row_floats() * 8, 2**64 - 1), 2**64 - 1)

    @staticmethod
    def of_cache(cache: KvCache) -> "KvGeometry":  # snapshot.rs:123-137
        return KvGeometry([cache.layer_kind(i) for i in range(cache.layer_count())],
                          cache.num_kv_heads(), cache.head_dim())


@dataclass
class LayerSnapshot:
    """itak_kv::LayerSnapshot (snapshot.rs:144-159): rows oldest first, flattened f32."""
    first_position: int
    keys: np.ndarray
    values: np.ndarray

    def rows(self, row_floats: int) -> int:
        return self.keys.size // row_floats if row_floats else 0


def _header(geometry: KvGeometry, token_count: int, fingerprint: bytes, blocks: int):
    h = N.ItkvHeader(token_count, geometry.num_kv_heads, geometry.head_dim, len(geometry.layers),
                     len(fingerprint), 0, 0)
    layers = (N.ItkvLayer * max(blocks, 1))()
    return h, layers


@dataclass
class KvSnapshot:
    """itak_kv::KvSnapshot (snapshot.rs:163-174): rows as f32, whatever they were encoded as.
    `to_bytes` writes the reference's version 1; bytes of version 2 (f16 rows, this library's
    own, from `capture_bytes(..., elem="f16")`) decode into the same f32 rows exactly."""
    geometry: KvGeometry
    model_fingerprint: str
    token_count: int
    layers: List[LayerSnapshot] = field(default_factory=list)

    def _raw(self):
        fp = self.model_fingerprint.encode()
        h, layers = _header(self.geometry, self.token_count, fp, len(self.layers))
        n = len(self.layers)
        kf, vf = (C.c_uint64 * max(n, 1))(), (C.c_uint64 * max(n, 1))()
        keys, values = (C.c_void_p * max(n, 1))(), (C.c_void_p * max(n, 1))()
        keep = []
        row = self.geometry.row_floats()
        for i, layer in enumerate(self.layers):
            k = np.ascontiguousarray(layer.keys, dtype=np.float32).reshape(-1)
            v = np.ascontiguousarray(layer.values, dtype=np.float32).reshape(-1)
            keep += [k, v]
            kf[i], vf[i] = k.size, v.size
            keys[i], values[i] = k.ctypes.data, v.ctypes.data
            if i < len(self.geometry.layers):
                kind = self.geometry.layers[i]
                layers[i].kind = N.LAYER_GLOBAL if kind.window() is None else N.LAYER_WINDOWED
                layers[i].window = kind.window() or 0
            layers[i].first_position = layer.first_position
            layers[i].rows = layer.rows(row) if row < 2**63 else 0
        return fp, h, layers, n, keys, kf, values, vf, keep

    def validate(self) -> None:  # snapshot.rs:187-236
        fp, h, layers, n, keys, kf, values, vf, keep = self._raw()
        _check_kv(None, N.load().itak_itkv_validate(C.byref(h), layers, n, kf, vf))

    def to_bytes(self) -> bytes:  # snapshot.rs:381-403
        fp, h, layers, n, keys, kf, values, vf, keep = self._raw()
        lib = N.load()
        written = C.c_uint64()
        _check_kv(None, lib.itak_itkv_encode(C.byref(h), fp, layers, n, keys, kf, values, vf, None,
                                             0, C.byref(written)))
        out = np.empty(written.value, dtype=np.uint8)
        _check_kv(None, lib.itak_itkv_encode(C.byref(h), fp, layers, n, keys, kf, values, vf,
                                             out.ctypes.data, out.size, C.byref(written)))
        return out.tobytes()

    @staticmethod
    def from_bytes(data: bytes) -> "KvSnapshot":  # snapshot.rs:405-509
        lib = N.load()
        buf = np.frombuffer(data, dtype=np.uint8)
        h = N.ItkvHeader()
        ptr = buf.ctypes.data if buf.size else C.cast(C.create_string_buffer(1), C.c_void_p)
        status = lib.itak_itkv_decode(ptr, buf.size, C.byref(h), None, 0)
        if status != N.OK:
            info = N.ErrorInfo()
            lib.itak_last_error_info(None, C.byref(info))
            if info.code != 17 or h.layer_count == 0:  # a real refusal, not "capacity too small"
                _raise_kv(None)
        layers = (N.ItkvLayer * max(int(h.layer_count), 1))()
        _check_kv(None, lib.itak_itkv_decode(ptr, buf.size, C.byref(h), layers, h.layer_count))
        kinds, blocks = [], []
        row = int(h.num_kv_heads * h.head_dim)
        for i in range(int(h.layer_count)):
            L = layers[i]
            kinds.append(LayerKind.Global if L.kind == N.LAYER_GLOBAL else LayerKind.windowed(int(L.window)))
            n = int(L.rows) * row
            wire = "<f2" if h.elem == N.ELEM_F16 else "<f4"
            keys = np.frombuffer(data, dtype=wire, count=n, offset=int(L.keys_offset)).astype(np.float32)
            vals = np.frombuffer(data, dtype=wire, count=n, offset=int(L.values_offset)).astype(np.float32)
            blocks.append(LayerSnapshot(int(L.first_position), keys, vals))
        fp = bytes(data[int(h.fingerprint_offset):int(h.fingerprint_offset + h.fingerprint_len)])
        return KvSnapshot(KvGeometry(kinds, int(h.num_kv_heads), int(h.head_dim)), fp.decode(),
                          int(h.token_count), blocks)

    @staticmethod
    def capture(cache: KvCache, model_fingerprint: str) -> "KvSnapshot":  # snapshot.rs:247-302
        return KvSnapshot.from_bytes(capture_bytes(cache, model_fingerprint))

    def restore(self, pool: KvPool) -> KvCache:  # snapshot.rs:321-334
        """A fresh slot of `pool` holding the snapshot (the reference builds a fresh KvCache)."""
        return restore_bytes(pool, self.to_bytes())

    def restore_checked(self, pool: KvPool, expected_geometry: KvGeometry,
                        expected_fingerprint: str) -> KvCache:  # snapshot.rs:351-371
        if self.geometry != expected_geometry:
            raise KvError("GeometryMismatch",
                          f"geometry mismatch: snapshot geometry ({len(self.geometry.layers)} layers, "
                          f"{self.geometry.num_kv_heads} KV heads, head dim {self.geometry.head_dim}) "
                          f"differs from the required geometry ({len(expected_geometry.layers)} "
                          f"layers, {expected_geometry.num_kv_heads} KV heads, head dim "
                          f"{expected_geometry.head_dim})")
        return restore_bytes(pool, self.to_bytes(), expected_fingerprint)


def capture_bytes(cache: KvCache, model_fingerprint: str, elem: str = "f32") -> bytes:
    """KvSnapshot::capture + to_bytes in one pass: device rows straight into ITKV bytes.
    elem="f32" is the reference's version 1; elem="f16" (f16 pools only) writes version 2,
    the pool's own halves: half the size, bit-identical on restore."""
    lib = N.load()
    fn = {"f32": lib.itak_kv_capture_itkv, "f16": lib.itak_kv_capture_itkv_f16}[elem]
    fp = model_fingerprint.encode()
    written = C.c_uint64()
    h = cache.pool._h
    _check_kv(h, fn(h, cache.slot, fp, len(fp), None, 0, C.byref(written)))
    out = np.empty(written.value, dtype=np.uint8)
    _check_kv(h, fn(h, cache.slot, fp, len(fp), out.ctypes.data, out.size, C.byref(written)))
    return out.tobytes()


def restore_bytes(pool: KvPool, data, expected_fingerprint: Optional[str] = None) -> KvCache:
    """KvSnapshot::from_bytes + restore_checked into a fresh slot of `pool`. `data` is bytes
    or a uint8 numpy array (which may wrap pinned host memory)."""
    lib = N.load()
    buf = data if isinstance(data, np.ndarray) else np.frombuffer(data, dtype=np.uint8)
    cache = pool.acquire()
    fp = expected_fingerprint.encode() if expected_fingerprint is not None else None
    status = lib.itak_kv_restore_itkv(pool._h, cache.slot, buf.ctypes.data, buf.size, fp,
                                      len(fp) if fp is not None else 0)
    if status != N.OK:
        try:
            _raise_kv(pool._h)
        finally:
            cache.release_slot()
    return cache
