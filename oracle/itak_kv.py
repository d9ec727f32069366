"""CPU restatement of the reference's prefix-snapshot crate for the oracle: the ITKV v1
wire format, KvSnapshot validate / capture / restore, and the FNV-1a hashes
(crates/itak-kv/src/snapshot.rs, hash.rs, error.rs). Test infrastructure only: nothing
the library ships imports this module.

Pinned by the reference's own cases (ported in tests/test_oracle_snapshot.py): the byte
layout table snapshot.rs:13-29, bytes_round_trip / restore_rebuilds_the_same_views /
restore_can_continue_appending / capture_refuses_a_divergent_cache /
decode_refuses_corruption / restore_checked_refuses_geometry_and_fingerprint and the
forged-header regressions (snapshot.rs:606-861), the sizing figures 106,496 / 272,629,760 /
3,653,238,784 (snapshot.rs:844-861), FNV offset basis and order sensitivity
(hash.rs:63-87), plus a hand-assembled byte string for the layout; prefix_discriminator by
literals folded by hand from the alternate offset basis (the empty input, one token, two
tokens: tests/test_oracle_snapshot.py).
"""
from __future__ import annotations

import struct
from dataclasses import dataclass, field
from typing import List, Sequence

import numpy as np

from . import AttentionError, KvCache, LayerKind

MAGIC = b"ITKV"                      # snapshot.rs:47
LAYER_HEADER_LEN = 28                # snapshot.rs:51
SNAPSHOT_FORMAT_VERSION = 1          # snapshot.rs:53
FNV_OFFSET = 0xCBF29CE484222325      # hash.rs:14
FNV_PRIME = 0x00000100000001B3       # hash.rs:16
ALT_OFFSET = 0x84222325CBF29CE4      # hash.rs:21
_M64 = (1 << 64) - 1
USIZE_MAX = _M64


class KvError(Exception):
    """itak_kv::KvError (error.rs:13-124) with its Display text (error.rs:141-188)."""

    def __init__(self, variant: str, message: str, **fields):
        self.variant, self.message, self.fields = variant, message, fields
        super().__init__(message)


def _inconsistent(detail: str) -> KvError:  # snapshot.rs:513-515
    return KvError("InconsistentSnapshot", f"inconsistent snapshot: {detail}")


def fnv1a(data: bytes, basis: int) -> int:  # hash.rs:24-31
    h = basis
    for b in data:
        h = ((h ^ b) * FNV_PRIME) & _M64
    return h


def checksum(data: bytes) -> int:  # hash.rs:59-61
    return fnv1a(data, FNV_OFFSET)


def prefix_hash(tokens: Sequence[int]) -> int:  # hash.rs:44-46
    return fnv1a(b"".join(struct.pack("<I", t) for t in tokens), FNV_OFFSET)


def prefix_discriminator(tokens: Sequence[int]) -> int:  # hash.rs:52-54
    return fnv1a(b"".join(struct.pack("<I", t) for t in tokens), ALT_OFFSET)


def _kind_debug(kind: LayerKind) -> str:
    w = kind.window()
    return "Global" if w is None else f"Windowed {{ window: {w} }}"


@dataclass
class KvGeometry:  # snapshot.rs:57-138
    layers: List[LayerKind]
    num_kv_heads: int
    head_dim: int

    def row_floats(self) -> int:
        return self.num_kv_heads * self.head_dim

    def row_floats_checked(self) -> int:  # snapshot.rs:84-94
        row = self.num_kv_heads * self.head_dim
        if row > USIZE_MAX:
            raise _inconsistent(f"KV row width overflows: {self.num_kv_heads} heads of dim "
                                f"{self.head_dim} have no usize product")
        return row

    def bytes_per_token(self) -> int:  # snapshot.rs:99-102
        per_layer = min(self.row_floats() * 8, _M64)
        return min(per_layer * len(self.layers), _M64)

    def stored_bytes_for(self, tokens: int) -> int:  # snapshot.rs:109-120
        per_row = min(self.row_floats() * 8, _M64)
        rows = 0
        for kind in self.layers:
            w = kind.window()
            rows = min(rows + (tokens if w is None else min(tokens, w)), _M64)
        return min(rows * per_row, _M64)

    @staticmethod
    def of_cache(cache: KvCache) -> "KvGeometry":  # snapshot.rs:123-137
        return KvGeometry([cache.layer_kind(i) for i in range(cache.layer_count())],
                          cache.num_kv_heads(), cache.head_dim())


@dataclass
class LayerSnapshot:  # snapshot.rs:144-159
    first_position: int
    keys: np.ndarray
    values: np.ndarray

    def rows(self, row_floats: int) -> int:
        return len(self.keys) // row_floats if row_floats else 0


@dataclass
class KvSnapshot:  # snapshot.rs:163-174
    geometry: KvGeometry
    model_fingerprint: str
    token_count: int
    layers: List[LayerSnapshot] = field(default_factory=list)

    def validate(self) -> None:  # snapshot.rs:187-236
        g = self.geometry
        if len(self.layers) != len(g.layers):
            raise _inconsistent(f"snapshot carries {len(self.layers)} layer blocks but its geometry "
                                f"has {len(g.layers)} layers")
        if g.num_kv_heads == 0 or g.head_dim == 0:
            raise _inconsistent("geometry has a zero KV head count or head dimension")
        row = g.row_floats_checked()
        for index, (kind, layer) in enumerate(zip(g.layers, self.layers)):
            w = kind.window()
            expected_rows = self.token_count if w is None else min(self.token_count, w)
            expected_first = self.token_count - expected_rows
            if layer.first_position != expected_first:
                raise _inconsistent(f"layer {index}: first stored position is "
                                    f"{layer.first_position} but {expected_first} follows from "
                                    f"token count {self.token_count} and kind {_kind_debug(kind)}")
            expected_floats = expected_rows * row
            if expected_floats > USIZE_MAX:
                raise _inconsistent(f"layer {index}: {expected_rows} rows of {row} floats overflow "
                                    "the float count")
            if len(layer.keys) != expected_floats or len(layer.values) != expected_floats:
                raise _inconsistent(f"layer {index}: holds {len(layer.keys)} key and "
                                    f"{len(layer.values)} value floats but {expected_rows} rows of "
                                    f"{row} floats were expected")

    @staticmethod
    def capture(cache: KvCache, model_fingerprint: str) -> "KvSnapshot":  # snapshot.rs:247-302
        geometry = KvGeometry.of_cache(cache)
        token_count = cache.next_position(0)
        layers = []
        for index in range(len(geometry.layers)):
            appended = cache.next_position(index)
            if appended != token_count:
                raise KvError("IncoherentCache",
                              f"incoherent cache: layer 0 has appended {token_count} positions but "
                              f"layer {index} has appended {appended}; a snapshot is one sequence")
            _, keys, values = cache.view(index).rows()
            visible = len(keys)
            layers.append(LayerSnapshot(token_count - visible,
                                        np.asarray(keys, dtype=np.float32).reshape(-1),
                                        np.asarray(values, dtype=np.float32).reshape(-1)))
        snapshot = KvSnapshot(geometry, model_fingerprint, token_count, layers)
        snapshot.validate()
        return snapshot

    def restore(self, store_f16: bool = False) -> KvCache:  # snapshot.rs:321-334
        self.validate()
        g = self.geometry
        try:
            cache = KvCache.new(g.layers, g.num_kv_heads, g.head_dim, store_f16=store_f16)
            for index, layer in enumerate(self.layers):
                row = g.row_floats()
                cache.restore_bulk(index, layer.first_position, layer.keys.reshape(-1, row),
                                   layer.values.reshape(-1, row))
        except AttentionError as e:
            raise KvError("Attention", f"attention: {e}", source=e) from e
        return cache

    def restore_checked(self, expected_geometry: KvGeometry, expected_fingerprint: str,
                        store_f16: bool = False) -> KvCache:  # snapshot.rs:351-371
        if self.geometry != expected_geometry:
            g, e = self.geometry, expected_geometry
            raise KvError("GeometryMismatch",
                          f"geometry mismatch: snapshot geometry ({len(g.layers)} layers, "
                          f"{g.num_kv_heads} KV heads, head dim {g.head_dim}) differs from the "
                          f"required geometry ({len(e.layers)} layers, {e.num_kv_heads} KV heads, "
                          f"head dim {e.head_dim})")
        if self.model_fingerprint != expected_fingerprint:
            raise KvError("FingerprintMismatch",
                          f"model fingerprint mismatch: need {expected_fingerprint}, snapshot "
                          f"carries {self.model_fingerprint}",
                          expected=expected_fingerprint, actual=self.model_fingerprint)
        return self.restore(store_f16)

    def to_bytes(self) -> bytes:  # snapshot.rs:381-403
        self.validate()
        out = bytearray()
        out += MAGIC
        out += struct.pack("<I", SNAPSHOT_FORMAT_VERSION)
        fingerprint = self.model_fingerprint.encode("utf-8")
        out += struct.pack("<I", len(fingerprint) & 0xFFFFFFFF)
        out += fingerprint
        out += struct.pack("<Q", self.token_count)
        out += struct.pack("<I", self.geometry.num_kv_heads & 0xFFFFFFFF)
        out += struct.pack("<I", self.geometry.head_dim & 0xFFFFFFFF)
        out += struct.pack("<I", len(self.geometry.layers) & 0xFFFFFFFF)
        row = self.geometry.row_floats()
        for kind, layer in zip(self.geometry.layers, self.layers):
            w = kind.window()
            out += bytes([0 if w is None else 1, 0, 0, 0])
            out += struct.pack("<Q", 0 if w is None else w)
            out += struct.pack("<Q", layer.first_position)
            out += struct.pack("<Q", layer.rows(row))
        for layer in self.layers:
            out += np.asarray(layer.keys, dtype="<f4").tobytes()
            out += np.asarray(layer.values, dtype="<f4").tobytes()
        out += struct.pack("<Q", checksum(bytes(out)))
        return bytes(out)

    @staticmethod
    def from_bytes(data: bytes) -> "KvSnapshot":  # snapshot.rs:405-509
        r = _Reader(data)
        if r.take(4) != MAGIC:
            raise KvError("BadMagic", "snapshot: bad magic", what="snapshot")
        version = r.u32()
        if version != SNAPSHOT_FORMAT_VERSION:
            raise KvError("UnsupportedVersion", f"snapshot: unsupported format version {version}",
                          what="snapshot", version=version)
        fingerprint_bytes = r.take(r.u32())
        try:
            model_fingerprint = fingerprint_bytes.decode("utf-8")
        except UnicodeDecodeError:
            raise _inconsistent("model fingerprint is not valid UTF-8") from None
        token_count = r.u64()
        num_kv_heads = r.u32()
        head_dim = r.u32()
        layer_count = r.u32()
        if layer_count > r.remaining() // LAYER_HEADER_LEN:
            raise _inconsistent(f"snapshot declares {layer_count} layers but only {r.remaining()} "
                                "bytes remain, not enough for the layer headers alone")
        kinds, blocks = [], []
        for _ in range(layer_count):
            tag = r.take(1)[0]
            if r.take(3) != b"\0\0\0":
                raise _inconsistent("layer header reserved bytes are not zero")
            window = r.u64()
            first_position = r.u64()
            row_count = r.u64()
            if tag == 0:
                kind = LayerKind.Global
            elif tag == 1:
                if window == 0:
                    raise _inconsistent("windowed layer carries a zero window")
                kind = LayerKind.Windowed(window)
            else:
                raise _inconsistent(f"layer kind tag {tag} is not a known kind")
            kinds.append(kind)
            blocks.append((first_position, row_count))
        geometry = KvGeometry(kinds, num_kv_heads, head_dim)
        row = geometry.row_floats_checked()
        layers = []
        for first_position, row_count in blocks:
            floats = row_count * row
            if floats > USIZE_MAX:
                raise _inconsistent("layer row count overflows the row width")
            keys = r.f32s(floats)
            values = r.f32s(floats)
            layers.append(LayerSnapshot(first_position, keys, values))
        stored = r.u64()
        if r.remaining() != 0:
            raise _inconsistent(f"{r.remaining()} trailing bytes after the checksum")
        computed = checksum(data[:len(data) - 8])
        if stored != computed:
            raise KvError("ChecksumMismatch",
                          f"snapshot checksum mismatch: stored {stored:#018x}, computed "
                          f"{computed:#018x}", stored=stored, computed=computed)
        snapshot = KvSnapshot(geometry, model_fingerprint, token_count, layers)
        snapshot.validate()
        return snapshot


class _Reader:  # snapshot.rs:520-604
    def __init__(self, data: bytes):
        self.data, self.at = data, 0

    def remaining(self) -> int:
        return len(self.data) - self.at

    def take(self, n: int) -> bytes:
        if self.remaining() < n:
            raise KvError("Truncated",
                          f"snapshot: truncated, needs {self.at + n} bytes, has {len(self.data)}",
                          what="snapshot", expected=self.at + n, actual=len(self.data))
        piece = self.data[self.at:self.at + n]
        self.at += n
        return piece

    def u32(self) -> int:
        return struct.unpack("<I", self.take(4))[0]

    def u64(self) -> int:
        return struct.unpack("<Q", self.take(8))[0]

    def f32s(self, count: int) -> np.ndarray:
        byte_count = count * 4
        if byte_count > USIZE_MAX:
            raise _inconsistent("float count overflows the byte count")
        return np.frombuffer(self.take(byte_count), dtype="<f4").copy()


# ---- version 2 (typed rows): not the reference's, this build's own extension ---------------
# v1 with one more u32 after the layer count, the element type of the rows (0 = f32,
# 1 = f16 bits), the rows in that type, and a trailer that is FNV-1a over the FNV-1a sums of
# consecutive 1 MiB blocks of the bytes before it (each sum as 8 little-endian bytes) instead
# of over the bytes themselves. Restated here independently of the library so that its
# encoder and decoder have something to be held to; `KvSnapshot.from_bytes` above stays the
# reference's reader and refuses version 2 by name.

TYPED_FORMAT_VERSION = 2
SUM_BLOCK = 1 << 20


def block_checksum(data: bytes, block_sum=checksum) -> int:
    """`block_sum` is FNV-1a 64 from the offset basis (hash.rs:59-61); the pure-Python one
    above by default, any faster restatement of it for inputs of many blocks."""
    sums = b"".join(struct.pack("<Q", block_sum(data[at:at + SUM_BLOCK]))
                    for at in range(0, len(data), SUM_BLOCK))
    return checksum(sums)


def to_bytes_f16(snapshot: KvSnapshot, block_sum=checksum) -> bytes:
    """Version 2 with f16 rows. The snapshot's f32 values must be exactly representable in
    f16 (they are when captured from an f16-storing cache)."""
    snapshot.validate()
    out = bytearray()
    out += MAGIC
    out += struct.pack("<I", TYPED_FORMAT_VERSION)
    fingerprint = snapshot.model_fingerprint.encode("utf-8")
    out += struct.pack("<I", len(fingerprint))
    out += fingerprint
    out += struct.pack("<Q", snapshot.token_count)
    out += struct.pack("<III", snapshot.geometry.num_kv_heads, snapshot.geometry.head_dim,
                       len(snapshot.geometry.layers))
    out += struct.pack("<I", 1)
    row = snapshot.geometry.row_floats()
    for kind, layer in zip(snapshot.geometry.layers, snapshot.layers):
        w = kind.window()
        out += bytes([0 if w is None else 1, 0, 0, 0])
        out += struct.pack("<QQQ", 0 if w is None else w, layer.first_position, layer.rows(row))
    for layer in snapshot.layers:
        for side in (layer.keys, layer.values):
            halves = np.asarray(side, dtype=np.float32).astype("<f2")
            assert np.array_equal(halves.astype(np.float32), np.asarray(side, dtype=np.float32)), \
                "rows are not f16 values"
            out += halves.tobytes()
    out += struct.pack("<Q", block_checksum(bytes(out), block_sum))
    return bytes(out)

