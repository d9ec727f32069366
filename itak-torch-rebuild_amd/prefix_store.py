"""The persistent prefix store: the Python mirror of the reference's `itak_kv::PrefixStore`
and its configuration (crates/itak-kv/src/store.rs, config.rs), over the C ABI.

The store itself is host code inside the library (entry files byte-identical to the
reference's). `restore_prefix` / `capture_and_put` are the two halves of the reference's
session flow (crates/wgpu-compute/src/session.rs:5000-5151) against a pool slot: a hit's
snapshot is read from disk into pinned host memory once and gathered into the slot from
there.
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass
from typing import List, Optional, Sequence, Union

import numpy as np

from . import _native as N
from .hip_compute import KvCache, KvPool
from .itak_kv import KvError, KvGeometry, KvSnapshot

DIR_ENV = "ITAK_KV_PREFIX_DIR"              # config.rs:19
MAX_BYTES_ENV = "ITAK_KV_PREFIX_MAX_BYTES"  # config.rs:23
ENABLE_ENV = "ITAK_KV_PREFIX_STORE"         # config.rs:28
DEFAULT_MAX_BYTES = 8 * 1024 * 1024 * 1024  # config.rs:31


def prefix_store_enabled_from(raw: Optional[str]) -> bool:  # config.rs:37-39: exact "1" enables
    return raw is not None and raw.strip() == "1"


def prefix_store_enabled() -> bool:  # config.rs:44-46
    return prefix_store_enabled_from(os.environ.get(ENABLE_ENV))


def max_bytes_from(raw: Optional[str]) -> int:  # config.rs:52-67
    if raw is None:
        return DEFAULT_MAX_BYTES
    text = raw.strip()
    digits = text[1:] if text.startswith("+") else text
    if digits and all("0" <= c <= "9" for c in digits) and 0 < int(digits) < 2 ** 64:
        return int(digits)
    return DEFAULT_MAX_BYTES


def default_root() -> str:  # config.rs:72-82
    home = os.environ.get("HOME")
    if home:
        return os.path.join(home, ".cache", "itak", "prefix-kv")
    import tempfile
    return os.path.join(tempfile.gettempdir(), "itak-prefix-kv")


def now_unix() -> int:  # store.rs:120-126
    return int(N.load().itak_kv_now_unix())


@dataclass
class StoreConfig:  # config.rs:88-121
    root: str
    max_bytes: int = DEFAULT_MAX_BYTES

    @staticmethod
    def from_env() -> "StoreConfig":
        root = os.environ.get(DIR_ENV) or default_root()
        return StoreConfig(root, max_bytes_from(os.environ.get(MAX_BYTES_ENV)))


@dataclass
class EntryMeta:  # store.rs:77-91
    file_name: str
    prefix_hash: int
    token_count: int
    bytes: int
    created_unix: int
    last_used_unix: int


@dataclass
class StoreStats:  # store.rs:108-116
    entries: int
    total_bytes: int
    max_bytes: int


@dataclass
class PrefixHit:  # store.rs:94-105
    token_count: int
    tokens: List[int]
    snapshot_bytes: bytes
    file_name: str

    @property
    def snapshot(self) -> KvSnapshot:
        return KvSnapshot.from_bytes(self.snapshot_bytes)


_FIELDS = {
    "TokenCountMismatch": ("snapshot", "tokens"), "PrefixHashMismatch": ("stored", "computed"),
    "SnapshotTokenMismatch": ("entry", "snapshot"), "EntryTooLarge": ("bytes", "cap"),
    "ChecksumMismatch": ("stored", "computed"), "Truncated": ("expected", "actual"),
}


def _raise_store(handle):
    lib = N.load()
    info = N.ErrorInfo()
    lib.itak_store_last_error_info(handle, C.byref(info))
    message = (lib.itak_store_last_error(handle) or b"").decode()
    name = N.STATUS_NAMES.get(info.code, f"Status{info.code}")
    fields = {}
    if name in _FIELDS:
        a, b = _FIELDS[name]
        fields = {a: int(info.a), b: int(info.b)}
    if name in ("Truncated", "BadMagic", "UnsupportedVersion", "Io"):
        fields["what"] = info.what.decode()
    raise KvError(name, message, **fields)


def _tokens(tokens: Sequence[int]) -> np.ndarray:
    return np.ascontiguousarray(tokens, dtype=np.uint32).reshape(-1)


class PrefixStore:
    """itak_kv::PrefixStore (store.rs:128-543)."""

    def __init__(self, handle, root: str):
        self._h = handle
        self._lib = N.load()
        self.root = root
        self.refusals: List[str] = []  # the reference's diag lines for refused entries
        self._drain()

    @staticmethod
    def open(config: Union[StoreConfig, str], max_bytes: Optional[int] = None) -> "PrefixStore":
        if not isinstance(config, StoreConfig):
            config = StoreConfig(str(config), DEFAULT_MAX_BYTES if max_bytes is None else max_bytes)
        lib = N.load()
        handle = C.c_void_p()
        status = lib.itak_store_open(config.root.encode(), config.max_bytes, C.byref(handle))
        if status != N.OK:
            _raise_store(None)
        return PrefixStore(handle, config.root)

    def close(self) -> None:
        if self._h:
            self._lib.itak_store_close(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _drain(self) -> None:
        text = (self._lib.itak_store_refusals(self._h) or b"").decode(errors="replace")
        if text:
            self.refusals.extend(line for line in text.split("\n") if line)
            self._lib.itak_store_clear_refusals(self._h)

    def _check(self, status: int) -> None:
        self._drain()
        if status != N.OK:
            _raise_store(self._h)

    def rescan(self) -> None:
        self._check(self._lib.itak_store_rescan(self._h))

    def stats(self) -> StoreStats:
        raw = N.StoreStats()
        self._check(self._lib.itak_store_get_stats(self._h, C.byref(raw)))
        return StoreStats(int(raw.entries), int(raw.total_bytes), int(raw.max_bytes))

    def entries(self) -> List[EntryMeta]:
        count = C.c_uint64()
        self._check(self._lib.itak_store_entries(self._h, None, 0, C.byref(count)))
        raw = (N.StoreEntry * max(1, count.value))()
        self._check(self._lib.itak_store_entries(self._h, raw, count.value, C.byref(count)))
        return [EntryMeta(e.file_name.decode(), int(e.prefix_hash), int(e.token_count), int(e.bytes),
                          int(e.created_unix), int(e.last_used_unix)) for e in raw[:count.value]]

    def put(self, tokens: Sequence[int], snapshot: Union[KvSnapshot, bytes, np.ndarray],
            now: int) -> None:
        data = snapshot.to_bytes() if isinstance(snapshot, KvSnapshot) else snapshot
        buf = data if isinstance(data, np.ndarray) else np.frombuffer(data, dtype=np.uint8)
        t = _tokens(tokens)
        self._check(self._lib.itak_store_put(self._h, t.ctypes.data if t.size else None, t.size,
                                             buf.ctypes.data, buf.size, now))

    def lookup(self, query: Sequence[int], expected_geometry: Optional[KvGeometry],
               expected_fingerprint: Optional[str], now: int) -> Optional[PrefixHit]:
        q = _tokens(query)
        header, layers = None, None
        if expected_geometry is not None:
            header = N.ItkvHeader()
            header.num_kv_heads = expected_geometry.num_kv_heads
            header.head_dim = expected_geometry.head_dim
            header.layer_count = len(expected_geometry.layers)
            layers = (N.ItkvLayer * max(1, len(expected_geometry.layers)))()
            for i, kind in enumerate(expected_geometry.layers):
                layers[i].kind = N.LAYER_WINDOWED if kind.is_windowed else N.LAYER_GLOBAL
                layers[i].window = kind.window_size or 0
        fp = expected_fingerprint.encode() if expected_fingerprint is not None else None
        hit = N.PrefixHit()
        self._check(self._lib.itak_store_lookup(
            self._h, q.ctypes.data if q.size else None, q.size,
            C.byref(header) if header is not None else None, layers, fp,
            len(fp) if fp is not None else 0, now, C.byref(hit)))
        if hit.token_count == 0:
            return None
        data = C.string_at(hit.snapshot, hit.snapshot_len)
        return PrefixHit(int(hit.token_count), [int(x) for x in q[:hit.token_count]], data,
                         hit.file_name.decode())

    def restore_prefix(self, cache: KvCache, tokens: Sequence[int], fingerprint: str,
                       now: Optional[int] = None) -> int:
        """restore_prefix_from_store (session.rs:5000-5053) into a fresh slot: tokens restored,
        0 when the caller has to prefill cold."""
        t = _tokens(tokens)
        fp = fingerprint.encode()
        matched = C.c_uint64()
        self._check(self._lib.itak_store_restore_prefix(
            self._h, cache.pool._h, cache.slot, t.ctypes.data if t.size else None, t.size, fp,
            len(fp), now_unix() if now is None else now, C.byref(matched)))
        return int(matched.value)

    def capture_and_put(self, cache: KvCache, tokens: Sequence[int], fingerprint: str,
                        now: Optional[int] = None, elem: str = "f32") -> None:
        """capture_and_store_prefix (session.rs:5056-5094). elem="f16" files an f16 pool's
        rows as they are (ITKV version 2) instead of widened to the reference's version 1."""
        t = _tokens(tokens)
        fp = fingerprint.encode()
        self._check(self._lib.itak_store_capture_and_put(
            self._h, cache.pool._h, cache.slot, t.ctypes.data if t.size else None, t.size, fp,
            len(fp), {"f32": N.ELEM_F32, "f16": N.ELEM_F16}[elem], now_unix() if now is None else now))
