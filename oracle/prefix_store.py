"""CPU restatement of the reference's persistent prefix store for the oracle
(crates/itak-kv/src/store.rs, config.rs): one file per entry under a root directory, keyed by
token prefix, bounded by a byte cap with LRU eviction. Test infrastructure only: nothing the
library ships imports this module.

Pinned by the reference's own cases (ported in tests/test_oracle_store.py): the entry layout
table store.rs:5-22 (assembled by hand in the test), the unit cases store.rs:700-808
(planted garbage entry, put/lookup round trip with restamp, longest prefix among nested
entries, mismatched / empty / oversize puts) and the integration cases
crates/itak-kv/tests/prefix_store.rs:57-201 (LRU eviction under the cap, forged entry refused
while the shorter honest prefix serves, geometry and fingerprint requirements, torn temp and
final files, persistence across reopen), plus the switch and cap parsing of config.rs:37-139.
"""
from __future__ import annotations

import os
import struct
from dataclasses import dataclass
from typing import List, Optional, Sequence

from .itak_kv import KvError, KvGeometry, KvSnapshot, prefix_discriminator, prefix_hash

ENTRY_MAGIC = b"ITKVPENT"        # store.rs:63
ENTRY_FORMAT_VERSION = 1         # store.rs:65
PREAMBLE_LEN = 72                # store.rs:67
LAST_USED_OFFSET = 24            # store.rs:69
ENTRY_SUFFIX = ".kv"             # store.rs:71
TEMP_PREFIX = ".tmp-"            # store.rs:73
DEFAULT_MAX_BYTES = 8 * 1024 * 1024 * 1024  # config.rs:31
_U64_MAX = (1 << 64) - 1


def prefix_store_enabled_from(raw: Optional[str]) -> bool:  # config.rs:37-39
    return raw is not None and raw.strip() == "1"


def max_bytes_from(raw: Optional[str]) -> int:  # config.rs:52-67
    if raw is None:
        return DEFAULT_MAX_BYTES
    text = raw.strip()
    # Rust's u64::from_str: optional '+', ASCII digits only, no overflow.
    digits = text[1:] if text.startswith("+") else text
    if digits and all("0" <= c <= "9" for c in digits) and 0 < int(digits) <= _U64_MAX:
        return int(digits)
    return DEFAULT_MAX_BYTES


@dataclass
class StoreConfig:  # config.rs:88-95
    root: str
    max_bytes: int = DEFAULT_MAX_BYTES


@dataclass
class EntryMeta:  # store.rs:77-91
    file_name: str
    prefix_hash: int
    token_count: int
    bytes: int
    created_unix: int
    last_used_unix: int


@dataclass
class PrefixHit:  # store.rs:94-105
    token_count: int
    tokens: List[int]
    snapshot: KvSnapshot


@dataclass
class StoreStats:  # store.rs:108-116
    entries: int
    total_bytes: int
    max_bytes: int


def _io(context: str, error: OSError) -> KvError:  # error.rs:127-133 with io::Error's Display
    message = f"{os.strerror(error.errno)} (os error {error.errno})"
    return KvError("Io", f"{context}: {message}", context=context, io_message=message)


@dataclass
class _Preamble:  # store.rs:546-553
    created_unix: int
    last_used_unix: int
    prefix_hash: int
    token_count: int
    payload_bytes: int


def encode_preamble(p: _Preamble) -> bytes:  # store.rs:555-567
    out = bytearray(PREAMBLE_LEN)
    out[0:8] = ENTRY_MAGIC
    out[8:12] = struct.pack("<I", ENTRY_FORMAT_VERSION)
    out[16:24] = struct.pack("<Q", p.created_unix)
    out[24:32] = struct.pack("<Q", p.last_used_unix)
    out[32:40] = struct.pack("<Q", p.prefix_hash)
    out[40:48] = struct.pack("<Q", p.token_count)
    out[48:56] = struct.pack("<Q", p.token_count * 4)
    out[56:64] = struct.pack("<Q", p.payload_bytes)
    return bytes(out)


def parse_preamble(data: bytes) -> _Preamble:  # store.rs:569-606
    if len(data) < PREAMBLE_LEN:
        raise KvError("Truncated", f"entry: truncated, needs {PREAMBLE_LEN} bytes, has {len(data)}",
                      what="entry", expected=PREAMBLE_LEN, actual=len(data))
    if data[0:8] != ENTRY_MAGIC:
        raise KvError("BadMagic", "entry: bad magic", what="entry")
    version = struct.unpack("<I", data[8:12])[0]
    if version != ENTRY_FORMAT_VERSION:
        raise KvError("UnsupportedVersion", f"entry: unsupported format version {version}",
                      what="entry", version=version)
    field = lambda at: struct.unpack("<Q", data[at:at + 8])[0]  # noqa: E731
    token_count = field(40)
    tokens_bytes = field(48)
    expected = min(token_count * 4, _U64_MAX)  # saturating_mul
    if tokens_bytes != expected:
        raise KvError("InconsistentSnapshot",
                      f"inconsistent snapshot: entry tokens_bytes is {tokens_bytes} but token count "
                      f"{token_count} implies {expected}")
    return _Preamble(field(16), field(24), field(32), token_count, field(56))


def _read_preamble(path: str) -> EntryMeta:  # store.rs:609-632
    try:
        with open(path, "rb") as f:
            head = f.read(PREAMBLE_LEN)
            size = os.fstat(f.fileno()).st_size
    except OSError as e:
        raise _io(f"open {path}", e) from None
    if len(head) < PREAMBLE_LEN:  # read_exact fails on a short file
        raise KvError("Io", f"read preamble of {path}: failed to fill whole buffer",
                      context=f"read preamble of {path}", io_message="failed to fill whole buffer")
    p = parse_preamble(head)
    return EntryMeta(os.path.basename(path), p.prefix_hash, p.token_count, size, p.created_unix,
                     p.last_used_unix)


def _read_entry_tokens(path: str) -> List[int]:  # store.rs:635-650
    try:
        with open(path, "rb") as f:
            data = f.read()
    except OSError as e:
        raise _io(f"read {path}", e) from None
    p = parse_preamble(data)
    end = PREAMBLE_LEN + p.token_count * 4
    if len(data) < end:
        raise KvError("Truncated", f"entry: truncated, needs {end} bytes, has {len(data)}",
                      what="entry", expected=end, actual=len(data))
    return list(struct.unpack(f"<{p.token_count}I", data[PREAMBLE_LEN:end]))


class PrefixStore:  # store.rs:128-543
    def __init__(self, root: str, max_bytes: int):
        self.root, self.max_bytes = root, max_bytes
        self._entries: List[EntryMeta] = []
        self.refusals: List[str] = []  # what the reference writes to its diag channel

    @staticmethod
    def open(config: StoreConfig) -> "PrefixStore":  # store.rs:147-168
        if config.max_bytes == 0:
            raise KvError("InvalidConfig", "invalid config: the store byte cap is zero")
        try:
            os.makedirs(config.root, exist_ok=True)
        except OSError as e:
            raise _io(f"create store root {config.root}", e) from None
        store = PrefixStore(config.root, config.max_bytes)
        store.rescan()
        return store

    def entries(self) -> List[EntryMeta]:  # store.rs:177-182: longest prefix first, stable
        return sorted(self._entries, key=lambda e: -e.token_count)

    def stats(self) -> StoreStats:  # store.rs:185-192
        return StoreStats(len(self._entries), self._total_bytes(), self.max_bytes)

    def _total_bytes(self) -> int:
        return sum(e.bytes for e in self._entries)

    def rescan(self) -> None:  # store.rs:204-224
        entries = []
        try:
            names = os.listdir(self.root)
        except OSError as e:
            raise _io(f"list store root {self.root}", e) from None
        for name in names:
            if name.startswith(TEMP_PREFIX) or not name.endswith(ENTRY_SUFFIX):
                continue
            try:
                entries.append(_read_preamble(os.path.join(self.root, name)))
            except KvError as error:
                self.refusals.append(f"prefix store refuses entry {name}: {error.message}")
        self._entries = entries

    def put(self, tokens: Sequence[int], snapshot: KvSnapshot, now: int) -> None:  # store.rs:236-300
        tokens = list(tokens)
        if not tokens:
            raise KvError("EmptyPrefix", "empty token prefix refused")
        if snapshot.token_count != len(tokens):
            raise KvError("TokenCountMismatch",
                          f"snapshot covers {snapshot.token_count} tokens but was offered under "
                          f"{len(tokens)} token ids", snapshot=snapshot.token_count,
                          tokens=len(tokens))
        payload = snapshot.to_bytes()
        key = prefix_hash(tokens)
        entry_bytes = PREAMBLE_LEN + len(tokens) * 4 + len(payload)
        if entry_bytes > self.max_bytes:
            raise KvError("EntryTooLarge",
                          f"entry of {entry_bytes} bytes exceeds the store cap of {self.max_bytes} "
                          "bytes", bytes=entry_bytes, cap=self.max_bytes)
        file_name = self._pick_file_name(tokens, key)
        path = os.path.join(self.root, file_name)
        temp_name = f"{TEMP_PREFIX}{file_name}-{os.getpid()}"
        temp_path = os.path.join(self.root, temp_name)
        preamble = encode_preamble(_Preamble(now, now, key, len(tokens), len(payload)))
        try:
            with open(temp_path, "wb") as f:
                f.write(preamble)
                f.write(struct.pack(f"<{len(tokens)}I", *tokens))
                f.write(payload)
                f.flush()
                os.fsync(f.fileno())
        except OSError as e:
            raise _io(f"write temp entry {temp_name}", e) from None
        try:
            os.rename(temp_path, path)
        except OSError as e:
            raise _io(f"rename entry {file_name}", e) from None
        self._entries = [e for e in self._entries if e.file_name != file_name]
        self._entries.append(EntryMeta(file_name, key, len(tokens), entry_bytes, now, now))
        self._evict_except(file_name)

    def lookup(self, query: Sequence[int], expected_geometry: Optional[KvGeometry],
               expected_fingerprint: Optional[str], now: int) -> Optional[PrefixHit]:  # store.rs:314-357
        query = list(query)
        candidates = sorted((e for e in self._entries if e.token_count <= len(query)),
                            key=lambda e: -e.token_count)
        for candidate in candidates:
            try:
                hit = self._verify_candidate(candidate, query, expected_geometry,
                                             expected_fingerprint)
            except KvError as error:
                self.refusals.append(
                    f"prefix store refuses entry {candidate.file_name}: {error.message}")
                continue
            if hit is None:
                continue
            self._touch(candidate.file_name, now)
            for meta in self._entries:
                if meta.file_name == candidate.file_name:
                    meta.last_used_unix = now
                    break
            return hit
        return None

    def _verify_candidate(self, meta: EntryMeta, query: List[int],
                          expected_geometry: Optional[KvGeometry],
                          expected_fingerprint: Optional[str]) -> Optional[PrefixHit]:  # store.rs:364-452
        path = os.path.join(self.root, meta.file_name)
        try:
            with open(path, "rb") as f:
                data = f.read()
        except OSError as e:
            raise _io(f"read entry {meta.file_name}", e) from None
        p = parse_preamble(data)
        if p.prefix_hash != meta.prefix_hash or p.token_count != meta.token_count:
            raise KvError("InconsistentSnapshot",
                          f"inconsistent snapshot: entry {meta.file_name} changed between scan and "
                          f"read (index hash {meta.prefix_hash:#x} / {meta.token_count} tokens, "
                          f"file hash {p.prefix_hash:#x} / {p.token_count} tokens)")
        tokens_end = PREAMBLE_LEN + p.token_count * 4
        if len(data) < tokens_end:
            raise KvError("Truncated",
                          f"entry: truncated, needs {tokens_end} bytes, has {len(data)}",
                          what="entry", expected=tokens_end, actual=len(data))
        tokens = list(struct.unpack(f"<{p.token_count}I", data[PREAMBLE_LEN:tokens_end]))
        computed = prefix_hash(tokens)
        if computed != p.prefix_hash:
            raise KvError("PrefixHashMismatch",
                          f"stored token ids hash to {computed:#018x}, not the entry key "
                          f"{p.prefix_hash:#018x}; entry refused", stored=p.prefix_hash,
                          computed=computed)
        if tokens != query[:len(tokens)]:
            return None
        payload = data[tokens_end:]
        if len(payload) != p.payload_bytes:
            raise KvError("Truncated",
                          f"entry payload: truncated, needs {p.payload_bytes} bytes, has "
                          f"{len(payload)}", what="entry payload", expected=p.payload_bytes,
                          actual=len(payload))
        snapshot = KvSnapshot.from_bytes(payload)
        if snapshot.token_count != p.token_count:
            raise KvError("SnapshotTokenMismatch",
                          f"entry preamble covers {p.token_count} tokens but its snapshot covers "
                          f"{snapshot.token_count}", entry=p.token_count,
                          snapshot=snapshot.token_count)
        if expected_geometry is not None and snapshot.geometry != expected_geometry:
            raise KvError("GeometryMismatch",
                          f"geometry mismatch: entry {meta.file_name} snapshot geometry differs "
                          "from the required geometry")
        if expected_fingerprint is not None and snapshot.model_fingerprint != expected_fingerprint:
            raise KvError("FingerprintMismatch",
                          f"model fingerprint mismatch: need {expected_fingerprint}, snapshot "
                          f"carries {snapshot.model_fingerprint}", expected=expected_fingerprint,
                          actual=snapshot.model_fingerprint)
        return PrefixHit(p.token_count, tokens, snapshot)

    def _pick_file_name(self, tokens: List[int], key: int) -> str:  # store.rs:458-503
        disc = prefix_discriminator(tokens)
        base = f"{key:016x}-{len(tokens)}-{disc:016x}"
        for counter in range(1024):
            name = f"{base}{ENTRY_SUFFIX}" if counter == 0 else f"{base}-c{counter}{ENTRY_SUFFIX}"
            path = os.path.join(self.root, name)
            indexed = any(e.file_name == name for e in self._entries)
            if not indexed and not os.path.exists(path):
                return name
            try:
                existing = _read_entry_tokens(path)
            except KvError:
                if indexed:
                    continue
                return name  # an unreadable stray file of that name is overwritten
            if existing == tokens:
                return name
        raise KvError("InvalidConfig",
                      f"invalid config: no free filename for prefix hash {key:#x} after 1024 "
                      "collisions; the store directory is not behaving like a prefix store")

    def _touch(self, file_name: str, now: int) -> None:  # store.rs:506-517
        path = os.path.join(self.root, file_name)
        try:
            with open(path, "r+b") as f:
                f.seek(LAST_USED_OFFSET)
                f.write(struct.pack("<Q", now))
        except OSError as e:
            raise _io(f"open entry {file_name} to restamp", e) from None

    def _evict_except(self, keep: str) -> None:  # store.rs:521-548
        while self._total_bytes() > self.max_bytes:
            victims = [e for e in self._entries if e.file_name != keep]
            if not victims:
                break
            victim = min(victims, key=lambda e: (e.last_used_unix, e.file_name)).file_name
            try:
                os.remove(os.path.join(self.root, victim))
            except OSError as e:
                raise _io(f"evict entry {victim}", e) from None
            self._entries = [e for e in self._entries if e.file_name != victim]
