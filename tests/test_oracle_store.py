"""The reference's prefix-store cases (crates/itak-kv/src/store.rs:700-808,
crates/itak-kv/tests/prefix_store.rs:57-201, config.rs:97-139) against the CPU oracle's
store AND against the library's store (host code: it runs without a GPU), and the two against
each other: the same puts leave byte-identical entry files, and each serves what the other
wrote."""
import os
import struct

import numpy as np
import pytest

import oracle
import oracle.itak_kv as okv
import oracle.prefix_store as ops
from helpers import pkg


def P():
    return pkg()


# ------------------------------------------------------------------ the reference's fixtures

def o_geometry():
    return okv.KvGeometry([oracle.LayerKind.Windowed(4), oracle.LayerKind.Global], 2, 3)


def snapshot_for(tokens, fingerprint):  # prefix_store.rs:26-45, f32 arithmetic as in Rust
    g = o_geometry()
    cache = oracle.KvCache.new(g.layers, g.num_kv_heads, g.head_dim)
    row = g.row_floats()
    for position, token in enumerate(tokens):
        for layer in range(len(g.layers)):
            k = [np.float32(token) + np.float32(position * 10 + layer + i) / np.float32(11.0)
                 for i in range(row)]
            v = [-(np.float32(token) + np.float32(position + layer * 3 + i) / np.float32(5.0))
                 for i in range(row)]
            cache.append(layer, np.array(k, np.float32), np.array(v, np.float32), position)
    return okv.KvSnapshot.capture(cache, fingerprint)


class OracleSide:
    """The oracle's store under the call shape the cases below use."""
    name = "oracle"

    def open(self, root, cap):
        return ops.PrefixStore.open(ops.StoreConfig(str(root), cap))

    def put(self, store, tokens, snapshot, now):
        store.put(tokens, snapshot, now)

    def lookup(self, store, query, geometry, fingerprint, now):
        hit = store.lookup(query, geometry, fingerprint, now)
        return None if hit is None else (hit.token_count, hit.tokens, hit.snapshot.to_bytes())

    def geometry(self, head_dim=3):
        g = o_geometry()
        g.head_dim = head_dim
        return g

    def error(self):
        return okv.KvError


class LibrarySide:
    """The library's store (C ABI) under the same call shape."""
    name = "library"

    def open(self, root, cap):
        return P().PrefixStore.open(str(root), cap)

    def put(self, store, tokens, snapshot, now):
        store.put(tokens, snapshot.to_bytes(), now)

    def lookup(self, store, query, geometry, fingerprint, now):
        hit = store.lookup(query, geometry, fingerprint, now)
        return None if hit is None else (hit.token_count, hit.tokens, hit.snapshot_bytes)

    def geometry(self, head_dim=3):
        return P().KvGeometry([P().LayerKind.Windowed(4), P().LayerKind.Global], 2, head_dim)

    def error(self):
        return P().KvError


SIDES = [OracleSide(), LibrarySide()]


@pytest.fixture(params=SIDES, ids=lambda s: s.name)
def side(request):
    return request.param


# ------------------------------------------------------------------------ config.rs cases

def test_enable_switch_is_exact_one_only():
    # config.rs:101-110, on the oracle and on the library's front end.
    for fn in (ops.prefix_store_enabled_from, P().prefix_store_enabled_from):
        assert fn("1") and fn(" 1 ")
        for raw in (None, "0", "true", "11", ""):
            assert not fn(raw)


def test_cap_parsing_falls_back_by_rule():
    # config.rs:112-121.
    for fn in (ops.max_bytes_from, P().max_bytes_from):
        assert fn(None) == 8 * 1024 ** 3
        assert fn("4096") == 4096 and fn(" 4096 ") == 4096
        for raw in ("0", "-1", "lots", ""):
            assert fn(raw) == 8 * 1024 ** 3


# ------------------------------------------------------------------------- store.rs cases

def test_entry_layout_is_the_documented_byte_table(tmp_path, side):
    # store.rs:5-22, assembled by hand.
    tokens = [10, 20, 30]
    snap = snapshot_for(tokens, "m")
    store = side.open(tmp_path, 1 << 30)
    side.put(store, tokens, snap, 1234)
    files = sorted(f for f in os.listdir(tmp_path) if f.endswith(".kv"))
    key, disc = okv.prefix_hash(tokens), okv.prefix_discriminator(tokens)
    assert files == [f"{key:016x}-3-{disc:016x}.kv"]
    payload = snap.to_bytes()
    want = (b"ITKVPENT" + struct.pack("<II", 1, 0) + struct.pack("<QQQQQQQ", 1234, 1234, key, 3, 12,
                                                                 len(payload), 0)
            + struct.pack("<3I", *tokens) + payload)
    assert len(want) == 72 + 12 + len(payload)
    assert open(tmp_path / files[0], "rb").read() == want
    assert not [f for f in os.listdir(tmp_path) if f.startswith(".tmp-")]


def test_open_refuses_a_planted_garbage_entry_by_name(tmp_path, side):
    # store.rs:700-723.
    planted = bytearray(72)
    planted[0:8] = b"ITKVPENT"
    planted[8:12] = struct.pack("<I", 1)
    planted[40:48] = struct.pack("<Q", 2 ** 64 - 1)
    planted[48:56] = struct.pack("<Q", 0)
    (tmp_path / "planted.kv").write_bytes(bytes(planted))
    store = side.open(tmp_path, 1 << 30)
    assert store.entries() == []
    assert any("planted.kv" in r and "entry tokens_bytes is 0 but token count "
               "18446744073709551615 implies 18446744073709551615" in r for r in store.refusals)


def test_put_lookup_round_trip(tmp_path, side):
    # store.rs:725-744.
    store = side.open(tmp_path, 1 << 30)
    tokens = [10, 20, 30, 40, 50]
    snap = snapshot_for(tokens, "model-a")
    side.put(store, tokens, snap, 100)
    count, got_tokens, got_bytes = side.lookup(store, [10, 20, 30, 40, 50, 60, 70], None, None, 200)
    assert count == 5 and list(got_tokens) == tokens
    assert got_bytes == snap.to_bytes()
    assert store.entries()[0].last_used_unix == 200
    reopened = side.open(tmp_path, 1 << 30)
    assert reopened.entries()[0].last_used_unix == 200
    assert reopened.entries()[0].created_unix == 100


def test_longest_prefix_wins_among_nested_entries(tmp_path, side):
    # store.rs:746-787.
    store = side.open(tmp_path, 1 << 30)
    for now, tokens in enumerate(([1, 2], [1, 2, 3, 4], [1, 2, 3, 4, 5, 6]), start=1):
        side.put(store, tokens, snapshot_for(tokens, "model-a"), now)
    assert side.lookup(store, [1, 2, 3, 4, 5, 6, 7, 8], None, None, 10)[0] == 6
    assert side.lookup(store, [1, 2, 3, 4, 99], None, None, 11)[0] == 4
    assert side.lookup(store, [1, 2, 77], None, None, 12)[0] == 2
    assert side.lookup(store, [9, 9], None, None, 13) is None
    assert [e.token_count for e in store.entries()] == [6, 4, 2]


def test_put_refuses_mismatched_and_oversize(tmp_path, side):
    # store.rs:789-808.
    store = side.open(tmp_path / "a", 1 << 30)
    tokens = [1, 2, 3]
    other = snapshot_for([7, 8], "model-a")
    with pytest.raises(side.error()) as e:
        side.put(store, tokens, other, 1)
    assert e.value.variant == "TokenCountMismatch"
    assert e.value.message == "snapshot covers 2 tokens but was offered under 3 token ids"
    with pytest.raises(side.error()) as e:
        side.put(store, [], other, 1)
    assert e.value.variant == "EmptyPrefix" and e.value.message == "empty token prefix refused"
    small = side.open(tmp_path / "b", 128)
    snap = snapshot_for(tokens, "model-a")
    with pytest.raises(side.error()) as e:
        side.put(small, tokens, snap, 1)
    assert e.value.variant == "EntryTooLarge"
    size = 72 + 12 + len(snap.to_bytes())
    assert e.value.message == f"entry of {size} bytes exceeds the store cap of 128 bytes"
    with pytest.raises(side.error()) as e:
        side.open(tmp_path / "c", 0)
    assert e.value.variant == "InvalidConfig"
    assert e.value.message == "invalid config: the store byte cap is zero"


# ------------------------------------------------------------------ prefix_store.rs cases

def test_eviction_respects_the_cap_and_lru_order(tmp_path, side):
    # prefix_store.rs:57-94.
    a, b, c = [1, 1, 1, 1], [2, 2, 2, 2], [3, 3, 3, 3]
    probe = side.open(tmp_path / "probe", 2 ** 64 - 1)
    side.put(probe, a, snapshot_for(a, "m"), 1)
    entry_bytes = probe.stats().total_bytes
    cap = entry_bytes * 2 + entry_bytes // 2
    store = side.open(tmp_path / "real", cap)
    side.put(store, a, snapshot_for(a, "m"), 1)
    side.put(store, b, snapshot_for(b, "m"), 2)
    assert side.lookup(store, [1, 1, 1, 1, 9], None, None, 3) is not None  # touch a
    side.put(store, c, snapshot_for(c, "m"), 4)
    stats = store.stats()
    assert stats.total_bytes <= cap and stats.entries == 2 and stats.max_bytes == cap
    assert side.lookup(store, b, None, None, 5) is None, "the LRU entry (b) must be evicted"
    assert side.lookup(store, a, None, None, 6) is not None
    assert side.lookup(store, c, None, None, 7) is not None
    assert len([f for f in os.listdir(tmp_path / "real") if f.endswith(".kv")]) == 2


def test_forged_entry_is_refused_and_shorter_honest_prefix_still_serves(tmp_path, side):
    # prefix_store.rs:96-137.
    store = side.open(tmp_path, 1 << 30)
    short, long = [5, 6], [5, 6, 7, 8]
    side.put(store, short, snapshot_for(short, "m"), 1)
    side.put(store, long, snapshot_for(long, "m"), 2)
    long_meta = [e for e in store.entries() if e.token_count == 4][0]
    path = tmp_path / long_meta.file_name
    data = bytearray(path.read_bytes())
    data[72:76] = bytes([0xEF, 0xBE, 0xAD, 0xDE])
    path.write_bytes(bytes(data))
    store = side.open(tmp_path, 1 << 30)
    count, tokens, _ = side.lookup(store, [5, 6, 7, 8, 9], None, None, 3)
    assert count == 2 and list(tokens) == short
    forged = okv.prefix_hash([0xDEADBEEF, 6, 7, 8])
    key = okv.prefix_hash(long)
    assert any(long_meta.file_name in r and
               f"stored token ids hash to {forged:#018x}, not the entry key {key:#018x}; entry "
               "refused" in r for r in store.refusals)


def test_geometry_and_fingerprint_requirements_refuse_at_lookup(tmp_path, side):
    # prefix_store.rs:139-166.
    store = side.open(tmp_path, 1 << 30)
    tokens = [3, 1, 4]
    side.put(store, tokens, snapshot_for(tokens, "model-a"), 1)
    assert side.lookup(store, tokens, side.geometry(head_dim=12), None, 2) is None
    assert side.lookup(store, tokens, None, "model-b", 3) is None
    assert any("need model-b, snapshot carries model-a" in r for r in store.refusals)
    assert any("snapshot geometry differs from the required geometry" in r for r in store.refusals)
    count, _, data = side.lookup(store, tokens, side.geometry(), "model-a", 4)
    assert count == 3
    okv.KvSnapshot.from_bytes(data).restore_checked(o_geometry(), "model-a")
    # A refused lookup does not restamp; the verified one does.
    assert store.entries()[0].last_used_unix == 4


def test_torn_temp_and_torn_final_files_are_ignored(tmp_path, side):
    # prefix_store.rs:168-187.
    (tmp_path / ".tmp-deadbeef-123.kv").write_bytes(b"half an entry")
    (tmp_path / "0123456789abcdef-4-0.kv").write_bytes(b"ITKV")
    store = side.open(tmp_path, 1 << 30)
    assert store.stats().entries == 0
    assert any("0123456789abcdef-4-0.kv" in r for r in store.refusals)
    assert not any(".tmp-" in r for r in store.refusals)
    tokens = [8, 8]
    side.put(store, tokens, snapshot_for(tokens, "m"), 1)
    assert side.lookup(store, [8, 8, 8], None, None, 2) is not None


def test_entries_survive_reopen(tmp_path, side):
    # prefix_store.rs:189-201.
    tokens = [42, 43, 44, 45, 46, 47]
    store = side.open(tmp_path, 1 << 30)
    side.put(store, tokens, snapshot_for(tokens, "m"), 10)
    del store
    store = side.open(tmp_path, 1 << 30)
    count, _, data = side.lookup(store, tokens + [48], None, None, 20)
    snap = okv.KvSnapshot.from_bytes(data)
    assert count == 6 and snap.token_count == 6
    assert snap.restore().next_position(0) == 6


# ------------------------------------------------------- beyond the reference's own cases

def test_a_truncated_payload_and_a_flipped_payload_byte_are_refused_by_name(tmp_path, side):
    store = side.open(tmp_path, 1 << 30)
    short, long = [1, 2], [1, 2, 3]
    side.put(store, short, snapshot_for(short, "m"), 1)
    side.put(store, long, snapshot_for(long, "m"), 2)
    path = tmp_path / [e for e in store.entries() if e.token_count == 3][0].file_name
    whole = path.read_bytes()
    path.write_bytes(whole[:-5])
    assert side.lookup(store, [1, 2, 3, 4], None, None, 3)[0] == 2
    assert any("entry payload: truncated, needs" in r for r in store.refusals)
    flipped = bytearray(whole)
    flipped[-20] ^= 0x40
    path.write_bytes(bytes(flipped))
    assert side.lookup(store, [1, 2, 3, 4], None, None, 4)[0] == 2
    assert any("snapshot checksum mismatch" in r for r in store.refusals)
    path.write_bytes(whole)
    assert side.lookup(store, [1, 2, 3, 4], None, None, 5)[0] == 3


def test_the_same_prefix_put_twice_replaces_its_entry(tmp_path, side):
    store = side.open(tmp_path, 1 << 30)
    tokens = [4, 5, 6]
    side.put(store, tokens, snapshot_for(tokens, "old"), 1)
    side.put(store, tokens, snapshot_for(tokens, "new"), 2)
    assert store.stats().entries == 1
    assert len([f for f in os.listdir(tmp_path) if f.endswith(".kv")]) == 1
    _, _, data = side.lookup(store, tokens, None, None, 3)
    assert okv.KvSnapshot.from_bytes(data).model_fingerprint == "new"
    assert store.entries()[0].created_unix == 2


def test_library_and_oracle_write_identical_files_and_serve_each_other(tmp_path):
    o, l = OracleSide(), LibrarySide()
    prefixes = [[1, 2], [1, 2, 3, 4], [9], [7, 7, 7, 7, 7, 7, 7]]
    so, sl = o.open(tmp_path / "o", 1 << 30), l.open(tmp_path / "l", 1 << 30)
    for now, tokens in enumerate(prefixes, start=5):
        snap = snapshot_for(tokens, "shared")
        o.put(so, tokens, snap, now)
        l.put(sl, tokens, snap, now)
    names_o, names_l = sorted(os.listdir(tmp_path / "o")), sorted(os.listdir(tmp_path / "l"))
    assert names_o == names_l and len(names_o) == 4
    for name in names_o:
        assert (tmp_path / "o" / name).read_bytes() == (tmp_path / "l" / name).read_bytes()
    assert [(e.file_name, e.prefix_hash, e.token_count, e.bytes, e.created_unix, e.last_used_unix)
            for e in so.entries()] == \
           [(e.file_name, e.prefix_hash, e.token_count, e.bytes, e.created_unix, e.last_used_unix)
            for e in sl.entries()]
    # Each reads the other's directory.
    cross_l, cross_o = l.open(tmp_path / "o", 1 << 30), o.open(tmp_path / "l", 1 << 30)
    for query in ([1, 2, 3, 4, 5], [1, 2, 8], [9, 9], [7] * 9, [3]):
        a, b = l.lookup(cross_l, query, None, None, 50), o.lookup(cross_o, query, None, None, 50)
        assert (a is None) == (b is None)
        if a is not None:
            assert a[0] == b[0] and list(a[1]) == list(b[1]) and a[2] == b[2]
    for name in names_o:  # both restamped the same entries in place
        assert (tmp_path / "o" / name).read_bytes() == (tmp_path / "l" / name).read_bytes()


@pytest.mark.parametrize("version", [1, 2])
def test_a_payload_read_in_pieces_is_served_whole_and_a_flip_in_any_piece_is_refused(tmp_path, version):
    """A payload larger than a few MB is not read and then summed: version 1 is read by a
    second thread while the byte-serial checksum follows it, version 2 (block sums) by several
    threads that each sum what they read. What comes out is what went in, and one flipped bit
    in the first, a middle or the last piece is still caught by name. (Library side only: the
    oracle's byte loop over 20 MB is what this path exists to avoid.)"""
    rng = np.random.default_rng(3)
    kvh, d, rows = 4, 128, 5000 * version
    geometry = P().KvGeometry([P().LayerKind.Global], kvh, d)
    keys = rng.standard_normal(rows * kvh * d, dtype=np.float32).astype(np.float16).astype(np.float32)
    values = rng.standard_normal(rows * kvh * d, dtype=np.float32).astype(np.float16).astype(np.float32)

    def encode(n):
        if version == 1:
            return P().KvSnapshot(geometry, "big", n, [P().LayerSnapshot(0, keys[:n * kvh * d],
                                                                         values[:n * kvh * d])]).to_bytes()
        snap = okv.KvSnapshot(okv.KvGeometry([oracle.LayerKind.Global], kvh, d), "big", n,
                              [okv.LayerSnapshot(0, keys[:n * kvh * d], values[:n * kvh * d])])
        return okv.to_bytes_f16(snap, lambda block: oracle.checksum(bytes(block)))

    data = encode(rows)
    assert len(data) > 20_000_000
    tokens = [int(t) for t in rng.integers(0, 1 << 20, size=rows)]
    short = tokens[:7]
    store = P().PrefixStore.open(str(tmp_path), 1 << 30)
    store.put(short, encode(7), 1)
    store.put(tokens, data, 2)
    hit = store.lookup(tokens + [5], geometry, "big", 3)
    assert hit.token_count == rows and hit.snapshot_bytes == data
    path = tmp_path / hit.file_name
    whole = path.read_bytes()
    payload_at = len(whole) - len(data)
    for offset in (payload_at + 100, payload_at + len(data) // 2, len(whole) - 9):
        flipped = bytearray(whole)
        flipped[offset] ^= 0x01
        path.write_bytes(bytes(flipped))
        store.refusals.clear()
        assert store.lookup(tokens + [5], geometry, "big", 4).token_count == 7
        assert any("snapshot checksum mismatch" in r for r in store.refusals), offset
    path.write_bytes(whole[:-3_000_000])  # the file ends inside a later piece
    store.refusals.clear()
    assert store.lookup(tokens + [5], geometry, "big", 5).token_count == 7
    assert any("entry payload: truncated, needs" in r for r in store.refusals)
    path.write_bytes(whole)
    assert store.lookup(tokens + [5], geometry, "big", 6).snapshot_bytes == data


def _corrupt(data, rng):
    """A seeded corruption of an entry file: a flipped bit, a cut, stray bytes, or an extreme
    value over a field of the header or of the snapshot's own header."""
    b = bytearray(data)
    extremes = (0, 1, 2, 0x80000000, 0xFFFFFFFF, 1 << 32, 1 << 61, (1 << 63) - 1, (1 << 64) - 1)
    for _ in range(int(rng.integers(1, 3))):
        kind = int(rng.integers(0, 5))
        if kind == 0 and b:
            b[int(rng.integers(0, len(b)))] ^= 1 << int(rng.integers(0, 8))
        elif kind == 1:
            del b[int(rng.integers(0, len(b) + 1)):]
        elif kind == 2 and len(b) >= 16:
            width = 8 if rng.integers(0, 2) else 4
            at = int(rng.integers(0, min(len(b), 240) - width + 1)) & ~3
            b[at:at + width] = int(extremes[int(rng.integers(0, len(extremes)))] % (1 << (8 * width))).to_bytes(width, "little")
        elif kind == 3:
            b += rng.integers(0, 256, size=int(rng.integers(1, 24)), dtype=np.uint8).tobytes()
        elif kind == 4 and len(b) > 12:
            at = int(rng.integers(0, len(b) - 4))
            del b[at:at + int(rng.integers(1, 17))]
    return bytes(b)


def test_corrupted_directories_are_indexed_refused_and_served_alike_by_library_and_oracle(tmp_path):
    """60 directories of honest entries, some then corrupted on disk (240 files in all): the
    library's store and the oracle's index the same entries, refuse the same files in the same
    words, serve the same prefixes with the same bytes, and leave the same files behind."""
    import shutil
    o, l = OracleSide(), LibrarySide()
    rng = np.random.default_rng(31)
    served = refused = 0

    def meta(store):
        return [(e.file_name, e.prefix_hash, e.token_count, e.bytes, e.created_unix, e.last_used_unix)
                for e in store.entries()]

    def said(store, root, but=()):  # the refusal lines, the directory's own path taken out
        return sorted(r.replace(str(root), "<root>") for r in store.refusals
                      if not any(name in r for name in but))

    def typed(store):
        # A corruption that writes 2 over the snapshot's version makes it the library's own typed
        # format: the reference's reader refuses the version by name, the library reads on and
        # refuses what follows. Both refuse; only the words differ, and are left out below.
        return [r.split()[4].rstrip(":") for r in store.refusals if r.endswith("unsupported format version 2")]

    for case in range(60):
        a, b = tmp_path / f"o{case}", tmp_path / f"l{case}"
        writer = o.open(a, 1 << 30)
        base = [int(t) for t in rng.integers(0, 9, size=2)]
        prefixes = [base, base + [int(rng.integers(0, 9))], base + [7, 7, int(rng.integers(0, 9))],
                    [int(t) for t in rng.integers(10, 20, size=int(rng.integers(1, 6)))]]
        for now, tokens in enumerate(prefixes, start=1):
            o.put(writer, tokens, snapshot_for(tokens, "m"), now)
        for name in sorted(os.listdir(a)):
            if rng.integers(0, 2):
                (a / name).write_bytes(_corrupt((a / name).read_bytes(), rng))
        if case % 7 == 0:
            (a / "stray.itkv").write_bytes(rng.integers(0, 256, size=int(rng.integers(0, 90)), dtype=np.uint8).tobytes())
        shutil.copytree(a, b)
        so, sl = o.open(a, 1 << 30), l.open(b, 1 << 30)
        assert meta(so) == meta(sl), case
        assert said(so, a, typed(so)) == said(sl, b, typed(so)), case
        assert len(so.refusals) == len(sl.refusals), case
        for now, tokens in enumerate(prefixes + [base + [7, 7, 7, 7]], start=10):
            query = tokens + [3]
            want, got = o.lookup(so, query, None, None, now), l.lookup(sl, query, None, None, now)
            assert (want is None) == (got is None), (case, tokens)
            if want is not None:
                assert want[0] == got[0] and list(want[1]) == list(got[1]) and want[2] == got[2], (case, tokens)
                served += 1
        assert said(so, a, typed(so)) == said(sl, b, typed(so)), case
        assert len(so.refusals) == len(sl.refusals), case
        refused += len(so.refusals)
        assert meta(so) == meta(sl), case
        assert sorted(os.listdir(a)) == sorted(os.listdir(b))
        for name in os.listdir(a):
            assert (a / name).read_bytes() == (b / name).read_bytes(), (case, name)
    assert served >= 100 and refused >= 60, (served, refused)
