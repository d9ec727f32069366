"""The oracle's restatement of the prefix-snapshot crate, pinned by the reference's own
cases (crates/itak-kv/src/snapshot.rs:606-861, hash.rs:63-87), by the published FNV-1a
test vectors, and by a snapshot assembled by hand from the layout table (snapshot.rs:13-29).
The library's host-side codec is then held to the oracle's bytes and refusals through the
C ABI (no GPU needed: the codec never touches the device)."""
import struct

import numpy as np
import pytest

import oracle
from oracle import itak_kv as okv
from helpers import pkg

LK = oracle.LayerKind


def geometry():  # snapshot.rs:610-621
    return okv.KvGeometry([LK.Windowed(4), LK.Global, LK.Windowed(4)], 2, 3)


def filled_cache(tokens, upto_layers=3):  # snapshot.rs:623-643
    g = geometry()
    cache = oracle.KvCache.new(g.layers, g.num_kv_heads, g.head_dim)
    row = g.row_floats()
    for position in range(tokens):
        for layer in range(upto_layers):
            k = (np.arange(row) + position * 100 + layer * 10).astype(np.float32) / np.float32(7.0)
            v = -((np.arange(row) + position * 50 + layer * 5).astype(np.float32)) / np.float32(3.0)
            cache.append(layer, k, v, position)
    return cache


def same_snapshot(a, b):
    assert a.geometry == b.geometry and a.model_fingerprint == b.model_fingerprint
    assert a.token_count == b.token_count and len(a.layers) == len(b.layers)
    for x, y in zip(a.layers, b.layers):
        assert x.first_position == y.first_position
        assert np.asarray(x.keys).tobytes() == np.asarray(y.keys).tobytes()
        assert np.asarray(x.values).tobytes() == np.asarray(y.values).tobytes()


# ---- hashes ---------------------------------------------------------------------------

def test_fnv1a_matches_the_published_vectors_and_the_reference_cases():
    # FNV-1a 64 test vectors of the algorithm's authors (empty, "a", "foobar").
    assert okv.checksum(b"") == 0xCBF29CE484222325 == oracle.checksum(b"")
    assert okv.checksum(b"a") == 0xAF63DC4C8601EC8C == oracle.checksum(b"a")
    assert okv.checksum(b"foobar") == 0x85944171F73967E8 == oracle.checksum(b"foobar")
    # hash.rs:67-87.
    assert okv.prefix_hash([1, 2, 3]) != okv.prefix_hash([3, 2, 1])
    assert okv.prefix_hash([1, 2, 3]) != okv.prefix_hash([1, 2, 4])
    assert okv.prefix_hash([1, 2]) != okv.prefix_hash([1, 2, 0])
    assert okv.prefix_hash([]) == 0xCBF29CE484222325
    assert okv.prefix_hash([7, 8, 9, 10]) != okv.prefix_discriminator([7, 8, 9, 10])
    assert okv.checksum(b"itkv") != okv.checksum(b"itkw")
    # Token ids enter as little-endian bytes (hash.rs:35-41): one token == its 4 bytes.
    assert okv.prefix_hash([0x04030201]) == okv.checksum(bytes([1, 2, 3, 4]))
    assert oracle.prefix_hash([7, 8, 9, 10]) == okv.prefix_hash([7, 8, 9, 10])


def test_prefix_discriminator_is_pinned_by_literals():
    # The discriminator is FNV-1a 64 from the alternate basis of hash.rs:21. No tokens give the
    # basis itself; the other two values were folded by hand (xor a byte, multiply by the prime
    # 0x100000001b3 modulo 2^64, four little-endian bytes per token), not by the code under
    # test: [1] and [0xDEADBEEF, 7].
    P = pkg()
    for fn in (okv.prefix_discriminator, P.prefix_discriminator):
        assert fn([]) == 0x84222325CBF29CE4
        assert fn([1]) == 0xB61D2746190C09B5
        assert fn([0xDEADBEEF, 7]) == 0x393DB72D40DB1AFD
    # The same fold from the standard basis, for contrast (hash.rs:44-46).
    assert okv.prefix_hash([1]) == 0xAD2ACA7747985764 == P.prefix_hash([1])


# ---- layout -----------------------------------------------------------------------------

def test_bytes_follow_the_layout_table():
    # One global layer, 1 KV head of dim 2, 2 tokens, fingerprint "ab": every field at the
    # offset the table of snapshot.rs:13-29 gives it.
    snap = okv.KvSnapshot(okv.KvGeometry([LK.Global], 1, 2), "ab", 2,
                          [okv.LayerSnapshot(0, np.array([1, 2, 3, 4], np.float32),
                                             np.array([5, 6, 7, 8], np.float32))])
    b = snap.to_bytes()
    assert b[0:4] == b"ITKV"
    assert struct.unpack_from("<I", b, 4)[0] == 1            # format_version
    assert struct.unpack_from("<I", b, 8)[0] == 2            # fingerprint_len
    assert b[12:14] == b"ab"
    assert struct.unpack_from("<Q", b, 14)[0] == 2           # token_count
    assert struct.unpack_from("<III", b, 22) == (1, 2, 1)    # kv heads, head dim, layer count
    assert b[34:38] == bytes([0, 0, 0, 0])                   # kind tag + 3 reserved
    assert struct.unpack_from("<QQQ", b, 38) == (0, 0, 2)    # window, first_position, row_count
    assert struct.unpack_from("<4f", b, 62) == (1, 2, 3, 4)  # keys
    assert struct.unpack_from("<4f", b, 78) == (5, 6, 7, 8)  # values
    assert len(b) == 94 + 8
    assert struct.unpack_from("<Q", b, 94)[0] == okv.checksum(b[:94])
    # A windowed layer writes tag 1 and its window.
    snap = okv.KvSnapshot(okv.KvGeometry([LK.Windowed(4)], 1, 1), "", 6,
                          [okv.LayerSnapshot(2, np.zeros(4, np.float32), np.zeros(4, np.float32))])
    b = snap.to_bytes()
    assert b[32] == 1 and struct.unpack_from("<QQQ", b, 36) == (4, 2, 4)


# ---- the reference's cases ----------------------------------------------------------------

def test_bytes_round_trip():  # snapshot.rs:645-652
    snapshot = okv.KvSnapshot.capture(filled_cache(10), "model-a")
    same_snapshot(okv.KvSnapshot.from_bytes(snapshot.to_bytes()), snapshot)
    # Windowed layers keep the last 4 rows, the global layer all 10.
    assert [l.first_position for l in snapshot.layers] == [6, 0, 6]
    assert [l.rows(6) for l in snapshot.layers] == [4, 10, 4]


def test_restore_rebuilds_the_same_views():  # snapshot.rs:654-676
    cache = filled_cache(10)
    restored = okv.KvSnapshot.capture(cache, "model-a").restore()
    for layer in range(3):
        assert restored.next_position(layer) == cache.next_position(layer)
        want, got = cache.view(layer).rows(), restored.view(layer).rows()
        for w, g in zip(want, got):
            assert np.asarray(w).tobytes() == np.asarray(g).tobytes()


def test_restore_can_continue_appending():  # snapshot.rs:678-691
    restored = okv.KvSnapshot.capture(filled_cache(6), "model-a").restore()
    for layer in range(3):
        restored.append(layer, np.full(6, 1.5, np.float32), np.full(6, -2.5, np.float32), 6)
    assert restored.next_position(0) == 7


def test_capture_refuses_a_divergent_cache():  # snapshot.rs:693-708
    with pytest.raises(okv.KvError) as e:
        okv.KvSnapshot.capture(filled_cache(1, upto_layers=1), "model-a")
    assert e.value.variant == "IncoherentCache"


def test_decode_refuses_corruption():  # snapshot.rs:710-729
    snapshot = okv.KvSnapshot.capture(filled_cache(5), "model-a")
    data = bytearray(snapshot.to_bytes())
    data[len(data) - 12] ^= 0xFF
    with pytest.raises(okv.KvError) as e:
        okv.KvSnapshot.from_bytes(bytes(data))
    assert e.value.variant == "ChecksumMismatch"
    with pytest.raises(okv.KvError) as e:
        okv.KvSnapshot.from_bytes(bytes(data[:8]))
    assert e.value.variant == "Truncated" and e.value.fields == {"what": "snapshot", "expected": 12, "actual": 8}
    bad = bytearray(snapshot.to_bytes())
    bad[0] = ord("X")
    with pytest.raises(okv.KvError) as e:
        okv.KvSnapshot.from_bytes(bytes(bad))
    assert e.value.variant == "BadMagic"


def test_restore_checked_refuses_geometry_and_fingerprint():  # snapshot.rs:731-753
    snapshot = okv.KvSnapshot.capture(filled_cache(4), "model-a")
    other = geometry()
    other.head_dim = 9
    with pytest.raises(okv.KvError) as e:
        snapshot.restore_checked(other, "model-a")
    assert e.value.variant == "GeometryMismatch"
    with pytest.raises(okv.KvError) as e:
        snapshot.restore_checked(geometry(), "model-b")
    assert e.value.variant == "FingerprintMismatch"
    snapshot.restore_checked(geometry(), "model-a")


def forged_layer_count():  # snapshot.rs:755-780
    b = b"ITKV" + struct.pack("<IIQIII", 1, 0, 0, 1, 1, 0xFFFFFFFF)
    assert len(b) == 32
    return b


def forged_overflow(heads, dim, token_count):  # snapshot.rs:794-812
    b = b"ITKV" + struct.pack("<II", 1, 1) + b"x" + struct.pack("<QIII", token_count, heads, dim, 1)
    b += bytes([0, 0, 0, 0]) + struct.pack("<QQQ", 0, 0, 0)
    return b + struct.pack("<Q", okv.checksum(b))


def test_decode_refuses_forged_headers():  # snapshot.rs:755-819
    for data in (forged_layer_count(), forged_overflow(65536, 65536, 1 << 32)):
        with pytest.raises(okv.KvError) as e:
            okv.KvSnapshot.from_bytes(data)
        assert e.value.variant == "InconsistentSnapshot"


def test_validate_refuses_geometry_whose_row_width_overflows():  # snapshot.rs:821-842
    foreign = okv.KvSnapshot(okv.KvGeometry([LK.Global], 1 << 32, 1 << 32), "x", 0,
                             [okv.LayerSnapshot(0, np.zeros(0, np.float32), np.zeros(0, np.float32))])
    with pytest.raises(okv.KvError) as e:
        foreign.validate()
    assert e.value.variant == "InconsistentSnapshot"


def test_glimmer_sizing_math():  # snapshot.rs:844-861
    g = okv.KvGeometry(oracle.glimmer_layer_pattern(), 2, 128)
    assert g.bytes_per_token() == 106_496
    assert g.stored_bytes_for(4096) == 272_629_760
    assert g.stored_bytes_for(131_072) == 3_653_238_784


# ---- the library's codec, through the C ABI, against the oracle ---------------------------------

def to_product(snapshot):
    P = pkg()
    kinds = [P.LayerKind.Global if k.window() is None else P.LayerKind.Windowed(k.window())
             for k in snapshot.geometry.layers]
    return P.KvSnapshot(P.KvGeometry(kinds, snapshot.geometry.num_kv_heads, snapshot.geometry.head_dim),
                        snapshot.model_fingerprint, snapshot.token_count,
                        [P.LayerSnapshot(l.first_position, l.keys, l.values) for l in snapshot.layers])


@pytest.mark.parametrize("tokens,fingerprint", [(10, "model-a"), (3, ""), (0, "x"), (5, "sha256:ä€𝄞")])
def test_library_encodes_and_decodes_the_oracles_bytes(tokens, fingerprint):
    snapshot = okv.KvSnapshot.capture(filled_cache(tokens), fingerprint)
    want = snapshot.to_bytes()
    assert to_product(snapshot).to_bytes() == want
    decoded = pkg().KvSnapshot.from_bytes(want)
    assert decoded.model_fingerprint == fingerprint and decoded.token_count == tokens
    assert decoded.geometry.num_kv_heads == 2 and decoded.geometry.head_dim == 3
    assert [k.window() for k in decoded.geometry.layers] == [4, None, 4]
    for got, ref in zip(decoded.layers, snapshot.layers):
        assert got.first_position == ref.first_position
        assert got.keys.tobytes() == ref.keys.tobytes() and got.values.tobytes() == ref.values.tobytes()
    assert decoded.to_bytes() == want


def test_library_hashes_match_the_oracle():
    P = pkg()
    rng = np.random.default_rng(0)
    blob = rng.integers(0, 256, size=10_001, dtype=np.uint8).tobytes()
    assert P.checksum(blob) == okv.checksum(blob)
    assert P.checksum(b"") == 0xCBF29CE484222325 and P.checksum(b"foobar") == 0x85944171F73967E8
    tokens = rng.integers(0, 2**32, size=257, dtype=np.uint64).astype(np.uint32).tolist()
    assert P.prefix_hash(tokens) == okv.prefix_hash(tokens)
    assert P.prefix_discriminator(tokens) == okv.prefix_discriminator(tokens)
    assert P.prefix_hash([]) == 0xCBF29CE484222325


def library_refusal(data):
    with pytest.raises(pkg().KvError) as e:
        pkg().KvSnapshot.from_bytes(data)
    return e.value


def oracle_refusal(data):
    with pytest.raises(okv.KvError) as e:
        okv.KvSnapshot.from_bytes(data)
    return e.value


def test_library_refuses_what_the_oracle_refuses_in_the_same_words():
    good = okv.KvSnapshot.capture(filled_cache(5), "model-a").to_bytes()
    cases = []
    flipped = bytearray(good); flipped[len(good) - 12] ^= 0xFF; cases.append(bytes(flipped))
    cases += [good[:8], good[:3], good[:40], good[:len(good) - 1], good + b"\0"]
    bad_magic = bytearray(good); bad_magic[0] = ord("X"); cases.append(bytes(bad_magic))
    # (Version 2 is the library's own typed format, which the reference's reader refuses by
    # name and the library reads: tests/test_gpu_snapshot.py. An unknown version is refused
    # by both.)
    version = bytearray(good); version[4] = 3; cases.append(bytes(version))
    cases += [forged_layer_count(), forged_overflow(65536, 65536, 1 << 32)]

    def resum(b):
        return bytes(b[:-8]) + struct.pack("<Q", okv.checksum(bytes(b[:-8])))
    reserved = bytearray(good); reserved[12 + 7 + 20 + 1] = 1; cases.append(resum(reserved))
    tag = bytearray(good); tag[12 + 7 + 20] = 7; cases.append(resum(tag))
    zero_window = bytearray(good); zero_window[12 + 7 + 20 + 4: 12 + 7 + 20 + 12] = bytes(8); cases.append(resum(zero_window))
    first = bytearray(good); first[12 + 7 + 20 + 12] ^= 1; cases.append(resum(first))
    utf8 = bytearray(good); utf8[12] = 0xFF; cases.append(resum(utf8))
    zero_heads = bytearray(good); zero_heads[12 + 7 + 8: 12 + 7 + 12] = bytes(4); cases.append(resum(zero_heads))
    for data in cases:
        want, got = oracle_refusal(data), library_refusal(data)
        assert (got.variant, got.message) == (want.variant, want.message), data[:48]
        for key in ("expected", "actual", "stored", "computed", "version"):
            if key in want.fields:
                assert got.fields[key] == want.fields[key]


def test_library_validate_matches_the_oracle_on_in_memory_snapshots():
    snapshot = okv.KvSnapshot.capture(filled_cache(6), "m")
    broken = []
    s = okv.KvSnapshot.capture(filled_cache(6), "m"); s.layers.pop(); broken.append(s)
    s = okv.KvSnapshot.capture(filled_cache(6), "m"); s.layers[1].keys = s.layers[1].keys[:-1]; broken.append(s)
    s = okv.KvSnapshot.capture(filled_cache(6), "m"); s.layers[0].first_position = 1; broken.append(s)
    s = okv.KvSnapshot.capture(filled_cache(6), "m"); s.token_count = 7; broken.append(s)
    broken.append(okv.KvSnapshot(okv.KvGeometry([LK.Global], 0, 4), "x", 0,
                                 [okv.LayerSnapshot(0, np.zeros(0, np.float32), np.zeros(0, np.float32))]))
    broken.append(okv.KvSnapshot(okv.KvGeometry([LK.Global], 1 << 32, 1 << 32), "x", 0,
                                 [okv.LayerSnapshot(0, np.zeros(0, np.float32), np.zeros(0, np.float32))]))
    to_product(snapshot).validate()
    for s in broken:
        with pytest.raises(okv.KvError) as want:
            s.validate()
        with pytest.raises(pkg().KvError) as got:
            to_product(s).validate()
        assert (got.value.variant, got.value.message) == (want.value.variant, want.value.message)
        with pytest.raises(pkg().KvError):
            to_product(s).to_bytes()
    g = pkg().KvGeometry([pkg().LayerKind.Global if i % 4 == 3 else pkg().LayerKind.Windowed(2048)
                          for i in range(52)], 2, 128)
    assert (g.bytes_per_token(), g.stored_bytes_for(4096), g.stored_bytes_for(131_072)) == \
        (106_496, 272_629_760, 3_653_238_784)


# ---- version 2 on the host (this library's own format; no counterpart in the reference) ----

def _fast_sum(data):  # FNV-1a 64 from the offset basis, the oracle's C restatement
    return oracle.checksum(bytes(data))


def test_block_checksum_is_the_sum_of_block_sums_at_every_boundary():
    P = pkg()
    rng = np.random.default_rng(2)
    B = okv.SUM_BLOCK
    assert P.checksum_blocks(b"") == okv.FNV_OFFSET == okv.block_checksum(b"")
    # (The library walks blocks in groups of four: sizes on both sides of a group's edge too.)
    for size in (1, 77, B - 1, B, B + 1, 2 * B, 3 * B + 5, 4 * B, 4 * B + 1, 5 * B + 17, 8 * B - 3, 9 * B):
        data = rng.integers(0, 256, size=size, dtype=np.uint8).tobytes()
        want = okv.block_checksum(data, _fast_sum)
        assert P.checksum_blocks(data) == want, size
        if size <= B:  # one block: the sum of one sum, not the plain checksum
            assert want == okv.checksum(struct.pack("<Q", _fast_sum(data)))
            assert want != _fast_sum(data)
    # Two blocks swapped, and a byte moved across a block edge, change it.
    data = bytearray(rng.integers(0, 256, size=2 * B, dtype=np.uint8).tobytes())
    swapped = bytes(data[B:]) + bytes(data[:B])
    assert P.checksum_blocks(bytes(data)) != P.checksum_blocks(swapped)
    assert _fast_sum(bytes(data[:77])) == okv.checksum(bytes(data[:77]))  # the C sum is the Python sum


def test_a_version_2_snapshot_of_several_blocks_decodes_and_a_flip_in_any_block_is_refused():
    P = pkg()
    rng = np.random.default_rng(4)
    kvh, d, rows = 2, 64, 2600  # 2600 x 128 halves x 2 sides: 1.3 MB, two blocks
    geometry = okv.KvGeometry([oracle.LayerKind.Global, oracle.LayerKind.windowed(2600)], kvh, d)
    layers = []
    for _ in range(2):
        k = rng.standard_normal(rows * kvh * d, dtype=np.float32).astype(np.float16).astype(np.float32)
        v = rng.standard_normal(rows * kvh * d, dtype=np.float32).astype(np.float16).astype(np.float32)
        layers.append(okv.LayerSnapshot(0, k, v))
    snap = okv.KvSnapshot(geometry, "typed", rows, layers)
    v2 = okv.to_bytes_f16(snap, _fast_sum)
    assert len(v2) > 2 * okv.SUM_BLOCK
    decoded = P.KvSnapshot.from_bytes(v2)
    assert decoded.token_count == rows and decoded.model_fingerprint == "typed"
    for got, want in zip(decoded.layers, layers):
        assert got.keys.tobytes() == want.keys.tobytes()
        assert got.values.tobytes() == want.values.tobytes()
    assert P.KvSnapshot.from_bytes(snap.to_bytes()).layers[1].values.tobytes() == layers[1].values.tobytes()
    for offset in (50, okv.SUM_BLOCK + 3, len(v2) - 9):
        bad = bytearray(v2)
        bad[offset] ^= 0x10
        with pytest.raises(P.KvError) as e:
            P.KvSnapshot.from_bytes(bytes(bad))
        assert e.value.variant == "ChecksumMismatch", offset
    # The version 1 trailer on version 2 bytes is refused: the two sums are different functions.
    forged = v2[:-8] + struct.pack("<Q", _fast_sum(v2[:-8]))
    with pytest.raises(P.KvError) as e:
        P.KvSnapshot.from_bytes(forged)
    assert e.value.variant == "ChecksumMismatch"


def _mutated(good, rng):
    """One seeded corruption of encoded bytes: flips, cuts, insertions and extreme field values,
    half of them with the trailer recomputed so that the checks behind the checksum are reached."""
    b = bytearray(good)
    extremes = (0, 1, 2, 3, 0x80000000, 0xFFFFFFFF, 1 << 32, 1 << 61, 1 << 62, (1 << 63) - 1, (1 << 64) - 1)
    for _ in range(int(rng.integers(1, 4))):
        kind = int(rng.integers(0, 6))
        if kind == 0 and b:
            b[int(rng.integers(0, len(b)))] ^= 1 << int(rng.integers(0, 8))
        elif kind == 1:
            del b[int(rng.integers(0, len(b) + 1)):]
        elif kind == 2 and len(b) >= 16:
            width = 8 if rng.integers(0, 2) else 4
            at = int(rng.integers(0, min(len(b) - 8, 200) - width + 1)) & ~3
            b[at:at + width] = int(extremes[int(rng.integers(0, len(extremes)))] % (1 << (8 * width))).to_bytes(width, "little")
        elif kind == 3:
            b += rng.integers(0, 256, size=int(rng.integers(1, 40)), dtype=np.uint8).tobytes()
        elif kind == 4 and len(b) > 12:
            at = int(rng.integers(0, len(b) - 4))
            del b[at:at + int(rng.integers(1, 33))]
        elif kind == 5 and len(b) >= 16:
            b[int(rng.integers(0, min(len(b) - 8, 200)))] = int(rng.integers(0, 256))
    if rng.integers(0, 2) and len(b) >= 8:
        b[-8:] = struct.pack("<Q", okv.checksum(bytes(b[:-8])))
    return bytes(b)


def test_seeded_corruptions_get_the_same_verdict_from_library_and_oracle():
    """600 corrupted snapshots: the library accepts exactly what the oracle accepts, with the same
    contents, and refuses the rest under the same variant, message and fields."""
    P = pkg()
    rng = np.random.default_rng(20)
    seeds = [okv.KvSnapshot.capture(filled_cache(n), fp).to_bytes()
             for n, fp in ((1, ""), (3, "m"), (5, "model-a"), (9, "längere-Kennung"))]
    accepted = refused = 0
    variants = set()
    for case in range(600):
        data = _mutated(seeds[case % len(seeds)], rng)
        if len(data) >= 8 and data[:4] == b"ITKV" and struct.unpack_from("<I", data, 4)[0] == 2:
            # The library's own typed format: the reference's reader refuses the version by
            # name, the library goes on to read it (and refuses these bytes for other reasons).
            assert oracle_refusal(data).variant == "UnsupportedVersion"
            library_refusal(data)
            continue
        try:
            want = okv.KvSnapshot.from_bytes(data)
        except okv.KvError as e:
            got = library_refusal(data)
            assert (got.variant, got.message) == (e.variant, e.message), (case, data[:64])
            for key in ("expected", "actual", "stored", "computed", "version"):
                if key in e.fields:
                    assert got.fields[key] == e.fields[key], (case, key)
            refused += 1
            variants.add(e.variant)
            continue
        got = P.KvSnapshot.from_bytes(data)
        assert got.token_count == want.token_count and got.model_fingerprint == want.model_fingerprint
        assert (got.geometry.num_kv_heads, got.geometry.head_dim) == (want.geometry.num_kv_heads, want.geometry.head_dim)
        assert [(k.is_windowed, k.window_size) for k in got.geometry.layers] == \
               [(k.is_windowed, k.window_size) for k in want.geometry.layers]
        assert len(got.layers) == len(want.layers)
        for x, y in zip(got.layers, want.layers):
            assert x.first_position == y.first_position
            assert np.asarray(x.keys).tobytes() == np.asarray(y.keys).tobytes()
            assert np.asarray(x.values).tobytes() == np.asarray(y.values).tobytes()
        accepted += 1
    assert accepted >= 10 and refused >= 400 and len(variants) >= 4, (accepted, refused, variants)
