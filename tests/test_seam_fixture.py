"""The reference's seam fixture (crates/itak-kv/tests/restore_fixture.rs:21-189): a small
model shape where a cold run (append the prefix, continue) and a restored run (append the
prefix, snapshot it through the prefix store, restore into a fresh cache, continue) must give
bitwise identical attention outputs and identical greedy streams. Run on the oracle (no GPU)
and on the device through the C ABI; the device's logits are also held to the oracle's."""
import json
import os

import numpy as np
import pytest

import oracle
import oracle.itak_kv as okv
import oracle.prefix_store as ops
from helpers import pkg

Q_HEADS, LOGITS = 4, 16
KV_HEADS, HEAD_DIM = 2, 8
ROW = KV_HEADS * HEAD_DIM
PREFIX = [11, 22, 33, 44, 55, 66, 77, 88, 99]
CONTINUATION = [5, 4, 3, 2, 1]
_M64 = (1 << 64) - 1


def lcg(seed, count):  # restore_fixture.rs:21-30
    state = max(seed, 1)
    out = np.empty(count, dtype=np.float32)
    for i in range(count):
        state = (state * 6_364_136_223_846_793_005 + 1_442_695_040_888_963_407) & _M64
        out[i] = np.float32((state >> 40) & 0xFFFFFFFF) / np.float32(1 << 24) - np.float32(0.5)
    return out


def rows(layer, position, token):  # restore_fixture.rs:48-55
    stream = lcg((layer << 40) | (position << 16) | token, 2 * ROW)
    return stream[:ROW], stream[ROW:]


def head_weights(layers):  # restore_fixture.rs:77-80
    w = np.empty((layers, LOGITS, Q_HEADS * HEAD_DIM), dtype=np.float32)
    for layer in range(layers):
        for o in range(LOGITS):
            for i in range(Q_HEADS * HEAD_DIM):
                w[layer, o, i] = np.float32((o * 31 + i * 7 + layer * 3) % 13) / np.float32(7.0) \
                    - np.float32(0.8)
    return w


class Side:
    """One implementation of the fixture's three moving parts: cache, attention, store."""

    def __init__(self, name):
        self.name = name
        self.P = pkg() if name == "device" else None

    def pattern(self):
        K = self.P.LayerKind if self.P else oracle.LayerKind
        return [K.Windowed(4), K.Global, K.Global, K.Windowed(4)]

    def new_cache(self):
        if self.P:
            return self.P.KvCache.new(self.pattern(), KV_HEADS, HEAD_DIM, elem="f32", capacity_rows=64)
        return oracle.KvCache.new(self.pattern(), KV_HEADS, HEAD_DIM)

    def attention(self, q, position, view):
        if self.P:
            return self.P.gqa_attention(q, 1, Q_HEADS, [position], view, self.P.AttentionParams.new())
        return oracle.gqa_attention(q, 1, Q_HEADS, [position], view, oracle.AttentionParams.new())

    def through_the_store(self, root, warm, query):
        """capture -> put -> lookup under geometry and fingerprint -> restore_checked."""
        if self.P:
            P = self.P
            store = P.PrefixStore.open(str(root), 1 << 30)
            geometry = P.KvGeometry(self.pattern(), KV_HEADS, HEAD_DIM)
            store.put(PREFIX, P.KvSnapshot.capture(warm, "fixture-model"), 100)
            hit = store.lookup(query, geometry, "fixture-model", 200)
            assert hit is not None and hit.token_count == len(PREFIX)
            return hit.snapshot.restore_checked(warm.pool, geometry, "fixture-model")
        store = ops.PrefixStore.open(ops.StoreConfig(str(root), 1 << 30))
        geometry = okv.KvGeometry(self.pattern(), KV_HEADS, HEAD_DIM)
        store.put(PREFIX, okv.KvSnapshot.capture(warm, "fixture-model"), 100)
        hit = store.lookup(query, geometry, "fixture-model", 200)
        assert hit is not None and hit.token_count == len(PREFIX)
        return hit.snapshot.restore_checked(geometry, "fixture-model")


def append_token(cache, position, token):
    for layer in range(4):
        k, v = rows(layer, position, token)
        cache.append(layer, k, v, position)


def logits_for(side, cache, position, token, w):  # restore_fixture.rs:66-85
    q = lcg(0x5EED ^ (position << 20) ^ token, Q_HEADS * HEAD_DIM)
    logits = np.zeros(LOGITS, dtype=np.float32)
    for layer in range(4):
        out = np.asarray(side.attention(q, position, cache.view(layer)), dtype=np.float32)
        logits = logits + w[layer] @ out
    return logits


def continue_run(side, cache, start, w):  # restore_fixture.rs:99-113
    all_logits, stream = [], []
    for step, token in enumerate(CONTINUATION):
        position = start + step
        append_token(cache, position, token)
        logits = logits_for(side, cache, position, token, w)
        stream.append(int(np.argmax(logits)))
        all_logits.append(logits)
    return np.stack(all_logits), stream


def view_rows(cache, layer):
    pos, keys, vals = cache.view(layer).rows()
    return (np.asarray(pos, dtype=np.int64).tobytes(), np.ascontiguousarray(keys).tobytes(),
            np.ascontiguousarray(vals).tobytes())


def run_fixture(side, root):  # restore_fixture.rs:116-189
    w = head_weights(4)
    cold = side.new_cache()
    for position, token in enumerate(PREFIX):
        append_token(cold, position, token)
    cold_logits, cold_stream = continue_run(side, cold, len(PREFIX), w)

    warm = side.new_cache() if not side.P else None
    if side.P:  # the restored cache goes into a second slot of the warm cache's pool
        pool = side.P.KvPool(side.pattern(), KV_HEADS, HEAD_DIM, elem="f32", max_slots=3,
                             capacity_rows=64)
        warm = pool.acquire()
    for position, token in enumerate(PREFIX):
        append_token(warm, position, token)
    restored = side.through_the_store(root, warm, PREFIX + CONTINUATION)

    prefix_only = side.new_cache()
    for position, token in enumerate(PREFIX):
        append_token(prefix_only, position, token)
    for layer in range(4):
        assert view_rows(restored, layer) == view_rows(prefix_only, layer), f"layer {layer}"
        assert restored.next_position(layer) == len(PREFIX)

    restored_logits, restored_stream = continue_run(side, restored, len(PREFIX), w)
    assert restored_stream == cold_stream
    assert restored_logits.tobytes() == cold_logits.tobytes()
    return cold_logits, cold_stream


def test_restored_cache_continues_bitwise_identically_on_the_oracle(tmp_path):
    logits, stream = run_fixture(Side("oracle"), tmp_path)
    assert logits.shape == (5, 16) and np.isfinite(logits).all() and len(stream) == 5


@pytest.mark.gpu
def test_restored_cache_continues_bitwise_identically_on_the_device(tmp_path):
    device_logits, device_stream = run_fixture(Side("device"), tmp_path / "device")
    oracle_logits, oracle_stream = run_fixture(Side("oracle"), tmp_path / "oracle")
    scale = float(np.max(np.abs(oracle_logits)))
    assert float(np.max(np.abs(device_logits - oracle_logits))) <= 1e-4 * scale
    assert device_stream == oracle_stream
    # The two stores hold the same file.
    dev_files = sorted(p.name for p in (tmp_path / "device").iterdir())
    assert dev_files == sorted(p.name for p in (tmp_path / "oracle").iterdir())
    for name in dev_files:
        assert (tmp_path / "device" / name).read_bytes() == (tmp_path / "oracle" / name).read_bytes()


# ---- the committed golden fixtures (tests/golden/, written by tests/golden/make_fixtures.py)

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def golden():
    meta = json.load(open(os.path.join(GOLDEN, "seam_fixture.json")))
    logits = np.stack([np.frombuffer(bytes.fromhex(h), dtype="<f4") for h in meta["logits_f32_hex"]])
    snapshot = open(os.path.join(GOLDEN, "seam_prefix.itkv"), "rb").read()
    entry = open(os.path.join(GOLDEN, "seam_entry.kv"), "rb").read()
    return meta, logits, snapshot, entry


def test_golden_files_are_what_the_oracle_and_the_library_produce(tmp_path):
    meta, logits, snapshot, entry = golden()
    # The oracle reproduces them.
    side = Side("oracle")
    got_logits, got_stream = run_fixture(side, tmp_path / "o")
    assert got_stream == meta["greedy_stream"]
    assert float(np.max(np.abs(got_logits - logits))) <= 1e-6 * float(np.max(np.abs(logits)))
    assert (tmp_path / "o" / meta["entry_file_name"]).read_bytes() == entry
    decoded = okv.KvSnapshot.from_bytes(snapshot)
    assert decoded.token_count == 9 and decoded.model_fingerprint == "fixture-model"
    assert okv.prefix_hash(PREFIX) == meta["prefix_hash"]
    assert okv.checksum(snapshot[:-8]) == meta["snapshot_checksum"]
    # The library's codec, hashes and store (host code: no GPU needed) agree with the files.
    P = pkg()
    assert P.prefix_hash(PREFIX) == meta["prefix_hash"]
    assert P.checksum(snapshot[:-8]) == meta["snapshot_checksum"]
    assert P.KvSnapshot.from_bytes(snapshot).to_bytes() == snapshot
    store = P.PrefixStore.open(str(tmp_path / "l"), 1 << 30)
    store.put(PREFIX, snapshot, 100)
    hit = store.lookup(PREFIX + CONTINUATION, None, "fixture-model", 200)
    assert hit is not None and hit.snapshot_bytes == snapshot
    assert (tmp_path / "l" / meta["entry_file_name"]).read_bytes() == entry
    # And a store directory holding the golden entry serves it.
    (tmp_path / "g").mkdir()
    (tmp_path / "g" / meta["entry_file_name"]).write_bytes(entry)
    for opened in (P.PrefixStore.open(str(tmp_path / "g"), 1 << 30),
                   ops.PrefixStore.open(ops.StoreConfig(str(tmp_path / "g"), 1 << 30))):
        hit = opened.lookup(PREFIX + [1], None, None, 300)
        assert hit is not None and hit.token_count == 9


@pytest.mark.gpu
def test_device_restores_the_golden_entry_and_reproduces_the_golden_stream(tmp_path):
    meta, logits, snapshot, entry = golden()
    P = pkg()
    side = Side("device")
    (tmp_path / meta["entry_file_name"]).write_bytes(entry)
    store = P.PrefixStore.open(str(tmp_path), 1 << 30)
    pool = P.KvPool(side.pattern(), KV_HEADS, HEAD_DIM, elem="f32", max_slots=2, capacity_rows=64)
    cache = pool.acquire()
    assert store.restore_prefix(cache, PREFIX + CONTINUATION, "fixture-model", now=300) == 9
    assert P.capture_bytes(cache, "fixture-model") == snapshot
    got_logits, got_stream = continue_run(side, cache, 9, head_weights(4))
    assert got_stream == meta["greedy_stream"]
    assert float(np.max(np.abs(got_logits - logits))) <= 1e-4 * float(np.max(np.abs(logits)))
    pool.close()
