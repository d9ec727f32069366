"""The prefix store against a device pool: the two halves of the reference's session flow
(crates/wgpu-compute/src/session.rs:5000-5151) through the C ABI. A slot's rows are captured
and filed under their tokens; a later, fresh slot finds the longest stored prefix, has it
gathered from the store's pinned buffer, and continues exactly as the first slot does. The
entries the device side writes are served by the oracle's store and the other way round."""
import numpy as np
import pytest
import torch

import oracle
import oracle.itak_kv as okv
import oracle.prefix_store as ops
from helpers import max_abs, normal, pkg

pytestmark = pytest.mark.gpu


def P():
    return pkg()


def view_bytes(cache, layer):
    pos, keys, vals = cache.view(layer).rows()
    return np.asarray(pos, dtype=np.int64).tobytes() + np.ascontiguousarray(keys).tobytes() + \
        np.ascontiguousarray(vals).tobytes()


def step(pool, cache, layer, q, k, v, q_heads):
    qd, kd, vd = (torch.from_numpy(np.ascontiguousarray(x)).cuda() for x in (q, k, v))
    out = torch.empty_like(qd)
    pool.attention_step_device(layer, [(cache, q.shape[0])], qd.data_ptr(), kd.data_ptr(),
                               vd.data_ptr(), out.data_ptr(), q_heads)
    pool.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("elem,kvh,d,q_heads", [("f16", 4, 128, 32), ("f32", 2, 16, 4)])
def test_a_stored_prefix_restores_into_a_fresh_slot_and_continues_identically(tmp_path, elem, kvh, d,
                                                                              q_heads):
    rng = np.random.default_rng(11)
    pattern = [P().LayerKind.windowed(24), P().LayerKind.Global, P().LayerKind.windowed(24)]
    pool = P().KvPool(pattern, kvh, d, elem=elem, max_slots=3, capacity_rows=256)
    store = P().PrefixStore.open(str(tmp_path), 1 << 30)
    tokens = [int(t) for t in rng.integers(0, 50000, size=77)]
    a = pool.acquire()
    for layer in range(3):  # the prompt, as three chunks
        for first, rows in ((0, 40), (40, 36), (76, 1)):
            step(pool, a, layer, normal(rng, rows, q_heads * d), normal(rng, rows, kvh * d),
                 normal(rng, rows, kvh * d), q_heads)
    store.capture_and_put(a, tokens, "model-x", now=100)
    assert store.stats().entries == 1
    assert store.entries()[0].token_count == 77 and store.entries()[0].created_unix == 100

    # A later sequence that shares the prompt and goes on.
    b = pool.acquire()
    matched = store.restore_prefix(b, tokens + [1, 2, 3], "model-x", now=200)
    assert matched == 77
    assert store.entries()[0].last_used_unix == 200
    for layer in range(3):
        assert b.next_position(layer) == 77
        assert view_bytes(a, layer) == view_bytes(b, layer)
    for _ in range(30):  # past the windowed layers' wrap
        for layer in range(3):
            q, k, v = normal(rng, 1, q_heads * d), normal(rng, 1, kvh * d), normal(rng, 1, kvh * d)
            assert step(pool, a, layer, q, k, v, q_heads).tobytes() == \
                step(pool, b, layer, q, k, v, q_heads).tobytes()
    # A shorter query than the entry, another model, a slot already in use: nothing restored,
    # by name, and the slot stays as it was.
    c = pool.acquire()
    assert store.restore_prefix(c, tokens[:50], "model-x") == 0
    assert store.restore_prefix(c, tokens, "model-y") == 0
    assert any("need model-y, snapshot carries model-x" in r for r in store.refusals)
    assert c.next_position(0) == 0
    assert store.restore_prefix(b, tokens, "model-x") == 0
    assert any("session position is 107, not 0" in r for r in store.refusals)
    # Filing a slot under a token list of another length is refused.
    with pytest.raises(P().KvError) as e:
        store.capture_and_put(a, tokens, "model-x")
    assert e.value.variant == "StepFailed"
    assert "session position 107 does not equal the 77 tokens to store under" in e.value.message
    pool.close()


def test_device_and_oracle_stores_serve_each_other(tmp_path):
    rng = np.random.default_rng(5)
    kvh, d, n = 2, 8, 19
    pattern = [P().LayerKind.windowed(6), P().LayerKind.Global]
    opattern = [oracle.LayerKind.windowed(6), oracle.LayerKind.Global]
    k, v = normal(rng, 2, n, kvh * d), normal(rng, 2, n, kvh * d)
    tokens = list(range(100, 100 + n))
    pool = P().KvPool(pattern, kvh, d, elem="f32", max_slots=2, capacity_rows=64)
    cache = pool.acquire()
    ref = oracle.KvCache.new(opattern, kvh, d)
    for layer in range(2):
        for p in range(n):
            cache.append(layer, k[layer, p], v[layer, p], p)
            ref.append(layer, k[layer, p], v[layer, p], p)
    # Device side writes, oracle reads.
    dev_store = P().PrefixStore.open(str(tmp_path / "dev"), 1 << 30)
    dev_store.capture_and_put(cache, tokens, "m", now=7)
    hit = ops.PrefixStore.open(ops.StoreConfig(str(tmp_path / "dev"), 1 << 30)).lookup(
        tokens + [1], okv.KvGeometry(opattern, kvh, d), "m", 8)
    assert hit is not None and hit.token_count == n
    assert hit.snapshot.to_bytes() == okv.KvSnapshot.capture(ref, "m").to_bytes()
    # Oracle writes, device side restores.
    ora_store = ops.PrefixStore.open(ops.StoreConfig(str(tmp_path / "ora"), 1 << 30))
    ora_store.put(tokens, okv.KvSnapshot.capture(ref, "m"), 9)
    fresh = pool.acquire()
    assert P().PrefixStore.open(str(tmp_path / "ora"), 1 << 30).restore_prefix(
        fresh, tokens + [5, 6], "m", now=10) == n
    for layer in range(2):
        assert view_bytes(fresh, layer) == view_bytes(cache, layer)
    files = sorted(p.name for p in (tmp_path / "dev").iterdir())
    assert files == sorted(p.name for p in (tmp_path / "ora").iterdir())
    pool.close()


@pytest.mark.parametrize("elem", ["f32", "f16"])
def test_an_entry_filed_from_a_slot_carries_the_trailer_an_independent_sum_gives(tmp_path, elem):
    """The store sums a captured payload while it writes it. What lands on disk must be what a
    capture into memory gives, trailer included, and the trailer what the oracle's restatement
    of the checksum (byte-serial for version 1, sum of block sums for version 2) computes."""
    import struct

    rng = np.random.default_rng(21)
    kvh, d, n = 4, 128, 1500  # 1500 x 512 x 2 sides: 6.1 MB of f32 rows, 3.1 MB of f16 rows
    pool = P().KvPool([P().LayerKind.Global, P().LayerKind.windowed(256)], kvh, d, elem="f16",
                      max_slots=2, capacity_rows=n + 8)
    cache = pool.acquire()
    k, v = normal(rng, n, kvh * d), normal(rng, n, kvh * d)
    cache.restore_bulk(0, 0, k, v)
    cache.restore_bulk(1, n - 256, k[n - 256:], v[n - 256:])
    tokens = [int(t) for t in rng.integers(0, 1 << 20, size=n)]
    store = P().PrefixStore.open(str(tmp_path), 1 << 30)
    store.capture_and_put(cache, tokens, "m", now=5, elem=elem)
    entry = (tmp_path / store.entries()[0].file_name).read_bytes()
    payload = entry[72 + 4 * n:]
    assert payload == P().capture_bytes(cache, "m", elem=elem)
    stored = struct.unpack("<Q", payload[-8:])[0]
    fast = lambda block: oracle.checksum(bytes(block))
    want = fast(payload[:-8]) if elem == "f32" else okv.block_checksum(payload[:-8], fast)
    assert stored == want
    fresh = pool.acquire()
    assert store.restore_prefix(fresh, tokens, "m", now=6) == n
    for layer in range(2):
        assert view_bytes(fresh, layer) == view_bytes(cache, layer)
    pool.close()
