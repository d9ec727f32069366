"""Prefix snapshots between the device cache and ITKV v1 bytes, through the C ABI, against
the oracle: capture is byte-identical to the oracle's capture of the same rows, restore
reproduces the device bytes of the captured slot, and the reference's refusals come back
by name (crates/itak-kv/src/snapshot.rs:247-371, tests :645-753)."""
import numpy as np
import pytest
import torch

import oracle
from oracle import itak_kv as okv
from helpers import normal, pkg

pytestmark = pytest.mark.gpu


def P():
    return pkg()


def fill(layers, kv_heads, head_dim, tokens, elem, seed, capacity=None):
    rng = np.random.default_rng(seed)
    pool = P().KvPool(layers, kv_heads, head_dim, elem=elem, max_slots=3,
                      capacity_rows=capacity or tokens + 40)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    ref = oracle.KvCache.new([oracle.LayerKind.Global] * layers, kv_heads, head_dim,
                             store_f16=(elem == "f16"))
    width = kv_heads * head_dim
    for layer in range(layers):
        k, v = normal(rng, tokens, width), normal(rng, tokens, width)
        if tokens:
            kd, vd = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
            pool.append_device(layer, [(cache, tokens)], kd.data_ptr(), vd.data_ptr())
            ref.restore_bulk(layer, 0, k, v)
    torch.cuda.synchronize()
    return pool, cache, ref


@pytest.mark.parametrize("elem,kv_heads,head_dim,tokens", [
    ("f32", 2, 3, 10), ("f32", 4, 64, 77), ("f16", 4, 128, 300), ("f16", 4, 128, 33), ("f16", 2, 20, 9),
    ("f16", 4, 128, 0)])
def test_capture_is_the_oracles_capture_byte_for_byte(elem, kv_heads, head_dim, tokens):
    pool, cache, ref = fill(3, kv_heads, head_dim, tokens, elem, seed=tokens + head_dim)
    got = P().capture_bytes(cache, "model-a")
    want = okv.KvSnapshot.capture(ref, "model-a").to_bytes()
    assert got == want
    snap = P().KvSnapshot.capture(cache, "model-a")
    assert snap.token_count == tokens and len(snap.layers) == 3
    assert snap.to_bytes() == want
    pool.close()


@pytest.mark.parametrize("elem,fingerprint", [("f32", "model-a"), ("f16", "m"), ("f16", "ab"),
                                               ("f16", "abc"), ("f16", "")])
def test_restore_rebuilds_the_device_rows_and_can_continue(elem, fingerprint):
    # snapshot.rs:654-691 on the device: the restored slot holds the captured slot's bytes
    # (whatever the payload's alignment inside the encoding: it starts where the fingerprint
    # ends), and appends continue at the next position.
    kv_heads, head_dim, tokens, layers = 4, 128, 70, 3
    pool, cache, ref = fill(layers, kv_heads, head_dim, tokens, elem, seed=11)
    data = P().capture_bytes(cache, fingerprint)
    restored = P().restore_bytes(pool, data, fingerprint)
    for layer in range(layers):
        assert restored.next_position(layer) == tokens
        a, b = cache.read_raw(layer), restored.read_raw(layer)
        assert a[0].tobytes() == b[0].tobytes() and a[1].tobytes() == b[1].tobytes()
    row = np.full(kv_heads * head_dim, 1.5, np.float32)
    for layer in range(layers):
        restored.append(layer, row, -row, tokens)
    assert restored.next_position(0) == tokens + 1
    # The same bytes from pinned host memory are gathered in place.
    pinned = torch.from_numpy(np.frombuffer(data, dtype=np.uint8).copy()).pin_memory()
    again = P().restore_bytes(pool, pinned.numpy(), fingerprint)
    for layer in range(layers):
        a, b = cache.read_raw(layer), again.read_raw(layer)
        assert a[0].tobytes() == b[0].tobytes() and a[1].tobytes() == b[1].tobytes()
    pool.close()


def test_an_f32_snapshot_restores_into_an_f16_pool_through_the_append_conversion():
    kv_heads, head_dim, tokens = 4, 128, 45
    pool32, cache32, ref32 = fill(2, kv_heads, head_dim, tokens, "f32", seed=3)
    data = P().capture_bytes(cache32, "m")
    pool16 = P().KvPool(2, kv_heads, head_dim, elem="f16", capacity_rows=tokens + 40)
    restored = P().restore_bytes(pool16, data, "m")
    for layer in range(2):
        _, keys, values = ref32.view(layer).rows()
        gk, gv = restored.read_raw(layer)
        assert np.array_equal(gk[:tokens], oracle.f32_to_f16_array(keys))
        assert np.array_equal(gv[:tokens], oracle.f32_to_f16_array(values))
    pool32.close()
    pool16.close()


def test_refusals_come_back_by_name():
    kv_heads, head_dim, tokens = 4, 128, 20
    pool, cache, ref = fill(2, kv_heads, head_dim, tokens, "f16", seed=5)
    data = P().capture_bytes(cache, "model-a")
    # snapshot.rs:693-708: layers that disagree on position.
    row = np.zeros(kv_heads * head_dim, np.float32)
    cache.append(0, row, row, tokens)
    with pytest.raises(P().KvError) as e:
        P().capture_bytes(cache, "model-a")
    assert e.value.variant == "IncoherentCache"
    assert e.value.message == (f"incoherent cache: layer 0 has appended {tokens + 1} positions but "
                               f"layer 1 has appended {tokens}; a snapshot is one sequence")
    # snapshot.rs:731-753.
    with pytest.raises(P().KvError) as e:
        P().restore_bytes(pool, data, "model-b")
    assert e.value.variant == "FingerprintMismatch"
    assert e.value.message == "model fingerprint mismatch: need model-b, snapshot carries model-a"
    other = P().KvPool(2, kv_heads, 64, elem="f16", capacity_rows=64)
    with pytest.raises(P().KvError) as e:
        P().restore_bytes(other, data, "model-a")
    assert e.value.variant == "GeometryMismatch"
    assert e.value.message == ("geometry mismatch: snapshot geometry (2 layers, 4 KV heads, head dim "
                               "128) differs from the required geometry (2 layers, 4 KV heads, head "
                               "dim 64)")
    other.close()
    # snapshot.rs:710-729 through the pool path.
    bad = bytearray(data)
    bad[len(bad) - 12] ^= 0xFF
    with pytest.raises(P().KvError) as e:
        P().restore_bytes(pool, bytes(bad))
    assert e.value.variant == "ChecksumMismatch"
    with pytest.raises(P().KvError) as e:
        P().restore_bytes(pool, data[:8])
    assert e.value.variant == "Truncated"
    # A refused restore leaves no slot behind: all three slots can still be acquired.
    extra = [pool.acquire(), pool.acquire()]
    assert len(extra) == 2
    # A snapshot longer than a slot is a capacity refusal, not a fault.
    small = P().KvPool(2, kv_heads, head_dim, elem="f16", capacity_rows=8)
    with pytest.raises(P().KvError) as e:
        P().restore_bytes(small, data, "model-a")
    assert e.value.variant == "Attention"
    small.close()
    pool.close()


def test_a_long_snapshot_round_trips_and_decodes_continue_identically():
    # 8192 tokens x 4 layers of the 30B-class row (64 MiB of f32 rows): capture, restore into
    # a second slot, then the same decode step on both slots gives bitwise the same output.
    kv_heads, head_dim, tokens, layers, q_heads = 4, 128, 8192, 4, 32
    pool, cache, ref = fill(layers, kv_heads, head_dim, tokens, "f16", seed=9, capacity=tokens + 8)
    data = P().capture_bytes(cache, "sha256:0123")
    restored = P().restore_bytes(pool, data, "sha256:0123")
    rng = np.random.default_rng(1)
    q = torch.from_numpy(normal(rng, 1, q_heads * head_dim)).cuda()
    k = torch.from_numpy(normal(rng, 1, kv_heads * head_dim)).cuda()
    v = torch.from_numpy(normal(rng, 1, kv_heads * head_dim)).cuda()
    outs = []
    for c in (cache, restored):
        out = torch.empty_like(q)
        pool.attention_step_device(1, [(c, 1)], q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                   out.data_ptr(), q_heads)
        torch.cuda.synchronize()
        outs.append(out.cpu().numpy().tobytes())
    assert outs[0] == outs[1]
    pool.close()


# ---- version 2: an f16 pool snapshotted in its own bytes (no counterpart in the reference) --


@pytest.mark.parametrize("pattern,kv_heads,head_dim,tokens", [
    (["G", "G"], 4, 128, 300), (["W40", "G", "W40"], 4, 128, 133), (["W8"], 2, 20, 5),
])
def test_f16_snapshots_are_half_the_size_and_restore_the_same_bits(pattern, kv_heads, head_dim, tokens):
    kinds = [P().LayerKind.Global if p == "G" else P().LayerKind.windowed(int(p[1:])) for p in pattern]
    okinds = [oracle.LayerKind.Global if p == "G" else oracle.LayerKind.windowed(int(p[1:]))
              for p in pattern]
    rng = np.random.default_rng(tokens)
    pool = P().KvPool(kinds, kv_heads, head_dim, elem="f16", max_slots=3, capacity_rows=tokens + 40)
    cache = pool.acquire()
    ref = oracle.KvCache.new(okinds, kv_heads, head_dim, store_f16=True)
    width = kv_heads * head_dim
    for layer in range(len(kinds)):
        k, v = normal(rng, tokens, width), normal(rng, tokens, width)
        for p in range(tokens):
            cache.append(layer, k[p], v[p], p)
            ref.append(layer, k[p], v[p], p)
    v1 = P().capture_bytes(cache, "m")
    v2 = P().capture_bytes(cache, "m", elem="f16")
    # The layout, restated independently: v1 plus an element-type word, rows as halves.
    assert v2 == okv.to_bytes_f16(okv.KvSnapshot.capture(ref, "m"))
    payload = sum(ref.stored_len(layer) for layer in range(len(kinds))) * width * 2
    assert len(v1) - len(v2) == payload * 2 - 4
    # The reference's reader refuses it by name; the library reads the same f32 rows from both.
    with pytest.raises(okv.KvError) as e:
        okv.KvSnapshot.from_bytes(v2)
    assert e.value.variant == "UnsupportedVersion" and e.value.fields["version"] == 2
    a, b = P().KvSnapshot.from_bytes(v1), P().KvSnapshot.from_bytes(v2)
    assert a.geometry == b.geometry and a.token_count == b.token_count
    for la, lb in zip(a.layers, b.layers):
        assert la.first_position == lb.first_position
        assert la.keys.tobytes() == lb.keys.tobytes() and la.values.tobytes() == lb.values.tobytes()
    # Restored from either version, the slot holds the captured slot's bits.
    r1 = P().restore_bytes(pool, v1, "m")
    r2 = P().restore_bytes(pool, v2, "m")
    for layer in range(len(kinds)):
        want = cache.view(layer).rows()
        for other in (r1, r2):
            got = other.view(layer).rows()
            assert all(np.asarray(x).tobytes() == np.asarray(y).tobytes() for x, y in zip(got, want))
    pool.close()


def test_f16_snapshots_stay_with_f16_pools_and_go_through_the_store(tmp_path):
    rng = np.random.default_rng(2)
    f32_pool = P().KvPool(1, 2, 8, elem="f32", max_slots=2)
    c32 = f32_pool.acquire()
    c32.append(0, normal(rng, 16), normal(rng, 16), 0)
    with pytest.raises(P().KvError) as e:  # a narrowing capture is refused
        P().capture_bytes(c32, "m", elem="f16")
    assert "would drop precision" in e.value.message
    f16_pool = P().KvPool(1, 2, 8, elem="f16", max_slots=3)
    c16 = f16_pool.acquire()
    tokens = [5, 6, 7]
    for p in range(3):
        c16.append(0, normal(rng, 16), normal(rng, 16), p)
    v2 = P().capture_bytes(c16, "m", elem="f16")
    with pytest.raises(P().KvError) as e:  # f16 rows are never widened into an f32 pool
        P().restore_bytes(f32_pool, v2, "m")
    assert "f16 snapshot restores only into an f16 pool" in e.value.message
    # The prefix store files and serves the typed snapshot like any other.
    store = P().PrefixStore.open(str(tmp_path), 1 << 20)
    store.put(tokens, v2, 10)
    fresh = f16_pool.acquire()
    assert store.restore_prefix(fresh, tokens + [8], "m", now=11) == 3
    assert np.asarray(fresh.view(0).rows()[1]).tobytes() == np.asarray(c16.view(0).rows()[1]).tobytes()
    # The session flow's write half in the pool's own bytes, then the oracle's store (the
    # reference's reader) walks past the typed entry by name.
    store.capture_and_put(c16, tokens, "m", now=12, elem="f16")
    assert store.stats().entries == 1
    assert (tmp_path / store.entries()[0].file_name).read_bytes().endswith(v2)
    import oracle.prefix_store as ops
    theirs = ops.PrefixStore.open(ops.StoreConfig(str(tmp_path), 1 << 20))
    assert theirs.lookup(tokens, None, None, 13) is None
    assert any("unsupported format version 2" in r for r in theirs.refusals)
    # A truncated typed snapshot is refused by name like a version 1 one.
    with pytest.raises(P().KvError) as e:
        P().KvSnapshot.from_bytes(v2[:-3])
    assert e.value.variant == "Truncated"
    bad = bytearray(v2); bad[4 + 4 + 4 + 1 + 8 + 12] = 9   # the element-type word
    with pytest.raises(P().KvError) as e:
        P().KvSnapshot.from_bytes(bytes(bad))
    assert e.value.variant in ("InconsistentSnapshot", "ChecksumMismatch")
    f32_pool.close(); f16_pool.close()
