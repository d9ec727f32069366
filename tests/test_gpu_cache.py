"""KV cache on the GPU through the C ABI: the reference's cache and checkpoint cases that
apply to global layers (crates/attention/tests/cache_tests.rs, checkpoint_tests.rs), and
bit-exact parity with the CPU oracle for append, truncate and restore."""
import numpy as np
import pytest

import oracle
from helpers import normal, pkg

pytestmark = pytest.mark.gpu


def P():
    return pkg()


def E(variant, **f):
    return P().AttentionError(variant, **f)


def row(kv_heads, head_dim, fill):
    return np.full(kv_heads * head_dim, fill, dtype=np.float32)


def k_row(kv_heads, head_dim, position):  # checkpoint_tests.rs:17-21
    e = np.arange(kv_heads * head_dim)
    return (position * 1000 + (e // head_dim) * 100 + (e % head_dim)).astype(np.float32)


def v_row(kv_heads, head_dim, position):  # checkpoint_tests.rs:25-29
    e = np.arange(kv_heads * head_dim)
    return (position * 1000 + 500 + (e // head_dim) * 100 + (e % head_dim)).astype(np.float32)


def view_snapshot(cache, layer):  # checkpoint_tests.rs:54-65, on either implementation
    pos, keys, vals = cache.view(layer).rows()
    return (np.asarray(pos, dtype=np.int64).tobytes() + np.ascontiguousarray(keys).tobytes()
            + np.ascontiguousarray(vals).tobytes())


def test_global_layer_keeps_everything():
    # cache_tests.rs:81-96.
    cache = P().KvCache.new([P().LayerKind.Global], 2, 2)
    for pos in range(10):
        cache.append(0, row(2, 2, pos), row(2, 2, pos), pos)
    assert cache.stored_len(0) == 10
    view = cache.view(0)
    assert view.len() == 10 and view.window() is None
    for pos in range(10):
        assert view.position_at(pos) == pos
        assert view.value(pos, 1)[0] == float(pos)
    assert view.position_at(10) is None and view.key(10, 0) is None


def test_append_rejects_bad_shapes_and_out_of_order_positions():
    # cache_tests.rs:98-131.
    cache = P().KvCache.new([P().LayerKind.Global], 2, 4)
    with pytest.raises(P().AttentionError) as e:
        cache.append(0, row(1, 4, 0.0), row(2, 4, 0.0), 0)
    assert e.value == E("ShapeMismatch", what="k", expected=8, actual=4)
    assert e.value.message == "k: got 4, expected 8"
    with pytest.raises(P().AttentionError) as e:
        cache.append(0, row(2, 4, 0.0), row(2, 4, 0.0), 1)
    assert e.value == E("OutOfOrderPosition", layer=0, expected=0, actual=1)
    assert cache.stored_len(0) == 0
    cache.append(0, row(2, 4, 0.0), row(2, 4, 0.0), 0)
    assert cache.stored_len(0) == 1


def test_invalid_layer_and_capacity_are_errors_not_faults():
    # cache_tests.rs:185-205, plus the pool's own bound.
    cache = P().KvCache.new([P().LayerKind.Global], 1, 1, capacity_rows=2)
    with pytest.raises(P().AttentionError) as e:
        cache.view(5)
    assert e.value == E("InvalidLayer", layer=5, layer_count=1)
    with pytest.raises(P().AttentionError) as e:
        cache.append(5, row(1, 1, 0.0), row(1, 1, 0.0), 0)
    assert e.value == E("InvalidLayer", layer=5, layer_count=1)
    assert cache.layer_kind(0) == P().LayerKind.Global
    cache.append(0, [1.0], [1.0], 0)
    cache.append(0, [2.0], [2.0], 1)
    with pytest.raises(P().AttentionError) as e:
        cache.append(0, [3.0], [3.0], 2)
    assert e.value.variant == "CapacityExceeded"
    assert cache.stored_len(0) == 2


@pytest.mark.parametrize("elem", ["f32", "f16"])
@pytest.mark.parametrize("kv_heads,head_dim", [(4, 64), (4, 128), (2, 3), (1, 1), (3, 20)])
def test_append_is_bit_exact_against_the_oracle(elem, kv_heads, head_dim):
    rng = np.random.default_rng(kv_heads * 1000 + head_dim)
    n = 37
    scale = np.float32(10.0) ** rng.integers(-8, 6, size=(n, 1)).astype(np.float32)
    k = normal(rng, n, kv_heads * head_dim) * scale
    v = normal(rng, n, kv_heads * head_dim) * scale
    k[3, 0], v[3, -1] = np.inf, -np.inf
    k[4, 0] = np.nan
    k[5, :] = 65520.0          # rounds to infinity in f16
    v[5, :] = 5.9604645e-08    # 2^-24: the smallest subnormal half
    gpu = P().KvCache.new([P().LayerKind.Global] * 2, kv_heads, head_dim, elem=elem,
                          capacity_rows=64)
    cpu = oracle.KvCache.new([oracle.LayerKind.Global] * 2, kv_heads, head_dim,
                             store_f16=(elem == "f16"))
    for layer in range(2):
        for p in range(n - layer):
            gpu.append(layer, k[p], v[p], p)
            cpu.append(layer, k[p], v[p], p)
    for layer in range(2):
        assert gpu.next_position(layer) == cpu.next_position(layer) == n - layer
        pos, gk, gv = gpu.view(layer).rows()
        cpos, ck, cv = cpu.view(layer).rows()
        assert np.array_equal(pos.astype(np.int64), cpos)
        if elem == "f16":
            ck, cv = oracle.f32_to_f16_array(ck), oracle.f32_to_f16_array(cv)
            assert np.array_equal(gk, ck) and np.array_equal(gv, cv)
        else:
            assert gk.tobytes() == ck.tobytes() and gv.tobytes() == cv.tobytes()


@pytest.mark.parametrize("start,rows", [(0, 128), (45, 300), (64, 129), (31, 2048)])
def test_chunk_append_is_bit_exact_and_leaves_its_neighbours_alone(start, rows):
    # A long run of rows appended in one call (a prefill chunk) at aligned and unaligned
    # positions: device bytes equal the host conversion, the rows before the run keep their
    # bytes, the rows after it are still zero.
    import torch

    kv_heads, head_dim = 4, 128
    width = kv_heads * head_dim
    rng = np.random.default_rng(start * 7 + rows)
    n = start + rows
    k, v = normal(rng, n, width), normal(rng, n, width)
    k[start + 1, 5], v[start + 2, 7], k[n - 1, 0] = np.nan, np.inf, 65520.0
    pool = P().KvPool(1, kv_heads, head_dim, elem="f16", capacity_rows=n + 70)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    kd, vd = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
    for p in range(start):  # one row at a time
        pool.append_device(0, [(cache, 1)], kd[p:].data_ptr(), vd[p:].data_ptr())
    pool.append_device(0, [(cache, rows)], kd[start:].data_ptr(), vd[start:].data_ptr())
    assert cache.next_position(0) == n
    gk, gv = cache.read_raw(0)
    want_k, want_v = oracle.f32_to_f16_array(k), oracle.f32_to_f16_array(v)
    assert np.array_equal(gk[:n].reshape(n, width), want_k)
    assert np.array_equal(gv[:n].reshape(n, width), want_v)
    assert not gk[n:].any() and not gv[n:].any()
    pool.close()


def test_f32_to_f16_conversion_matches_the_oracle_on_every_rounding_class():
    import torch

    rng = np.random.default_rng(99)
    bits = rng.integers(0, 2**32, size=1 << 22, dtype=np.uint64).astype(np.uint32)
    edges = []
    for e in range(256):
        for frac in (0, 1, 0xFFF, 0x1000, 0x1001, 0x1FFF, 0x2000, 0x2FFF, 0x3000, 0x3001,
                     0x7FEFFF, 0x7FF000, 0x7FF001, 0x7FFFFF, 0x400000, 0x123456):
            edges += [(e << 23) | frac, 0x80000000 | (e << 23) | frac]
    # Every f32 whose top 19 bits vary and whose low 13 bits sit on / next to the tie.
    hi = np.arange(0, 1 << 19, dtype=np.uint32) << 13
    ties = np.concatenate([hi | 0x1000, hi | 0x0FFF, hi | 0x1001, hi])
    bits = np.concatenate([bits, np.array(edges, dtype=np.uint32), ties])
    pool = P().KvPool(1, 1, 8, elem="f16", capacity_rows=1)
    src = torch.from_numpy(bits.view(np.int32)).cuda()
    dst = torch.empty(bits.size, dtype=torch.int16, device="cuda")
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    pool.convert_f32_to_f16_device(src.data_ptr(), dst.data_ptr(), bits.size)
    torch.cuda.synchronize()
    got = dst.cpu().numpy().view(np.uint16)
    want = oracle.f32_to_f16_array(bits.view(np.float32))
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, [(hex(bits[i]), hex(got[i]), hex(want[i])) for i in bad[:5]]
    pool.close()


def test_global_rewind_truncates_and_keeps_the_prefix():
    # checkpoint_tests.rs:163-181, against the oracle fed only the kept prefix.
    G = P().LayerKind.Global
    cache = P().KvCache.new([G], 2, 2)
    for p in range(5):
        cache.append(0, k_row(2, 2, p), v_row(2, 2, p), p)
    cp = cache.checkpoint(3)
    assert cp.saved_bytes() == 0 and cache.checkpoint_active() and cp.base(0) == 5
    for p in (5, 6, 7):
        cache.append(0, k_row(2, 2, p), v_row(2, 2, p), p)
    assert cache.stored_len(0) == 8
    cache.rewind_to(cp, 6)
    cache.release(cp)
    assert not cache.checkpoint_active()
    ref = oracle.KvCache.new([oracle.LayerKind.Global], 2, 2)
    for p in range(6):
        ref.append(0, k_row(2, 2, p), v_row(2, 2, p), p)
    assert view_snapshot(cache, 0) == view_snapshot(ref, 0)
    assert cache.stats()[0].appended == 6 and cache.stored_len(0) == 6
    # The sequence continues with no seam (checkpoint_tests.rs:139-143).
    cache.append(0, k_row(2, 2, 6), v_row(2, 2, 6), 6)
    ref.append(0, k_row(2, 2, 6), v_row(2, 2, 6), 6)
    assert view_snapshot(cache, 0) == view_snapshot(ref, 0)


def test_rewind_to_a_checkpoint_taken_before_any_append():
    # checkpoint_tests.rs:183-207 on two global layers.
    G = P().LayerKind.Global
    cache = P().KvCache.new([G, G], 1, 2)
    cp = cache.checkpoint(2)
    assert cp.base(0) == 0 and cp.base(1) == 0
    for layer in range(2):
        for p in (0, 1):
            cache.append(layer, k_row(1, 2, p), v_row(1, 2, p), p)
    cache.rewind_to(cp, 0)
    cache.release(cp)
    for layer in range(2):
        assert cache.stats()[layer].appended == 0
        assert cache.view(layer).is_empty()
    raw_k, raw_v = cache.read_raw(0)
    assert not raw_k.any() and not raw_v.any()  # scrubbed: as if never appended


def test_checkpoint_contract_violations_are_named_refusals():
    # checkpoint_tests.rs:232-316 (the cases that do not need a ring).
    G = P().LayerKind.Global
    cache = P().KvCache.new([G, G], 1, 2)
    for layer in range(2):
        for p in (0, 1):
            cache.append(layer, k_row(1, 2, p), v_row(1, 2, p), p)
    with pytest.raises(P().AttentionError) as e:
        cache.checkpoint(0)
    assert e.value == E("ZeroDimension", what="max_round_tokens")
    cp = cache.checkpoint(2)
    with pytest.raises(P().AttentionError) as e:
        cache.checkpoint(1)
    assert e.value == E("CheckpointBusy")
    for layer in range(2):
        for p in (2, 3):
            cache.append(layer, k_row(1, 2, p), v_row(1, 2, p), p)
    with pytest.raises(P().AttentionError) as e:
        cache.append(0, k_row(1, 2, 4), v_row(1, 2, 4), 4)
    assert e.value == E("CheckpointRangeExceeded", layer=0, position=4, limit=4)
    with pytest.raises(P().AttentionError) as e:
        cache.rewind_to(cp, 1)
    assert e.value == E("RewindOutOfRange", layer=0, base=2, appended=4, target=1)
    assert e.value.message == "rewind target 1 is outside layer 0's checkpoint range [2, 4]"
    with pytest.raises(P().AttentionError) as e:
        cache.rewind_to(cp, 5)
    assert e.value == E("RewindOutOfRange", layer=0, base=2, appended=4, target=5)
    assert cache.stats()[0].appended == 4
    cache.release(cp)
    for call in (lambda: cache.rewind_to(cp, 2), lambda: cache.release(cp)):
        with pytest.raises(P().AttentionError) as e:
            call()
        assert e.value.variant == "StaleCheckpoint"
    other = P().KvCache.new([G, G], 1, 2)
    for layer in range(2):
        for p in (0, 1):
            other.append(layer, k_row(1, 2, p), v_row(1, 2, p), p)
    foreign = other.checkpoint(2)
    mine = cache.checkpoint(2)
    with pytest.raises(P().AttentionError) as e:
        cache.rewind_to(foreign, 2)
    assert e.value.variant == "StaleCheckpoint"
    cache.release(mine)
    other.release(foreign)


@pytest.mark.parametrize("elem", ["f32", "f16"])
def test_bulk_restore_matches_append_replay_bitwise(elem):
    # cache_tests.rs:218-283 with global layers, plus continuation.
    rng = np.random.default_rng(5)
    kv_heads, head_dim, tokens, layers = 2, 24, 19, 3
    k = normal(rng, layers, tokens + 1, kv_heads * head_dim)
    v = normal(rng, layers, tokens + 1, kv_heads * head_dim)
    G = P().LayerKind.Global
    replay = P().KvCache.new([G] * layers, kv_heads, head_dim, elem=elem, capacity_rows=32)
    bulk = P().KvCache.new([G] * layers, kv_heads, head_dim, elem=elem, capacity_rows=32)
    for layer in range(layers):
        for p in range(tokens):
            replay.append(layer, k[layer, p], v[layer, p], p)
        bulk.restore_bulk(layer, 0, k[layer, :tokens], v[layer, :tokens])
    for layer in range(layers):
        assert bulk.next_position(layer) == tokens
        assert view_snapshot(bulk, layer) == view_snapshot(replay, layer)
        replay.append(layer, k[layer, tokens], v[layer, tokens], tokens)
        bulk.append(layer, k[layer, tokens], v[layer, tokens], tokens)
        assert view_snapshot(bulk, layer) == view_snapshot(replay, layer)
        rk, rv = replay.read_raw(layer)
        bk, bv = bulk.read_raw(layer)
        assert rk.tobytes() == bk.tobytes() and rv.tobytes() == bv.tobytes()


def test_bulk_restore_refusals_are_named():
    # cache_tests.rs:285-322 (global-layer cases).
    G = P().LayerKind.Global
    cache = P().KvCache.new([G, G], 1, 2)
    with pytest.raises(P().AttentionError) as e:
        cache.restore_bulk(1, 3, np.zeros(4), np.zeros(4))
    assert e.value == E("ShapeMismatch", what="bulk restore first position (global layer)",
                        expected=0, actual=3)
    cache.append(0, row(1, 2, 1.0), row(1, 2, 1.0), 0)
    with pytest.raises(P().AttentionError) as e:
        cache.restore_bulk(0, 0, np.zeros(2), np.zeros(2))
    assert e.value == E("BulkRestoreNotFresh", layer=0, appended=1)
    with pytest.raises(P().AttentionError) as e:
        cache.restore_bulk(1, 0, np.zeros(4), np.zeros(2))
    assert e.value == E("ShapeMismatch", what="bulk restore rows", expected=2, actual=4)
    with pytest.raises(P().AttentionError) as e:
        cache.restore_bulk(1, 0, np.zeros(3), np.zeros(3))
    assert e.value == E("ShapeMismatch", what="bulk restore rows", expected=3, actual=3)
    with pytest.raises(P().AttentionError) as e:
        cache.restore_bulk(7, 0, np.zeros(2), np.zeros(2))
    assert e.value == E("InvalidLayer", layer=7, layer_count=2)


def test_f16_snapshot_restores_raw_and_pinned_host_sources_are_read_in_place():
    import torch

    rng = np.random.default_rng(8)
    kv_heads, head_dim, tokens, layers = 4, 128, 50, 3
    k32 = normal(rng, layers, tokens, kv_heads * head_dim)
    v32 = normal(rng, layers, tokens, kv_heads * head_dim)
    want_k, want_v = oracle.f32_to_f16_array(k32), oracle.f32_to_f16_array(v32)
    pool = P().KvPool(layers, kv_heads, head_dim, elem="f16", max_slots=3, capacity_rows=64)
    a, b, c = pool.acquire(), pool.acquire(), pool.acquire()
    # a: f32 snapshot in pinned host memory, converted by the gather kernel.
    pk = torch.from_numpy(k32).pin_memory()
    pv = torch.from_numpy(v32).pin_memory()
    row_elems = tokens * kv_heads * head_dim
    a.restore_snapshot_ptrs(tokens, [(0, tokens, pk[l].data_ptr(), pv[l].data_ptr())
                                     for l in range(layers)], src_f16=False)
    # b: f16 snapshot (raw bits) in pinned host memory.
    hk = torch.from_numpy(want_k.view(np.int16)).pin_memory()
    hv = torch.from_numpy(want_v.view(np.int16)).pin_memory()
    b.restore_snapshot_ptrs(tokens, [(0, tokens, hk[l].data_ptr(), hv[l].data_ptr())
                                     for l in range(layers)], src_f16=True)
    # c: f32 snapshot already on the device, layer by layer.
    dk, dv = torch.from_numpy(k32).cuda(), torch.from_numpy(v32).cuda()
    for l in range(layers):
        c.restore_bulk_ptr(l, 0, dk[l].data_ptr(), dv[l].data_ptr(), row_elems, src_f16=False)
    for cache in (a, b, c):
        for l in range(layers):
            assert cache.next_position(l) == tokens
            _, gk, gv = cache.view(l).rows()
            assert np.array_equal(gk.reshape(tokens, -1), want_k[l])
            assert np.array_equal(gv.reshape(tokens, -1), want_v[l])
    # Snapshot validation (crates/itak-kv/src/snapshot.rs:187-236) happens before any write.
    d = P().KvPool(layers, kv_heads, head_dim, elem="f16", capacity_rows=64).acquire()
    with pytest.raises(P().StepFailed):
        d.restore_snapshot_ptrs(tokens, [(0, tokens - 1, pk[l].data_ptr(), pv[l].data_ptr())
                                         for l in range(layers)], src_f16=False)
    with pytest.raises(P().StepFailed):
        d.restore_snapshot_ptrs(tokens, [(0, tokens, pk[0].data_ptr(), pv[0].data_ptr())],
                                src_f16=False)
    assert all(d.next_position(l) == 0 for l in range(layers))
    f32pool = P().KvCache.new([P().LayerKind.Global], kv_heads, head_dim, elem="f32",
                              capacity_rows=64)
    with pytest.raises(P().AttentionError) as e:
        f32pool.restore_bulk(0, 0, want_k[0], want_v[0])
    assert e.value.variant == "Unsupported"


def test_a_snapshot_whose_layers_lie_in_different_allocations_of_different_kinds():
    # The library asks the runtime what kind of memory a source is once per device allocation
    # and answers the rest from that allocation's extent: sources in two device allocations
    # (one of them large enough to hold several layers), in pinned host memory and in ordinary
    # host memory, mixed within one snapshot and given as a prebuilt layer table, each land
    # where a snapshot from one place lands.
    import torch

    rng = np.random.default_rng(21)
    kv_heads, head_dim, tokens, layers = 2, 128, 70, 6
    width = kv_heads * head_dim
    k32, v32 = normal(rng, layers, tokens, width), normal(rng, layers, tokens, width)
    want_k, want_v = oracle.f32_to_f16_array(k32), oracle.f32_to_f16_array(v32)
    big = torch.from_numpy(np.concatenate([k32[:3], v32[:3]])).cuda()          # layers 0-2, K then V
    other = torch.from_numpy(k32[3:5]).cuda()                                    # K of layers 3, 4
    pinned = torch.from_numpy(v32[3:5]).pin_memory()                             # V of layers 3, 4
    plain_k, plain_v = np.ascontiguousarray(k32[5]), np.ascontiguousarray(v32[5])  # layer 5: staged
    table = []
    for l in range(layers):
        if l < 3:
            table.append((0, tokens, big[l].data_ptr(), big[3 + l].data_ptr()))
        elif l < 5:
            table.append((0, tokens, other[l - 3].data_ptr(), pinned[l - 3].data_ptr()))
        else:
            table.append((0, tokens, plain_k.ctypes.data, plain_v.ctypes.data))
    pool = P().KvPool(layers, kv_heads, head_dim, elem="f16", max_slots=2, capacity_rows=96)
    a, b = pool.acquire(), pool.acquire()
    a.restore_snapshot_ptrs(tokens, P().KvCache.snapshot_layer_table(table), src_f16=False)
    b.restore_snapshot_ptrs(tokens, table, src_f16=False)
    for cache in (a, b):
        for l in range(layers):
            assert cache.next_position(l) == tokens
            _, gk, gv = cache.view(l).rows()
            assert np.array_equal(gk.reshape(tokens, -1), want_k[l]), l
            assert np.array_equal(gv.reshape(tokens, -1), want_v[l]), l


def test_batched_truncate_then_reappend_is_bitwise_never_appended():
    import torch

    rng = np.random.default_rng(21)
    kv_heads, head_dim, layers, slots = 4, 128, 3, 4
    base, block = 40, 7
    pool = P().KvPool(layers, kv_heads, head_dim, elem="f16", max_slots=2 * slots,
                      capacity_rows=64)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    spec = [pool.acquire() for _ in range(slots)]   # append 7, truncate r, re-append
    never = [pool.acquire() for _ in range(slots)]  # only ever sees the kept rows
    k = normal(rng, slots, base + 2 * block, kv_heads * head_dim)
    v = normal(rng, slots, base + 2 * block, kv_heads * head_dim)
    kd, vd = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
    rejected = rng.integers(0, 6, size=slots, endpoint=True)
    rejected[0], rejected[1] = 0, 6
    keep = base + block - rejected
    for layer in range(layers):
        for s in range(slots):
            pool.append_device(layer, [(spec[s], base + block)], kd[s].data_ptr(),
                               vd[s].data_ptr())
            pool.append_device(layer, [(never[s], int(keep[s]))], kd[s].data_ptr(),
                               vd[s].data_ptr())
    pool.truncate(spec, keep)
    for s in range(slots):
        for layer in range(layers):
            assert spec[s].next_position(layer) == keep[s]
            sk, sv = spec[s].read_raw(layer)
            nk, nv = never[s].read_raw(layer)
            assert sk.tobytes() == nk.tobytes() and sv.tobytes() == nv.tobytes()
    # Re-append different rows after the kept prefix on both: still identical.
    for layer in range(layers):
        for s in range(slots):
            off = base + block
            for c in (spec[s], never[s]):
                pool.append_device(layer, [(c, block)], kd[s, off:].data_ptr(),
                                   vd[s, off:].data_ptr())
    for s in range(slots):
        for layer in range(layers):
            sk, sv = spec[s].read_raw(layer)
            nk, nv = never[s].read_raw(layer)
            assert sk.tobytes() == nk.tobytes() and sv.tobytes() == nv.tobytes()
            ref = oracle.f32_to_f16_array(np.concatenate([k[s, :keep[s]], k[s, off:off + block]]))
            assert np.array_equal(sk[:keep[s] + block].reshape(keep[s] + block, -1), ref)
    with pytest.raises(P().AttentionError) as e:
        pool.truncate([spec[0]], [10_000])
    assert e.value.variant == "RewindOutOfRange"
    pool.close()


def test_slots_are_independent_and_reset_gives_a_fresh_cache():
    G = P().LayerKind.Global
    pool = P().KvPool([G], 1, 4, elem="f32", max_slots=2, capacity_rows=8)
    a, b = pool.acquire(), pool.acquire()
    with pytest.raises(P().AttentionError) as e:
        pool.acquire()
    assert e.value.variant == "NoFreeSlot"
    a.append(0, [1, 2, 3, 4], [5, 6, 7, 8], 0)
    b.append(0, [9, 9, 9, 9], [7, 7, 7, 7], 0)
    b.append(0, [8, 8, 8, 8], [6, 6, 6, 6], 1)
    assert a.stored_len(0) == 1 and b.stored_len(0) == 2
    assert a.view(0).key(0, 0).tolist() == [1, 2, 3, 4]
    assert b.view(0).value(1, 0).tolist() == [6, 6, 6, 6]
    cp = a.checkpoint(2)
    a.reset()
    assert a.stored_len(0) == 0 and not a.checkpoint_active()
    with pytest.raises(P().AttentionError) as e:
        a.release(cp)
    assert e.value.variant == "StaleCheckpoint"
    rk, rv = a.read_raw(0)
    assert not rk.any() and not rv.any()
    assert b.stored_len(0) == 2
    a.release_slot()
    c = pool.acquire()
    assert c.slot == a.slot and c.stored_len(0) == 0


def test_getters_refuse_null_outputs_by_name():
    # Nothing aborts across the boundary: a null out pointer is an InvalidArgument refusal.
    pool = P().KvPool(1, 2, 8, elem="f32", capacity_rows=8)
    cache = pool.acquire()
    lib = P()._native.load()
    cp = cache.checkpoint(1)
    raw = P()._native.CheckpointRaw()
    for status in (lib.itak_kv_stored_len(pool._h, cache.slot, 0, None),
                   lib.itak_kv_next_position(pool._h, cache.slot, 0, None),
                   lib.itak_kv_checkpoint_active(pool._h, cache.slot, None),
                   lib.itak_kv_checkpoint_bases(pool._h, cache.slot, raw, None),
                   lib.itak_kv_checkpoint_bases(pool._h, cache.slot, None, None)):
        assert status == 17, status
        assert b"null" in lib.itak_last_error(pool._h)
    cache.release(cp)
    pool.close()


def test_debug_channel_reports_cache_and_attention_events(capfd):
    # attention::diag (crates/attention/src/diag.rs): the events the reference logs (cache built,
    # append, checkpoint, rewind, release, gqa_attention, bulk restore) each give one line, and
    # nothing is printed once the switch is off again.
    import torch
    kv_heads, d = 2, 128
    P().set_debug_enabled(True)
    try:
        pool = P().KvPool(1, kv_heads, d, elem="f16", capacity_rows=64)
        pool.set_stream(torch.cuda.current_stream().cuda_stream)
        cache = pool.acquire()
        for p in range(3):
            cache.append(0, k_row(kv_heads, d, p), v_row(kv_heads, d, p), p)
        cp = cache.checkpoint(4)
        cache.append(0, k_row(kv_heads, d, 3), v_row(kv_heads, d, 3), 3)
        q = normal(np.random.default_rng(0), 1, 4 * d)
        P().gqa_attention(q, 1, 4, [3], cache.view(0))
        cache.rewind_to(cp, 3)
        cache.release(cp)
        with pytest.raises(P().AttentionError):
            cache.append(0, k_row(kv_heads, d, 9), v_row(kv_heads, d, 9), 9)
    finally:
        P().set_debug_enabled(False)
    err = capfd.readouterr().err
    lines = [l[len("[itak_hip_kv::diag] "):] for l in err.splitlines() if l.startswith("[itak_hip_kv::diag] ")]
    assert lines[0].startswith("kv pool built layers=1 kv_heads=2 head_dim=128 elem=f16 slots=")
    assert "append layer=0 slot=0 rows=1 kind=global stored=3" in lines
    assert "checkpoint slot=0 serial=1 max_round_tokens=4 saved_bytes=0" in lines
    assert any(l.startswith("gqa_attention layer=0 items=1 queries=1 q_heads=4 kv_heads=2 view_len=4 window=0")
               for l in lines)
    assert "rewind slot=0 serial=1 target=3" in lines
    assert "release slot=0 serial=1" in lines
    assert any(l.startswith("refused code=") and "position" in l for l in lines)
    cache.append(0, k_row(kv_heads, d, 3), v_row(kv_heads, d, 3), 3)
    assert "[itak_hip_kv::diag]" not in capfd.readouterr().err
    pool.close()


def test_the_mfma_probe_reports_its_work_and_both_clocks():
    # A measurement aid, not part of the path: the call launches, says how many floating-point
    # operations the launch held, and leaves the ticks of the two clocks in device memory.
    import torch
    pool = P().KvPool(1, 1, 128, elem="f16", capacity_rows=64)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    clocks = torch.zeros(2, dtype=torch.int64, device="cuda")
    flops = pool.probe_mfma(True, 64, clocks.data_ptr())
    pool.synchronize()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    assert flops == 2 * cus * 4 * 64 * 32 * 16384
    shader, constant = clocks.cpu().tolist()
    assert shader > 0 and constant > 0 and 5 <= shader / constant <= 30   # 0.5 to 3 GHz against 100 MHz
    assert pool.probe_mfma(False, 1) == 2 * cus * 4 * 32 * 16384
    with pytest.raises(Exception, match="trips"):
        pool.probe_mfma(True, 0)
    src = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    pool.probe_read_device(src.data_ptr(), 1 << 20)   # launches and reads, nothing to compare
    pool.synchronize()
    with pytest.raises(Exception, match="multiple of 16"):
        pool.probe_read_device(src.data_ptr(), 24)
    pool.close()


def test_a_read_that_starts_past_the_end_is_refused_without_a_wrapped_sum():
    pool = P().KvPool(1, 1, 16, elem="f32", capacity_rows=8)
    cache = pool.acquire()
    k = np.ones((3, 16), dtype=np.float32)
    for i in range(3):
        cache.append(0, k[i], k[i], i)
    with pytest.raises(P().AttentionError) as e:
        cache.read_rows(0, 2 ** 64 - 4, 64)      # a first row computed as 3 - 7 and the like
    assert "18446744073709551615" in str(e.value) and "expected 3" in str(e.value)
    pool.close()


def test_a_restore_from_device_memory_is_ordered_by_the_stream_and_one_from_host_memory_is_done_on_return():
    import torch
    kvh, d, n = 2, 64, 500
    row = kvh * d
    rng = np.random.default_rng(11)
    k, v = normal(rng, n, row), normal(rng, n, row)
    pool = P().KvPool(1, kvh, d, elem="f32", max_slots=2, capacity_rows=n + 8)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    a, b = pool.acquire(), pool.acquire()
    # Device rows: the call returns with the gather enqueued; what reads the cache next on the
    # same stream (here the read-back) comes after it.
    kd, vd = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
    a.restore_bulk_ptr(0, 0, kd.data_ptr(), vd.data_ptr(), n * row, src_f16=False)
    _, gk, gv = a.read_rows(0, 0, n)
    assert np.array_equal(np.asarray(gk).reshape(n, row), k) and np.array_equal(np.asarray(gv).reshape(n, row), v)
    # Pinned host rows are the caller's again when the call returns: overwritten at once, the
    # cache still holds what they were.
    kp, vp = torch.from_numpy(k.copy()).pin_memory(), torch.from_numpy(v.copy()).pin_memory()
    b.restore_bulk_ptr(0, 0, kp.data_ptr(), vp.data_ptr(), n * row, src_f16=False)
    kp.zero_(); vp.zero_()
    _, gk, gv = b.read_rows(0, 0, n)
    assert np.array_equal(np.asarray(gk).reshape(n, row), k) and np.array_equal(np.asarray(gv).reshape(n, row), v)
    pool.close()
