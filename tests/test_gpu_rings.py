"""Windowed (ring) layers on the GPU through the C ABI: the reference's ring cases
(crates/attention/tests/cache_tests.rs:37-79, 218-322, checkpoint_tests.rs:79-337,
attention_tests.rs windowed cases) on the device front end, and parity with the CPU oracle
for append, rewind, restore, snapshots and attention on windowed layers.

The device ring is window + headroom rows (position p in row p % ring): rewinds move a
length instead of restoring saved rows, so the cases here check what the reference's own tests
check, the visible rows and positions, not raw storage.

Tolerances: f32 KV outputs within 1e-5 of the oracle relative to the largest output
magnitude; f16 KV outputs within 2e-3 max-abs of the oracle over the same f16-rounded cache;
rows bit-exact."""
import numpy as np
import pytest

import oracle
from helpers import max_abs, normal, pkg, rel_err

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


def append(cache, layer, kv_heads, head_dim, position):
    cache.append(layer, k_row(kv_heads, head_dim, position), v_row(kv_heads, head_dim, position),
                 position)


def append_all(cache, kv_heads, head_dim, positions):
    for p in positions:
        for layer in range(cache.layer_count()):
            append(cache, layer, kv_heads, head_dim, p)


def view_snapshot(cache, layer):  # checkpoint_tests.rs:54-65, on either implementation
    pos, keys, vals = cache.view(layer).rows()
    keys, vals = np.asarray(keys), np.asarray(vals)
    if keys.dtype == np.uint16:  # f16 storage: compare as the values they hold
        keys, vals = keys.view(np.float16).astype(np.float32), vals.view(np.float16).astype(np.float32)
    return (np.asarray(pos, dtype=np.int64).tobytes() + np.ascontiguousarray(keys).tobytes()
            + np.ascontiguousarray(vals).tobytes())


def W(window):
    return P().LayerKind.windowed(window)


def device_cache(pattern, kv_heads, head_dim, positions, **kw):
    cache = P().KvCache.new(pattern, kv_heads, head_dim, **kw)
    append_all(cache, kv_heads, head_dim, positions)
    return cache


def oracle_cache(pattern, kv_heads, head_dim, positions, store_f16=False):
    cache = oracle.KvCache.new(pattern, kv_heads, head_dim, store_f16=store_f16)
    append_all(cache, kv_heads, head_dim, positions)
    return cache


@pytest.mark.parametrize("elem", ["f32", "f16"])
def test_ring_buffer_wraps_and_evicts_oldest(elem):
    # cache_tests.rs:37-62.
    cache = P().KvCache.new([W(4)], 1, 1, elem=elem)
    for pos in range(7):
        cache.append(0, row(1, 1, pos), row(1, 1, pos), pos)
    assert cache.stored_len(0) == 4
    assert cache.next_position(0) == 7
    view = cache.view(0)
    assert view.len() == 4 and not view.is_empty() and view.window() == 4
    for vi, expected in enumerate([3, 4, 5, 6]):
        assert view.position_at(vi) == expected
        assert view.value(vi, 0).tolist() == [float(expected)]
        assert view.key(vi, 0).tolist() == [float(expected)]
    assert view.position_at(4) is None
    stats = cache.stats()
    assert stats[0].appended == 7 and stats[0].stored == 4


def test_ring_buffer_holds_exactly_the_glimmer_window():
    # cache_tests.rs:64-79, through the device append so that the ring wraps in one call
    # sequence of block appends as a session would issue them.
    import torch
    pool = P().KvPool([W(2048)], 2, 4, elem="f32", ring_headroom=64)
    cache = pool.acquire()
    rows = np.repeat(np.arange(2050, dtype=np.float32)[:, None], 8, axis=1)
    dev = torch.from_numpy(rows).cuda()
    for first in range(0, 2050, 64):
        n = min(64, 2050 - first)
        pool.append_device(0, [(cache, n)], dev[first:].data_ptr(), dev[first:].data_ptr())
    pool.synchronize()
    assert cache.stored_len(0) == 2048
    view = cache.view(0)
    assert view.position_at(0) == 2
    assert view.position_at(2047) == 2049
    assert view.value(0, 0)[0] == 2.0
    assert view.value(2047, 1)[0] == 2049.0
    pos, keys, _ = view.rows()
    assert pos.tolist() == list(range(2, 2050))
    assert keys[:, 0, 0].tolist() == [float(p) for p in range(2, 2050)]
    pool.close()


def test_mixed_pattern_keeps_layers_apart():
    # cache_tests.rs:148-183's pattern: windowed, global, windowed, each layer its own rows.
    pattern = [W(4), P().LayerKind.Global, W(4)]
    opattern = [oracle.LayerKind.windowed(4), oracle.LayerKind.Global, oracle.LayerKind.windowed(4)]
    cache = device_cache(pattern, 2, 3, range(11))
    ref = oracle_cache(opattern, 2, 3, range(11))
    for layer in range(3):
        assert cache.stored_len(layer) == ref.stored_len(layer)
        assert view_snapshot(cache, layer) == view_snapshot(ref, layer)
        assert cache.layer_kind(layer).window() == ref.layer_kind(layer).window()
    stats = cache.stats()
    assert [s.stored for s in stats] == [4, 11, 4]


@pytest.mark.parametrize("elem", ["f32", "f16"])
def test_windowed_rewind_restores_rows_evicted_by_speculative_appends(elem):
    # checkpoint_tests.rs:79-117.
    pattern = [W(4)]
    cache = device_cache(pattern, 1, 2, range(6), elem=elem)
    committed = view_snapshot(cache, 0)
    cp = cache.checkpoint(3)
    assert cache.checkpoint_active()
    assert cp.base(0) == 6
    for p in (6, 7, 8):
        append(cache, 0, 1, 2, p)
    assert view_snapshot(cache, 0) != committed
    cache.rewind_to(cp, 6)
    cache.release(cp)
    assert not cache.checkpoint_active()
    assert view_snapshot(cache, 0) == committed
    stats = cache.stats()
    assert stats[0].appended == 6 and stats[0].stored == 4
    fresh = device_cache(pattern, 1, 2, range(6), elem=elem)
    q = np.array([0.5, -0.25], dtype=np.float32)
    after = P().gqa_attention(q, 1, 1, [5], cache.view(0), P().AttentionParams.new())
    never = P().gqa_attention(q, 1, 1, [5], fresh.view(0), P().AttentionParams.new())
    assert after.tobytes() == never.tobytes()


def test_windowed_rewind_to_mid_block_keeps_exactly_the_committed_prefix():
    # checkpoint_tests.rs:119-144.
    pattern = [W(4)]
    cache = device_cache(pattern, 2, 2, range(6))
    cp = cache.checkpoint(3)
    for p in (6, 7, 8):
        append(cache, 0, 2, 2, p)
    cache.rewind_to(cp, 7)
    cache.release(cp)
    assert view_snapshot(cache, 0) == view_snapshot(device_cache(pattern, 2, 2, range(7)), 0)
    assert cache.stats()[0].appended == 7
    append(cache, 0, 2, 2, 7)
    assert view_snapshot(cache, 0) == view_snapshot(device_cache(pattern, 2, 2, range(8)), 0)


def test_windowed_checkpoint_saved_slots_wrap_the_ring():
    # checkpoint_tests.rs:146-161.
    pattern = [W(4)]
    cache = device_cache(pattern, 1, 2, range(7))
    cp = cache.checkpoint(2)
    for p in (7, 8):
        append(cache, 0, 1, 2, p)
    cache.rewind_to(cp, 7)
    cache.release(cp)
    assert view_snapshot(cache, 0) == view_snapshot(device_cache(pattern, 1, 2, range(7)), 0)
    assert cache.stats()[0].appended == 7


def test_rewind_to_a_checkpoint_taken_before_any_append():
    # checkpoint_tests.rs:183-207.
    pattern = [W(4), P().LayerKind.Global]
    cache = P().KvCache.new(pattern, 1, 2)
    cp = cache.checkpoint(2)
    assert cp.base(0) == 0 and cp.base(1) == 0
    append_all(cache, 1, 2, [0, 1])
    cache.rewind_to(cp, 0)
    cache.release(cp)
    for layer in range(2):
        assert cache.stats()[layer].appended == 0
        assert cache.view(layer).is_empty()
    append_all(cache, 1, 2, [0, 1])
    reference = device_cache(pattern, 1, 2, [0, 1])
    for layer in range(2):
        assert view_snapshot(cache, layer) == view_snapshot(reference, layer)


def test_second_rewind_restores_the_snapshot_again():
    # checkpoint_tests.rs:209-230.
    pattern = [W(4)]
    cache = device_cache(pattern, 1, 2, range(6))
    committed = view_snapshot(cache, 0)
    cp = cache.checkpoint(3)
    for p in (6, 7, 8):
        append(cache, 0, 1, 2, p)
    cache.rewind_to(cp, 6)
    append(cache, 0, 1, 2, 6)
    assert view_snapshot(cache, 0) != committed
    cache.rewind_to(cp, 6)
    cache.release(cp)
    assert view_snapshot(cache, 0) == committed


def test_checkpoint_contract_violations_are_named_refusals():
    # checkpoint_tests.rs:232-316 on the windowed + global pattern.
    pattern = [W(4), P().LayerKind.Global]
    cache = device_cache(pattern, 1, 2, [0, 1])
    with pytest.raises(P().AttentionError) as e:
        cache.checkpoint(0)
    assert e.value == E("ZeroDimension", what="max_round_tokens")
    with pytest.raises(P().AttentionError) as e:
        cache.checkpoint(5)
    assert e.value == E("CheckpointTooDeep", max_round_tokens=5, window=4)
    assert e.value.message == ("checkpoint round bound 5 exceeds the smallest sliding window 4: a "
                               "round that long would overwrite a ring slot twice and no rewind "
                               "could be exact")
    cp = cache.checkpoint(2)
    with pytest.raises(P().AttentionError) as e:
        cache.checkpoint(1)
    assert e.value == E("CheckpointBusy")
    append_all(cache, 1, 2, [2, 3])
    with pytest.raises(P().AttentionError) as e:
        append(cache, 0, 1, 2, 4)
    assert e.value == E("CheckpointRangeExceeded", layer=0, position=4, limit=4)
    with pytest.raises(P().AttentionError) as e:
        cache.rewind_to(cp, 1)
    assert e.value == E("RewindOutOfRange", layer=0, base=2, appended=4, target=1)
    with pytest.raises(P().AttentionError) as e:
        cache.rewind_to(cp, 5)
    assert e.value == E("RewindOutOfRange", layer=0, base=2, appended=4, target=5)
    assert cache.stats()[0].appended == 4
    cache.release(cp)
    for call in (lambda: cache.rewind_to(cp, 2), lambda: cache.release(cp)):
        with pytest.raises(P().AttentionError) as e:
            call()
        assert e.value.variant == "StaleCheckpoint"


def test_checkpoint_reports_the_bytes_the_reference_would_save():
    # checkpoint_tests.rs:318-337: 39 windowed layers x 17 rows x (K + V) x 256 floats x 4 B.
    pattern = [W(2048) if (i + 1) % 4 else P().LayerKind.Global for i in range(52)]
    cache = P().KvCache.new(pattern, 2, 128, elem="f16", capacity_rows=64)
    cp = cache.checkpoint(17)
    assert cp.saved_bytes() == 39 * 17 * 2 * 256 * 4 == 1_357_824
    cache.release(cp)


def test_the_rings_headroom_bounds_blocks_rounds_and_truncates():
    import torch
    pool = P().KvPool([W(64)], 1, 8, elem="f32", ring_headroom=16)  # ring: 96 rows
    cache = pool.acquire()
    rows = torch.zeros(64, 8, device="cuda")
    # 32 = ring - window rows fit one block, 33 do not.
    with pytest.raises(P().AttentionError) as e:
        pool.append_device(0, [(cache, 33)], rows.data_ptr(), rows.data_ptr())
    assert e.value.variant == "CapacityExceeded" and "ring headroom" in e.value.message
    assert cache.next_position(0) == 0
    for _ in range(4):
        pool.append_device(0, [(cache, 32)], rows.data_ptr(), rows.data_ptr())
    assert cache.next_position(0) == 128
    # A round longer than the ring can undo by itself (ring - window = 32 rows) is taken all
    # the same, as the reference takes any round up to the window: the checkpoint sets the rows
    # it may overwrite aside (the deep-round test below rewinds one).
    cp = cache.checkpoint(33)
    cache.release(cp)
    with pytest.raises(P().AttentionError) as e:
        cache.checkpoint(65)
    assert e.value == E("CheckpointTooDeep", max_round_tokens=65, window=64)
    pool.truncate([cache.slot], [100])   # 28 positions back: inside the 32 spare rows
    assert cache.next_position(0) == 100
    with pytest.raises(P().AttentionError) as e:
        pool.truncate([cache.slot], [90])  # the rows up to 128 are still in the ring
    assert e.value.variant == "CapacityExceeded"
    assert cache.next_position(0) == 100
    cp = cache.checkpoint(32)  # exactly the bound
    pool.append_device(0, [(cache, 32)], rows.data_ptr(), rows.data_ptr())
    cache.rewind_to(cp, 100)
    cache.release(cp)
    assert cache.next_position(0) == 100
    pool.close()


@pytest.mark.parametrize("elem", ["f32", "f16"])
def test_bulk_restore_matches_append_replay_on_rings(elem):
    # cache_tests.rs:218-283: windowed and global layers, restored rows == replayed rows,
    # and the continuation stays identical.
    rng = np.random.default_rng(5)
    kv_heads, head_dim, tokens, window = 2, 16, 45, 8
    pattern = [W(window), P().LayerKind.Global, W(window)]
    k = normal(rng, 3, tokens + 3, kv_heads * head_dim)
    v = normal(rng, 3, tokens + 3, kv_heads * head_dim)
    replay = P().KvCache.new(pattern, kv_heads, head_dim, elem=elem, capacity_rows=64)
    bulk = P().KvCache.new(pattern, kv_heads, head_dim, elem=elem, capacity_rows=64)
    for layer in range(3):
        for p in range(tokens):
            replay.append(layer, k[layer, p], v[layer, p], p)
        first = 0 if layer == 1 else tokens - window
        bulk.restore_bulk(layer, first, k[layer, first:tokens], v[layer, first:tokens])
    for layer in range(3):
        assert bulk.next_position(layer) == tokens
        assert view_snapshot(bulk, layer) == view_snapshot(replay, layer)
        for p in range(tokens, tokens + 3):
            replay.append(layer, k[layer, p], v[layer, p], p)
            bulk.append(layer, k[layer, p], v[layer, p], p)
            assert view_snapshot(bulk, layer) == view_snapshot(replay, layer)


def test_bulk_restore_refusals_on_rings_are_named():
    # cache_tests.rs:285-322.
    pattern = [W(4), P().LayerKind.Global]
    cache = P().KvCache.new(pattern, 1, 2)
    with pytest.raises(P().AttentionError) as e:
        cache.restore_bulk(0, 0, np.zeros(10, np.float32), np.zeros(10, np.float32))
    assert e.value == E("ShapeMismatch", what="bulk restore rows (windowed layer)", expected=4,
                        actual=5)
    with pytest.raises(P().AttentionError) as e:
        cache.restore_bulk(1, 3, np.zeros(4, np.float32), np.zeros(4, np.float32))
    assert e.value == E("ShapeMismatch", what="bulk restore first position (global layer)",
                        expected=0, actual=3)
    cache.restore_bulk(0, 9, np.ones(8, np.float32), np.ones(8, np.float32))
    assert cache.next_position(0) == 13 and cache.stored_len(0) == 4
    with pytest.raises(P().AttentionError) as e:
        cache.restore_bulk(0, 0, np.zeros(2, np.float32), np.zeros(2, np.float32))
    assert e.value == E("BulkRestoreNotFresh", layer=0, appended=13)


def test_a_ring_rewound_to_empty_restores_like_a_fresh_one():
    # restore_bulk needs a fresh layer (cache.rs:524-529); a layer rewound to position 0 is
    # fresh by that rule, and rows the restore does not write must read as a fresh cache's
    # zeros, not as what the ring held before.
    cache = P().KvCache.new([W(4)], 1, 2)
    ref = oracle.KvCache.new([oracle.LayerKind.windowed(4)], 1, 2)
    for p in range(12):
        append(cache, 0, 1, 2, p)
    cache.pool.truncate([cache.slot], [0])
    rows = np.arange(1, 7, dtype=np.float32).reshape(3, 2)
    cache.restore_bulk(0, 10, rows, rows)   # positions 10..12; position 9 is in view, unwritten
    ref.restore_bulk(0, 10, rows, rows)
    assert cache.next_position(0) == 13 and cache.stored_len(0) == 4
    assert view_snapshot(cache, 0) == view_snapshot(ref, 0)
    assert cache.view(0).key(0, 0).tolist() == [0.0, 0.0]


def test_a_restored_ring_cannot_be_cut_back_under_its_snapshot():
    # A snapshot of a windowed layer carries its last `window` rows only. The query appended
    # after a cut stands at the new length and sees `window` positions down from there: the cut
    # may go to first + window - 1 (the resident session's rewind by one after a stored prefix
    # covered the whole prompt) and no further.
    pool = P().KvPool([W(8)], 1, 2, elem="f32", ring_headroom=16)
    cache = pool.acquire()
    rows = np.arange(16, dtype=np.float32).reshape(8, 2)
    cache.restore_bulk(0, 40, rows, rows)          # positions 40..47
    for p in range(48, 52):
        cache.append(0, [float(p)] * 2, [float(p)] * 2, p)
    pool.truncate([cache.slot], [49])
    assert cache.view(0).rows()[0].tolist() == list(range(41, 49))
    with pytest.raises(P().AttentionError) as e:
        pool.truncate([cache.slot], [46])
    assert e.value == E("RewindOutOfRange", layer=0, base=47, appended=49, target=46)
    pool.truncate([cache.slot], [48])
    assert cache.view(0).rows()[0].tolist() == list(range(40, 48))
    # One further: position 47 goes, and the next row appended sees 40..47 again.
    pool.truncate([cache.slot], [47])
    cache.append(0, [47.5] * 2, [47.5] * 2, 47)
    positions, keys, _ = cache.view(0).rows()
    assert positions.tolist() == list(range(40, 48))
    assert keys.reshape(8, 2)[:, 0].tolist() == [0.0, 2.0, 4.0, 6.0, 8.0, 10.0, 12.0, 47.5]
    pool.close()


# ------------------------------------------------------------------------------ attention


def pair(window, kv_heads, head_dim, elem, rows=0, seed=0, headroom=0, capacity=64):
    """A one-layer windowed cache on the device and in the oracle, filled with the same rows."""
    rng = np.random.default_rng(seed)
    pool = P().KvPool([W(window)], kv_heads, head_dim, elem=elem, capacity_rows=capacity,
                      ring_headroom=headroom)
    cache = pool.acquire()
    ref = oracle.KvCache.new([oracle.LayerKind.windowed(window)], kv_heads, head_dim,
                             store_f16=(elem == "f16"))
    if rows:
        k = normal(rng, rows, kv_heads * head_dim)
        v = normal(rng, rows, kv_heads * head_dim)
        first = max(0, rows - window)
        cache.restore_bulk(0, first, k[first:], v[first:])
        ref.restore_bulk(0, first, k[first:], v[first:])
    return pool, cache, ref, rng


def test_windowed_layer_provably_cannot_see_beyond_the_window():
    # attention_tests.rs windowed case (tests/test_oracle_attention.py pins the oracle on it):
    # with window 2 the query at position 3 averages the values at 2 and 3 only.
    cache = P().KvCache.new([W(2)], 1, 1)
    for p, val in enumerate([100.0, 200.0, 1.0, 3.0]):
        cache.append(0, [0.0], [val], p)
    out = P().gqa_attention([1.0], 1, 1, [3], cache.view(0), P().AttentionParams.new())
    assert abs(float(out[0]) - 2.0) < 1e-6


@pytest.mark.parametrize("elem", ["f32", "f16"])
@pytest.mark.parametrize("window,n,qh,kvh,d,softcap", [
    (16, 50, 4, 4, 8, 0.0),
    (7, 23, 6, 3, 4, 2.0),
    (256, 1000, 32, 4, 128, 0.0),   # the MFMA shapes, ring wrapped three times
    (100, 333, 8, 2, 128, 30.0),
    (64, 40, 8, 2, 64, 0.0),        # not yet full
])
def test_view_attention_matches_the_oracle_on_windowed_layers(elem, window, n, qh, kvh, d, softcap):
    pool, cache, ref, rng = pair(window, kvh, d, elem, rows=n, seed=n + d)
    params = dict(softcap=softcap)
    tol = (lambda a, b: rel_err(a, b) <= 1e-5) if elem == "f32" else (lambda a, b: max_abs(a, b) <= 2e-3)
    for positions in ([n - 1], [n - 2, n - 1], [n - 1, n - 2], [n + 3],
                      list(range(n - min(7, n), n))):
        positions = [p for p in positions if p > n - min(n, window) - 1]
        q = normal(rng, len(positions), qh * d)
        got = P().gqa_attention(q, len(positions), qh, positions, cache.view(0),
                                P().AttentionParams(**params))
        want = oracle.gqa_attention(q, len(positions), qh, positions, ref.view(0),
                                    oracle.AttentionParams(**params))
        assert tol(got, want), positions
    # A query whose whole window has left the ring sees nothing: refused by name.
    if n > window + 1:
        old = n - window - 1
        with pytest.raises(P().AttentionError) as e:
            P().gqa_attention(normal(rng, 1, qh * d), 1, qh, [old], cache.view(0),
                              P().AttentionParams.new())
        assert e.value == E("NoVisibleKeys", position=old)
    pool.close()


def run_steps(pool, cache, ref, rng, q_heads, steps, elem, softcap=0.0):
    """Device steps of the given row counts against the oracle's append-then-attend loop."""
    import torch
    kvh, d = pool.num_kv_heads, pool.head_dim
    worst = 0.0
    for rows in steps:
        base = cache.next_position(0)
        q = normal(rng, rows, q_heads * d)
        k = normal(rng, rows, kvh * d)
        v = normal(rng, rows, kvh * d)
        qd, kd, vd = (torch.from_numpy(x).cuda() for x in (q, k, v))
        out = torch.empty_like(qd)
        pool.attention_step_device(0, [(cache, rows)], qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                                   out.data_ptr(), q_heads, softcap=softcap)
        pool.synchronize()
        want = oracle.attention_step(ref, 0, q, k, v, q_heads, base,
                                     oracle.AttentionParams(softcap=softcap), threads=8)
        got = out.cpu().numpy().reshape(-1)
        err = rel_err(got, want) if elem == "f32" else max_abs(got, want)
        worst = max(worst, err)
        assert err <= (1e-5 if elem == "f32" else 2e-3), (rows, base, err)
        assert cache.next_position(0) == ref.next_position(0) == base + rows
    return worst


@pytest.mark.parametrize("elem,window,q_heads,kvh,d,steps,headroom", [
    ("f32", 16, 4, 2, 8, [1] * 40 + [5, 3, 7, 1, 1], 8),
    ("f32", 100, 8, 2, 64, [33, 1, 1, 20, 64, 1], 64),
    ("f16", 64, 32, 4, 128, [1] * 150, 0),                    # decode through two wraps
    ("f16", 64, 32, 4, 128, [7, 1, 7, 7, 1, 8, 2] * 12, 0),   # verify blocks (split-K kernel)
    ("f16", 128, 32, 4, 128, [100, 1, 64, 33, 128, 7, 1, 128, 90], 128),  # block kernel
    ("f16", 300, 8, 8, 128, [256, 256, 17, 256, 1, 200], 256),            # MHA, two tiles per wavefront
    ("f16", 96, 16, 2, 64, [1, 5, 40, 1, 1, 64], 64),                     # generic f16 path
    ("f16", 1500, 32, 4, 128, [256] * 7 + [1, 256], 256),  # block kernel, deep ring, through a wrap
])
def test_steps_on_a_windowed_layer_match_the_oracle(elem, window, q_heads, kvh, d, steps, headroom):
    pool, cache, ref, rng = pair(window, kvh, d, elem, seed=window + d, headroom=headroom)
    run_steps(pool, cache, ref, rng, q_heads, steps, elem)
    assert view_snapshot(cache, 0) == view_snapshot(ref, 0)
    pool.close()


@pytest.mark.parametrize("window,headroom,d,q_heads", [(7, 16, 128, 32), (20, 40, 128, 32), (7, 16, 64, 16),
                                                        (40, 50, 128, 8), (70, 20, 128, 32)])
def test_blocks_on_rings_of_one_to_three_storage_blocks_leave_exactly_their_rows(window, headroom, d, q_heads):
    # Blocks of eight rows or more are stored by writing whole 32-row storage blocks back. On a
    # ring of one or two storage blocks, consecutive position blocks are the same storage block:
    # a block that crosses a 32-row boundary must still leave its first rows in place. The
    # cache is compared after every step.
    pool, cache, ref, rng = pair(window, 4, d, "f16", seed=window + headroom, headroom=headroom)
    most = min(headroom, 64)
    for rows in [5, 16, 9, 16, 16, 8, 13, 16, 12, 16, 16, 10, most, 1, most, 11, most]:
        rows = min(rows, most)
        run_steps(pool, cache, ref, rng, q_heads, [rows], "f16")
        assert view_snapshot(cache, 0) == view_snapshot(ref, 0), (rows, cache.next_position(0))
    pool.close()


def test_steps_with_softcap_and_several_slots_on_a_mixed_pattern():
    import torch
    rng = np.random.default_rng(9)
    kvh, d, q_heads, window = 4, 128, 32, 48
    pattern = [W(window), P().LayerKind.Global]
    opattern = [oracle.LayerKind.windowed(window), oracle.LayerKind.Global]
    pool = P().KvPool(pattern, kvh, d, elem="f16", max_slots=3, capacity_rows=400)
    caches = [pool.acquire() for _ in range(3)]
    refs = [oracle.KvCache.new(opattern, kvh, d, store_f16=True) for _ in range(3)]
    for step, rows_per_slot in enumerate([(60, 5, 130), (1, 1, 1), (7, 1, 3), (1, 7, 1)] + [(1, 1, 1)] * 60):
        rows_per_slot = [min(r, 64) for r in rows_per_slot]
        for layer in range(2):
            total = sum(rows_per_slot)
            q = normal(rng, total, q_heads * d)
            k = normal(rng, total, kvh * d)
            v = normal(rng, total, kvh * d)
            qd, kd, vd = (torch.from_numpy(x).cuda() for x in (q, k, v))
            out = torch.empty_like(qd)
            pool.attention_step_device(layer, list(zip(caches, rows_per_slot)), qd.data_ptr(),
                                       kd.data_ptr(), vd.data_ptr(), out.data_ptr(), q_heads,
                                       softcap=20.0)
            pool.synchronize()
            got = out.cpu().numpy()
            r0 = 0
            for s, rows in enumerate(rows_per_slot):
                base = refs[s].next_position(layer)
                want = oracle.attention_step(refs[s], layer, q[r0:r0 + rows], k[r0:r0 + rows],
                                             v[r0:r0 + rows], q_heads, base,
                                             oracle.AttentionParams(softcap=20.0), threads=8)
                assert max_abs(got[r0:r0 + rows].reshape(-1), want) <= 2e-3, (step, layer, s)
                r0 += rows
    for s in range(3):
        for layer in range(2):
            assert view_snapshot(caches[s], layer) == view_snapshot(refs[s], layer)
    pool.close()


@pytest.mark.parametrize("elem", ["f32", "f16"])
def test_speculative_rounds_on_a_windowed_layer_rewind_to_the_exact_continuation(elem):
    # SPEC-itak-spec 5.2-5.3 as checkpoint_tests.rs:79-117 exercises it, with attention: a
    # round appends a verify block, is cut back to what was accepted, and the next tokens see
    # exactly what a cache that only ever held the accepted rows shows them.
    import torch
    window, kvh, d, q_heads = 40, 4, 128, 32
    pool, cache, ref, rng = pair(window, kvh, d, elem, seed=3)
    run_steps(pool, cache, ref, rng, q_heads, [1] * 50, elem)
    for accepted in (0, 3, 6, 7, 1, 0, 5) * 4:
        base = cache.next_position(0)
        cp, rcp = cache.checkpoint(8), ref.checkpoint(8)
        run_steps(pool, cache, ref, rng, q_heads, [8], elem)
        cache.rewind_to(cp, base + 1 + accepted)
        ref.rewind_to(rcp, base + 1 + accepted)
        cache.release(cp)
        ref.release(rcp)
        assert view_snapshot(cache, 0) == view_snapshot(ref, 0)
        run_steps(pool, cache, ref, rng, q_heads, [1], elem)
    pool.close()


@pytest.mark.parametrize("elem", ["f32", "f16"])
def test_rounds_deeper_than_the_ring_headroom_rewind_from_the_checkpoints_saved_rows(elem):
    # KvCache::checkpoint takes any round up to the smallest window and saves the ring slots the
    # round may overwrite (cache.rs:634-697); rewind_to puts back those the dropped positions
    # took (cache.rs:792-812). The device ring undoes ring - window = 32 positions by itself; a
    # deeper round (several blocks, each within the headroom) needs the saved rows: after every
    # rewind the view and the next tokens' attention equal the oracle's, through second rewinds
    # inside one checkpoint, rewinds below an earlier one, a round accepted whole, and a shallow
    # round's leftovers under a deep one.
    window, kvh, d, q_heads = 64, 4, 128, 32
    pool, cache, ref, rng = pair(window, kvh, d, elem, seed=11, headroom=32)
    run_steps(pool, cache, ref, rng, q_heads, [1] * 70 + [8] * 5, elem)   # wrapped once
    for depth, blocks, cuts in (
            (64, [32, 32], [40]),            # the whole window, rewound past the headroom
            (60, [20, 20, 20], [48, 10]),    # second rewind below the first, more tokens between
            (56, [28, 28], [5, 15, 2]),
            (48, [16, 32], [48]),            # nothing dropped
            (50, [25, 25], [1]),
            (8, [8], [3]),                   # shallow: leaves dropped rows in the headroom ...
            (64, [30, 30, 4], [0]),          # ... under a deep round that drops everything
            (40, [8] * 5, [33])):
        base = cache.next_position(0)
        cp, rcp = cache.checkpoint(depth), ref.checkpoint(depth)
        run_steps(pool, cache, ref, rng, q_heads, blocks, elem)
        for i, cut in enumerate(cuts):
            cache.rewind_to(cp, base + cut)
            ref.rewind_to(rcp, base + cut)
            assert cache.next_position(0) == ref.next_position(0) == base + cut
            assert view_snapshot(cache, 0) == view_snapshot(ref, 0), (depth, cut)
            if i + 1 < len(cuts):   # the round goes on before the next cut
                run_steps(pool, cache, ref, rng, q_heads, [min(depth - cut, 12)], elem)
        cache.release(cp)
        ref.release(rcp)
        run_steps(pool, cache, ref, rng, q_heads, [1, 1, 5], elem)
        assert view_snapshot(cache, 0) == view_snapshot(ref, 0), depth
    # The round bound still holds while the checkpoint is live, with the reference's fields.
    base = cache.next_position(0)
    cp, rcp = cache.checkpoint(40), ref.checkpoint(40)
    run_steps(pool, cache, ref, rng, q_heads, [32], elem)
    import torch
    z = torch.zeros(9, kvh * d, device="cuda")
    with pytest.raises(P().AttentionError) as e:
        pool.append_device(0, [(cache, 9)], z.data_ptr(), z.data_ptr())
    assert e.value.variant == "CheckpointRangeExceeded"
    cache.rewind_to(cp, base)
    ref.rewind_to(rcp, base)
    cache.release(cp)
    ref.release(rcp)
    assert view_snapshot(cache, 0) == view_snapshot(ref, 0)
    pool.close()


def test_a_deep_round_on_a_hybrid_pattern_saves_only_the_layers_that_need_it():
    # Windows 64 and 70 with 32 rows of headroom give rings of 96 and 128 rows: a round of 50
    # outgrows the first ring's 32 spare rows and not the second's 58; the global layer
    # truncates. All three must come back to the oracle's views.
    import torch
    kvh, d, q_heads = 2, 128, 8
    pattern = [W(64), P().LayerKind.Global, W(70)]
    rpattern = [oracle.LayerKind.windowed(64), oracle.LayerKind.Global, oracle.LayerKind.windowed(70)]
    pool = P().KvPool(pattern, kvh, d, elem="f16", capacity_rows=512, ring_headroom=32)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    ref = oracle.KvCache.new(rpattern, kvh, d, store_f16=True)
    rng = np.random.default_rng(21)

    def step(rows):
        base = cache.next_position(0)
        for layer in range(3):
            q, k, v = normal(rng, rows, q_heads * d), normal(rng, rows, kvh * d), normal(rng, rows, kvh * d)
            qd, kd, vd = (torch.from_numpy(x).cuda() for x in (q, k, v))
            out = torch.empty_like(qd)
            pool.attention_step_device(layer, [(cache, rows)], qd.data_ptr(), kd.data_ptr(),
                                       vd.data_ptr(), out.data_ptr(), q_heads)
            pool.synchronize()
            want = oracle.attention_step(ref, layer, q, k, v, q_heads, base, threads=4)
            assert max_abs(out.cpu().numpy().reshape(-1), want) <= 2e-3, (layer, base, rows)

    for rows in [25] * 6:
        step(rows)
    for depth, blocks, cut in ((50, [25, 25], 7), (64, [32, 32], 33), (50, [20, 30], 50)):
        base = cache.next_position(0)
        cp, rcp = cache.checkpoint(depth), ref.checkpoint(depth)
        for rows in blocks:
            step(rows)
        cache.rewind_to(cp, base + cut)
        ref.rewind_to(rcp, base + cut)
        cache.release(cp)
        ref.release(rcp)
        for layer in range(3):
            assert view_snapshot(cache, layer) == view_snapshot(ref, layer), (depth, layer)
        step(1)
        step(4)
    pool.close()


# ------------------------------------------------------------------------------ snapshots


@pytest.mark.parametrize("elem", ["f32", "f16"])
def test_snapshots_of_a_hybrid_cache_round_trip_and_match_the_oracles_bytes(elem):
    import oracle.itak_kv as okv
    kvh, d, window, tokens = 2, 16, 8, 21
    pattern = [W(window), P().LayerKind.Global, W(window)]
    opattern = [oracle.LayerKind.windowed(window), oracle.LayerKind.Global,
                oracle.LayerKind.windowed(window)]
    rng = np.random.default_rng(31)
    k = normal(rng, 3, tokens, kvh * d)
    v = normal(rng, 3, tokens, kvh * d)
    pool = P().KvPool(pattern, kvh, d, elem=elem, max_slots=2, capacity_rows=64)
    cache = pool.acquire()
    ref = oracle.KvCache.new(opattern, kvh, d, store_f16=(elem == "f16"))
    for layer in range(3):
        for p in range(tokens):
            cache.append(layer, k[layer, p], v[layer, p], p)
            ref.append(layer, k[layer, p], v[layer, p], p)
    data = P().capture_bytes(cache, "hybrid-test")
    want = okv.KvSnapshot.capture(ref, "hybrid-test").to_bytes()
    assert data == want
    # Restored into a fresh slot (and into a fresh oracle cache), then continued: the rings
    # hold the same positions and the next rows land in the same places.
    restored = P().restore_bytes(pool, data, expected_fingerprint="hybrid-test")
    ref2 = okv.KvSnapshot.from_bytes(want).restore(store_f16=(elem == "f16"))
    for layer in range(3):
        assert restored.next_position(layer) == tokens
        assert view_snapshot(restored, layer) == view_snapshot(cache, layer) == view_snapshot(ref2, layer)
    more_k = normal(rng, 3, 12, kvh * d)
    more_v = normal(rng, 3, 12, kvh * d)
    for layer in range(3):
        for i in range(12):
            restored.append(layer, more_k[layer, i], more_v[layer, i], tokens + i)
            ref2.append(layer, more_k[layer, i], more_v[layer, i], tokens + i)
        assert view_snapshot(restored, layer) == view_snapshot(ref2, layer)
    assert P().capture_bytes(restored, "x") == okv.KvSnapshot.capture(ref2, "x").to_bytes()
    # A snapshot of another pattern is refused by name before anything is written.
    other_pool = P().KvPool([W(window), P().LayerKind.Global, W(window + 1)], kvh, d, elem=elem)
    with pytest.raises(P().KvError) as e:
        P().restore_bytes(other_pool, data)
    assert e.value.variant == "GeometryMismatch"
    other_pool.close()
    pool.close()


# ---------------------------------------------------------------- Compute::attention mirror


@pytest.mark.parametrize("elem,d", [("f32", 16), ("f16", 16), ("f16", 128)])
def test_compute_attention_on_a_hybrid_model_takes_any_number_of_rows(elem, d):
    # cpu.rs:586-646 on the reference model's kind of pattern: the host-pointer call rotates
    # Q and K on the sliding-window layers (interleaved RoPE at the SWA base, each row at its
    # position; global layers are NoPE), then appends and attends row by row in the
    # reference, so a prompt longer than the device ring's headroom (and longer than the
    # window) must come out the same, and decoding on from it too.
    rng = np.random.default_rng(41)
    SW, G = P().LayerKind.SlidingWindow, P().LayerKind.Global
    # (head_dim 128 on an f16 pool is the MFMA path: single rows and short blocks rotate inside
    # the attention launch, long blocks by a launch of their own before the block kernel.)
    cfg = P().GlimmerConfig(layers=[SW, SW, G], q_heads=8, kv_heads=2, key_length=d,
                            value_length=d, sliding_window=20, rope_freq_base_swa=10000.0)
    ref = oracle.KvCache.new([oracle.LayerKind.windowed(20), oracle.LayerKind.windowed(20),
                              oracle.LayerKind.Global], cfg.kv_heads, cfg.key_length,
                             store_f16=(elem == "f16"))
    hc = P().HipCompute.new(elem=elem, capacity_rows=512)
    cache = P().PositionCache()
    for rows in (150, 1, 1, 65, 5, 1):
        for layer, kind in enumerate(cfg.layers):
            q = normal(rng, rows, cfg.q_width())
            k = normal(rng, rows, cfg.k_width())
            v = normal(rng, rows, cfg.v_width())
            got = hc.attention(P().AttentionRequest(q, k, v, layer, kind, cfg), cache)
            want = oracle.compute_attention(ref, layer, q, k, v, cfg.q_heads, cache.position(),
                                            cfg.rope_freq_base_swa, threads=8)
            if elem == "f32":
                assert rel_err(got, want) <= 1e-5, (rows, layer)
            else:
                assert max_abs(got, want) <= 2e-3, (rows, layer)
        cache.advance(rows)
    dev = hc.kv_cache()
    for layer in range(3):
        assert dev.next_position(layer) == 223
        assert view_snapshot(dev, layer) == view_snapshot(ref, layer)
    # A speculative round through the Compute-level calls, on the hybrid cache.
    cp = hc.cache_checkpoint(4)
    rcp = ref.checkpoint(4)
    for layer, kind in enumerate(cfg.layers):
        q, k, v = normal(rng, 4, cfg.q_width()), normal(rng, 4, cfg.k_width()), normal(rng, 4, cfg.v_width())
        hc.attention(P().AttentionRequest(q, k, v, layer, kind, cfg), cache)
        oracle.compute_attention(ref, layer, q, k, v, cfg.q_heads, 223, cfg.rope_freq_base_swa,
                                 threads=8)
    hc.cache_rewind(cp, 225)
    ref.rewind_to(rcp, 225)
    hc.cache_release(cp)
    ref.release(rcp)
    for layer in range(3):
        assert view_snapshot(dev, layer) == view_snapshot(ref, layer)


def test_compute_attention_refuses_a_bad_swa_base_on_sliding_layers_only():
    # rope_interleaved's refusals (crates/torch-math/src/rope_interleaved.rs:72-99) surface
    # under the attention step; a global layer never looks at the base.
    SW, G = P().LayerKind.SlidingWindow, P().LayerKind.Global
    cfg = P().GlimmerConfig(layers=[SW, G], q_heads=4, kv_heads=2, key_length=8, value_length=8,
                            sliding_window=6, rope_freq_base_swa=1.0)
    hc = P().HipCompute.new(elem="f32", capacity_rows=32)
    cache = P().PositionCache()
    q, k, v = np.ones(32, np.float32), np.ones(16, np.float32), np.ones(16, np.float32)
    with pytest.raises(P().StepFailed) as e:
        hc.attention(P().AttentionRequest(q, k, v, 0, SW, cfg), cache)
    assert e.value.step == "attention" and "rope: base must be finite and > 1" in e.value.detail
    assert hc.kv_cache().next_position(0) == 0
    out = hc.attention(P().AttentionRequest(q, k, v, 1, G, cfg), cache)
    assert np.allclose(out, 1.0)


@pytest.mark.gpu
@pytest.mark.parametrize("kvh,d", [(4, 128), (2, 64)])
def test_chunk_appends_into_a_ring_land_where_row_appends_would(kvh, d):
    """Chunks of 128 rows and more go into a ring as whole 32-row blocks (in two pieces where
    they wrap) with the rows before the first block boundary and after the last one beside them:
    after every chunk the view holds exactly what the oracle's row-by-row appends leave, and a
    rewind into the chunk still finds the rows the chunk must not have touched."""
    import torch
    window, headroom = 200, 320
    pool, cache, ref, rng = pair(window, kvh, d, "f16", headroom=headroom)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    for rows in (128, 129, 31, 320, 1, 160, 255, 128, 7, 300, 192):  # starts at 0, 128, 257, 288, ...
        base = cache.next_position(0)
        k, v = normal(rng, rows, kvh * d), normal(rng, rows, kvh * d)
        kd, vd = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
        pool.append_device(0, [(cache, rows)], kd.data_ptr(), vd.data_ptr())
        pool.synchronize()
        for i in range(rows):
            ref.append(0, k[i], v[i], base + i)
        assert cache.next_position(0) == ref.next_position(0) == base + rows
        assert view_snapshot(cache, 0) == view_snapshot(ref, 0), (rows, base)
    # A truncate into the last chunk keeps every row of the window before the cut: the chunk's
    # whole-block stores wrote nothing outside its own rows.
    end = cache.next_position(0)
    cut = end - 100
    pool.truncate([cache], [cut])
    def values_of(rows):  # f16 storage compared as the values it holds
        rows = np.asarray(rows)
        if rows.dtype == np.uint16:
            rows = rows.view(np.float16)
        return rows.astype(np.float32).reshape(window, -1)

    pos, keys, _ = ref.view(0).rows()
    got_pos, got_k, _ = cache.view(0).rows()
    got_pos = list(np.asarray(got_pos, dtype=np.int64))
    assert got_pos == list(range(cut - window, cut))
    ref_pos = list(np.asarray(pos, dtype=np.int64))
    # The oracle's view (uncut) and the cut view overlap on positions [end - window, cut).
    lo = end - window
    a = values_of(got_k)[lo - (cut - window):]
    b = values_of(keys)[: cut - lo]
    assert ref_pos[0] == lo and a.tobytes() == b.tobytes()
    pool.close()
