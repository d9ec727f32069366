"""The reference's cache KATs (crates/attention/tests/cache_tests.rs) against the CPU oracle."""
import numpy as np
import pytest

import oracle
from oracle import Err, KvCache, LayerKind, glimmer_layer_pattern

U64_MAX = 2**64 - 1


def row(kv_heads, head_dim, fill):
    return np.full(kv_heads * head_dim, fill, dtype=np.float32)


def test_glimmer_pattern_is_39_windowed_13_global():
    # cache_tests.rs:11-35.
    pattern = glimmer_layer_pattern()
    assert len(pattern) == 52
    assert [i for i, k in enumerate(pattern) if k == LayerKind.Global] == list(range(3, 52, 4))
    assert sum(1 for k in pattern if k.window() is not None) == 39
    assert all(k.window() == 2048 for k in pattern if k.window() is not None)


def test_ring_buffer_wraps_and_evicts_oldest():
    # cache_tests.rs:37-62.
    cache = KvCache.new([LayerKind.windowed(4)], 1, 1)
    for pos in range(7):
        cache.append(0, row(1, 1, pos), row(1, 1, pos), pos)
    assert cache.stored_len(0) == 4
    assert cache.next_position(0) == 7
    view = cache.view(0)
    assert view.len() == 4 and not view.is_empty()
    for vi, expected in enumerate([3, 4, 5, 6]):
        assert view.position_at(vi) == expected
        assert view.value(vi, 0).tolist() == [float(expected)]
        assert view.key(vi, 0).tolist() == [float(expected)]
    assert view.position_at(4) is None
    stats = cache.stats()
    assert stats[0].appended == 7 and stats[0].stored == 4


def test_ring_buffer_holds_exactly_the_glimmer_window():
    # cache_tests.rs:64-79.
    cache = KvCache.new([LayerKind.windowed(2048)], 2, 4)
    for pos in range(2050):
        k = row(2, 4, pos)
        cache.append(0, k, k, pos)
    assert cache.stored_len(0) == 2048
    view = cache.view(0)
    assert view.position_at(0) == 2
    assert view.position_at(2047) == 2049
    assert view.value(0, 0)[0] == 2.0
    assert view.value(2047, 1)[0] == 2049.0


def test_global_layer_keeps_everything():
    # cache_tests.rs:81-96.
    cache = KvCache.new([LayerKind.Global], 2, 2)
    for pos in range(10):
        cache.append(0, row(2, 2, pos), row(2, 2, pos), pos)
    assert cache.stored_len(0) == 10
    view = cache.view(0)
    assert view.len() == 10 and view.window() is None
    for pos in range(10):
        assert view.position_at(pos) == pos
        assert view.value(pos, 1)[0] == float(pos)


def test_append_rejects_bad_shapes_and_out_of_order_positions():
    # cache_tests.rs:98-131.
    cache = KvCache.new([LayerKind.Global], 2, 4)
    with pytest.raises(oracle.AttentionError) as e:
        cache.append(0, row(1, 4, 0.0), row(2, 4, 0.0), 0)
    assert e.value == Err("ShapeMismatch", what="k", expected=8, actual=4)
    with pytest.raises(oracle.AttentionError) as e:
        cache.append(0, row(2, 4, 0.0), row(1, 4, 0.0), 0)
    assert e.value == Err("ShapeMismatch", what="v", expected=8, actual=4)
    with pytest.raises(oracle.AttentionError) as e:
        cache.append(0, row(2, 4, 0.0), row(2, 4, 0.0), 1)
    assert e.value == Err("OutOfOrderPosition", layer=0, expected=0, actual=1)
    assert "expected position 0, got 1" in e.value.message
    assert cache.stored_len(0) == 0
    cache.append(0, row(2, 4, 0.0), row(2, 4, 0.0), 0)
    assert cache.stored_len(0) == 1


def test_construction_rejects_zero_dimensions_and_window():
    # cache_tests.rs:133-159.
    with pytest.raises(oracle.AttentionError) as e:
        KvCache.new([], 2, 128)
    assert e.value == Err("ZeroDimension", what="layer pattern")
    with pytest.raises(oracle.AttentionError) as e:
        KvCache.new([LayerKind.Global], 0, 128)
    assert e.value == Err("ZeroDimension", what="num_kv_heads")
    with pytest.raises(oracle.AttentionError) as e:
        KvCache.new([LayerKind.Global], 2, 0)
    assert e.value == Err("ZeroDimension", what="head_dim")
    with pytest.raises(oracle.AttentionError) as e:
        LayerKind.windowed(0)
    assert e.value == Err("InvalidWindow", window=0)
    with pytest.raises(oracle.AttentionError) as e:
        KvCache.new([LayerKind.Windowed(0)], 2, 128)
    assert e.value == Err("InvalidWindow", window=0)


def test_construction_refuses_sizes_that_overflow():
    # cache_tests.rs:161-183.
    with pytest.raises(oracle.AttentionError) as e:
        KvCache.new([LayerKind.Windowed(U64_MAX)], 2, 128)
    assert e.value == Err("SizeOverflow", what="windowed layer storage")
    with pytest.raises(oracle.AttentionError) as e:
        KvCache.new([LayerKind.Global], U64_MAX, 2)
    assert e.value == Err("SizeOverflow", what="kv row length")


def test_invalid_layer_is_an_error_not_a_panic():
    # cache_tests.rs:185-205.
    cache = KvCache.new([LayerKind.Global], 1, 1)
    with pytest.raises(oracle.AttentionError) as e:
        cache.view(5)
    assert e.value == Err("InvalidLayer", layer=5, layer_count=1)
    with pytest.raises(oracle.AttentionError) as e:
        cache.append(5, row(1, 1, 0.0), row(1, 1, 0.0), 0)
    assert e.value == Err("InvalidLayer", layer=5, layer_count=1)
    assert cache.layer_kind(0) == LayerKind.Global


def test_empty_view_is_empty_and_indexes_to_none():
    # cache_tests.rs:207-216.
    cache = KvCache.new([LayerKind.windowed(8)], 1, 2)
    view = cache.view(0)
    assert view.is_empty() and view.len() == 0
    assert view.position_at(0) is None
    assert view.key(0, 0) is None
    assert view.window() == 8


def rows_for(layer, position, row_len):
    # cache_tests.rs:232-240; the divisions are f32 divisions of exactly representable ints.
    i = np.arange(row_len)
    k = ((position * 100 + layer * 10 + i).astype(np.float32) / np.float32(7.0)).astype(np.float32)
    v = (-((position * 50 + layer * 5 + i).astype(np.float32)) / np.float32(3.0)).astype(np.float32)
    return k, v


def test_bulk_restore_matches_append_replay_bitwise():
    # cache_tests.rs:218-283.
    pattern = [LayerKind.windowed(4), LayerKind.Global, LayerKind.windowed(4)]
    kv_heads, head_dim = 2, 3
    row_len = kv_heads * head_dim
    tokens = 9
    replay = KvCache.new(pattern, kv_heads, head_dim)
    for position in range(tokens):
        for layer in range(len(pattern)):
            k, v = rows_for(layer, position, row_len)
            replay.append(layer, k, v, position)
    bulk = KvCache.new(pattern, kv_heads, head_dim)
    for layer, kind in enumerate(pattern):
        if kind.window() is None:
            first, count = 0, tokens
        else:
            count = min(tokens, kind.window())
            first = tokens - count
        keys, values = [], []
        for position in range(first, first + count):
            k, v = rows_for(layer, position, row_len)
            keys.append(k)
            values.append(v)
        bulk.restore_bulk(layer, first, np.concatenate(keys), np.concatenate(values))
    for layer in range(len(pattern)):
        assert bulk.next_position(layer) == tokens
        want, got = replay.view(layer), bulk.view(layer)
        assert got.len() == want.len()
        for slot in range(want.len()):
            assert got.position_at(slot) == want.position_at(slot)
            for head in range(kv_heads):
                assert got.key(slot, head).tobytes() == want.key(slot, head).tobytes()
                assert got.value(slot, head).tobytes() == want.value(slot, head).tobytes()
        k, v = rows_for(layer, tokens, row_len)
        replay.append(layer, k, v, tokens)
        bulk.append(layer, k, v, tokens)
        pw, kw, vw = replay.view(layer).rows()
        pg, kg, vg = bulk.view(layer).rows()
        assert np.array_equal(pw, pg) and kw.tobytes() == kg.tobytes() and vw.tobytes() == vg.tobytes()


def test_bulk_restore_refusals_are_named():
    # cache_tests.rs:285-322.
    pattern = [LayerKind.windowed(4), LayerKind.Global]
    cache = KvCache.new(pattern, 1, 2)
    with pytest.raises(oracle.AttentionError) as e:
        cache.restore_bulk(0, 0, np.zeros(10), np.zeros(10))
    assert e.value == Err("ShapeMismatch", what="bulk restore rows (windowed layer)", expected=4,
                          actual=5)
    with pytest.raises(oracle.AttentionError) as e:
        cache.restore_bulk(1, 3, np.zeros(4), np.zeros(4))
    assert e.value == Err("ShapeMismatch", what="bulk restore first position (global layer)",
                          expected=0, actual=3)
    cache.append(0, row(1, 2, 1.0), row(1, 2, 1.0), 0)
    with pytest.raises(oracle.AttentionError) as e:
        cache.restore_bulk(0, 0, np.zeros(2), np.zeros(2))
    assert e.value == Err("BulkRestoreNotFresh", layer=0, appended=1)
    fresh = KvCache.new(pattern, 1, 2)
    with pytest.raises(oracle.AttentionError) as e:
        fresh.restore_bulk(0, 0, np.zeros(4), np.zeros(2))
    assert e.value == Err("ShapeMismatch", what="bulk restore rows", expected=2, actual=4)
