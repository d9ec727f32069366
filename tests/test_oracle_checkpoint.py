"""The reference's checkpoint/rewind KATs (crates/attention/tests/checkpoint_tests.rs)
against the CPU oracle. Rows carry exactly representable integers so equality is exact."""
import numpy as np
import pytest

import oracle
from oracle import AttentionParams, Err, KvCache, LayerKind, glimmer_layer_pattern, gqa_attention


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
    for layer in range(cache.layer_count()):
        for p in positions:
            append(cache, layer, kv_heads, head_dim, p)


def view_snapshot(cache, layer):  # checkpoint_tests.rs:54-65
    view = cache.view(layer)
    out = []
    for vi in range(view.len()):
        out.append(np.float32(view.position_at(vi)).tobytes())
        for head in range(view.num_kv_heads()):
            out.append(view.key(vi, head).tobytes())
            out.append(view.value(vi, head).tobytes())
    return b"".join(out)


def reference_cache(pattern, kv_heads, head_dim, positions):
    cache = KvCache.new(pattern, kv_heads, head_dim)
    append_all(cache, kv_heads, head_dim, positions)
    return cache


def test_windowed_rewind_restores_rows_evicted_by_speculative_appends():
    # checkpoint_tests.rs:79-117.
    pattern = [LayerKind.windowed(4)]
    cache = reference_cache(pattern, 1, 2, range(6))
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
    fresh = reference_cache(pattern, 1, 2, range(6))
    q = [0.5, -0.25]
    after = gqa_attention(q, 1, 1, [5], cache.view(0), AttentionParams.new())
    never = gqa_attention(q, 1, 1, [5], fresh.view(0), AttentionParams.new())
    assert after.tobytes() == never.tobytes()


def test_windowed_rewind_to_mid_block_keeps_exactly_the_committed_prefix():
    # checkpoint_tests.rs:119-144.
    pattern = [LayerKind.windowed(4)]
    cache = reference_cache(pattern, 2, 2, range(6))
    cp = cache.checkpoint(3)
    for p in (6, 7, 8):
        append(cache, 0, 2, 2, p)
    cache.rewind_to(cp, 7)
    cache.release(cp)
    assert view_snapshot(cache, 0) == view_snapshot(reference_cache(pattern, 2, 2, range(7)), 0)
    assert cache.stats()[0].appended == 7
    append(cache, 0, 2, 2, 7)
    assert view_snapshot(cache, 0) == view_snapshot(reference_cache(pattern, 2, 2, range(8)), 0)


def test_windowed_checkpoint_saved_slots_wrap_the_ring():
    # checkpoint_tests.rs:146-161.
    pattern = [LayerKind.windowed(4)]
    cache = reference_cache(pattern, 1, 2, range(7))
    cp = cache.checkpoint(2)
    for p in (7, 8):
        append(cache, 0, 1, 2, p)
    cache.rewind_to(cp, 7)
    cache.release(cp)
    assert view_snapshot(cache, 0) == view_snapshot(reference_cache(pattern, 1, 2, range(7)), 0)
    assert cache.stats()[0].appended == 7


def test_global_rewind_truncates_and_keeps_the_prefix():
    # checkpoint_tests.rs:163-181.
    pattern = [LayerKind.Global]
    cache = reference_cache(pattern, 2, 2, range(5))
    cp = cache.checkpoint(3)
    assert cp.saved_bytes() == 0
    for p in (5, 6, 7):
        append(cache, 0, 2, 2, p)
    assert cache.stored_len(0) == 8
    cache.rewind_to(cp, 6)
    cache.release(cp)
    assert view_snapshot(cache, 0) == view_snapshot(reference_cache(pattern, 2, 2, range(6)), 0)
    assert cache.stats()[0].appended == 6
    assert cache.stored_len(0) == 6


def test_rewind_to_a_checkpoint_taken_before_any_append():
    # checkpoint_tests.rs:183-207.
    pattern = [LayerKind.windowed(4), LayerKind.Global]
    cache = KvCache.new(pattern, 1, 2)
    cp = cache.checkpoint(2)
    assert cp.base(0) == 0 and cp.base(1) == 0
    append_all(cache, 1, 2, [0, 1])
    cache.rewind_to(cp, 0)
    cache.release(cp)
    for layer in range(2):
        assert cache.stats()[layer].appended == 0
        assert cache.view(layer).is_empty()
    append_all(cache, 1, 2, [0, 1])
    reference = reference_cache(pattern, 1, 2, [0, 1])
    for layer in range(2):
        assert view_snapshot(cache, layer) == view_snapshot(reference, layer)


def test_second_rewind_restores_the_snapshot_again():
    # checkpoint_tests.rs:209-230.
    pattern = [LayerKind.windowed(4)]
    cache = reference_cache(pattern, 1, 2, range(6))
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
    # checkpoint_tests.rs:232-316.
    pattern = [LayerKind.windowed(4), LayerKind.Global]
    cache = reference_cache(pattern, 1, 2, [0, 1])
    with pytest.raises(oracle.AttentionError) as e:
        cache.checkpoint(0)
    assert e.value == Err("ZeroDimension", what="max_round_tokens")
    with pytest.raises(oracle.AttentionError) as e:
        cache.checkpoint(5)
    assert e.value == Err("CheckpointTooDeep", max_round_tokens=5, window=4)
    cp = cache.checkpoint(2)
    with pytest.raises(oracle.AttentionError) as e:
        cache.checkpoint(1)
    assert e.value == Err("CheckpointBusy")
    append_all(cache, 1, 2, [2, 3])
    with pytest.raises(oracle.AttentionError) as e:
        cache.append(0, k_row(1, 2, 4), v_row(1, 2, 4), 4)
    assert e.value == Err("CheckpointRangeExceeded", layer=0, position=4, limit=4)
    with pytest.raises(oracle.AttentionError) as e:
        cache.rewind_to(cp, 1)
    assert e.value == Err("RewindOutOfRange", layer=0, base=2, appended=4, target=1)
    with pytest.raises(oracle.AttentionError) as e:
        cache.rewind_to(cp, 5)
    assert e.value == Err("RewindOutOfRange", layer=0, base=2, appended=4, target=5)
    assert cache.stats()[0].appended == 4
    cache.release(cp)
    with pytest.raises(oracle.AttentionError) as e:
        cache.rewind_to(cp, 2)
    assert e.value.variant == "StaleCheckpoint"
    with pytest.raises(oracle.AttentionError) as e:
        cache.release(cp)
    assert e.value.variant == "StaleCheckpoint"
    other = reference_cache(pattern, 1, 2, [0, 1])
    foreign = other.checkpoint(2)
    mine = cache.checkpoint(2)
    with pytest.raises(oracle.AttentionError) as e:
        cache.rewind_to(foreign, 2)
    assert e.value.variant == "StaleCheckpoint"
    cache.release(mine)
    other.release(foreign)


def test_checkpoint_memory_bound_at_glimmer_geometry():
    # checkpoint_tests.rs:318-337.
    cache = KvCache.new(glimmer_layer_pattern(), 2, 128)
    append_all(cache, 2, 128, [0])
    cp = cache.checkpoint(17)
    assert cp.base(0) == 1 and cp.base(51) == 1
    assert cp.max_round_tokens() == 17
    assert cp.saved_bytes() == 39 * 17 * 2048 == 1_357_824
    cache.release(cp)
