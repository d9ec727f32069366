"""The reference's device-ring KATs (crates/wgpu-compute/src/session.rs:6091-6120, 6183-6268)
against the oracle's restatement, and the library's ring against the restatement: a restore
puts every row into the ring slot the runs name."""
import numpy as np
import pytest

import oracle
from oracle.device_ring import prefix_slot_runs, prefix_visible_range, ring_capacity
from helpers import pkg


def test_ring_capacity_is_window_plus_cap_headroom():
    # session.rs:6091-6120.
    assert ring_capacity(2048, 64) == 2111
    assert ring_capacity(2048, 32) == 2079
    assert ring_capacity(2048, 1) == 2048
    assert ring_capacity(4, 64) == 67


def test_prefix_visible_range_is_the_snapshot_rule():
    # session.rs:6183-6202.
    assert prefix_visible_range(None, 0) == (0, 0)
    assert prefix_visible_range(None, 70) == (0, 70)
    assert prefix_visible_range(4, 3) == (0, 3)
    assert prefix_visible_range(4, 4) == (0, 4)
    assert prefix_visible_range(4, 70) == (66, 4)


def test_prefix_slot_runs_remap_the_windowed_ring():
    # session.rs:6204-6268.
    assert prefix_slot_runs(False, 0, 70, 67) == [(0, 0, 70)]
    assert prefix_slot_runs(True, 10, 4, 67) == [(0, 10, 4)]
    assert prefix_slot_runs(True, 66, 4, 67) == [(0, 66, 1), (1, 0, 3)]
    for cap in (1, 4, 32, 64):
        ring = 4 + cap - 1
        for position in range(300):
            first, rows = prefix_visible_range(4, position)
            runs = prefix_slot_runs(True, first, rows, ring)
            assert len(runs) <= 2
            assert sum(r[2] for r in runs) == rows
            slots = [r[1] + i for r in runs for i in range(r[2])]
            assert slots == [p % ring for p in range(first, first + rows)]


def test_the_oracles_snapshots_follow_the_visible_range_rule():
    # The CPU cache's own view and the device-session rule describe the same rows.
    cache = oracle.KvCache.new([oracle.LayerKind.windowed(4), oracle.LayerKind.Global], 1, 2)
    for p in range(70):
        for layer in range(2):
            cache.append(layer, [float(p)] * 2, [float(-p)] * 2, p)
        for layer, window in ((0, 4), (1, None)):
            first, rows = prefix_visible_range(window, p + 1)
            view = cache.view(layer)
            assert (view.position_at(0), view.len()) == (first, rows)


@pytest.mark.gpu
@pytest.mark.parametrize("elem", ["f32", "f16"])
@pytest.mark.parametrize("window,headroom,position", [(4, 64, 70), (4, 1, 70), (100, 28, 1000),
                                                      (100, 28, 60), (33, 31, 64)])
def test_a_restore_lands_in_the_slots_the_runs_name(elem, window, headroom, position):
    P = pkg()
    kvh, d = 2, 16
    pool = P.KvPool([P.LayerKind.windowed(window)], kvh, d, elem=elem, ring_headroom=headroom)
    cache = pool.acquire()
    first, rows = prefix_visible_range(window, position)
    rng = np.random.default_rng(position)
    k = rng.standard_normal((rows, kvh * d), dtype=np.float32)
    v = rng.standard_normal((rows, kvh * d), dtype=np.float32)
    cache.restore_bulk(0, first, k, v)
    raw_k, raw_v = cache.read_raw(0)
    ring = raw_k.shape[0]
    assert ring % 32 == 0 and ring >= window + headroom  # the library's ring: whole 32-row blocks
    as_f32 = (lambda a: a.view(np.float16).astype(np.float32)) if elem == "f16" else (lambda a: a)
    want_k = k.astype(np.float16).astype(np.float32) if elem == "f16" else k
    want_v = v.astype(np.float16).astype(np.float32) if elem == "f16" else v
    touched = np.zeros(ring, dtype=bool)
    for row, slot, count in prefix_slot_runs(True, first, rows, ring):
        got_k = as_f32(raw_k[slot:slot + count]).reshape(count, -1)
        got_v = as_f32(raw_v[slot:slot + count]).reshape(count, -1)
        assert np.array_equal(got_k, want_k[row:row + count])
        assert np.array_equal(got_v, want_v[row:row + count])
        touched[slot:slot + count] = True
    assert not as_f32(raw_k[~touched]).any() and not as_f32(raw_v[~touched]).any()
    pool.close()
