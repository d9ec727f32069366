"""The reference's attention KATs (crates/attention/tests/attention_tests.rs) run against
the CPU oracle, plus closed forms and an independent float64 reference that pin what
those hand values leave open (softmax weights over many keys, the softcap extension)."""
import numpy as np
import pytest

import oracle
from oracle import AttentionParams, Err, KvCache, LayerKind, gqa_attention, kv_head_for_query_head


def cache_with(kind, kv_heads, head_dim, rows, store_f16=False):
    """attention_tests.rs:12-23."""
    cache = KvCache.new([kind], kv_heads, head_dim, store_f16)
    for pos, (k, v) in enumerate(rows):
        cache.append(0, k, v, pos)
    return cache


def close(actual, expected, tol):
    return abs(float(actual) - expected) <= tol


def test_windowed_layer_provably_cannot_see_beyond_the_window():
    # attention_tests.rs:29-45: window 2 at position 2 averages (3 + 5) / 2, never 336.
    rows = [([1.0], [1000.0]), ([1.0], [3.0]), ([1.0], [5.0])]
    cache = cache_with(LayerKind.windowed(2), 1, 1, rows)
    out = gqa_attention([1.0], 1, 1, [2], cache.view(0), AttentionParams.new())
    assert close(out[0], 4.0, 1e-6), out[0]


def test_global_layer_sees_everything():
    # attention_tests.rs:47-61.
    rows = [([1.0], [1000.0]), ([1.0], [3.0]), ([1.0], [5.0])]
    cache = cache_with(LayerKind.Global, 1, 1, rows)
    out = gqa_attention([1.0], 1, 1, [2], cache.view(0), AttentionParams.new())
    assert close(out[0], 336.0, 1e-3), out[0]


def test_causal_mask_blocks_future_positions():
    # attention_tests.rs:63-85.
    rows = [([0.0], [1.0]), ([10.0], [100.0]), ([10.0], [1000.0])]
    cache = cache_with(LayerKind.Global, 1, 1, rows)
    out = gqa_attention([1.0, 1.0], 2, 1, [0, 1], cache.view(0), AttentionParams.new())
    assert close(out[0], 1.0, 1e-6), out[0]
    assert 99.9 < out[1] < 100.0, out[1]
    # Closed form for the second query: softmax over scores (0, 10).
    expect = (1.0 + 100.0 * np.exp(10.0)) / (1.0 + np.exp(10.0))
    assert close(out[1], expect, 1e-4)


def test_gqa_head_sharing_glimmer_shape_32_to_2():
    # attention_tests.rs:87-114.
    for h in range(32):
        assert kv_head_for_query_head(h, 32, 2) == (0 if h < 16 else 1)
    rows = [([1.0, 0.0, 1.0, 0.0], [10.0, 0.0, 20.0, 0.0])]
    cache = cache_with(LayerKind.Global, 2, 2, rows)
    q = [1.0, 0.0] * 32
    out = gqa_attention(q, 1, 32, [0], cache.view(0), AttentionParams.new())
    for h in range(32):
        expected = 10.0 if h < 16 else 20.0
        assert close(out[h * 2], expected, 1e-6), (h, out[h * 2])
        assert close(out[h * 2 + 1], 0.0, 1e-6)


def test_gqa_head_sharing_smaller_ratio_4_to_2():
    # attention_tests.rs:116-140.
    for h, expected in [(0, 0), (1, 0), (2, 1), (3, 1)]:
        assert kv_head_for_query_head(h, 4, 2) == expected
    cache = cache_with(LayerKind.Global, 2, 1, [([1.0, 1.0], [7.0, 9.0])])
    out = gqa_attention([1.0] * 4, 1, 4, [0], cache.view(0), AttentionParams.new())
    for h, expected in [(0, 7.0), (1, 7.0), (2, 9.0), (3, 9.0)]:
        assert close(out[h], expected, 1e-6), (h, out[h])


def test_scale_defaults_to_one_over_sqrt_head_dim_and_is_a_parameter():
    # attention_tests.rs:142-150.
    params = AttentionParams.new()
    assert close(params.scale_for(128), 0.08838835, 1e-7)
    assert close(params.scale_for(1), 1.0, 1e-7)
    assert close(AttentionParams.with_scale(0.25).scale_for(128), 0.25, 1e-7)
    assert AttentionParams() == params
    # The C side applies the same default: one key at score q.k*scale, two keys with
    # scores (0, ln 3 / scale * scale) give weights 1/4, 3/4 only if scale is 1/sqrt(d).
    d = 16
    k1 = np.zeros(d, dtype=np.float32)
    k2 = np.zeros(d, dtype=np.float32)
    k2[0] = np.log(3.0) * 4.0  # q.k2 * (1/4) = ln 3
    q = np.zeros(d, dtype=np.float32)
    q[0] = 1.0
    cache = cache_with(LayerKind.Global, 1, d, [(k1, np.full(d, 0.0)), (k2, np.full(d, 4.0))])
    out = gqa_attention(q, 1, 1, [1], cache.view(0), AttentionParams.new())
    assert close(out[0], 3.0, 1e-5)
    out = gqa_attention(q, 1, 1, [1], cache.view(0), AttentionParams.with_scale(0.5))
    assert close(out[0], 4.0 * 9.0 / 10.0, 1e-5)  # weights 1/10, 9/10


def test_attention_validation_is_named_errors_not_panics():
    # attention_tests.rs:152-212.
    cache = KvCache.new([LayerKind.Global], 2, 2)
    with pytest.raises(oracle.AttentionError) as e:
        gqa_attention([1.0, 0.0, 1.0, 0.0], 1, 2, [0], cache.view(0), AttentionParams.new())
    assert e.value == Err("NoVisibleKeys", position=0)
    assert "query at position 0 has no visible keys" in e.value.message

    cache = cache_with(LayerKind.Global, 2, 2, [([1.0, 0.0, 1.0, 0.0], [1.0, 0.0, 1.0, 0.0])])
    view = cache.view(0)
    with pytest.raises(oracle.AttentionError) as e:
        gqa_attention([1.0] * 6, 1, 3, [0], view, AttentionParams.new())
    assert e.value == Err("NonDivisibleHeads", num_q_heads=3, num_kv_heads=2)
    with pytest.raises(oracle.AttentionError) as e:
        gqa_attention([1.0], 1, 2, [0], view, AttentionParams.new())
    assert e.value == Err("ShapeMismatch", what="q", expected=4, actual=1)
    with pytest.raises(oracle.AttentionError) as e:
        gqa_attention([1.0] * 4, 2, 2, [0], view, AttentionParams.new())
    assert e.value == Err("ShapeMismatch", what="query_positions", expected=2, actual=1)
    with pytest.raises(oracle.AttentionError) as e:
        kv_head_for_query_head(0, 3, 2)
    assert e.value == Err("NonDivisibleHeads", num_q_heads=3, num_kv_heads=2)


# --- what the hand values leave open -------------------------------------------------

def naive_f64(q, keys, vals, positions, key_positions, q_heads, scale, window=None, softcap=0.0):
    """Independent float64 reference in the pattern of
    crates/cpu-compute/tests/forward_tests.rs:490-514 (plain softmax, no shared code)."""
    nq = len(positions)
    kv_heads, d = keys.shape[1], keys.shape[2]
    group = q_heads // kv_heads
    q = q.reshape(nq, q_heads, d).astype(np.float64)
    out = np.zeros((nq, q_heads, d))
    for qi, p in enumerate(positions):
        vis = [j for j, kp in enumerate(key_positions)
               if kp <= p and (window is None or kp > p - window)]
        for h in range(q_heads):
            kh = h // group
            s = keys[vis, kh].astype(np.float64) @ q[qi, h] * scale
            if softcap > 0:
                s = softcap * np.tanh(s / softcap)
            w = np.exp(s - s.max())
            w /= w.sum()
            out[qi, h] = w @ vals[vis, kh].astype(np.float64)
    return out.reshape(-1)


@pytest.mark.parametrize("kind,n,qh,kvh,d,softcap", [
    (LayerKind.Global, 37, 8, 2, 16, 0.0),
    (LayerKind.Global, 130, 32, 4, 64, 0.0),
    (LayerKind.windowed(16), 50, 4, 4, 8, 0.0),
    (LayerKind.Global, 64, 8, 1, 32, 5.0),
    (LayerKind.windowed(7), 23, 6, 3, 4, 2.0),
])
def test_matches_an_independent_float64_reference(kind, n, qh, kvh, d, softcap):
    rng = np.random.default_rng(1234 + n)
    keys = rng.standard_normal((n, kvh, d), dtype=np.float32) * 2
    vals = rng.standard_normal((n, kvh, d), dtype=np.float32)
    cache = cache_with(kind, kvh, d, [(keys[i], vals[i]) for i in range(n)])
    positions = [n - 1, max(n - 5, 0), n // 2]
    if kind.window() is not None:
        positions = [n - 1, n - 2]  # older positions have lost part of their window to the ring
    q = rng.standard_normal((len(positions), qh, d), dtype=np.float32)
    view = cache.view(0)
    first = view.position_at(0)
    stored = slice(first, n)
    got = gqa_attention(q, len(positions), qh, positions, view,
                        AttentionParams(softcap=softcap))
    want = naive_f64(q, keys[stored], vals[stored], positions, list(range(first, n)), qh,
                     1.0 / np.sqrt(d), kind.window(), softcap)
    assert np.max(np.abs(got - want)) < 2e-5


def test_equal_keys_average_and_single_key_copies_value():
    rng = np.random.default_rng(7)
    d, n = 8, 9
    k = rng.standard_normal(d).astype(np.float32)
    vals = rng.standard_normal((n, 1, d)).astype(np.float32)
    cache = cache_with(LayerKind.Global, 1, d, [(k, vals[i]) for i in range(n)])
    q = rng.standard_normal(d).astype(np.float32)
    out = gqa_attention(q, 1, 1, [n - 1], cache.view(0))
    assert np.allclose(out, vals[:, 0].mean(axis=0), atol=1e-6)
    out = gqa_attention(q, 1, 1, [0], cache.view(0))
    assert np.array_equal(out, vals[0, 0])  # weight exactly 1: bit-for-bit the value row


def test_softcap_formula_invariants_and_reference_kats():
    # torch-math/src/logits.rs:65-70 and muse-glimmer/src/model.rs:921-934.
    assert abs(oracle.logit_softcap(20.0, 20.0) - 15.231883119915298) < 1e-4
    assert abs(oracle.logit_softcap(10.0, 20.0) - 9.242343) < 1e-4
    assert oracle.logit_softcap(0.0, 20.0) == 0.0
    assert oracle.logit_softcap(5.0, 20.0) == -oracle.logit_softcap(-5.0, 20.0)
    assert abs(oracle.logit_softcap(1e9, 30.0)) <= 30.0
    # In attention: cap -> infinity recovers the uncapped result, and a finite cap changes it.
    rng = np.random.default_rng(3)
    n, d = 40, 16
    keys = rng.standard_normal((n, 1, d), dtype=np.float32) * 3
    vals = rng.standard_normal((n, 1, d), dtype=np.float32)
    cache = cache_with(LayerKind.Global, 1, d, [(keys[i], vals[i]) for i in range(n)])
    q = rng.standard_normal(d).astype(np.float32) * 3
    plain = gqa_attention(q, 1, 1, [n - 1], cache.view(0))
    huge = gqa_attention(q, 1, 1, [n - 1], cache.view(0), AttentionParams(softcap=1e9))
    capped = gqa_attention(q, 1, 1, [n - 1], cache.view(0), AttentionParams(softcap=1.0))
    assert np.max(np.abs(plain - huge)) < 1e-5
    assert np.max(np.abs(plain - capped)) > 1e-3


def test_f16_storage_is_f32_math_over_round_tripped_rows():
    rng = np.random.default_rng(11)
    n, kvh, d, qh = 33, 2, 16, 4
    keys = rng.standard_normal((n, kvh, d), dtype=np.float32)
    vals = rng.standard_normal((n, kvh, d), dtype=np.float32)
    a = cache_with(LayerKind.Global, kvh, d, [(keys[i], vals[i]) for i in range(n)], True)
    rk = keys.astype(np.float16).astype(np.float32)
    rv = vals.astype(np.float16).astype(np.float32)
    b = cache_with(LayerKind.Global, kvh, d, [(rk[i], rv[i]) for i in range(n)], False)
    q = rng.standard_normal((1, qh, d), dtype=np.float32)
    assert np.array_equal(gqa_attention(q, 1, qh, [n - 1], a.view(0)),
                          gqa_attention(q, 1, qh, [n - 1], b.view(0)))
    _, ka, va = a.view(0).rows()
    assert np.array_equal(ka, rk) and np.array_equal(va, rv)


def test_threads_do_not_change_results_and_step_equals_append_then_attend():
    rng = np.random.default_rng(5)
    kvh, d, qh, rows = 2, 8, 4, 6
    q = rng.standard_normal((rows, qh * d), dtype=np.float32)
    k = rng.standard_normal((rows, kvh * d), dtype=np.float32)
    v = rng.standard_normal((rows, kvh * d), dtype=np.float32)
    a = KvCache.new([LayerKind.Global], kvh, d)
    b = KvCache.new([LayerKind.Global], kvh, d)
    got = oracle.attention_step(a, 0, q, k, v, qh, 0, threads=4)
    want = []
    for i in range(rows):  # cpu.rs:592-646
        b.append(0, k[i], v[i], i)
        want.append(gqa_attention(q[i], 1, qh, [i], b.view(0)))
    assert np.array_equal(got, np.concatenate(want))
    # Block form with the causal mask is the same thing on a global layer.
    blk = gqa_attention(q, rows, qh, list(range(rows)), b.view(0), threads=3)
    assert np.array_equal(blk, got)
    with pytest.raises(oracle.AttentionError) as e:
        oracle.attention_step(a, 0, q, k, v, qh, 0)  # position 0 but the cache is at 6
    assert e.value.variant == "StepFailed"
