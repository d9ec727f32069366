"""The oracle's norm, RoPE and gate functions (the steps between the Q/K projections and
attention, and the gate after it), pinned by the reference's own known answers
(crates/torch-math/src/norm.rs:59-93, rope_interleaved.rs:122-200, rope.rs tests,
crates/cpu-compute/src/cpu.rs:867-881) and by closed forms."""
import math

import numpy as np

import oracle


def close(a, b, tol):
    return np.max(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64))) <= tol


def test_rms_norm_known_answers():
    ones = np.ones(4, np.float32)
    assert close(oracle.rms_norm([2, 2, 2, 2], ones, 1e-6), [1, 1, 1, 1], 1e-5)          # norm.rs:60-65
    assert close(oracle.rms_norm([1, 2, 3, 4], ones, 1e-5), [0.36515, 0.73030, 1.09545, 1.46061], 1e-4)
    assert close(oracle.rms_norm([2, 2, 2, 2], 2 * ones, 1e-6), [2, 2, 2, 2], 1e-5)      # norm.rs:76-80
    assert abs(oracle.rms_norm([2, 2, 2, 2], ones, 4.0)[0] - 1 / math.sqrt(2)) < 1e-6    # norm.rs:82-90
    # cpu.rs:867-881: per-head rows of width 2.
    inv = 1.0 / math.sqrt(12.5 + 1e-6)
    out = oracle.rms_norm([3, 4], [1, 1], 1e-6)
    assert abs(out[0] - 3 * inv) < 1e-6 and abs(out[1] - 4 * inv) < 1e-6
    assert abs(oracle.rms_norm([0, 2], [1, 1], 1e-6)[1] - 2 / math.sqrt(2 + 1e-6)) < 1e-6
    # Scale invariance (up to eps) and an independent float64 evaluation.
    rng = np.random.default_rng(0)
    x, w = rng.standard_normal(128).astype(np.float32), rng.standard_normal(128).astype(np.float32)
    want = (x.astype(np.float64) / np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-6) * w).astype(np.float32)
    assert np.array_equal(oracle.rms_norm(x, w, 1e-6), want)
    assert close(oracle.rms_norm(8 * x, w, 1e-12), oracle.rms_norm(x, w, 1e-12), 1e-5)


def test_rope_interleaved_known_rotations():
    # rope_interleaved.rs:126-147: adjacent pairing, rates 1 and 10000^(-1/2).
    out = oracle.rope_interleaved([1, 0, 1, 0], 1, 10_000.0)
    assert close(out, [0.5403023058681398, 0.8414709848078965, 0.9999500004166653,
                       0.009999833334166664], 1e-5)
    # The half-split form pairs (0, 2) and (1, 3): a different answer on the same input.
    assert not close(oracle.rope_half_split_partial([1, 0, 1, 0], 1, 10_000.0), out, 1e-2)
    x = np.array([1, 2, 3, 4], np.float32)
    assert np.array_equal(oracle.rope_interleaved(x, 0, 500_000.0), x)                   # :150-155
    turned = oracle.rope_interleaved(x, 7, 500_000.0)
    assert abs(float(np.sum(turned.astype(np.float64) ** 2)) - 30.0) < 0.01              # :156-160
    # Partial rotary (rope_interleaved.rs:163-190): the tail passes through.
    out = oracle.rope_interleaved([1, 0, 1, 0, 9, -4, 7, 3], 1, 10_000.0, rotary_dim=4)
    assert close(out, [0.5403023058681398, 0.8414709848078965, 0.9999500004166653,
                       0.009999833334166664, 9, -4, 7, 3], 1e-5)
    # Rotations compose: position a then b (as angles add) equals position a + b.
    rng = np.random.default_rng(1)
    y = rng.standard_normal(64).astype(np.float32)
    assert close(oracle.rope_interleaved(oracle.rope_interleaved(y, 5, 1e6), 9, 1e6),
                 oracle.rope_interleaved(y, 14, 1e6), 1e-5)


def test_rope_half_split_partial_agrees_with_the_full_form_and_passes_the_tail():
    rng = np.random.default_rng(2)
    y = rng.standard_normal(32).astype(np.float32)
    assert np.array_equal(oracle.rope_half_split_partial(y, 11, 1e4), oracle.rope_half_split(y, 11, 1e4))
    out = oracle.rope_half_split_partial(y, 11, 1e4, rotary_dim=8)
    assert np.array_equal(out[8:], y[8:]) and not np.array_equal(out[:8], y[:8])
    # Pair i joins channel i with channel i + rotary_dim/2 (rope.rs:104-114).
    e = np.zeros(8, np.float32); e[0] = 1
    out = oracle.rope_half_split_partial(e, 1, 10_000.0, rotary_dim=4)
    assert close(out, [math.cos(1), 0, math.sin(1), 0, 0, 0, 0, 0], 1e-6)


def test_sigmoid_and_gate():
    assert oracle.sigmoid(0.0) == 0.5
    for x in (0.3, 2.0, 17.0, 88.0, 200.0):
        assert abs(oracle.sigmoid(x) + oracle.sigmoid(-x) - 1.0) < 1e-6
        assert abs(oracle.sigmoid(x) - 1.0 / (1.0 + math.exp(-x))) < 1e-6
    assert oracle.sigmoid(-200.0) == 0.0 and oracle.sigmoid(200.0) == 1.0  # no overflow either way
    out = oracle.attn_gate([2.0, -4.0, 1.0], [0.0, 0.0, 100.0])
    assert np.array_equal(out, np.array([1.0, -2.0, 1.0], np.float32))


def test_attention_prep_composes_norm_then_rope_per_head():
    rng = np.random.default_rng(3)
    rows = rng.standard_normal((3, 2 * 8)).astype(np.float32)
    w = rng.standard_normal(8).astype(np.float32)
    out = oracle.attention_prep(rows, 2, 8, 40, w, 1e-6, 1e4, interleaved=True)
    for r in range(3):
        for h in range(2):
            want = oracle.rope_interleaved(oracle.rms_norm(rows[r, h * 8:(h + 1) * 8], w, 1e-6), 40 + r, 1e4)
            assert np.array_equal(out[r, h * 8:(h + 1) * 8], want)
    assert np.array_equal(oracle.attention_prep(rows, 2, 8, 40, None, 1e-6, 0.0), rows)
