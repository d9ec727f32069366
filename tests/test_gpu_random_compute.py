"""Compute::attention (the host-pointer call of the drop-in boundary, cpu.rs:506-655) on randomly
drawn hybrid models: element type, head_dim, heads, the sliding window, the pattern of
sliding-window and global layers and the lengths of the calls (single rows, short blocks, prompts
longer than the window and than the device ring's headroom) are drawn per seed. After every
sequence the device cache holds, layer by layer, the rows the CPU oracle holds, bit for bit,
rotated keys of sliding-window layers included; outputs to the usual bars (f16 KV 2e-3 max-abs,
f32 KV 1e-5 relative). A failure names its seed."""
import numpy as np
import pytest

import oracle
from helpers import max_abs, normal, pkg, rel_err

pytestmark = pytest.mark.gpu

# (Among them the seeds on which keys rotated inside the attention launch, with the hardware's
# sine and cosine, once came out one f16 step from the oracle's; the call rotates by the
# preparation launch since.)
# 5253 and 5604: a rotated f32 key one and three units in the last place off while the kernel took
# the rotation frequencies from the device library's pow (a last bit that the position
# multiplies); they come from the host's now.
SEEDS = sorted({*range(24), 35, 44, 47, 100, 113, 146, 5253, 5604})


def P():
    return pkg()


def view_bytes(cache, layer):
    pos, keys, vals = cache.view(layer).rows()
    keys, vals = np.asarray(keys), np.asarray(vals)
    if keys.dtype == np.uint16:
        keys, vals = keys.view(np.float16).astype(np.float32), vals.view(np.float16).astype(np.float32)
    return (np.asarray(pos, dtype=np.int64).tobytes(), np.ascontiguousarray(keys).tobytes(),
            np.ascontiguousarray(vals).tobytes())


@pytest.mark.parametrize("seed", SEEDS)
def test_compute_attention_on_random_hybrid_models(seed):
    rng = np.random.default_rng(seed + 31337)
    elem = "f16" if seed % 3 else "f32"
    d = int(rng.choice([16, 64, 128] if elem == "f32" else [16, 64, 96, 128, 128, 256]))
    kvh = int(rng.choice([1, 2, 4]))
    group = int(rng.choice([1, 2, 3, 4, 8]))
    window = int(rng.choice([rng.integers(2, 30), rng.integers(30, 300)]))
    SW, G = P().LayerKind.SlidingWindow, P().LayerKind.Global
    layers = [SW if rng.random() < 0.6 else G for _ in range(int(rng.integers(1, 4)))]
    base = float(rng.choice([10000.0, 500000.0]))
    steps = [int(rng.choice([1, 1, rng.integers(2, 9), rng.integers(9, 70), rng.integers(70, 260)]))
             for _ in range(int(rng.integers(3, 8)))]
    cfg = P().GlimmerConfig(layers=layers, q_heads=kvh * group, kv_heads=kvh, key_length=d, value_length=d,
                            sliding_window=window, rope_freq_base_swa=base)
    ref = oracle.KvCache.new([oracle.LayerKind.windowed(window) if k is SW else oracle.LayerKind.Global
                              for k in layers], kvh, d, store_f16=(elem == "f16"))
    hc = P().HipCompute.new(elem=elem, capacity_rows=sum(steps) + 16)
    cache = P().PositionCache()
    for rows in steps:
        for layer, kind in enumerate(layers):
            q, k, v = normal(rng, rows, cfg.q_width()), normal(rng, rows, cfg.k_width()), normal(rng, rows, cfg.v_width())
            got = hc.attention(P().AttentionRequest(q, k, v, layer, kind, cfg), cache)
            want = oracle.compute_attention(ref, layer, q, k, v, cfg.q_heads, cache.position(), base, threads=8)
            err = rel_err(got, want) if elem == "f32" else max_abs(got, want)
            assert err <= (1e-5 if elem == "f32" else 2e-3), (seed, rows, layer, err)
        cache.advance(rows)
    dev = hc.kv_cache()
    for layer in range(len(layers)):
        assert dev.next_position(layer) == ref.next_position(layer) == sum(steps)
        assert view_bytes(dev, layer) == view_bytes(ref, layer), (seed, layer)
