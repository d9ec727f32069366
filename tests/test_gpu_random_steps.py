"""Batched steps at randomly drawn shapes against the CPU oracle: element type, head_dim, KV heads,
group size (divisors of sixteen and not), number of slots, prefix lengths and row counts (single
rows, blocks of up to 64, chunks, long chunks) are drawn per seed, so that the planner's choices
(one or two column tiles, splits, deep ring, runs taken in reverse, fused appends) are met in
combinations the hand-written cases do not list. Global layers are checked on sampled rows at
their full context, windowed layers on every row; stored rows bit for bit in both.

Bars as everywhere: f16 KV 2e-3 max-abs, f32 KV 1e-5 relative. A failure names its seed."""
import numpy as np
import pytest
import torch

import oracle
from helpers import max_abs, normal, pkg

pytestmark = pytest.mark.gpu

THREADS = 8


def P():
    return pkg()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def shape_of(rng, seed):
    elem = "f16" if seed % 5 else "f32"
    d = int(rng.choice([64, 128] if elem == "f32" else [64, 96, 128, 128, 128, 256]))
    kvh = int(rng.choice([1, 2, 4, 8]))
    group = int(rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 12, 16]))
    return elem, d, kvh, kvh * group


def check_outputs(elem, got, want, what):
    err = max_abs(got, want)
    if elem == "f32":
        err /= max(1e-6, float(np.abs(want).max()))
    assert err <= (2e-3 if elem == "f16" else 1e-5), (*what, err)


def view_bytes(cache):
    pos, keys, vals = cache.view(0).rows()
    keys, vals = np.asarray(keys), np.asarray(vals)
    if keys.dtype == np.uint16:
        keys, vals = keys.view(np.float16).astype(np.float32), vals.view(np.float16).astype(np.float32)
    return (np.asarray(pos, dtype=np.int64).tobytes(), np.ascontiguousarray(keys).tobytes(),
            np.ascontiguousarray(vals).tobytes())


@pytest.mark.parametrize("seed", range(30))
def test_steps_on_a_global_layer_at_random_shapes(seed):
    rng = np.random.default_rng(seed)
    elem, d, kvh, q_heads = shape_of(rng, seed)
    slots = int(rng.choice([1, 1, 1, 2, 3, 5]))
    softcap = float(rng.choice([0.0, 0.0, 30.0]))
    long_prefix = 9000 if rng.random() < 0.3 else 3001
    prefixes = [int(rng.choice([0, rng.integers(1, 200), rng.integers(200, 3000),
                                rng.integers(3000, long_prefix)])) for _ in range(slots)]
    kinds = ["row", "block", "chunk", "long"] if slots == 1 else ["row", "row", "block", "chunk"]

    def draw():
        return {"row": 1, "block": int(rng.integers(2, 65)), "chunk": int(rng.integers(65, 400)),
                "long": int(rng.integers(400, 1700))}[str(rng.choice(kinds))]

    steps = [[draw() for _ in range(slots)] for _ in range(3)]
    row = kvh * d
    pool = P().KvPool([P().LayerKind.Global], kvh, d, elem=elem, max_slots=slots,
                      capacity_rows=max(prefixes) + sum(max(s) for s in steps) + 8)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    caches = [pool.acquire() for _ in range(slots)]
    refs = [oracle.KvCache.new([oracle.LayerKind.Global], kvh, d, store_f16=(elem == "f16")) for _ in range(slots)]
    for cache, ref, n in zip(caches, refs, prefixes):
        if n:
            k, v = normal(rng, n, row), normal(rng, n, row)
            kd, vd = dev(k), dev(v)
            pool.append_device(0, [(cache, n)], kd.data_ptr(), vd.data_ptr())
            torch.cuda.synchronize()
            ref.restore_bulk(0, 0, k, v)
    for rows in steps:
        total = sum(rows)
        q, k, v = normal(rng, total, q_heads * d), normal(rng, total, row), normal(rng, total, row)
        qd, kd, vd = dev(q), dev(k), dev(v)
        out = torch.empty_like(qd)
        pool.attention_step_device(0, list(zip(caches, rows)), qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                                   out.data_ptr(), q_heads, softcap=softcap)
        torch.cuda.synchronize()
        got, at = out.cpu().numpy(), 0
        for cache, ref, n in zip(caches, refs, rows):
            base = ref.next_position(0)
            for i in range(n):
                ref.append(0, k[at + i], v[at + i], base + i)
            # Causal attention of a row depends on nothing after it: sampled rows are evaluated
            # over the cache that already holds the whole step.
            pick = sorted({0, n - 1, n // 2, *rng.integers(0, n, size=min(n, 12)).tolist()})
            want = oracle.gqa_attention(q[at:at + n][pick], len(pick), q_heads, [base + i for i in pick],
                                        ref.view(0), oracle.AttentionParams(softcap=softcap),
                                        threads=THREADS).reshape(len(pick), -1)
            check_outputs(elem, got[at:at + n][pick], want, (seed, rows, n, base))
            _, gk, gv = cache.read_rows(0, base, n)
            if elem == "f16":
                assert np.array_equal(gk.reshape(n, row), oracle.f32_to_f16_array(k[at:at + n])), (seed, rows, n)
                assert np.array_equal(gv.reshape(n, row), oracle.f32_to_f16_array(v[at:at + n])), (seed, rows, n)
            else:
                assert np.array_equal(np.asarray(gk).reshape(n, row), k[at:at + n]), (seed, rows, n)
                assert np.array_equal(np.asarray(gv).reshape(n, row), v[at:at + n]), (seed, rows, n)
            at += n
    pool.close()


@pytest.mark.parametrize("seed", range(30))
def test_steps_on_a_windowed_layer_at_random_shapes(seed):
    rng = np.random.default_rng(seed + 7000)
    elem, d, kvh, q_heads = shape_of(rng, seed)
    window = int(rng.choice([rng.integers(2, 64), rng.integers(64, 400), rng.integers(400, 2100)]))
    headroom = int(rng.choice([64, 128, 256]))
    slots = int(rng.choice([1, 1, 2, 3]))
    softcap = float(rng.choice([0.0, 0.0, 30.0]))

    def draw():
        rows = {"row": 1, "block": int(rng.integers(2, 65)),
                "chunk": int(rng.integers(65, 257))}[str(rng.choice(["row", "row", "block", "chunk"]))]
        return min(headroom, rows)

    steps = [[draw() for _ in range(slots)] for _ in range(int(rng.integers(6, 14)))]
    row = kvh * d
    pool = P().KvPool([P().LayerKind.windowed(window)], kvh, d, elem=elem, max_slots=slots, capacity_rows=64,
                      ring_headroom=headroom)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    caches = [pool.acquire() for _ in range(slots)]
    refs = [oracle.KvCache.new([oracle.LayerKind.windowed(window)], kvh, d, store_f16=(elem == "f16"))
            for _ in range(slots)]
    for rows in steps:
        total = sum(rows)
        q, k, v = normal(rng, total, q_heads * d), normal(rng, total, row), normal(rng, total, row)
        qd, kd, vd = dev(q), dev(k), dev(v)
        out = torch.empty_like(qd)
        pool.attention_step_device(0, list(zip(caches, rows)), qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                                   out.data_ptr(), q_heads, softcap=softcap)
        torch.cuda.synchronize()
        got, at = out.cpu().numpy(), 0
        for cache, ref, n in zip(caches, refs, rows):
            base = ref.next_position(0)
            want = oracle.attention_step(ref, 0, q[at:at + n], k[at:at + n], v[at:at + n], q_heads, base,
                                         oracle.AttentionParams(softcap=softcap), threads=THREADS)
            check_outputs(elem, got[at:at + n].reshape(-1), want, (seed, rows, n, base))
            assert view_bytes(cache) == view_bytes(ref), (seed, rows, n, base)
            at += n
    pool.close()
