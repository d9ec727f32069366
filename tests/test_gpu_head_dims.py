"""f16 pools at head_dim 64, 96 and 256 run on the block kernel (head_dim is a template argument of
it): decode steps, speculative blocks that append their own rows, prefill chunks, windowed rings
and ragged batches, against the CPU oracle evaluated over the same f16-rounded cache.

Bars as everywhere: outputs within 2e-3 max-abs, stored rows bit-exact."""
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


def make(kinds, okinds, kv_heads, d, slots, capacity, **kw):
    pool = P().KvPool(kinds, kv_heads, d, elem="f16", max_slots=slots, capacity_rows=capacity, **kw)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    caches = [pool.acquire() for _ in range(slots)]
    refs = [oracle.KvCache.new(okinds, kv_heads, d, store_f16=True) for _ in range(slots)]
    return pool, caches, refs


def step(pool, caches, refs, rng, rows, q_heads, softcap=0.0, layer=0):
    """One batched step: `rows[i]` new rows for slot i (0 = the slot sits this step out)."""
    kvh, d = pool.num_kv_heads, pool.head_dim
    total = sum(rows)
    q, k, v = normal(rng, total, q_heads * d), normal(rng, total, kvh * d), normal(rng, total, kvh * d)
    qd, kd, vd = dev(q), dev(k), dev(v)
    out = torch.empty_like(qd)
    items = [(c, r) for c, r in zip(caches, rows) if r]
    pool.attention_step_device(layer, items, qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                               out.data_ptr(), q_heads, softcap=softcap)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    at = 0
    for ref, r in zip(refs, rows):
        if not r:
            continue
        base = ref.next_position(layer)
        want = oracle.attention_step(ref, layer, q[at:at + r], k[at:at + r], v[at:at + r], q_heads, base,
                                     oracle.AttentionParams(softcap=softcap), threads=THREADS)
        err = max_abs(got[at:at + r].reshape(-1), want)
        assert err <= 2e-3, (rows, base, r, err)
        at += r


@pytest.mark.parametrize("d,q_heads,kv_heads", [(64, 32, 4), (64, 8, 8), (64, 24, 8), (256, 16, 4), (256, 8, 1),
                                                  (96, 32, 32), (96, 32, 8), (96, 12, 4)])
@pytest.mark.parametrize("softcap", [0.0, 30.0])
def test_decode_steps_blocks_and_chunks(d, q_heads, kv_heads, softcap):
    G = P().LayerKind.Global
    rng = np.random.default_rng(d + q_heads)
    pool, caches, refs = make([G], [oracle.LayerKind.Global], kv_heads, d, 1, 1400)
    cache, ref = caches[0], refs[0]
    row = kv_heads * d
    # A prompt's first chunk (no prefix), then decode rows, blocks that append their own rows
    # (up to 64 at head_dim 64 and 96, up to 16 at 256), blocks behind the append launch, a second
    # chunk.
    kept = []
    for rows in (300, 1, 1, 7, 16, 1, 17, 40, 64, 65, 1, 330, 1, 3):
        base = ref.next_position(0)
        kvh = pool.num_kv_heads
        q, k, v = normal(rng, rows, q_heads * d), normal(rng, rows, row), normal(rng, rows, row)
        kept.append((base, k, v))
        qd, kd, vd = dev(q), dev(k), dev(v)
        out = torch.empty_like(qd)
        pool.attention_step_device(0, [(cache, rows)], qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                                   out.data_ptr(), q_heads, softcap=softcap)
        torch.cuda.synchronize()
        want = oracle.attention_step(ref, 0, q, k, v, q_heads, base,
                                     oracle.AttentionParams(softcap=softcap), threads=THREADS)
        err = max_abs(out.cpu().numpy().reshape(-1), want)
        assert err <= 2e-3, (rows, base, err)
        assert cache.next_position(0) == base + rows and kvh == kv_heads
    # What the steps stored is what the append kernel stores: the rounded rows, bit for bit.
    for base, k, v in kept:
        _, gk, gv = cache.read_rows(0, base, len(k))
        assert np.array_equal(gk.reshape(len(k), row), oracle.f32_to_f16_array(k)), base
        assert np.array_equal(gv.reshape(len(v), row), oracle.f32_to_f16_array(v)), base
    pool.close()


@pytest.mark.parametrize("d,q_heads,kv_heads", [(64, 32, 4), (256, 8, 2), (96, 16, 4)])
def test_ragged_batches_split_their_contexts(d, q_heads, kv_heads):
    # Slots of very different lengths in one launch, long enough that the planner splits the
    # context (the merge of head dims other than 128 is the general merge kernel), a slot that
    # starts empty, steps that mix decode rows with a block and a chunk.
    G = P().LayerKind.Global
    rng = np.random.default_rng(d)
    pool, caches, refs = make([G], [oracle.LayerKind.Global], kv_heads, d, 4, 5200)
    row = kv_heads * d
    for cache, ref, n in zip(caches, refs, (5000, 37, 0, 1900)):
        if n:
            k, v = normal(rng, n, row), normal(rng, n, row)
            kd, vd = dev(k), dev(v)
            pool.append_device(0, [(cache, n)], kd.data_ptr(), vd.data_ptr())
            torch.cuda.synchronize()
            ref.restore_bulk(0, 0, k, v)
    for rows in ([1, 1, 1, 1], [1, 1, 1, 1], [7, 7, 7, 7], [1, 0, 5, 1], [1, 1, 100, 9], [16, 1, 1, 70]):
        step(pool, caches, refs, rng, rows, q_heads)
    pool.close()


@pytest.mark.parametrize("d,q_heads,kv_heads,window", [(64, 32, 4, 256), (64, 8, 2, 100), (256, 8, 2, 128),
                                                         (96, 8, 2, 100)])
@pytest.mark.parametrize("softcap", [0.0, 30.0])
def test_windowed_layers_beside_global_ones(d, q_heads, kv_heads, window, softcap):
    # A windowed ring and a global layer in one pool; the ring wraps several times, by single
    # rows, blocks and chunks (within the ring's headroom).
    K, OK = P().LayerKind, oracle.LayerKind
    rng = np.random.default_rng(window + d)
    pool, caches, refs = make([K.windowed(window), K.Global], [OK.windowed(window), OK.Global],
                              kv_heads, d, 1, 1300, ring_headroom=160)
    for rows in (90, 1, 1, 33, 150, 1, 7, 16, 1, 64, 128, 1, 160, 1, 1, 12):
        for layer in (0, 1):
            step(pool, caches, refs, rng, [rows], q_heads, softcap=softcap, layer=layer)
    pool.close()


def test_head_dim_64_rewinds_a_speculative_round():
    # Verify, reject, re-append: the cache after truncate-then-reappend equals never having
    # appended (raw bytes), at a head_dim the block kernel appends for.
    d, q_heads, kv_heads = 64, 32, 4
    G = P().LayerKind.Global
    rng = np.random.default_rng(5)
    pool, caches, refs = make([G], [oracle.LayerKind.Global], kv_heads, d, 2, 700)
    step(pool, caches, refs, rng, [500, 411], q_heads)
    for keep in ((3, 0), (7, 1), (0, 6)):
        before = [r.next_position(0) for r in refs]
        cps = [r.checkpoint(7) for r in refs]
        step(pool, caches, refs, rng, [7, 7], q_heads)
        pool.truncate(caches, [b + k for b, k in zip(before, keep)])
        for r, cp, b, k in zip(refs, cps, before, keep):
            r.rewind_to(cp, b + k)
            r.release(cp)
        step(pool, caches, refs, rng, [1, 1], q_heads)
    pool.close()


@pytest.mark.parametrize("elem,d,q_heads,kv_heads,rows,ctx,window", [
    ("f16", 64, 32, 4, 1, 3000, None),     # splits merged by the general merge kernel, which applies the gate
    ("f16", 64, 32, 4, 1, 20, None),       # one split: the gate is a launch of its own
    ("f16", 64, 8, 2, 7, 500, 128),        # a block on a ring
    ("f16", 64, 32, 4, 150, 200, None),    # a chunk behind the append launch
    ("f16", 256, 16, 4, 1, 2500, None),
    ("f16", 256, 8, 2, 12, 300, None),
    ("f16", 96, 32, 8, 1, 3000, None),
    ("f16", 96, 8, 8, 9, 300, 128),
    ("f32", 64, 32, 4, 1, 2500, None),     # the f32 matrix-pipe kernel at head_dim 64
    ("f32", 64, 32, 4, 40, 600, None),
])
def test_norms_rotation_and_gate_around_the_step(elem, d, q_heads, kv_heads, rows, ctx, window):
    # The fused preparation (RMS norms, rotation, append) and the output gate at the head dims
    # whose steps run on the block kernel or the f32 kernel: the preparation is a launch of its
    # own there, the gate is applied by whichever kernel writes the output.
    from test_gpu_prep import run_case
    run_case(elem, q_heads, kv_heads, d, ctx=ctx, rows=rows, norm=True, rope_base=1e6, interleaved=True,
             rotary=0, gate=True, seed=ctx + rows, window=window)
    # (Normed in both: the case's raw Q and K are drawn at three and two times unit scale, past
    # what f16 operands hold to 2e-3 without the norm.)
    run_case(elem, q_heads, kv_heads, d, ctx=ctx, rows=rows, norm=True, rope_base=1e4, interleaved=False,
             rotary=d // 2, gate=True, seed=ctx + rows + 1, window=window)
