"""Steps on f32 pools of head_dim 128 (the reference's own storage type) run on the f32 MFMA
kernel: decode rows, verify blocks and prefill chunks as tiles of 16 query vectors; other head
dims stay on the generic kernel. Both are held to the oracle within 1e-5 relative to the largest
output magnitude, the f32 bar."""
import numpy as np
import pytest
import torch

import oracle
from helpers import normal, pkg, rel_err

pytestmark = pytest.mark.gpu


def P():
    return pkg()


def run(ctxs, rows, q_heads, kv_heads, window=None, softcap=0.0, steps=3, seed=0, d=128):
    rng = np.random.default_rng(seed)
    width = kv_heads * d
    kind = P().LayerKind.Global if window is None else P().LayerKind.windowed(window)
    okind = oracle.LayerKind.Global if window is None else oracle.LayerKind.windowed(window)
    pool = P().KvPool([kind], kv_heads, d, elem="f32", max_slots=len(ctxs),
                      capacity_rows=max(ctxs) + steps * rows + 3)
    caches, refs = [], []
    for n0 in ctxs:
        cache = pool.acquire()
        ref = oracle.KvCache.new([okind], kv_heads, d)
        if n0:
            k0, v0 = normal(rng, n0, width), normal(rng, n0, width)
            first = 0 if window is None else max(0, n0 - window)
            cache.restore_bulk(0, first, k0[first:], v0[first:])
            ref.restore_bulk(0, first, k0[first:], v0[first:])
        caches.append(cache)
        refs.append(ref)
    for step in range(steps):
        total = rows * len(ctxs)
        q, k, v = normal(rng, total, q_heads * d), normal(rng, total, width), normal(rng, total, width)
        qd, kd, vd = (torch.from_numpy(x).cuda() for x in (q, k, v))
        out = torch.empty_like(qd)
        pool.attention_step_device(0, [(c, rows) for c in caches], qd.data_ptr(), kd.data_ptr(),
                                   vd.data_ptr(), out.data_ptr(), q_heads, softcap=softcap)
        pool.synchronize()
        got = out.cpu().numpy()
        for s, (cache, ref) in enumerate(zip(caches, refs)):
            part = slice(s * rows, (s + 1) * rows)
            want = oracle.attention_step(ref, 0, q[part], k[part], v[part], q_heads,
                                         ctxs[s] + step * rows,
                                         oracle.AttentionParams(softcap=softcap), threads=8)
            assert rel_err(got[part].reshape(-1), want) <= 1e-5, (step, s, ctxs[s])
            assert cache.next_position(0) == ref.next_position(0)
    # The rows the steps appended are the reference's rows, bit for bit.
    for cache, ref in zip(caches, refs):
        _, gk, gv = cache.view(0).rows()
        _, wk, wv = ref.view(0).rows()
        assert np.asarray(gk).tobytes() == np.asarray(wk).tobytes()
        assert np.asarray(gv).tobytes() == np.asarray(wv).tobytes()
    pool.close()


@pytest.mark.parametrize("ctx", [0, 1, 30, 31, 32, 33, 300, 4097])
def test_decode_at_every_block_edge(ctx):
    run([ctx], rows=1, q_heads=32, kv_heads=4, seed=ctx)


@pytest.mark.parametrize("q_heads,kv_heads,rows", [(4, 4, 1), (4, 4, 8), (8, 4, 3), (16, 2, 2),
                                                  (32, 4, 2), (16, 1, 1)])
def test_groups_and_short_blocks(q_heads, kv_heads, rows):
    run([200], rows=rows, q_heads=q_heads, kv_heads=kv_heads, seed=q_heads + rows)


def test_ragged_slots_in_one_launch():
    run([5, 1000, 64, 2300, 0], rows=1, q_heads=32, kv_heads=4, seed=3)
    run([700, 33], rows=2, q_heads=32, kv_heads=4, seed=4)


@pytest.mark.parametrize("ctx,window", [(50, 100), (500, 100), (500, 64), (3000, 1024)])
def test_sliding_window_layers_through_the_ring(ctx, window):
    run([ctx], rows=1, q_heads=32, kv_heads=4, window=window, steps=70, seed=ctx + window)


def test_softcap_and_a_block_of_rows_on_a_ring():
    run([900], rows=1, q_heads=32, kv_heads=4, softcap=20.0, seed=8)
    run([400, 90], rows=2, q_heads=32, kv_heads=4, window=128, steps=40, seed=9)


@pytest.mark.parametrize("ctxs,rows,q_heads,kv_heads,window,softcap", [
    ([300], 3, 32, 4, None, 0.0),            # 24 vectors: two tiles, the second half empty
    ([2100, 700, 0, 45], 8, 32, 4, None, 0.0),   # verify blocks, four slots
    ([1000], 64, 32, 4, None, 30.0),         # the reference's prefill chunk
    ([0], 300, 32, 4, None, 0.0),            # a prompt's first chunk: tiles see different runs of keys
    ([500], 200, 40, 8, None, 0.0),          # a group of five: tiles straddle rows
    ([900], 40, 16, 2, 256, 0.0),            # a block on a ring, the window inside the block's span
    ([3000, 100], 20, 12, 4, 1024, 0.0),
])
def test_blocks_of_any_length_run_as_tiles_of_sixteen_vectors(ctxs, rows, q_heads, kv_heads, window, softcap):
    run(ctxs, rows=rows, q_heads=q_heads, kv_heads=kv_heads, window=window, softcap=softcap, steps=2,
        seed=rows + len(ctxs))


@pytest.mark.parametrize("ctxs,rows,q_heads,kv_heads,window", [
    ([512], 1, 32, 4, None),                 # configs[0]: the reference's CPU-runnable case
    ([0, 31, 1000], 1, 8, 2, None), ([700], 2, 32, 4, None), ([300, 64], 8, 32, 4, None),
    ([0], 200, 16, 4, None), ([900], 1, 32, 4, 256), ([600], 30, 8, 8, 128)])
def test_head_dim_64_runs_on_the_same_kernel(ctxs, rows, q_heads, kv_heads, window):
    run(ctxs, rows=rows, q_heads=q_heads, kv_heads=kv_heads, window=window, steps=3, seed=rows + 64, d=64)


def test_other_head_dims_keep_the_generic_kernel():
    run([300], rows=1, q_heads=8, kv_heads=2, d=96, seed=11)
    run([300], rows=3, q_heads=4, kv_heads=2, d=256, seed=12)
