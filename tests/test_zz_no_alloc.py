"""itak_attention_step_device_noalloc: the step entry point that allocates nothing (its split
workspace is a static device array inside the library). It has no counterpart in the
reference; its contract is itak_attention_step_device's, so every call here is made twice,
through both entry points on twin pools, and compared: caches bit for bit, outputs to the f16
bar (2e-3 max-abs; the two run the same kernels, so they are in fact equal). Calls go through
the C ABI (ctypes table of the package)."""
import ctypes as C
import math

import numpy as np
import pytest
import torch

import oracle
from helpers import max_abs, normal, pkg

pytestmark = pytest.mark.gpu

Q_HEADS, KV_HEADS, D = 32, 4, 128
ROW = KV_HEADS * D


def P():
    return pkg()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def call(pool, name, layer, items, q, k, v, out):
    """One raw C-ABI call of either step entry point."""
    lib = P()._native.load()
    raw = (P()._native.BatchItem * len(items))()
    for i, (cache, rows) in enumerate(items):
        raw[i].slot, raw[i].rows = cache.slot, rows
    return getattr(lib, name)(pool._h, layer, raw, len(items), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                              out.data_ptr(), Q_HEADS, C.c_float(math.nan), C.c_float(0.0))


def twin_pools(slots, capacity, in_launch, elem="f16"):
    pools = []
    for _ in range(2):
        pool = P().KvPool(1, KV_HEADS, D, elem=elem, max_slots=slots, capacity_rows=capacity,
                          merge_in_launch=in_launch)
        pool.set_stream(torch.cuda.current_stream().cuda_stream)
        pools.append((pool, [pool.acquire() for _ in range(slots)]))
    return pools


def run_both(pools, contexts, rows, seed):
    """Fills every slot of both pools with the same rows, then makes the same step through
    itak_attention_step_device on the first pool and the allocation-free call on the second."""
    rng = np.random.default_rng(seed)
    slots = len(contexts)
    ks = [normal(rng, n + rows, ROW) for n in contexts]
    vs = [normal(rng, n + rows, ROW) for n in contexts]
    q = dev(normal(rng, slots * rows, Q_HEADS * D))
    k_new = dev(np.concatenate([ks[s][contexts[s]:] for s in range(slots)]))
    v_new = dev(np.concatenate([vs[s][contexts[s]:] for s in range(slots)]))
    outs = []
    for (pool, caches), name in zip(pools, ("itak_attention_step_device",
                                            "itak_attention_step_device_noalloc")):
        pool.truncate(caches[:slots], [0] * slots)
        for s in range(slots):
            kd, vd = dev(ks[s]), dev(vs[s])
            pool.append_device(0, [(caches[s], contexts[s])], kd.data_ptr(), vd.data_ptr())
            pool.synchronize()
        out = torch.full((slots * rows, Q_HEADS * D), float("nan"), device="cuda")
        st = call(pool, name, 0, [(caches[s], rows) for s in range(slots)], q, k_new, v_new, out)
        assert st == 0, P()._native.load().itak_last_error(pool._h)
        pool.synchronize()
        outs.append(out.cpu().numpy())
    got_ref, got = outs
    assert np.isfinite(got).all()
    assert max_abs(got, got_ref) <= 2e-3
    assert np.array_equal(got, got_ref)  # the same kernels over the same plan
    for s in range(slots):
        n = contexts[s] + rows
        a, b = pools[0][1][s].read_rows(0, 0, n), pools[1][1][s].read_rows(0, 0, n)
        assert np.array_equal(a[1], b[1]) and np.array_equal(a[2], b[2])
        assert np.array_equal(b[1].reshape(n, ROW), oracle.f32_to_f16_array(ks[s]))
    return got, ks, vs, q.cpu().numpy()


@pytest.mark.parametrize("in_launch", [False, True])
def test_two_calls_in_a_row_the_second_smaller(in_launch):
    pools = twin_pools(1, 4200, in_launch)
    got, ks, vs, q = run_both(pools, [4096], 1, seed=1)
    ref = oracle.KvCache.new([oracle.LayerKind.Global], KV_HEADS, D, store_f16=True)
    ref.restore_bulk(0, 0, ks[0][:4096], vs[0][:4096])
    want = oracle.attention_step(ref, 0, q, ks[0][4096:], vs[0][4096:], Q_HEADS, 4096, threads=8)
    assert max_abs(got.reshape(-1), want) <= 2e-3
    # The second call is smaller: fewer splits, so part of what the first left in the array is
    # not touched again.
    run_both(pools, [1000], 1, seed=2)
    run_both(pools, [200], 1, seed=3)
    for pool, _ in pools:
        pool.close()


@pytest.mark.parametrize("in_launch", [False, True])
def test_batches_and_speculative_blocks(in_launch):
    pools = twin_pools(4, 8300, in_launch)
    run_both(pools, [8192, 8192, 8192, 8192], 7, seed=4)   # the verify block of the benchmark
    run_both(pools, [3000, 257, 5000], 1, seed=5)          # a smaller, ragged decode batch
    run_both(pools, [600], 3, seed=6)
    for pool, _ in pools:
        pool.close()


def test_a_step_beyond_the_static_workspace_is_refused_before_anything_changes():
    # A 64-row block over 4096 positions splits into many workgroups of 128 query vectors each:
    # about 18 MB of partials, more than the static array's 8 MiB.
    ctx, rows = 4096, 64
    pool = P().KvPool(1, KV_HEADS, D, elem="f16", max_slots=1, capacity_rows=ctx + rows)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    zeros = torch.zeros(ctx, ROW, device="cuda")
    pool.append_device(0, [(cache, ctx)], zeros.data_ptr(), zeros.data_ptr())
    pool.synchronize()
    q = torch.zeros(rows, Q_HEADS * D, device="cuda")
    kv = torch.zeros(rows, ROW, device="cuda")
    out = torch.zeros_like(q)
    items = [(cache, rows)]
    st = call(pool, "itak_attention_step_device_noalloc", 0, items, q, kv, kv, out)
    assert st == 19  # ITAK_CAPACITY_EXCEEDED
    message = P()._native.load().itak_last_error(pool._h).decode()
    assert "allocation-free entry point holds" in message, message
    assert cache.next_position(0) == ctx  # nothing was appended
    # The allocating entry point takes the same step.
    assert call(pool, "itak_attention_step_device", 0, items, q, kv, kv, out) == 0
    pool.synchronize()
    assert cache.next_position(0) == ctx + rows
    # A long block needs no split workspace at all and goes through.
    rows2 = 2048
    pool2 = P().KvPool(1, KV_HEADS, D, elem="f16", max_slots=1, capacity_rows=ctx + rows2)
    pool2.set_stream(torch.cuda.current_stream().cuda_stream)
    cache2 = pool2.acquire()
    pool2.append_device(0, [(cache2, ctx)], zeros.data_ptr(), zeros.data_ptr())
    q2 = torch.zeros(rows2, Q_HEADS * D, device="cuda")
    kv2 = torch.zeros(rows2, ROW, device="cuda")
    out2 = torch.zeros_like(q2)
    assert call(pool2, "itak_attention_step_device_noalloc", 0, [(cache2, rows2)], q2, kv2, kv2, out2) == 0
    pool2.synchronize()
    assert cache2.next_position(0) == ctx + rows2
    pool.close()
    pool2.close()


def captured_on_first_use(pools, contexts, rows):
    """The callers the entry point is for: its very first call on a pool is made under stream
    capture (nothing before it has sized a workspace), the graph is replayed with new inputs
    in the captured buffers, and every replay equals the eager call of the allocating entry
    point on a twin pool, bit for bit."""
    rng = np.random.default_rng(8)
    stream = torch.cuda.current_stream()
    for pool, caches in pools:
        for s, n in enumerate(contexts):
            kd = dev(normal(np.random.default_rng(100 + s), n, ROW))
            pool.append_device(0, [(caches[s], n)], kd.data_ptr(), kd.data_ptr())
            pool.synchronize()
    inputs = [tuple(normal(rng, len(contexts) * rows, w) for w in (Q_HEADS * D, ROW, ROW)) for _ in range(2)]
    q, k, v = (dev(x) for x in inputs[0])
    out = torch.full((len(contexts) * rows, Q_HEADS * D), float("nan"), device="cuda")
    (eager_pool, eager_caches), (pool, caches) = pools
    items = [(c, rows) for c in caches]

    def step():
        assert call(pool, "itak_attention_step_device_noalloc", 0, items, q, k, v, out) == 0, \
            P()._native.load().itak_last_error(pool._h)
        pool.truncate(caches, contexts)

    side = torch.cuda.Stream()
    side.wait_stream(stream)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        pool.set_stream(side.cuda_stream)
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.synchronize()
    pool.set_stream(stream.cuda_stream)
    for replay in range(4):
        for t, x in zip((q, k, v), inputs[replay % 2]):
            t.copy_(torch.from_numpy(x))
        want = torch.full_like(out, float("nan"))
        assert call(eager_pool, "itak_attention_step_device", 0, [(c, rows) for c in eager_caches],
                    q, k, v, want) == 0
        eager_pool.truncate(eager_caches, contexts)
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.isfinite(out).all(), replay
        assert torch.equal(out, want), replay
    for p, _ in pools:
        p.close()


@pytest.mark.parametrize("in_launch", [False, True])
def test_the_call_is_captured_into_a_graph_on_its_first_use_and_replays(in_launch):
    captured_on_first_use(twin_pools(2, 2200, in_launch), [2048, 700], 3)


@pytest.mark.parametrize("elem,rows", [("f16", 16), ("f32", 1), ("f32", 3)])
def test_the_other_kernels_workspaces_are_captured_on_first_use_too(elem, rows):
    # A 16-row block goes to the block kernel with its context split (partials and a merge of
    # their own), an f32 pool to the f32 kernel: each sizes its workspace by its own plan, and
    # each must find the static array bound when the first call is the captured one.
    captured_on_first_use(twin_pools(2, 2200, False, elem), [2048, 700], rows)


def test_two_pools_on_two_streams_take_the_static_workspace_in_turn():
    # Every pool and stream of a device shares the one static array. Eager calls on different
    # streams are ordered by the library (each waits, on the device, for the array's last user);
    # without that the launches of the two streams overlap and one step's merge reads the
    # other's partials. Two pools with different batch shapes, each on a stream of its own,
    # call in turn with no host synchronisation in between; every output equals the allocating
    # entry point's on a twin pool, bit for bit.
    shapes = [([4096, 3000, 2500, 3900], 1), ([2048, 1800], 3)]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    rounds = 12
    rng = np.random.default_rng(31)
    sides = []
    for (contexts, rows), stream in zip(shapes, streams):
        slots = len(contexts)
        pools = []
        for _ in range(2):  # the allocating twin, then the allocation-free pool
            pool = P().KvPool(1, KV_HEADS, D, elem="f16", max_slots=slots, capacity_rows=max(contexts) + 16)
            pool.set_stream(stream.cuda_stream)
            pools.append((pool, [pool.acquire() for _ in range(slots)]))
        fill = [dev(normal(rng, n, ROW)) for n in contexts]
        inputs = [tuple(dev(normal(rng, slots * rows, w)) for w in (Q_HEADS * D, ROW, ROW))
                  for _ in range(rounds)]
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            for pool, caches in pools:
                for c, kd, n in zip(caches, fill, contexts):
                    pool.append_device(0, [(c, n)], kd.data_ptr(), kd.data_ptr())
        outs = [[torch.full((slots * rows, Q_HEADS * D), float("nan"), device="cuda")
                 for _ in range(rounds)] for _ in range(2)]
        sides.append((pools, contexts, rows, inputs, outs))
    torch.cuda.synchronize()
    for r in range(rounds):
        for pools, contexts, rows, inputs, outs in sides:
            q, k, v = inputs[r]
            for which, name in enumerate(("itak_attention_step_device", "itak_attention_step_device_noalloc")):
                pool, caches = pools[which]
                st = call(pool, name, 0, [(c, rows) for c in caches], q, k, v, outs[which][r])
                assert st == 0, P()._native.load().itak_last_error(pool._h)
                pool.truncate(caches, contexts)
    torch.cuda.synchronize()
    for pools, contexts, rows, inputs, outs in sides:
        for r in range(rounds):
            assert torch.isfinite(outs[1][r]).all(), r
            assert torch.equal(outs[0][r], outs[1][r]), r
        for pool, _ in pools:
            pool.close()
