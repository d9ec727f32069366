"""Steps captured into a HIP graph and replayed: what a serving loop (and bench.py) does with the
step entry points. A step over several layers, followed by the truncate that takes its rows back,
is captured once; every replay must give what the same calls give eagerly, bit for bit (the same
kernels over the same plan), with the inputs it finds in the buffers at replay time, with eager
work of the same library and synchronisations between the replays, and the cache must be left as
an eager step leaves it. The eager result itself is held to the CPU oracle.

Covered: a decode row, a ragged decode batch, speculative blocks that append their own rows (the
split-K kernel's and the block kernel's forms), a chunk behind an append launch with split
contexts and a merge launch, f32 pools, and a windowed ring beside a global layer."""
import numpy as np
import pytest
import torch

import oracle
from helpers import max_abs, normal, pkg, rel_err

pytestmark = pytest.mark.gpu

THREADS = 8
Q_HEADS, KV_HEADS, D = 32, 4, 128
ROW = KV_HEADS * D


def P():
    return pkg()


def capture(pool, stream, fn):
    """One call of fn captured into a graph on a side stream (the pool launches on it meanwhile)."""
    side = torch.cuda.Stream()
    side.wait_stream(stream)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        pool.set_stream(side.cuda_stream)
        with torch.cuda.graph(graph, stream=side):
            fn()
    torch.cuda.synchronize()
    pool.set_stream(stream.cuda_stream)
    return graph


CASES = [
    # elem, windows per layer, contexts per slot, rows per slot
    ("f16", [None, None, None], [1000], 1),              # decode: split-K over the context, merge launch
    ("f16", [None, None], [3000, 37, 900], 1),           # ragged decode batch
    ("f16", [None, None], [2048, 2048], 7),              # verify blocks, rows appended by the split-K kernel
    ("f16", [None, None], [1500], 40),                   # a block the block kernel appends, stored by stage
    ("f16", [None, None], [600], 300),                   # a chunk: append launch, two tiles, splits, merge
    ("f16", [64, None], [500], 1),                       # a ring that has wrapped, beside a global layer
    ("f16", [100, None], [400], 24),                     # a block on the ring
    ("f32", [None, None], [1000], 1),                    # f32 pool: decode
    ("f32", [None, None], [700, 90], 5),                 # f32 pool: blocks in a batch
]


@pytest.mark.parametrize("elem,windows,contexts,rows", CASES)
def test_replays_of_a_captured_step_equal_the_eager_step(elem, windows, contexts, rows):
    K, OK = P().LayerKind, oracle.LayerKind
    kinds = [K.Global if w is None else K.windowed(w) for w in windows]
    okinds = [OK.Global if w is None else OK.windowed(w) for w in windows]
    layers, slots = len(windows), len(contexts)
    rng = np.random.default_rng(sum(contexts) + rows)
    stream = torch.cuda.current_stream()
    pool = P().KvPool(kinds, KV_HEADS, D, elem=elem, max_slots=slots, capacity_rows=max(contexts) + rows + 8,
                      ring_headroom=64)
    pool.set_stream(stream.cuda_stream)
    caches = [pool.acquire() for _ in range(slots)]
    # One single-layer oracle cache per slot and layer: each is stepped and rewound on its own.
    refs = [[oracle.KvCache.new([kind], KV_HEADS, D, store_f16=(elem == "f16")) for kind in okinds]
            for _ in range(slots)]
    for cache, ref, n in zip(caches, refs, contexts):
        for layer in range(layers):
            k, v = normal(rng, n, ROW), normal(rng, n, ROW)
            piece = n if windows[layer] is None else 50  # a ring takes what its headroom holds
            for first in range(0, n, piece):
                m = min(piece, n - first)
                kd, vd = torch.from_numpy(k[first:first + m]).cuda(), torch.from_numpy(v[first:first + m]).cuda()
                pool.append_device(layer, [(cache, m)], kd.data_ptr(), vd.data_ptr())
                pool.synchronize()
            if windows[layer] is None:
                ref[layer].restore_bulk(0, 0, k, v)
            else:
                for i in range(n):
                    ref[layer].append(0, k[i], v[i], i)
    total = slots * rows
    inputs = [tuple(normal(rng, layers * total, w).reshape(layers, total, w) for w in (Q_HEADS * D, ROW, ROW))
              for _ in range(2)]
    q, kn, vn = (torch.from_numpy(x).cuda() for x in inputs[0])
    out = torch.empty_like(q)
    items = [(c, rows) for c in caches]

    def step():
        for layer in range(layers):
            pool.attention_step_device(layer, items, q[layer].data_ptr(), kn[layer].data_ptr(),
                                       vn[layer].data_ptr(), out[layer].data_ptr(), Q_HEADS)
        pool.truncate(caches, contexts)

    def eager():
        out.fill_(float("nan"))
        step()
        torch.cuda.synchronize()
        return out.cpu().numpy().copy()

    want = [None, None]
    want[0] = eager()
    # The eager result against the oracle, which appends, attends and is rewound to the context.
    for layer in range(layers):
        for s, ref in enumerate(refs):
            rows_of = slice(s * rows, (s + 1) * rows)
            cp = ref[layer].checkpoint(rows)
            ref_want = oracle.attention_step(ref[layer], 0, inputs[0][0][layer][rows_of],
                                             inputs[0][1][layer][rows_of], inputs[0][2][layer][rows_of],
                                             Q_HEADS, contexts[s], threads=THREADS)
            got = want[0][layer][rows_of].reshape(-1)
            err = max_abs(got, ref_want) if elem == "f16" else rel_err(got, ref_want)
            assert err <= (2e-3 if elem == "f16" else 1e-5), (layer, s, err)
            ref[layer].rewind_to(cp, contexts[s])
            ref[layer].release(cp)

    graph = capture(pool, stream, step)
    # A second pool of the same library doing eager work between the replays.
    other = P().KvPool(1, KV_HEADS, D, elem="f16", capacity_rows=300)
    other.set_stream(stream.cuda_stream)
    oc = other.acquire()
    ok = torch.from_numpy(normal(rng, 200, ROW)).cuda()
    other.append_device(0, [(oc, 200)], ok.data_ptr(), ok.data_ptr())
    oq, oo = torch.from_numpy(normal(rng, 1, Q_HEADS * D)).cuda(), torch.empty(1, Q_HEADS * D, device="cuda")

    for replay in range(5):
        which = replay % 2
        # New contents in the captured buffers every other replay.
        for t, x in zip((q, kn, vn), inputs[which]):
            t.copy_(torch.from_numpy(x))
        if want[which] is None:
            want[which] = eager()
        out.fill_(float("nan"))
        other.attention_step_device(0, [(oc, 1)], oq.data_ptr(), ok.data_ptr(), ok.data_ptr(), oo.data_ptr(), Q_HEADS)
        other.truncate([oc], [200])
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        assert np.isfinite(got).all(), replay
        assert np.array_equal(got, want[which]), (replay, float(np.abs(got - want[which]).max()))
    # The cache after the replays is the cache after an eager step: the rows of the last replay
    # sit behind the context (dropped), every slot stands at its context, and a further eager
    # step matches the oracle.
    for cache, n in zip(caches, contexts):
        for layer in range(layers):
            assert cache.next_position(layer) == n
    q1, k1, v1 = normal(rng, slots, Q_HEADS * D), normal(rng, slots, ROW), normal(rng, slots, ROW)
    qd, kd, vd = (torch.from_numpy(x).cuda() for x in (q1, k1, v1))
    od = torch.empty_like(qd)
    pool.attention_step_device(0, [(c, 1) for c in caches], qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                               od.data_ptr(), Q_HEADS)
    pool.synchronize()
    last = od.cpu().numpy()
    for s, ref in enumerate(refs):
        ref_want = oracle.attention_step(ref[0], 0, q1[s:s + 1], k1[s:s + 1], v1[s:s + 1], Q_HEADS, contexts[s],
                                         threads=THREADS)
        err = max_abs(last[s], ref_want) if elem == "f16" else rel_err(last[s], ref_want)
        assert err <= (2e-3 if elem == "f16" else 1e-5), (s, err)
    other.close()
    pool.close()


@pytest.mark.parametrize("rows", [1, 20])
def test_replays_of_a_captured_prepared_step_equal_the_eager_step(rows):
    # The step with its norms, rotation and output gate (a preparation launch of its own from nine
    # rows on): captured, replayed with new inputs, compared with the eager call bit for bit. The
    # eager call itself is held to the oracle by the preparation's own tests.
    ctx, layers = 700, 2
    rng = np.random.default_rng(rows)
    stream = torch.cuda.current_stream()
    pool = P().KvPool(layers, KV_HEADS, D, elem="f16", capacity_rows=ctx + rows + 8)
    pool.set_stream(stream.cuda_stream)
    cache = pool.acquire()
    for layer in range(layers):
        kd = torch.from_numpy(normal(rng, ctx, ROW)).cuda()
        pool.append_device(layer, [(cache, ctx)], kd.data_ptr(), kd.data_ptr())
        pool.synchronize()
    qw, kw = (torch.from_numpy(1.0 + 0.1 * normal(rng, D)).cuda() for _ in range(2))
    inputs = [tuple(normal(rng, layers * rows, w).reshape(layers, rows, w)
                    for w in (Q_HEADS * D, ROW, ROW, Q_HEADS * D)) for _ in range(2)]
    q, kn, vn, gate = (torch.from_numpy(x).cuda() for x in inputs[0])
    out = torch.empty_like(q)

    def step():
        for layer in range(layers):
            pool.attention_prep_step_device(
                layer, [(cache, rows)], q[layer].data_ptr(), kn[layer].data_ptr(), vn[layer].data_ptr(),
                out[layer].data_ptr(), Q_HEADS, q_norm_ptr=qw.data_ptr(), k_norm_ptr=kw.data_ptr(), eps=1e-6,
                rope_base=1e6, interleaved=True, rotary_dim=0, gate_ptr=gate[layer].data_ptr())
        pool.truncate([cache], [ctx])

    def eager():
        out.fill_(float("nan"))
        step()
        torch.cuda.synchronize()
        return out.cpu().numpy().copy()

    want = [eager(), None]
    graph = capture(pool, stream, step)
    for replay in range(4):
        which = replay % 2
        for t, x in zip((q, kn, vn, gate), inputs[which]):
            t.copy_(torch.from_numpy(x))
        if want[which] is None:
            want[which] = eager()
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        assert np.isfinite(got).all(), replay
        assert np.array_equal(got, want[which]), (replay, float(np.abs(got - want[which]).max()))
    assert cache.next_position(0) == ctx
    pool.close()
