"""Values and keys that are not finite, planted at random in steps of randomly drawn shapes.

gqa_attention reads the key and value rows of the positions a query sees and of no others
(crates/attention/src/attention.rs:160-173), so what is not finite reaches exactly the rows that
see it: an infinite or NaN value the channels it stands in, a key whose score is NaN the whole
output row (the running maximum passes over a NaN, as the reference's comparison does, and the
weight and the sum are NaN). The kernels share operands among the rows of a step and among the
keys of a block, and clear or redo what a row must not see; here the shapes, the places and the
planted values are drawn per seed and the outputs are compared with the oracle element for
element: the same elements NaN, the same elements infinite with the same sign, the finite ones
within the pool's bar.

One limit is kept out of the draw: on f16 pools the softmax weights enter the matrix pipe as f16,
so a weight below about 2^-24 of the row's largest is zero there, and zero times an infinite
value is NaN where the reference has an infinity. Scores that far apart do not come from
N(0, 1) inputs; an infinite key under a softcap makes them (its capped score of +-cap stands 2 *
cap from the others), so with a softcap the planted keys are NaN only.

The seed lists hold the seeds that failed while the kernels were written (a wavefront or tile
holding one row of a step of several; a NaN score as the only one a wavefront sees in its
block) and some that never did. The pools say `q_two_halves=False`: as two halves an infinite
key channel scores NaN where one product scores an infinity (the flag's text in the header), and
the planted keys include infinities."""
import numpy as np
import pytest
import torch

import oracle
from helpers import normal, pkg

pytestmark = pytest.mark.gpu

NOT_FINITE = [np.inf, -np.inf, np.nan]


def P():
    return pkg()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def plant(rng, a, lo, hi, count, nan_only=False):
    for _ in range(count):
        if hi > lo:
            r, c, x = int(rng.integers(lo, hi)), int(rng.integers(0, a.shape[1])), NOT_FINITE[int(rng.integers(0, 3))]
            a[r, c] = np.nan if nan_only else x


def same_elements(elem, got, want, what):
    got, want = got.reshape(-1), want.reshape(-1)
    off = np.flatnonzero(np.isnan(got) != np.isnan(want))
    assert off.size == 0, (what, "NaN at", off[:6], "got", got[off[:6]], "want", want[off[:6]])
    inf = np.isinf(want)
    assert np.array_equal(np.isinf(got), inf), (what, "inf at", np.flatnonzero(np.isinf(got) != inf)[:6])
    assert np.array_equal(np.sign(got[inf]), np.sign(want[inf])), (what, "sign of an infinity")
    fin = np.isfinite(want)
    if fin.any():
        scale = 1.0 if elem == "f16" else max(1e-6, float(np.abs(want[fin]).max()))
        err = float(np.max(np.abs(got[fin] - want[fin]))) / scale
        assert err <= (2e-3 if elem == "f16" else 1e-5), (what, "error", err)


@pytest.mark.parametrize("seed", [6, 28, 34, 38, 50, 55, 58, 63, 116, 133, 143, 167, 194, 229, 249, 275,
                                  0, 1, 2, 3, 296, 297, 298, 299])
def test_one_step_with_values_planted_near_the_edges_of_its_rows_masks(seed):
    rng = np.random.default_rng(seed)
    elem = str(rng.choice(["f16", "f16", "f16", "f32"]))
    d = int(rng.choice([64, 128] if elem == "f32" else [64, 96, 128, 128, 256]))
    kvh = int(rng.choice([1, 2, 4]))
    group = int(rng.choice([1, 2, 4, 5, 8, 16]))
    rows = int(rng.choice([rng.integers(2, 9), rng.integers(9, 65), rng.integers(65, 300)]))
    window = None if rng.random() < 0.5 else int(rng.choice([rng.integers(4, 64), rng.integers(64, 400)]))
    ctx = int(rng.choice([rng.integers(1, 100), rng.integers(100, 1500)]))
    what = (seed, elem, d, kvh, group, rows, window, ctx)
    width, q_heads = kvh * d, kvh * group
    data = np.random.default_rng(seed)
    k, v = normal(data, ctx + rows, width), normal(data, ctx + rows, width)
    q = normal(data, rows, q_heads * d)
    # Cached rows within reach of the step's first and last windows, then the step's own rows.
    for _ in range(int(rng.integers(0, 4))):
        back = int(rng.integers(1, min(ctx, (window or ctx) + rows + 2) + 1))
        v[ctx - back, int(rng.integers(0, width))] = NOT_FINITE[int(rng.integers(0, 3))]
    plant(rng, v[ctx:], 0, rows, int(rng.integers(0, 4)))

    okind = oracle.LayerKind.Global if window is None else oracle.LayerKind.windowed(window)
    pkind = P().LayerKind.Global if window is None else P().LayerKind.windowed(window)
    pool = P().KvPool([pkind], kvh, d, elem=elem, capacity_rows=ctx + rows + 8, ring_headroom=max(64, rows),
                      q_two_halves=False)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    kd, vd, qd = dev(k), dev(v), dev(q)
    for p0 in range(0, ctx, 40):  # a ring takes no more than its headroom at a time
        pool.append_device(0, [(cache, min(40, ctx - p0))], kd[p0:].data_ptr(), vd[p0:].data_ptr())
    out = torch.empty_like(qd)
    pool.attention_step_device(0, [(cache, rows)], qd.data_ptr(), kd[ctx:].data_ptr(), vd[ctx:].data_ptr(),
                               out.data_ptr(), q_heads)
    pool.synchronize()
    ref = oracle.KvCache.new([okind], kvh, d, store_f16=(elem == "f16"))
    first = 0 if window is None else max(0, ctx - window)
    ref.restore_bulk(0, first, k[first:ctx], v[first:ctx])
    want = oracle.attention_step(ref, 0, q, k[ctx:], v[ctx:], q_heads, ctx, threads=8)
    pool.close()
    same_elements(elem, out.cpu().numpy(), want, what)


@pytest.mark.parametrize("seed,keys", [(248, False), (7, False), (19, False), (363, False), (367, False),
                                       (1005, True), (1015, True), (1016, True), (1024, True), (1034, True),
                                       (1067, True), (1081, True), (1112, True), (1117, True), (1208, True),
                                       (1230, True), (1001, True), (1002, True)])
def test_batched_steps_with_values_and_keys_planted(seed, keys):
    rng = np.random.default_rng(seed)
    elem = "f16" if seed % 4 else "f32"
    d = int(rng.choice([64, 128] if elem == "f32" else [64, 96, 128, 128, 128, 256]))
    kvh = int(rng.choice([1, 2, 4]))
    group = int(rng.choice([1, 2, 3, 4, 5, 8, 16]))
    q_heads = kvh * group
    slots = int(rng.choice([1, 1, 2, 3, 4]))
    softcap = float(rng.choice([0.0, 0.0, 30.0]))
    window = None if rng.random() < 0.5 else int(rng.choice([rng.integers(2, 64), rng.integers(64, 400),
                                                             rng.integers(400, 1200)]))
    headroom = int(rng.choice([64, 128, 256]))
    prefixes = [int(rng.choice([0, rng.integers(1, 200), rng.integers(200, 3000), rng.integers(3000, 12000)]))
                for _ in range(slots)]

    def draw():
        kind = str(rng.choice(["row", "block", "block", "mid", "chunk"]))
        n = {"row": 1, "block": int(rng.integers(2, 9)), "mid": int(rng.integers(9, 65)),
             "chunk": int(rng.integers(65, 300))}[kind]
        return min(n, headroom) if window is not None else n

    steps = [[draw() for _ in range(slots)] for _ in range(3)]
    row = kvh * d
    nan_keys = softcap > 0  # see the module's note on f16 weights
    okind = oracle.LayerKind.Global if window is None else oracle.LayerKind.windowed(window)
    pkind = P().LayerKind.Global if window is None else P().LayerKind.windowed(window)
    pool = P().KvPool([pkind], kvh, d, elem=elem, max_slots=slots, ring_headroom=headroom,
                      capacity_rows=max(prefixes) + sum(max(s) for s in steps) + 8, q_two_halves=False)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    caches = [pool.acquire() for _ in range(slots)]
    refs = [oracle.KvCache.new([okind], kvh, d, store_f16=(elem == "f16")) for _ in range(slots)]
    for cache, ref, n in zip(caches, refs, prefixes):
        if n:
            k, v = normal(rng, n, row), normal(rng, n, row)
            near = max(0, n - (window or n) - 40)
            plant(rng, v, near, n, int(rng.integers(0, 4)))
            if keys:
                plant(rng, k, near, n, int(rng.integers(0, 2)), nan_keys)
            first = 0 if window is None else max(0, n - window)
            kd, vd = dev(k[first:]), dev(v[first:])
            cache.restore_bulk_ptr(0, first, kd.data_ptr(), vd.data_ptr(), (n - first) * row, src_f16=False)
            torch.cuda.synchronize()
            ref.restore_bulk(0, first, k[first:], v[first:])
    for rows in steps:
        total = sum(rows)
        q, k, v = normal(rng, total, q_heads * d), normal(rng, total, row), normal(rng, total, row)
        plant(rng, v, 0, total, int(rng.integers(0, 4)))
        if keys:
            plant(rng, k, 0, total, int(rng.integers(0, 2)), nan_keys)
        qd, kd, vd = dev(q), dev(k), dev(v)
        out = torch.empty_like(qd)
        pool.attention_step_device(0, list(zip(caches, rows)), qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                                   out.data_ptr(), q_heads, softcap=softcap)
        torch.cuda.synchronize()
        got, at = out.cpu().numpy(), 0
        for ref, n in zip(refs, rows):
            base = ref.next_position(0)
            want = oracle.attention_step(ref, 0, q[at:at + n], k[at:at + n], v[at:at + n], q_heads, base,
                                         oracle.AttentionParams(softcap=softcap), threads=8)
            same_elements(elem, got[at:at + n], want, (seed, elem, d, kvh, group, window, rows, n, base))
            at += n
    pool.close()


@pytest.mark.parametrize("elem,d", [("f16", 128), ("f16", 64), ("f32", 128)])
def test_a_nan_key_that_is_the_only_key_a_row_sees_in_its_block(elem, d):
    # Six rows from position 190: row 2 stands at 192, the first position of a 32-key block, and
    # its own key is NaN. Whatever wavefront takes that block has nothing else to show for row
    # 2; rows 3 to 5 see the key beside finite ones. All four come out NaN in the key's KV head.
    kvh, group, ctx, rows = 2, 3, 190, 6
    q_heads, width = kvh * group, kvh * d
    rng = np.random.default_rng(5)
    k, v, q = normal(rng, ctx + rows, width), normal(rng, ctx + rows, width), normal(rng, rows, q_heads * d)
    k[ctx + 2, d + 49] = np.nan
    pool = P().KvPool([P().LayerKind.Global], kvh, d, elem=elem, capacity_rows=ctx + rows + 8, q_two_halves=False)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    kd, vd, qd = dev(k), dev(v), dev(q)
    pool.append_device(0, [(cache, ctx)], kd.data_ptr(), vd.data_ptr())
    out = torch.empty_like(qd)
    pool.attention_step_device(0, [(cache, rows)], qd.data_ptr(), kd[ctx:].data_ptr(), vd[ctx:].data_ptr(),
                               out.data_ptr(), q_heads)
    pool.synchronize()
    got = out.cpu().numpy().reshape(rows, q_heads, d)
    pool.close()
    assert np.isnan(got[2:, group:]).all()
    assert np.isfinite(got[:2]).all() and np.isfinite(got[:, :group]).all()
    ref = oracle.KvCache.new([oracle.LayerKind.Global], kvh, d, store_f16=(elem == "f16"))
    ref.restore_bulk(0, 0, k[:ctx], v[:ctx])
    want = oracle.attention_step(ref, 0, q, k[ctx:], v[ctx:], q_heads, ctx, threads=8)
    same_elements(elem, got, want, (elem, d))
