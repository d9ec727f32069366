"""Value rows that are not finite, in steps of several rows.

gqa_attention never reads the value row of a key a query does not see
(crates/attention/src/attention.rs:160-173): an infinity or a NaN in a value row reaches the
outputs of exactly the query rows that see the key. In a step of several rows those are not
all the rows: a later row of the same step is seen by the rows from it on, and on a
sliding-window layer a ring row inside the first row's window lies outside the last row's. The
matrix-pipe kernels multiply one shared value operand for all rows of a step, and a masked
key's zero weight times such a value is NaN. The split-K kernels (f16 pools at head_dim 128,
steps of up to 8 rows: decode batches and speculative blocks), the f32 kernel and the block
kernel (longer blocks and prefill chunks; every step at head dims 64, 96 and 256) take the
product row by row in the blocks where that can happen, and are compared with the oracle
element for element: the same elements NaN, the same elements infinite with the same sign, the
finite ones within the pool's bar (`exact=True`; `exact=False` is the weaker check a kernel
that keeps the shared product would be held to: rows that see the key not finite where the
oracle's are, everything finite within the bar)."""
import numpy as np
import pytest
import torch

import oracle
from helpers import normal, pkg

pytestmark = pytest.mark.gpu

Q_HEADS, KV_HEADS = 32, 4


def P():
    return pkg()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def same_elements(got, want, bar, what, exact=True):
    got, want = np.asarray(got, dtype=np.float32).reshape(-1), np.asarray(want, dtype=np.float32).reshape(-1)
    if exact:
        assert np.array_equal(np.isnan(got), np.isnan(want)), \
            (what, "NaN at", np.flatnonzero(np.isnan(got) != np.isnan(want))[:8])
        inf = np.isinf(want)
        assert np.array_equal(np.isinf(got), inf), (what, "inf at", np.flatnonzero(np.isinf(got) != inf)[:8])
        assert np.array_equal(np.sign(got[inf]), np.sign(want[inf])), what
    else:
        # The shared product: what the oracle has not finite is not finite, and what else is
        # not finite is NaN in a channel that some row of the step has not finite.
        assert not np.isfinite(got[~np.isfinite(want)]).any(), what
        stray = np.isfinite(want) & ~np.isfinite(got)
        width = got.size // ROWS_OF[what]
        bad_channels = (~np.isfinite(want)).reshape(-1, width).any(axis=0)
        assert np.isnan(got[stray]).all() and bad_channels[np.flatnonzero(stray) % width].all(), what
        want = np.where(stray, np.nan, want)
    fin = np.isfinite(want)
    assert fin.any() and (~fin).any(), what   # the case plants values that some rows see
    scale = 1.0 if bar == 2e-3 else float(np.max(np.abs(want[fin])))
    assert float(np.max(np.abs(got[fin] - want[fin]))) / scale <= bar, what


def run_step(elem, d, kind, ctx, rows, plant_new, plant_old, seed, chunk=40):
    """`ctx` cached rows, then one step of `rows` rows; `plant_*` write non-finite values into the
    new and the cached value rows. Returns (device output, oracle output)."""
    rng = np.random.default_rng(seed)
    width = KV_HEADS * d
    k, v = normal(rng, ctx + rows, width), normal(rng, ctx + rows, width)
    q = normal(rng, rows, Q_HEADS * d)
    plant_old(v[:ctx])
    plant_new(v[ctx:])
    okind = oracle.LayerKind.Global if kind is None else oracle.LayerKind.windowed(kind)
    pkind = P().LayerKind.Global if kind is None else P().LayerKind.windowed(kind)
    pool = P().KvPool([pkind], KV_HEADS, d, elem=elem, capacity_rows=ctx + rows + 8,
                      ring_headroom=max(64, rows))
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    kd, vd, qd = dev(k), dev(v), dev(q)
    for p0 in range(0, ctx, chunk):  # a ring takes no more than its headroom at a time
        n = min(chunk, ctx - p0)
        pool.append_device(0, [(cache, n)], kd[p0:].data_ptr(), vd[p0:].data_ptr())
    out = torch.empty_like(qd)
    pool.attention_step_device(0, [(cache, rows)], qd.data_ptr(), kd[ctx:].data_ptr(),
                               vd[ctx:].data_ptr(), out.data_ptr(), Q_HEADS)
    pool.synchronize()
    ref = oracle.KvCache.new([okind], KV_HEADS, d, store_f16=(elem == "f16"))
    first = 0 if kind is None else max(0, ctx - kind)
    ref.restore_bulk(0, first, k[first:ctx], v[first:ctx])
    want = oracle.attention_step(ref, 0, q, k[ctx:], v[ctx:], Q_HEADS, ctx, threads=8)
    pool.close()
    return out.cpu().numpy().reshape(rows, -1), want.reshape(rows, -1)


def nothing(_):
    pass


# (element type, head_dim, rows of the step, context, exact): the split-K kernels' three tile
# counts, the f32 kernel, then the block kernel's mid-size blocks and a head_dim it takes alone.
SHAPES = [("f16", 128, 2, 700, True), ("f16", 128, 4, 700, True), ("f16", 128, 7, 700, True),
          ("f16", 128, 8, 2100, True), ("f32", 128, 2, 700, True), ("f32", 128, 6, 700, True),
          ("f16", 128, 24, 700, True), ("f16", 128, 64, 700, True), ("f16", 64, 4, 700, True),
          ("f16", 128, 96, 700, True), ("f16", 128, 200, 300, True), ("f16", 64, 40, 700, True),
          ("f16", 96, 5, 700, True), ("f16", 96, 40, 700, True), ("f16", 96, 130, 300, True),
          ("f16", 256, 3, 700, True), ("f16", 64, 130, 300, True)]
ROWS_OF = {}


@pytest.mark.parametrize("elem,d,rows,ctx,exact", SHAPES)
def test_a_later_row_of_the_step_holds_values_that_are_not_finite(elem, d, rows, ctx, exact):
    def plant(v_new):
        v_new[rows - 1, 5] = np.inf                 # the last row: only its own queries see it
        v_new[rows // 2, d + 9] = -np.inf           # a middle row, another KV head
        v_new[rows // 2, 2 * d + 1] = np.nan
    got, want = run_step(elem, d, None, ctx, rows, plant, nothing, seed=rows)
    # What the reference does, spelled out: row 0 sees none of it.
    assert np.isfinite(want[0]).all()
    ROWS_OF[(elem, d, rows, ctx)] = rows
    same_elements(got, want, 2e-3 if elem == "f16" else 1e-5, (elem, d, rows, ctx), exact)


@pytest.mark.parametrize("elem,d,rows,exact", [("f16", 128, 4, True), ("f16", 128, 7, True), ("f32", 128, 4, True),
                                                ("f16", 128, 20, True), ("f16", 64, 4, True),
                                                ("f16", 128, 80, True), ("f16", 96, 6, True),
                                                ("f16", 96, 70, True)])
def test_a_ring_row_inside_the_first_rows_window_and_outside_the_lasts(elem, d, rows, exact):
    window, ctx = 96, 333
    def plant(v_old):
        v_old[ctx + 1 - window, 3] = np.inf         # the oldest position row 0 sees; row 1 does not
        v_old[ctx + 2 - window, d + 4] = np.nan     # rows 0 and 1 see it, row 2 does not
        v_old[ctx - window, 7] = -np.inf            # nobody sees it
    got, want = run_step(elem, d, window, ctx, rows, nothing, plant, seed=50 + rows, chunk=40)
    assert np.isfinite(want[rows - 1]).all() and not np.isfinite(want[0]).all()
    ROWS_OF[(elem, d, rows)] = rows
    same_elements(got, want, 2e-3 if elem == "f16" else 1e-5, (elem, d, rows), exact)


def test_finite_steps_are_untouched_by_the_exact_path():
    # The same shapes with nothing planted: the row-by-row products never run, and the outputs
    # meet the bar as before.
    for elem, d, rows, ctx, _ in SHAPES[:4]:
        rng = np.random.default_rng(1)
        got, want = run_step(elem, d, None, ctx, rows, nothing, nothing, seed=200 + rows)
        assert np.isfinite(got).all()
        assert float(np.max(np.abs(got - want))) <= 2e-3
