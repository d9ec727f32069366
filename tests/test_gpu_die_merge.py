"""Split merges on the units' compute dies (ITAK_POOL_DIE_MERGE) against the merge launch (the
default) and against the oracle.

A batched step whose (sequence, KV head) units deal out evenly over the device's eight compute
dies places every split of a unit on one die; the last workgroup of a unit to finish merges the
unit's partials from that die's L2 (csrc/attn_splitk_f16_die.hip). The two plans cut the
context at other places, so the f16 roundings of the softmax weights differ between them as
they differ from the oracle's f32 weights: the forms agree to 2e-4 (observed: a few 1e-5, what
either is from the oracle), stored rows bit for bit, and both meet the oracle's bar (2e-3 max-abs on f16 KV, gqa_attention in
crates/attention/src/attention.rs:104-215). The library's diagnostic line names the form each
launch took, which is how the tests know that the form under test ran.

The form rests on the device dealing workgroup i of a launch to compute die i % 8. Every such
launch checks it, and itak_pool_synchronize reports a launch that was dealt otherwise
(ITAK_STEP_FAILED) instead of returning its outputs; that has been seen once in some thousand
launches, on a launch of 16 workgroups. A test that meets the report skips: the contract of the
opt-in form is results equal to the merge launch's, or that report."""
import re

import numpy as np
import pytest
import torch

import oracle
from helpers import max_abs, normal, pkg

pytestmark = pytest.mark.gpu

D = 128
FORMS_AGREE = 2e-4


def P():
    return pkg()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def merge_forms(capfd):
    """The merge= fields of the diagnostic lines printed since the last call."""
    return re.findall(r"merge=(\w+)", capfd.readouterr().err)


def synchronize_or_skip(pool):
    try:
        pool.synchronize()
    except P().StepFailed as e:
        if "another compute die" in str(e):
            pytest.skip(f"the device dealt a launch otherwise and the library said so: {e}")
        raise


class Twin:
    """Two pools fed alike: one merges on the dies, one keeps the merge launch."""

    def __init__(self, kinds, kv_heads, slots, capacity, lengths, rng, ring_headroom=0):
        self.kv_heads, self.width = kv_heads, kv_heads * D
        self.pools = [P().KvPool(kinds, kv_heads, D, elem="f16", max_slots=slots,
                                 capacity_rows=capacity, die_merge=form, ring_headroom=ring_headroom,
                                 q_two_halves=False)  # (the two forms exclude each other)
                      for form in (True, False)]
        self.caches = []
        self.k0 = [normal(rng, int(n), self.width) for n in lengths]
        self.v0 = [normal(rng, int(n), self.width) for n in lengths]
        for pool in self.pools:
            pool.set_stream(torch.cuda.current_stream().cuda_stream)
            caches = [pool.acquire() for _ in lengths]
            for layer in range(kinds if isinstance(kinds, int) else len(kinds)):
                window = None if isinstance(kinds, int) else kinds[layer].window_size
                for c, k, v in zip(caches, self.k0, self.v0):
                    if len(k) and window:  # what a prefill leaves in the ring: the last rows
                        first = max(0, len(k) - window)
                        c.restore_bulk(layer, first, k[first:], v[first:])
                    elif len(k):
                        kd, vd = dev(k), dev(v)
                        pool.append_device(layer, [(c, len(k))], kd.data_ptr(), vd.data_ptr())
                        torch.cuda.synchronize()
            self.caches.append(caches)

    def step(self, layer, rows, q, k, v, q_heads, capfd, softcap=0.0, order=None):
        """Runs the step on both pools; returns (on-die output, merge-launch output, forms)."""
        order = list(range(len(rows))) if order is None else order
        qd, kd, vd = dev(q), dev(k), dev(v)
        outs, forms = [], []
        for pool, caches in zip(self.pools, self.caches):
            out = torch.empty_like(qd)
            capfd.readouterr()
            P().set_debug_enabled(True)
            try:
                pool.attention_step_device(layer, [(caches[s], rows[i]) for i, s in enumerate(order)],
                                           qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), out.data_ptr(),
                                           q_heads, softcap=softcap)
                synchronize_or_skip(pool)
            finally:
                P().set_debug_enabled(False)
            forms.append(merge_forms(capfd))
            outs.append(out.cpu().numpy())
        return outs[0], outs[1], forms

    def close(self):
        for pool in self.pools:
            pool.close()


def oracle_rows(k0, v0, q, k, v, q_heads, kv_heads, kind=None, softcap=0.0):
    ref = oracle.KvCache.new([kind or oracle.LayerKind.Global], kv_heads, D, store_f16=True)
    window = None if kind is None else kind.window_size
    first = 0 if window is None else max(0, len(k0) - window)
    ref.restore_bulk(0, first, k0[first:], v0[first:])
    return oracle.attention_step(ref, 0, q, k, v, q_heads, len(k0),
                                 params=oracle.AttentionParams(softcap=softcap), threads=8)


def test_ragged_decode_batch_merges_on_the_dies(capfd):
    rng = np.random.default_rng(11)
    slots, kv_heads, q_heads = 16, 4, 32
    lengths = rng.integers(200, 5000, size=slots)
    lengths[0], lengths[1] = 4999, 200
    twin = Twin(1, kv_heads, slots, 5200, lengths, rng)
    for step in range(3):
        q = normal(rng, slots, q_heads * D)
        k, v = normal(rng, slots, twin.width), normal(rng, slots, twin.width)
        order = list(rng.permutation(slots))
        on_die, launch, forms = twin.step(0, [1] * slots, q, k, v, q_heads, capfd, order=order)
        assert forms == [["on_die"], ["launch"]], forms
        assert max_abs(on_die, launch) <= FORMS_AGREE
        for i, s in enumerate(order):
            if i % 4 == 0:
                want = oracle_rows(twin.k0[s], twin.v0[s], q[i:i + 1], k[i:i + 1], v[i:i + 1], q_heads, kv_heads)
                assert max_abs(on_die[i], want.reshape(-1)) <= 2e-3, (step, s)
            twin.k0[s] = np.concatenate([twin.k0[s], k[i:i + 1]])
            twin.v0[s] = np.concatenate([twin.v0[s], v[i:i + 1]])
    for a, b in zip(*twin.caches):
        assert a.read_raw(0)[0].tobytes() == b.read_raw(0)[0].tobytes()
        assert a.read_raw(0)[1].tobytes() == b.read_raw(0)[1].tobytes()
    twin.close()


@pytest.mark.parametrize("rows,softcap", [(4, 0.0), (4, 30.0), (3, 0.0), (2, 0.0), (7, 0.0)])
def test_speculative_blocks_merge_on_the_dies(capfd, rows, softcap):
    # 3 and 4 rows of 8 heads are a two-tile unit, 2 rows a one-tile unit; 7 rows are more than
    # 32 query vectors per KV head and keep the merge launch.
    rng = np.random.default_rng(100 + rows)
    slots, kv_heads, q_heads, ctx = 4, 4, 32, 2100
    lengths = [ctx, ctx + 17, ctx - 40, ctx + 3]
    twin = Twin(1, kv_heads, slots, ctx + 64, lengths, rng)
    q = normal(rng, slots * rows, q_heads * D)
    k, v = normal(rng, slots * rows, twin.width), normal(rng, slots * rows, twin.width)
    on_die, launch, forms = twin.step(0, [rows] * slots, q, k, v, q_heads, capfd, softcap=softcap)
    assert forms == [["launch" if rows == 7 else "on_die"], ["launch"]], forms
    assert max_abs(on_die, launch) <= FORMS_AGREE
    for s in range(slots):
        at = slice(s * rows, (s + 1) * rows)
        want = oracle_rows(twin.k0[s], twin.v0[s], q[at], k[at], v[at], q_heads, kv_heads, softcap=softcap)
        assert max_abs(on_die[at], want.reshape(rows, -1)) <= 2e-3, s
    for a, b in zip(*twin.caches):
        assert a.read_raw(0)[0].tobytes() == b.read_raw(0)[0].tobytes()
        assert a.read_raw(0)[1].tobytes() == b.read_raw(0)[1].tobytes()
    twin.close()


@pytest.mark.parametrize("kv_heads,slots", [(8, 1), (8, 3), (2, 4), (1, 8), (2, 9)])
def test_kv_head_counts_that_deal_out_over_eight_dies(capfd, kv_heads, slots):
    rng = np.random.default_rng(7 * kv_heads + slots)
    q_heads = kv_heads * 4
    lengths = [9000 + 31 * s for s in range(slots)]
    twin = Twin(1, kv_heads, slots, 9400, lengths, rng)
    q = normal(rng, slots, q_heads * D)
    k, v = normal(rng, slots, twin.width), normal(rng, slots, twin.width)
    on_die, launch, forms = twin.step(0, [1] * slots, q, k, v, q_heads, capfd)
    # 9 sequences over 4 groups of dies leave one group a third more than its share: the merge launch.
    assert forms == [["launch" if slots == 9 else "on_die"], ["launch"]], forms
    assert max_abs(on_die, launch) <= FORMS_AGREE
    want = oracle_rows(twin.k0[0], twin.v0[0], q[:1], k[:1], v[:1], q_heads, kv_heads)
    assert max_abs(on_die[0], want.reshape(-1)) <= 2e-3
    twin.close()


def test_batches_that_do_not_deal_out_keep_the_merge_launch(capfd):
    rng = np.random.default_rng(5)
    kv_heads, q_heads = 4, 32
    # Two sequences of very different length (one die group would carry thirty times the
    # other's work), then a single one (four units for eight dies).
    twin = Twin(1, kv_heads, 2, 9100, [300, 9000], rng)
    q = normal(rng, 2, q_heads * D)
    k, v = normal(rng, 2, twin.width), normal(rng, 2, twin.width)
    _, _, forms = twin.step(0, [1, 1], q, k, v, q_heads, capfd)
    assert forms == [["launch"], ["launch"]], forms
    _, _, forms = twin.step(0, [1], q[:1], k[:1], v[:1], q_heads, capfd, order=[1])
    assert forms == [["launch"], ["launch"]], forms
    twin.close()


def test_windowed_layers_merge_on_the_dies(capfd):
    rng = np.random.default_rng(9)
    slots, kv_heads, q_heads, window = 8, 4, 32, 4096
    kinds = [P().LayerKind.windowed(window)]
    lengths = [3500 + 1397 * s for s in range(slots)]  # inside the window up to several wraps
    twin = Twin(kinds, kv_heads, slots, 16384, lengths, rng, ring_headroom=64)
    for rows in (1, 4):
        q = normal(rng, slots * rows, q_heads * D)
        k, v = normal(rng, slots * rows, twin.width), normal(rng, slots * rows, twin.width)
        on_die, launch, forms = twin.step(0, [rows] * slots, q, k, v, q_heads, capfd)
        assert forms == [["on_die"], ["launch"]], forms
        assert max_abs(on_die, launch) <= FORMS_AGREE
        for s in (0, 3, 7):
            at = slice(s * rows, (s + 1) * rows)
            want = oracle_rows(twin.k0[s], twin.v0[s], q[at], k[at], v[at], q_heads, kv_heads,
                               kind=oracle.LayerKind.windowed(window))
            assert max_abs(on_die[at], want.reshape(rows, -1)) <= 2e-3, (rows, s)
        for s in range(slots):
            at = slice(s * rows, (s + 1) * rows)
            twin.k0[s] = np.concatenate([twin.k0[s], k[at]])
            twin.v0[s] = np.concatenate([twin.v0[s], v[at]])
    twin.close()


def test_tickets_are_left_clean_between_launches_of_different_shapes(capfd):
    # Launch after launch on one stream with no synchronisation in between, the batch shape
    # changing every time: each launch finds every ticket at zero or its merges would run early
    # or never.
    rng = np.random.default_rng(21)
    slots, kv_heads, q_heads = 16, 4, 32
    lengths = [1500 + 211 * s for s in range(slots)]
    twin = Twin(1, kv_heads, slots, 6000, lengths, rng)
    shapes = [(list(range(16)), 1), ([0, 5, 9, 12], 7), (list(range(8)), 2), (list(range(16)), 1),
              ([1, 2, 3, 4, 6, 7, 8, 10], 4), (list(range(16)), 3)]
    inputs = []
    for order, rows in shapes:
        n = len(order) * rows
        inputs.append((dev(normal(rng, n, q_heads * D)), dev(normal(rng, n, twin.width)),
                       dev(normal(rng, n, twin.width))))
    outs = []
    for pool, caches in zip(twin.pools, twin.caches):
        mine = []
        for (order, rows), (qd, kd, vd) in zip(shapes, inputs):
            out = torch.empty_like(qd)
            pool.attention_step_device(0, [(caches[s], rows) for s in order], qd.data_ptr(),
                                       kd.data_ptr(), vd.data_ptr(), out.data_ptr(), q_heads)
            mine.append(out)
        synchronize_or_skip(pool)
        outs.append([o.cpu().numpy() for o in mine])
    for a, b in zip(*outs):
        assert np.isfinite(a).all()
        assert max_abs(a, b) <= FORMS_AGREE
    twin.close()
