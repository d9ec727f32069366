"""The split merge done inside the attention launch (ITAK_POOL_MERGE_IN_LAUNCH): decode steps
and speculative blocks of f16 pools whose workgroups exchange their partials through a buffer
instead of leaving them to a merge launch. Same bars as the default form: caches bit-exact,
outputs within 2e-3 max-abs of the oracle over the same f16-rounded cache; and the two forms
agree with each other far inside that bar."""
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


def pool_of(pattern, slots, capacity, in_launch, kv_heads=KV_HEADS):
    pool = P().KvPool(pattern, kv_heads, D, elem="f16", max_slots=slots, capacity_rows=capacity,
                      merge_in_launch=in_launch)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    return pool


def step(pool, cache, layer, k, v, q, rows, q_heads=Q_HEADS, softcap=0.0):
    """Fills the cache with all but the last `rows` rows, then steps the last rows."""
    ctx = k.shape[0] - rows
    kd, vd, qd = dev(k), dev(v), dev(q)
    out = torch.empty_like(qd)
    pool.append_device(layer, [(cache, ctx)], kd.data_ptr(), vd.data_ptr())
    pool.attention_step_device(layer, [(cache, rows)], qd.data_ptr(), kd[ctx:].data_ptr(),
                               vd[ctx:].data_ptr(), out.data_ptr(), q_heads, softcap=softcap)
    pool.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("ctx", [31, 129, 1000, 4096, 7777, 16384])
@pytest.mark.parametrize("softcap", [0.0, 30.0])
def test_decode_step_merged_in_launch_matches_oracle_and_default_form(ctx, softcap):
    rng = np.random.default_rng(ctx)
    k, v = normal(rng, ctx + 1, ROW), normal(rng, ctx + 1, ROW)
    q = normal(rng, 1, Q_HEADS * D)
    outs = []
    for in_launch in (True, False):
        pool = pool_of(1, 1, ctx + 1, in_launch)
        cache = pool.acquire()
        outs.append(step(pool, cache, 0, k, v, q, 1, softcap=softcap))
        _, gk, gv = cache.read_rows(0, 0, ctx + 1)
        assert np.array_equal(gk.reshape(ctx + 1, ROW), oracle.f32_to_f16_array(k))
        assert np.array_equal(gv.reshape(ctx + 1, ROW), oracle.f32_to_f16_array(v))
        pool.close()
    ref = oracle.KvCache.new([oracle.LayerKind.Global], KV_HEADS, D, store_f16=True)
    ref.restore_bulk(0, 0, k[:ctx], v[:ctx])
    want = oracle.attention_step(ref, 0, q, k[ctx:], v[ctx:], Q_HEADS, ctx,
                                 oracle.AttentionParams(softcap=softcap), threads=8)
    assert max_abs(outs[0].reshape(-1), want) <= 2e-3
    assert max_abs(outs[0], outs[1]) <= 1e-4  # different kernels round Q and P at different points


@pytest.mark.parametrize("group", [1, 2, 4, 16])
def test_other_group_sizes(group):
    ctx, kv_heads = 2500, 2
    q_heads = kv_heads * group
    rng = np.random.default_rng(group)
    k, v = normal(rng, ctx + 1, kv_heads * D), normal(rng, ctx + 1, kv_heads * D)
    q = normal(rng, 1, q_heads * D)
    pool = pool_of(1, 1, ctx + 1, True, kv_heads=kv_heads)
    cache = pool.acquire()
    got = step(pool, cache, 0, k, v, q, 1, q_heads=q_heads)
    pool.close()
    ref = oracle.KvCache.new([oracle.LayerKind.Global], kv_heads, D, store_f16=True)
    ref.restore_bulk(0, 0, k[:ctx], v[:ctx])
    want = oracle.attention_step(ref, 0, q, k[ctx:], v[ctx:], q_heads, ctx, threads=8)
    assert max_abs(got.reshape(-1), want) <= 2e-3


def test_many_steps_reuse_the_exchange_buffer():
    # Forty consecutive decode steps of two slots: every step finds the buffer as the last left it.
    slots, ctx0, steps = 2, 3000, 40
    rng = np.random.default_rng(7)
    pool = pool_of(1, slots, ctx0 + 37 * slots + steps + 1, True)
    caches = [pool.acquire() for _ in range(slots)]
    refs = []
    for s in range(slots):
        n = ctx0 + 37 * s
        k, v = normal(rng, n, ROW), normal(rng, n, ROW)
        kd, vd = dev(k), dev(v)
        pool.append_device(0, [(caches[s], n)], kd.data_ptr(), vd.data_ptr())
        pool.synchronize()
        ref = oracle.KvCache.new([oracle.LayerKind.Global], KV_HEADS, D, store_f16=True)
        ref.restore_bulk(0, 0, k, v)
        refs.append(ref)
    for t in range(steps):
        q = normal(rng, slots, Q_HEADS * D)
        k, v = normal(rng, slots, ROW), normal(rng, slots, ROW)
        qd, kd, vd = dev(q), dev(k), dev(v)
        out = torch.empty_like(qd)
        pool.attention_step_device(0, [(c, 1) for c in caches], qd.data_ptr(), kd.data_ptr(),
                                   vd.data_ptr(), out.data_ptr(), Q_HEADS)
        pool.synchronize()
        got = out.cpu().numpy()
        for s in range(slots):
            pos = refs[s].next_position(0)
            want = oracle.attention_step(refs[s], 0, q[s:s + 1], k[s:s + 1], v[s:s + 1], Q_HEADS, pos,
                                         threads=8)
            assert max_abs(got[s], want) <= 2e-3, (t, s)
    pool.close()


def test_windowed_layer_decode():
    window, ctx = 512, 3000
    rng = np.random.default_rng(11)
    k, v = normal(rng, ctx + 1, ROW), normal(rng, ctx + 1, ROW)
    q = normal(rng, 1, Q_HEADS * D)
    pool = pool_of([P().LayerKind.windowed(window)], 1, ctx + 8, True)
    cache = pool.acquire()
    first = ctx - window
    cache.restore_bulk(0, first, k[first:ctx], v[first:ctx])
    qd, kd, vd = dev(q), dev(k[ctx:]), dev(v[ctx:])
    out = torch.empty_like(qd)
    pool.attention_step_device(0, [(cache, 1)], qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                               out.data_ptr(), Q_HEADS)
    pool.synchronize()
    ref = oracle.KvCache.new([oracle.LayerKind.windowed(window)], KV_HEADS, D, store_f16=True)
    ref.restore_bulk(0, first, k[first:ctx], v[first:ctx])
    want = oracle.attention_step(ref, 0, q, k[ctx:], v[ctx:], Q_HEADS, ctx, threads=8)
    assert max_abs(out.cpu().numpy().reshape(-1), want) <= 2e-3
    pool.close()


def test_speculative_block_merged_in_launch():
    # Seven rows per slot: the general split-K kernel's exchange (64 query vectors per KV head).
    slots, ctx, rows = 2, 2048, 7
    rng = np.random.default_rng(13)
    pool = pool_of(1, slots, ctx + rows, True)
    caches = [pool.acquire() for _ in range(slots)]
    ks = [normal(rng, ctx + rows, ROW) for _ in range(slots)]
    vs = [normal(rng, ctx + rows, ROW) for _ in range(slots)]
    q = normal(rng, slots * rows, Q_HEADS * D)
    for s in range(slots):
        kd, vd = dev(ks[s]), dev(vs[s])
        pool.append_device(0, [(caches[s], ctx)], kd.data_ptr(), vd.data_ptr())
        pool.synchronize()
    kd = dev(np.concatenate([ks[s][ctx:] for s in range(slots)]))
    vd = dev(np.concatenate([vs[s][ctx:] for s in range(slots)]))
    qd = dev(q)
    out = torch.empty_like(qd)
    pool.attention_step_device(0, [(c, rows) for c in caches], qd.data_ptr(), kd.data_ptr(),
                               vd.data_ptr(), out.data_ptr(), Q_HEADS)
    pool.synchronize()
    got = out.cpu().numpy()
    for s in range(slots):
        ref = oracle.KvCache.new([oracle.LayerKind.Global], KV_HEADS, D, store_f16=True)
        ref.restore_bulk(0, 0, ks[s][:ctx], vs[s][:ctx])
        want = oracle.attention_step(ref, 0, q[s * rows:(s + 1) * rows], ks[s][ctx:], vs[s][ctx:],
                                     Q_HEADS, ctx, threads=8)
        assert max_abs(got[s * rows:(s + 1) * rows].reshape(-1), want) <= 2e-3
    pool.close()


def test_a_wait_that_runs_out_is_reported_and_the_pool_recovers():
    # With a spin limit of 0 every consumer looks once: whether the partials were there in time
    # is up to the machine, so either outcome is accepted, but a give-up must surface at the
    # next synchronize as StepFailed, and the step after it must be right again.
    ctx = 4096
    rng = np.random.default_rng(17)
    k, v = normal(rng, ctx + 2, ROW), normal(rng, ctx + 2, ROW)
    q = normal(rng, 2, Q_HEADS * D)
    pool = pool_of(1, 1, ctx + 2, True)
    cache = pool.acquire()
    kd, vd, qd = dev(k), dev(v), dev(q)
    out = torch.empty_like(qd)
    pool.append_device(0, [(cache, ctx)], kd.data_ptr(), vd.data_ptr())
    pool.synchronize()
    pool.set_merge_spin_limit(0)
    pool.attention_step_device(0, [(cache, 1)], qd.data_ptr(), kd[ctx:].data_ptr(),
                               vd[ctx:].data_ptr(), out.data_ptr(), Q_HEADS)
    gave_up = False
    try:
        pool.synchronize()
    except P().StepFailed as e:
        gave_up = True
        assert "gave up waiting" in str(e)
    ref = oracle.KvCache.new([oracle.LayerKind.Global], KV_HEADS, D, store_f16=True)
    ref.restore_bulk(0, 0, k[:ctx], v[:ctx])
    want0 = oracle.attention_step(ref, 0, q[:1], k[ctx:ctx + 1], v[ctx:ctx + 1], Q_HEADS, ctx, threads=8)
    if not gave_up:
        assert max_abs(out[0].cpu().numpy(), want0) <= 2e-3
    pool.set_merge_spin_limit(1 << 17)
    pool.attention_step_device(0, [(cache, 1)], qd[1:].data_ptr(), kd[ctx + 1:].data_ptr(),
                               vd[ctx + 1:].data_ptr(), out[1:].data_ptr(), Q_HEADS)
    pool.synchronize()
    want1 = oracle.attention_step(ref, 0, q[1:], k[ctx + 1:], v[ctx + 1:], Q_HEADS, ctx + 1, threads=8)
    assert max_abs(out[1].cpu().numpy(), want1) <= 2e-3
    pool.close()
