"""The five benchmark configurations, end to end through the C ABI, against the CPU oracle.

Bars: append / truncate / restore bit-exact; f32-KV outputs within 1e-5 (relative to the
largest output magnitude); f16-KV outputs within 2e-3 max-abs of the oracle evaluated over
the same f16-rounded cache. Inputs are seeded N(0,1) from numpy's default_rng."""
import numpy as np
import pytest
import torch

import oracle
from helpers import max_abs, normal, pkg, rel_err

pytestmark = pytest.mark.gpu

Q_HEADS, KV_HEADS, D = 32, 4, 128
ROW = KV_HEADS * D
THREADS = 8


def P():
    return pkg()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def oracle_cache(layers, kv_heads, d, f16):
    return oracle.KvCache.new([oracle.LayerKind.Global] * layers, kv_heads, d, store_f16=f16)


def test_config1_f32_single_layer_decode():
    # 32 Q / 4 KV heads, head_dim 64, f32 KV, 512 cached positions + 1 new token, scale 1/8.
    rng = np.random.default_rng(1)
    d, ctx = 64, 512
    k, v = normal(rng, ctx + 1, KV_HEADS * d), normal(rng, ctx + 1, KV_HEADS * d)
    q = normal(rng, 1, Q_HEADS * d)
    pool = P().KvPool(1, KV_HEADS, d, elem="f32", capacity_rows=ctx + 1)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    kd, vd, qd = dev(k), dev(v), dev(q)
    out = torch.empty_like(qd)
    pool.append_device(0, [(cache, ctx)], kd.data_ptr(), vd.data_ptr())
    pool.attention_step_device(0, [(cache, 1)], qd.data_ptr(), kd[ctx:].data_ptr(),
                               vd[ctx:].data_ptr(), out.data_ptr(), Q_HEADS, scale=0.125)
    torch.cuda.synchronize()
    ref = oracle_cache(1, KV_HEADS, d, False)
    ref.restore_bulk(0, 0, k[:ctx], v[:ctx])
    want = oracle.attention_step(ref, 0, q, k[ctx:], v[ctx:], Q_HEADS, ctx,
                                 oracle.AttentionParams(scale=0.125))
    assert cache.next_position(0) == ctx + 1
    _, gk, gv = cache.view(0).rows()
    assert gk.tobytes() == k.tobytes() and gv.tobytes() == v.tobytes()  # append is bit-exact
    assert rel_err(out.cpu().numpy().reshape(-1), want) <= 1e-5
    # The host-pointer path (Compute::attention) gives the same result.
    hc = P().HipCompute.new(elem="f32", capacity_rows=ctx + 1)
    cfg = P().GlimmerConfig(layers=[P().LayerKind.Global], q_heads=Q_HEADS, kv_heads=KV_HEADS,
                            key_length=d, value_length=d)
    pc = P().PositionCache()
    hc.attention(P().AttentionRequest(np.zeros((ctx, Q_HEADS * d), np.float32), k[:ctx], v[:ctx], 0,
                                      P().LayerKind.Global, cfg), pc)
    pc.advance(ctx)
    got = hc.attention(P().AttentionRequest(q, k[ctx:], v[ctx:], 0, P().LayerKind.Global, cfg), pc)
    assert rel_err(got, want) <= 1e-5
    pool.close()


@pytest.mark.parametrize("softcap", [0.0, 30.0])
def test_config2_30b_class_decode_step_all_layers(softcap):
    # 48 layers, f16 KV at context 4096, K pre-rotated with RoPE base 1e6, 1 token appended
    # per layer, scale 1/sqrt(128); the variant applies softcap 30.
    layers, ctx = 48, 4096
    rng = np.random.default_rng(2)
    pool = P().KvPool(layers, KV_HEADS, D, elem="f16", capacity_rows=ctx + 1)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    worst = 0.0
    for layer in range(layers):
        k = oracle.rope_rows(normal(rng, ctx + 1, KV_HEADS, D), 0, 1e6).reshape(ctx + 1, ROW)
        v = normal(rng, ctx + 1, ROW)
        q = normal(rng, 1, Q_HEADS * D)
        kd, vd, qd = dev(k), dev(v), dev(q)
        out = torch.empty_like(qd)
        pool.append_device(layer, [(cache, ctx)], kd.data_ptr(), vd.data_ptr())
        pool.attention_step_device(layer, [(cache, 1)], qd.data_ptr(), kd[ctx:].data_ptr(),
                                   vd[ctx:].data_ptr(), out.data_ptr(), Q_HEADS, softcap=softcap)
        torch.cuda.synchronize()
        if True:  # every layer is checked against the oracle
            ref = oracle_cache(1, KV_HEADS, D, True)
            ref.restore_bulk(0, 0, k[:ctx], v[:ctx])
            want = oracle.attention_step(ref, 0, q, k[ctx:], v[ctx:], Q_HEADS, ctx,
                                         oracle.AttentionParams(softcap=softcap), threads=THREADS)
            worst = max(worst, max_abs(out.cpu().numpy().reshape(-1), want))
            _, gk, gv = cache.read_rows(layer, 0, ctx + 1)
            assert np.array_equal(gk.reshape(ctx + 1, ROW), oracle.f32_to_f16_array(k))
            assert np.array_equal(gv.reshape(ctx + 1, ROW), oracle.f32_to_f16_array(v))
    assert all(s.appended == ctx + 1 for s in cache.stats())
    assert worst <= 2e-3, worst
    pool.close()


def test_config3_ragged_continuous_batching_decode():
    # 16 slots, ragged context 256..16384, one token appended per slot, per-slot masking.
    slots, layers = 16, 2
    rng = np.random.default_rng(3)
    lengths = rng.integers(256, 16384, size=slots, endpoint=True)
    lengths[0], lengths[1] = 256, 16384
    pool = P().KvPool(layers, KV_HEADS, D, elem="f16", max_slots=slots, capacity_rows=16385)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    caches = [pool.acquire() for _ in range(slots)]
    ks = [normal(rng, int(n) + 1, ROW) for n in lengths]
    vs = [normal(rng, int(n) + 1, ROW) for n in lengths]
    for layer in range(layers):
        q = normal(rng, slots, Q_HEADS * D)
        for s in range(slots):
            kd, vd = dev(ks[s]), dev(vs[s])
            pool.append_device(layer, [(caches[s], int(lengths[s]))], kd.data_ptr(), vd.data_ptr())
        torch.cuda.synchronize()
        new_k = dev(np.stack([ks[s][-1] for s in range(slots)]))
        new_v = dev(np.stack([vs[s][-1] for s in range(slots)]))
        qd = dev(q)
        out = torch.empty_like(qd)
        # A shuffled slot order: the slot table, not the position in the batch, addresses KV.
        order = rng.permutation(slots)
        items = [(caches[s], 1) for s in order]
        ord_k, ord_v = new_k[order].contiguous(), new_v[order].contiguous()
        pool.attention_step_device(layer, items, qd.data_ptr(), ord_k.data_ptr(),
                                   ord_v.data_ptr(), out.data_ptr(), Q_HEADS)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        for i, s in enumerate(order):
            n = int(lengths[s])
            assert caches[s].next_position(layer) == n + 1
            ref = oracle_cache(1, KV_HEADS, D, True)
            ref.restore_bulk(0, 0, ks[s][:n], vs[s][:n])
            want = oracle.attention_step(ref, 0, q[i], ks[s][n:], vs[s][n:], Q_HEADS, n,
                                         threads=THREADS)
            assert max_abs(got[i], want) <= 2e-3, (layer, s, n)
            _, gk, _ = caches[s].read_rows(layer, n, 1)
            assert np.array_equal(gk.reshape(-1), oracle.f32_to_f16_array(ks[s][n]))
    pool.close()


def test_config4_speculative_verify_then_truncate():
    # 4 slots at context 8192, 7 query rows (last accepted + 6 drafts) appended, causal
    # inside the block, then a seeded number of rejected positions (0..6) rolled back.
    slots, layers, ctx, block = 4, 2, 8192, 7
    rng = np.random.default_rng(4)
    pool = P().KvPool(layers, KV_HEADS, D, elem="f16", max_slots=2 * slots,
                      capacity_rows=ctx + 2 * block)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    spec = [pool.acquire() for _ in range(slots)]
    never = [pool.acquire() for _ in range(slots)]
    k = normal(rng, slots, ctx + 2 * block, ROW)
    v = normal(rng, slots, ctx + 2 * block, ROW)
    kd, vd = dev(k), dev(v)
    rejected = rng.integers(0, 6, size=slots, endpoint=True)
    rejected[0], rejected[1] = 0, 6
    keep = ctx + block - rejected
    for layer in range(layers):
        q = normal(rng, slots * block, Q_HEADS * D)
        qd = dev(q)
        out = torch.empty_like(qd)
        for s in range(slots):
            for c in (spec[s], never[s]):
                pool.append_device(layer, [(c, ctx)], kd[s].data_ptr(), vd[s].data_ptr())
        blk_k = kd[:, ctx:ctx + block].contiguous()
        blk_v = vd[:, ctx:ctx + block].contiguous()
        pool.attention_step_device(layer, [(c, block) for c in spec], qd.data_ptr(),
                                   blk_k.data_ptr(), blk_v.data_ptr(), out.data_ptr(), Q_HEADS)
        torch.cuda.synchronize()
        got = out.cpu().numpy().reshape(slots, block, -1)
        for s in range(slots):
            ref = oracle_cache(1, KV_HEADS, D, True)
            ref.restore_bulk(0, 0, k[s, :ctx], v[s, :ctx])
            want = oracle.attention_step(ref, 0, q[s * block:(s + 1) * block],
                                         k[s, ctx:ctx + block], v[s, ctx:ctx + block], Q_HEADS,
                                         ctx, threads=THREADS).reshape(block, -1)
            assert max_abs(got[s], want) <= 2e-3, (layer, s)
    # Rollback, then the kept prefix is what a slot that appended only those rows holds.
    pool.truncate(spec, keep)
    for layer in range(layers):
        for s in range(slots):
            pool.append_device(layer, [(never[s], int(keep[s] - ctx))], kd[s, ctx:].data_ptr(),
                               vd[s, ctx:].data_ptr())
    torch.cuda.synchronize()
    for layer in range(layers):
        for s in range(slots):
            assert spec[s].next_position(layer) == never[s].next_position(layer) == keep[s]
            sk, sv = spec[s].read_raw(layer)
            nk, nv = never[s].read_raw(layer)
            assert sk.tobytes() == nk.tobytes() and sv.tobytes() == nv.tobytes()
    # Re-append the same rows: bit-identical to a slot that never rolled back.
    for layer in range(layers):
        for s in range(slots):
            r = int(rejected[s])
            if r:
                pool.append_device(layer, [(spec[s], r)], kd[s, int(keep[s]):].data_ptr(),
                                   vd[s, int(keep[s]):].data_ptr())
            _, gk, gv = spec[s].read_rows(layer, ctx, block)
            assert np.array_equal(gk.reshape(block, ROW),
                                  oracle.f32_to_f16_array(k[s, ctx:ctx + block]))
            assert np.array_equal(gv.reshape(block, ROW),
                                  oracle.f32_to_f16_array(v[s, ctx:ctx + block]))
    pool.close()


def test_config5_snapshot_restore_all_layers_is_bit_exact():
    # An 8192-token prefix snapshot for all 48 layers in pinned host memory, restored by
    # the gather kernel: (a) f32 rows (the ITKV payload type) converted like append does,
    # (b) f16 rows copied raw. Device rows must equal the host conversion bit for bit.
    layers, tokens = 48, 8192
    rng = np.random.default_rng(5)
    pool = P().KvPool(layers, KV_HEADS, D, elem="f16", max_slots=2, capacity_rows=tokens + 16)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    a, b = pool.acquire(), pool.acquire()
    snap_k = torch.empty((layers, tokens, ROW), dtype=torch.float32).pin_memory()
    snap_v = torch.empty((layers, tokens, ROW), dtype=torch.float32).pin_memory()
    for layer in range(layers):
        snap_k[layer] = torch.from_numpy(normal(rng, tokens, ROW))
        snap_v[layer] = torch.from_numpy(normal(rng, tokens, ROW))
    want_k = oracle.f32_to_f16_array(snap_k.numpy())
    want_v = oracle.f32_to_f16_array(snap_v.numpy())
    a.restore_snapshot_ptrs(tokens, [(0, tokens, snap_k[l].data_ptr(), snap_v[l].data_ptr())
                                     for l in range(layers)], src_f16=False)
    half_k = torch.from_numpy(want_k.view(np.int16)).pin_memory()
    half_v = torch.from_numpy(want_v.view(np.int16)).pin_memory()
    b.restore_snapshot_ptrs(tokens, [(0, tokens, half_k[l].data_ptr(), half_v[l].data_ptr())
                                     for l in range(layers)], src_f16=True)
    for cache in (a, b):
        for layer in range(layers):
            assert cache.next_position(layer) == tokens
            kk, vv = cache.read_raw(layer)
            assert np.array_equal(kk[:tokens].reshape(tokens, ROW), want_k[layer])
            assert np.array_equal(vv[:tokens].reshape(tokens, ROW), want_v[layer])
            assert not kk[tokens:].any() and not vv[tokens:].any()
    pool.close()


def test_config5_chunked_causal_prefill_over_a_long_prefix():
    # A 2048-row chunk attends over a 30720-token prefix plus itself (causal), f16-valued
    # Q/K/V, f32 accumulate. The oracle evaluates a seeded subset of rows at full context.
    prefix, chunk = 30720, 2048
    rng = np.random.default_rng(6)
    f16 = lambda a: a.astype(np.float16).astype(np.float32)  # noqa: E731
    k, v = f16(normal(rng, prefix + chunk, ROW)), f16(normal(rng, prefix + chunk, ROW))
    q = f16(normal(rng, chunk, Q_HEADS * D))
    pool = P().KvPool(1, KV_HEADS, D, elem="f16", capacity_rows=prefix + chunk)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    kd, vd, qd = dev(k), dev(v), dev(q)
    out = torch.empty_like(qd)
    cache.restore_bulk_ptr(0, 0, kd.data_ptr(), vd.data_ptr(), prefix * ROW, src_f16=False)
    pool.attention_step_device(0, [(cache, chunk)], qd.data_ptr(), kd[prefix:].data_ptr(),
                               vd[prefix:].data_ptr(), out.data_ptr(), Q_HEADS)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert cache.next_position(0) == prefix + chunk
    ref = oracle_cache(1, KV_HEADS, D, True)
    ref.restore_bulk(0, 0, k, v)
    rows = sorted({0, 1, 63, 64, 1023, chunk - 1, *rng.integers(0, chunk, size=10).tolist()})
    want = oracle.gqa_attention(q[rows], len(rows), Q_HEADS, [prefix + r for r in rows],
                                ref.view(0), threads=THREADS).reshape(len(rows), -1)
    assert max_abs(got[rows], want) <= 2e-3
    _, gk, _ = cache.read_rows(0, prefix, chunk)
    assert np.array_equal(gk.reshape(chunk, ROW), oracle.f32_to_f16_array(k[prefix:]))
    pool.close()


def test_reduced_prefill_matches_the_oracle_on_every_row():
    # The same path at a size the oracle covers completely, from an empty cache and over a
    # prefix, with and without softcap.
    rng = np.random.default_rng(7)
    # (The last two: contexts short enough that the row tiles are left unsplit although the
    # launch is far from filling the device; a prompt's first chunk.)
    for prefix, chunk, softcap in ((0, 200, 0.0), (333, 150, 30.0), (0, 520, 0.0), (500, 390, 0.0)):
        k, v = normal(rng, prefix + chunk, ROW), normal(rng, prefix + chunk, ROW)
        q = normal(rng, chunk, Q_HEADS * D)
        pool = P().KvPool(1, KV_HEADS, D, elem="f16", capacity_rows=prefix + chunk)
        pool.set_stream(torch.cuda.current_stream().cuda_stream)
        cache = pool.acquire()
        kd, vd, qd = dev(k), dev(v), dev(q)
        out = torch.empty_like(qd)
        if prefix:
            pool.append_device(0, [(cache, prefix)], kd.data_ptr(), vd.data_ptr())
        pool.attention_step_device(0, [(cache, chunk)], qd.data_ptr(), kd[prefix:].data_ptr(),
                                   vd[prefix:].data_ptr(), out.data_ptr(), Q_HEADS,
                                   softcap=softcap)
        torch.cuda.synchronize()
        ref = oracle_cache(1, KV_HEADS, D, True)
        if prefix:
            ref.restore_bulk(0, 0, k[:prefix], v[:prefix])
        want = oracle.attention_step(ref, 0, q, k[prefix:], v[prefix:], Q_HEADS, prefix,
                                     oracle.AttentionParams(softcap=softcap), threads=THREADS)
        assert max_abs(out.cpu().numpy().reshape(-1), want) <= 2e-3
        pool.close()


@pytest.mark.parametrize("q_heads,kv_heads", [(40, 8), (12, 4), (24, 4), (28, 4)])
def test_prefill_chunks_with_groups_that_do_not_divide_sixteen(q_heads, kv_heads):
    # Groups of 5, 3, 6 and 7 Q heads per KV head (40 / 8 is a common model shape): the block
    # kernel pads a row's heads to 8 (or 4) MFMA columns instead of leaving such models to the
    # generic kernel. A chunk over a prefix and a prompt's first chunk, every row checked.
    rng = np.random.default_rng(q_heads)
    row = kv_heads * D
    for prefix, chunk in ((700, 300), (0, 260)):
        k, v = normal(rng, prefix + chunk, row), normal(rng, prefix + chunk, row)
        q = normal(rng, chunk, q_heads * D)
        pool = P().KvPool(1, kv_heads, D, elem="f16", capacity_rows=prefix + chunk)
        pool.set_stream(torch.cuda.current_stream().cuda_stream)
        cache = pool.acquire()
        kd, vd, qd = dev(k), dev(v), dev(q)
        out = torch.empty_like(qd)
        if prefix:
            pool.append_device(0, [(cache, prefix)], kd.data_ptr(), vd.data_ptr())
        pool.attention_step_device(0, [(cache, chunk)], qd.data_ptr(), kd[prefix:].data_ptr(),
                                   vd[prefix:].data_ptr(), out.data_ptr(), q_heads)
        torch.cuda.synchronize()
        ref = oracle_cache(1, kv_heads, D, True)
        if prefix:
            ref.restore_bulk(0, 0, k[:prefix], v[:prefix])
        want = oracle.attention_step(ref, 0, q, k[prefix:], v[prefix:], q_heads, prefix, threads=THREADS)
        assert max_abs(out.cpu().numpy().reshape(-1), want) <= 2e-3
        pool.close()


def test_prefill_with_scores_that_climb_and_fall_along_the_context():
    # Key magnitudes ramp up and down along the context, so the softmax reference maximum
    # moves many times, by little and by a lot, and long runs of keys sit far below it; group sizes 8 and 2; with and without softcap.
    rng = np.random.default_rng(8)
    for q_heads, prefix, chunk, softcap in ((32, 700, 90, 0.0), (8, 259, 77, 0.0), (32, 420, 40, 50.0)):
        n = prefix + chunk
        ramp = 0.25 + 1.5 * np.abs(np.sin(np.arange(n, dtype=np.float32) * (7.0 / n)))[:, None]
        k, v = normal(rng, n, ROW) * ramp, normal(rng, n, ROW)
        q = normal(rng, chunk, q_heads * D)
        pool = P().KvPool(1, KV_HEADS, D, elem="f16", capacity_rows=n)
        pool.set_stream(torch.cuda.current_stream().cuda_stream)
        cache = pool.acquire()
        kd, vd, qd = dev(k), dev(v), dev(q)
        out = torch.empty_like(qd)
        pool.append_device(0, [(cache, prefix)], kd.data_ptr(), vd.data_ptr())
        pool.attention_step_device(0, [(cache, chunk)], qd.data_ptr(), kd[prefix:].data_ptr(),
                                   vd[prefix:].data_ptr(), out.data_ptr(), q_heads,
                                   softcap=softcap)
        torch.cuda.synchronize()
        ref = oracle_cache(1, KV_HEADS, D, True)
        ref.restore_bulk(0, 0, k[:prefix], v[:prefix])
        want = oracle.attention_step(ref, 0, q, k[prefix:], v[prefix:], q_heads, prefix,
                                     oracle.AttentionParams(softcap=softcap), threads=THREADS)
        assert max_abs(out.cpu().numpy().reshape(-1), want) <= 2e-3
        pool.close()
