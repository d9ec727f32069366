"""GQA attention on the GPU through the C ABI: the reference's attention cases
(crates/attention/tests/attention_tests.rs) and the Compute::attention contract
(crates/cpu-compute/src/cpu.rs:506-655, tests/forward_tests.rs), checked against the oracle.

Tolerances: f32 KV outputs within 1e-5 of the oracle relative to the largest output
magnitude; f16 KV outputs within 2e-3 max-abs of the oracle run over the same f16-rounded
cache."""
import numpy as np
import pytest

import oracle
from helpers import max_abs, normal, pkg, rel_err

pytestmark = pytest.mark.gpu

F32_REL = 1e-5
F16_ABS = 2e-3


def P():
    return pkg()


def E(variant, **f):
    return P().AttentionError(variant, **f)


def both(kv_heads, head_dim, rows, elem="f32", layers=1, capacity=None):
    """The same rows appended to a GPU cache and to the oracle."""
    cap = capacity or max(16, len(rows) + 8)
    g = P().KvCache.new([P().LayerKind.Global] * layers, kv_heads, head_dim, elem=elem,
                        capacity_rows=cap)
    c = oracle.KvCache.new([oracle.LayerKind.Global] * layers, kv_heads, head_dim,
                           store_f16=(elem == "f16"))
    if len(rows):
        k = np.stack([np.asarray(r[0], dtype=np.float32).reshape(-1) for r in rows])
        v = np.stack([np.asarray(r[1], dtype=np.float32).reshape(-1) for r in rows])
        for layer in range(layers):
            g.restore_bulk(layer, 0, k, v)
            c.restore_bulk(layer, 0, k, v)
    return g, c


def close(a, b, tol):
    return abs(float(a) - b) <= tol


def test_global_layer_sees_everything():
    # attention_tests.rs:47-61.
    g, _ = both(1, 1, [([1.0], [1000.0]), ([1.0], [3.0]), ([1.0], [5.0])])
    out = P().gqa_attention([1.0], 1, 1, [2], g.view(0), P().AttentionParams.new())
    assert close(out[0], 336.0, 1e-3), out[0]


def test_causal_mask_blocks_future_positions():
    # attention_tests.rs:63-85.
    g, _ = both(1, 1, [([0.0], [1.0]), ([10.0], [100.0]), ([10.0], [1000.0])])
    out = P().gqa_attention([1.0, 1.0], 2, 1, [0, 1], g.view(0), P().AttentionParams.new())
    assert close(out[0], 1.0, 1e-6), out[0]
    assert 99.9 < out[1] < 100.0, out[1]


def test_gqa_head_sharing_glimmer_shape_32_to_2():
    # attention_tests.rs:87-114.
    g, _ = both(2, 2, [([1.0, 0.0, 1.0, 0.0], [10.0, 0.0, 20.0, 0.0])])
    out = P().gqa_attention([1.0, 0.0] * 32, 1, 32, [0], g.view(0), P().AttentionParams.new())
    for h in range(32):
        assert close(out[h * 2], 10.0 if h < 16 else 20.0, 1e-6), (h, out[h * 2])
        assert close(out[h * 2 + 1], 0.0, 1e-6)


def test_gqa_head_sharing_smaller_ratio_4_to_2():
    # attention_tests.rs:116-140.
    g, _ = both(2, 1, [([1.0, 1.0], [7.0, 9.0])])
    out = P().gqa_attention([1.0] * 4, 1, 4, [0], g.view(0), P().AttentionParams.new())
    for h, expected in [(0, 7.0), (1, 7.0), (2, 9.0), (3, 9.0)]:
        assert close(out[h], expected, 1e-6), (h, out[h])


def test_attention_validation_is_named_errors_not_faults():
    # attention_tests.rs:152-212.
    empty = P().KvCache.new([P().LayerKind.Global], 2, 2)
    with pytest.raises(P().AttentionError) as e:
        P().gqa_attention([1.0, 0.0, 1.0, 0.0], 1, 2, [0], empty.view(0))
    assert e.value == E("NoVisibleKeys", position=0)
    g, _ = both(2, 2, [([1.0, 0.0, 1.0, 0.0], [1.0, 0.0, 1.0, 0.0])])
    view = g.view(0)
    with pytest.raises(P().AttentionError) as e:
        P().gqa_attention([1.0] * 6, 1, 3, [0], view)
    assert e.value == E("NonDivisibleHeads", num_q_heads=3, num_kv_heads=2)
    with pytest.raises(P().AttentionError) as e:
        P().gqa_attention([1.0], 1, 2, [0], view)
    assert e.value == E("ShapeMismatch", what="q", expected=4, actual=1)
    with pytest.raises(P().AttentionError) as e:
        P().gqa_attention([1.0] * 4, 2, 2, [0], view)
    assert e.value == E("ShapeMismatch", what="query_positions", expected=2, actual=1)
    assert P().gqa_attention([], 0, 2, [], view).size == 0


def test_scale_is_a_parameter_and_softcap_follows_the_formula():
    d = 16
    k1, k2 = np.zeros(d, dtype=np.float32), np.zeros(d, dtype=np.float32)
    k2[0] = np.log(3.0) * 4.0
    q = np.zeros(d, dtype=np.float32)
    q[0] = 1.0
    g, c = both(1, d, [(k1, np.full(d, 0.0)), (k2, np.full(d, 4.0))])
    A = P().AttentionParams
    assert close(P().gqa_attention(q, 1, 1, [1], g.view(0), A.new())[0], 3.0, 1e-5)
    assert close(P().gqa_attention(q, 1, 1, [1], g.view(0), A.with_scale(0.5))[0], 3.6, 1e-5)
    # Softcap: scores (0, 2 ln 3) at scale 0.5 become cap*tanh(s/cap).
    cap = 1.5
    got = P().gqa_attention(q, 1, 1, [1], g.view(0), A(scale=0.5, softcap=cap))[0]
    want = oracle.gqa_attention(q, 1, 1, [1], c.view(0),
                                oracle.AttentionParams(scale=0.5, softcap=cap))[0]
    assert close(got, want, 1e-5)
    assert close(got, 4.0 * np.exp(cap * np.tanh(2 * np.log(3.0) / cap))
                 / (1 + np.exp(cap * np.tanh(2 * np.log(3.0) / cap))), 1e-5)


@pytest.mark.parametrize("elem", ["f32", "f16"])
@pytest.mark.parametrize("n,qh,kvh,d,nq,softcap", [
    (513, 32, 4, 64, 1, 0.0),     # the CPU-runnable decode shape
    (300, 32, 4, 128, 1, 0.0),
    (300, 32, 4, 128, 7, 30.0),   # verify-block shape with softcap
    (77, 8, 8, 32, 3, 0.0),       # MHA
    (130, 6, 2, 20, 5, 0.0),      # head_dim % 4 == 0 but not a power of two
    (45, 4, 2, 3, 2, 0.0),        # scalar path
    (1000, 16, 1, 256, 2, 0.0),   # MQA, largest head_dim
    (9, 2, 1, 1, 9, 0.0),
])
def test_matches_the_oracle_on_seeded_shapes(elem, n, qh, kvh, d, nq, softcap):
    rng = np.random.default_rng(n * 7 + d)
    keys = normal(rng, n, kvh * d)
    vals = normal(rng, n, kvh * d)
    g, c = both(kvh, d, list(zip(keys, vals)), elem=elem)
    q = normal(rng, nq, qh * d)
    positions = list(range(n - nq, n))
    params = dict(softcap=softcap)
    got = P().gqa_attention(q, nq, qh, positions, g.view(0), P().AttentionParams(**params))
    want = oracle.gqa_attention(q, nq, qh, positions, c.view(0), oracle.AttentionParams(**params))
    if elem == "f32":
        assert rel_err(got, want) <= F32_REL
    else:
        assert max_abs(got, want) <= F16_ABS
    # Arbitrary (non-consecutive, repeated, future) positions take the explicit-position path.
    positions = [n - 1, 0, n // 2, n + 5][:nq] + [n // 3] * max(0, nq - 4)
    got = P().gqa_attention(q, nq, qh, positions, g.view(0), P().AttentionParams(**params))
    want = oracle.gqa_attention(q, nq, qh, positions, c.view(0), oracle.AttentionParams(**params))
    assert (rel_err(got, want) <= F32_REL) if elem == "f32" else (max_abs(got, want) <= F16_ABS)
    # Consecutive positions ahead of the stored rows: every query sees the whole cache.
    positions = list(range(n + 2, n + 2 + nq))
    got = P().gqa_attention(q, nq, qh, positions, g.view(0), P().AttentionParams(**params))
    want = oracle.gqa_attention(q, nq, qh, positions, c.view(0), oracle.AttentionParams(**params))
    assert (rel_err(got, want) <= F32_REL) if elem == "f32" else (max_abs(got, want) <= F16_ABS)


def glimmer_cfg(layers=2, q_heads=8, kv_heads=2, d=16):
    return P().GlimmerConfig(layers=[P().LayerKind.Global] * layers, q_heads=q_heads,
                             kv_heads=kv_heads, key_length=d, value_length=d)


def test_compute_attention_is_append_then_attend_per_row():
    # cpu.rs:586-646; incremental decode equals one-shot prefill (forward_tests.rs:641-719).
    rng = np.random.default_rng(17)
    cfg = glimmer_cfg()
    G = P().LayerKind.Global
    rows = 11
    q = normal(rng, 2, rows, cfg.q_width())
    k = normal(rng, 2, rows, cfg.k_width())
    v = normal(rng, 2, rows, cfg.v_width())
    one_shot = P().HipCompute.new(elem="f32", capacity_rows=32)
    stepwise = P().HipCompute.new(elem="f32", capacity_rows=32)
    cache_a, cache_b = P().PositionCache(), P().PositionCache()
    ref = oracle.KvCache.new([oracle.LayerKind.Global] * 2, cfg.kv_heads, cfg.key_length)
    outs = []
    for layer in range(2):
        outs.append(one_shot.attention(
            P().AttentionRequest(q[layer], k[layer], v[layer], layer, G, cfg), cache_a))
        want = oracle.attention_step(ref, layer, q[layer], k[layer], v[layer], cfg.q_heads, 0)
        assert rel_err(outs[layer], want) <= F32_REL
    cache_a.advance(rows)
    for i in range(rows):
        for layer in range(2):
            o = stepwise.attention(
                P().AttentionRequest(q[layer, i], k[layer, i], v[layer, i], layer, G, cfg), cache_b)
            assert rel_err(o, outs[layer].reshape(rows, -1)[i]) <= 2 * F32_REL
        cache_b.advance(1)
    a, b = one_shot.kv_cache(), stepwise.kv_cache()
    for layer in range(2):
        ak, av = a.read_raw(layer)
        bk, bv = b.read_raw(layer)
        assert ak.tobytes() == bk.tobytes() and av.tobytes() == bv.tobytes()


def test_compute_attention_refusals_follow_the_reference():
    rng = np.random.default_rng(4)
    cfg = glimmer_cfg()
    G = P().LayerKind.Global
    hc = P().HipCompute.new(elem="f32", capacity_rows=16)
    cache = P().PositionCache()
    with pytest.raises(P().StepFailed) as e:
        hc.cache_checkpoint(3)
    assert e.value.step == "cache_checkpoint" and "no KV state exists yet" in e.value.detail
    q, k, v = normal(rng, cfg.q_width()), normal(rng, cfg.k_width()), normal(rng, cfg.v_width())
    with pytest.raises(P().StepFailed) as e:
        hc.attention(P().AttentionRequest(q[:-1], k, v, 0, G, cfg), cache)
    assert "not a whole number" in e.value.detail
    with pytest.raises(P().StepFailed) as e:
        hc.attention(P().AttentionRequest(q, k[:-1], v, 0, G, cfg), cache)
    assert "key/value projections hold" in e.value.detail
    with pytest.raises(P().StepFailed) as e:
        hc.attention(P().AttentionRequest(q, k, v, 0, P().LayerKind.SlidingWindow, cfg), cache)
    assert "does not match the config's kind" in e.value.detail
    hc.attention(P().AttentionRequest(q, k, v, 0, G, cfg), cache)
    # The model did not advance the position cache: the next call must refuse
    # (forward_tests.rs:1153-1181), and keep refusing until reset.
    with pytest.raises(P().StepFailed) as e:
        hc.attention(P().AttentionRequest(q, k, v, 0, G, cfg), cache)
    assert "is at position 1 but the sequence cache is at position 0" in e.value.detail
    other = glimmer_cfg(kv_heads=4)
    with pytest.raises(P().StepFailed) as e:
        hc.attention(P().AttentionRequest(q, np.tile(k, 2), np.tile(v, 2), 0, G, other), cache)
    assert "different shape" in e.value.detail
    hc.reset()
    hc.attention(P().AttentionRequest(q, k, v, 0, G, cfg), cache)


def test_speculative_round_trip_rewind_restores_the_exact_continuation():
    # itak-spec round order (session.rs:616-831): checkpoint -> verify block -> rewind ->
    # release, and forward_tests.rs:1097-1151: the continuation after a rewind equals the
    # continuation of a backend that never speculated.
    rng = np.random.default_rng(23)
    cfg = glimmer_cfg(layers=2, q_heads=8, kv_heads=2, d=32)
    G = P().LayerKind.Global
    prompt, block, accepted = 20, 7, 2
    total = prompt + block + 4
    q = normal(rng, 2, total, cfg.q_width())
    k = normal(rng, 2, total, cfg.k_width())
    v = normal(rng, 2, total, cfg.v_width())

    def forward(hc, cache, lo, hi, qq=q, kk=k, vv=v):
        outs = [hc.attention(P().AttentionRequest(qq[l, lo:hi], kk[l, lo:hi], vv[l, lo:hi], l, G,
                                                  cfg), cache) for l in range(2)]
        cache.advance(hi - lo)
        return outs

    spec, plain = P().HipCompute.new(elem="f16", capacity_rows=64), \
        P().HipCompute.new(elem="f16", capacity_rows=64)
    cs, cp_ = P().PositionCache(), P().PositionCache()
    forward(spec, cs, 0, prompt)
    forward(plain, cp_, 0, prompt)
    handle = spec.cache_checkpoint(block)
    assert handle.base(0) == prompt and handle.saved_bytes() == 0
    # Verify block with draft rows that will be rejected (different K/V than the truth).
    kk, vv = k.copy(), v.copy()
    kk[:, prompt + 1 + accepted:prompt + block] += 3.0
    vv[:, prompt + 1 + accepted:prompt + block] -= 2.0
    forward(spec, cs, prompt, prompt + block, kk=kk, vv=vv)
    with pytest.raises(P().StepFailed) as e:  # one row past the round bound
        spec.attention(P().AttentionRequest(q[0, 0], k[0, 0], v[0, 0], 0, G, cfg), cs)
    assert "outside the live checkpoint's saved range" in e.value.detail
    keep = prompt + 1 + accepted
    spec.cache_rewind(handle, keep)
    cs.rewind_to(keep)
    spec.cache_release(handle)
    forward(plain, cp_, prompt, keep)
    a = forward(spec, cs, keep, total)
    b = forward(plain, cp_, keep, total)
    for l in range(2):
        assert a[l].tobytes() == b[l].tobytes()
        sk, sv = spec.kv_cache().read_raw(l)
        pk, pv = plain.kv_cache().read_raw(l)
        assert sk.tobytes() == pk.tobytes() and sv.tobytes() == pv.tobytes()
    with pytest.raises(P().StepFailed) as e:
        spec.cache_release(handle)
    assert "not this cache's live checkpoint" in e.value.detail


@pytest.mark.parametrize("rows,ctx,softcap", [
    (9, 3000, 0.0), (40, 5000, 0.0),
    # 8 to 40 key blocks per compute unit in all: the block kernel's deep-ring instantiation.
    (130, 2100, 25.0), (64, 4096, 0.0), (48, 6000, 0.0),
    # between 256 and 520 key blocks: still one tile per wavefront, rows appended by the kernel
    (24, 9000, 0.0), (64, 16384, 30.0),
])
def test_mid_size_blocks_split_over_the_context(rows, ctx, softcap):
    # Blocks too long for the decode kernel and too short to fill the device by rows alone:
    # the block kernel cuts the context into splits and the merge launch joins them.
    # Row r at position ctx + r sees keys 0..ctx+r (causal inside the block).
    import torch

    q_heads, kv_heads, d = 32, 4, 128
    rng = np.random.default_rng(rows)
    n = ctx + rows
    k, v = normal(rng, n, kv_heads * d), normal(rng, n, kv_heads * d)
    q = normal(rng, rows, q_heads * d)
    pool = P().KvPool(1, kv_heads, d, elem="f16", capacity_rows=n)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    kd, vd, qd = [torch.from_numpy(a).cuda() for a in (k, v, q)]
    out = torch.empty_like(qd)
    pool.append_device(0, [(cache, ctx)], kd.data_ptr(), vd.data_ptr())
    pool.attention_step_device(0, [(cache, rows)], qd.data_ptr(), kd[ctx:].data_ptr(),
                               vd[ctx:].data_ptr(), out.data_ptr(), q_heads, softcap=softcap)
    torch.cuda.synchronize()
    ref = oracle.KvCache.new([oracle.LayerKind.Global], kv_heads, d, store_f16=True)
    ref.restore_bulk(0, 0, k[:ctx], v[:ctx])
    want = oracle.attention_step(ref, 0, q, k[ctx:], v[ctx:], q_heads, ctx,
                                 oracle.AttentionParams(softcap=softcap), threads=8)
    assert max_abs(out.cpu().numpy().reshape(-1), want) <= 2e-3
    # Blocks of up to 64 rows bring their rows along (the block kernel appends them itself):
    # what the cache then holds is what a separate append leaves, bit for bit.
    _, rk, rv = ref.view(0).rows()
    _, ck, cv = cache.view(0).rows()
    as_f32 = lambda a: np.asarray(a).view(np.float16).astype(np.float32) if np.asarray(a).dtype == np.uint16 \
        else np.asarray(a, dtype=np.float32)
    assert as_f32(ck).tobytes() == as_f32(rk).tobytes()
    assert as_f32(cv).tobytes() == as_f32(rv).tobytes()
    pool.close()


@pytest.mark.parametrize("window", [None, 512])
def test_a_step_that_mixes_decode_rows_a_verify_block_and_a_prefill_chunk(window):
    # Continuous batching: one call carries slots that decode one row, a slot that verifies an
    # 8-row block and a slot that prefills a 300-row chunk (a prompt's first chunk and a later
    # one). Every slot's rows against the oracle, and the lengths afterwards.
    import torch
    q_heads, kv_heads, d = 32, 4, 128
    rng = np.random.default_rng(77)
    kind = P().LayerKind.Global if window is None else P().LayerKind.windowed(window)
    okind = oracle.LayerKind.Global if window is None else oracle.LayerKind.windowed(window)
    plan = [(3000, 1), (517, 1), (2100, 8), (0, 300), (1030, 300), (8000, 1)]   # (context, rows)
    if window is not None:   # a ring takes a block no longer than its headroom
        plan = [(3000, 1), (517, 1), (2100, 8), (0, 200), (1030, 200), (8000, 1)]
    pool = P().KvPool([kind], kv_heads, d, elem="f16", max_slots=len(plan), capacity_rows=8400,
                      ring_headroom=224)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    caches, refs = [], []
    for ctx, _ in plan:
        c = pool.acquire()
        r = oracle.KvCache.new([okind], kv_heads, d, store_f16=True)
        if ctx:
            k, v = normal(rng, ctx, kv_heads * d), normal(rng, ctx, kv_heads * d)
            kd, vd = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
            for p0 in range(0, ctx, 200):
                n = min(200, ctx - p0)
                pool.append_device(0, [(c, n)], kd[p0:].data_ptr(), vd[p0:].data_ptr())
            first = 0 if window is None else max(0, ctx - window)
            r.restore_bulk(0, first, k[first:], v[first:])
        caches.append(c); refs.append(r)
    for step in range(2):
        rows = [n for _, n in plan]
        total = sum(rows)
        q = normal(rng, total, q_heads * d)
        k, v = normal(rng, total, kv_heads * d), normal(rng, total, kv_heads * d)
        qd, kd, vd = (torch.from_numpy(a).cuda() for a in (q, k, v))
        out = torch.empty_like(qd)
        pool.attention_step_device(0, list(zip(caches, rows)), qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                                   out.data_ptr(), q_heads)
        pool.synchronize()
        got = out.cpu().numpy()
        row0 = 0
        for s, n in enumerate(rows):
            base = refs[s].next_position(0)
            want = oracle.attention_step(refs[s], 0, q[row0:row0 + n], k[row0:row0 + n], v[row0:row0 + n],
                                         q_heads, base, threads=8)
            assert max_abs(got[row0:row0 + n].reshape(-1), want) <= 2e-3, (step, s)
            assert caches[s].next_position(0) == refs[s].next_position(0) == base + n
            row0 += n
    pool.close()


@pytest.mark.parametrize("rows", [9, 40, 64])
def test_blocks_that_append_their_own_rows_convert_every_class_of_value_as_append_does(rows):
    # NaNs with payloads and either sign, infinities (a pair that cancels in a sum included),
    # overflow, subnormals and ties among the new rows: the stored bits equal the append kernel's.
    # (The outputs of such a step are NaN in any implementation and are not compared.)
    import torch
    kv_heads, d, ctx = 4, 128, 700
    rng = np.random.default_rng(rows)
    k, v = normal(rng, ctx + rows, kv_heads * d), normal(rng, ctx + rows, kv_heads * d)
    specials = np.array([np.nan, -np.nan, np.inf, -np.inf, 65504.0, 65520.0, 1e9, -7e4, 6e-8, -3e-8,
                         5.9604645e-8, 2.9802322e-8, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 0.0, -0.0],
                        dtype=np.float32)
    payload = np.array([0x7fc12345, 0xffa00001, 0x7f800001, 0xff812345], dtype=np.uint32).view(np.float32)
    for arr in (k, v):
        tail = arr[ctx:].reshape(-1)
        idx = rng.choice(tail.size, size=400, replace=False)
        tail[idx[:300]] = rng.choice(specials, size=300)
        tail[idx[300:]] = rng.choice(payload, size=100)
        tail[:4] = [np.inf, -np.inf, 1.0, 2.0]      # one piece whose sum is a NaN without a NaN in it
    q = normal(rng, rows, 32 * d)
    pools = [P().KvPool(1, kv_heads, d, elem="f16", capacity_rows=ctx + rows) for _ in range(2)]
    caches = [p.acquire() for p in pools]
    kd, vd, qd = (torch.from_numpy(a).cuda() for a in (k, v, q))
    out = torch.empty_like(qd)
    for p, c in zip(pools, caches):
        p.set_stream(torch.cuda.current_stream().cuda_stream)
        p.append_device(0, [(c, ctx)], kd.data_ptr(), vd.data_ptr())
    pools[0].attention_step_device(0, [(caches[0], rows)], qd.data_ptr(), kd[ctx:].data_ptr(),
                                   vd[ctx:].data_ptr(), out.data_ptr(), 32)
    pools[1].append_device(0, [(caches[1], rows)], kd[ctx:].data_ptr(), vd[ctx:].data_ptr())
    pools[0].synchronize()
    a, b = caches[0].read_raw(0), caches[1].read_raw(0)
    assert a[0].tobytes() == b[0].tobytes() and a[1].tobytes() == b[1].tobytes()
    want = oracle.f32_to_f16_array(k[ctx:]).reshape(rows, kv_heads, d)
    assert a[0][ctx:ctx + rows].view(np.uint16).tobytes() == np.asarray(want).view(np.uint16).tobytes()
    for p in pools:
        p.close()


@pytest.mark.parametrize("rows,ctx,window,group", [
    (64, 4096, None, 8), (33, 1000, None, 8), (16, 4100, None, 8), (17, 31, None, 8),
    (64, 200, None, 4), (40, 3000, None, 2), (64, 4096 + 13, None, 8),
    (64, 5000, 1024, 8), (20, 2030, 1024, 8), (48, 1000, 256, 4), (31, 10000, None, 8),
    # groups that do not divide 16 take padded columns: 5 heads in 8, 3 in 4, 6 in 8, 12 in 16
    (40, 1500, None, 5), (64, 900, None, 3), (30, 2000, 512, 6), (20, 1200, None, 12), (64, 700, None, 16)])
def test_blocks_that_append_their_own_rows_leave_the_cache_as_a_separate_append_does(rows, ctx, window,
                                                                                     group):
    # The block kernel's one-tile form takes the new rows as parameters: converted in the
    # prologue, written over the tail blocks in LDS by every workgroup that reads them, stored
    # to the planes by one workgroup per KV head. Outputs against the oracle, stored rows bit for
    # bit against a pool that appended first (through the append kernel), and the next steps on
    # top of them; global and sliding-window layers (rings wrapped), several slots at once.
    import torch
    kv_heads, d = 4, 128
    q_heads = kv_heads * group
    rng = np.random.default_rng(rows * 7 + ctx)
    kind = P().LayerKind.Global if window is None else P().LayerKind.windowed(window)
    okind = oracle.LayerKind.Global if window is None else oracle.LayerKind.windowed(window)
    slots = 2
    pool = P().KvPool([kind], kv_heads, d, elem="f16", max_slots=slots, capacity_rows=ctx + 4 * rows + 8,
                      ring_headroom=64)
    plain = P().KvPool([kind], kv_heads, d, elem="f16", max_slots=slots, capacity_rows=ctx + 4 * rows + 8,
                       ring_headroom=64)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    plain.set_stream(torch.cuda.current_stream().cuda_stream)
    caches = [pool.acquire() for _ in range(slots)]
    pcaches = [plain.acquire() for _ in range(slots)]
    refs = [oracle.KvCache.new([okind], kv_heads, d, store_f16=True) for _ in range(slots)]
    ctxs = [ctx, max(ctx - 37, 1)]
    for s in range(slots):
        k, v = normal(rng, ctxs[s], kv_heads * d), normal(rng, ctxs[s], kv_heads * d)
        kd, vd = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
        for p0 in range(0, ctxs[s], 64):
            n = min(64, ctxs[s] - p0)
            pool.append_device(0, [(caches[s], n)], kd[p0:].data_ptr(), vd[p0:].data_ptr())
            plain.append_device(0, [(pcaches[s], n)], kd[p0:].data_ptr(), vd[p0:].data_ptr())
        for i in range(ctxs[s]):
            refs[s].append(0, k[i], v[i], i)
    for step_rows in (rows, rows, 1, max(rows // 2, 9)):
        per = [step_rows, max(step_rows - 3, 9)]   # the second slot's block is a little shorter
        total = sum(per)
        q = normal(rng, total, q_heads * d)
        k, v = normal(rng, total, kv_heads * d), normal(rng, total, kv_heads * d)
        qd, kd, vd = (torch.from_numpy(a).cuda() for a in (q, k, v))
        out = torch.empty_like(qd)
        pool.attention_step_device(0, list(zip(caches, per)), qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                                   out.data_ptr(), q_heads)
        plain.append_device(0, list(zip(pcaches, per)), kd.data_ptr(), vd.data_ptr())
        pool.synchronize()
        got = out.cpu().numpy()
        row0 = 0
        for s in range(slots):
            base = refs[s].next_position(0)
            want = oracle.attention_step(refs[s], 0, q[row0:row0 + per[s]], k[row0:row0 + per[s]],
                                         v[row0:row0 + per[s]], q_heads, base, threads=8)
            assert max_abs(got[row0:row0 + per[s]].reshape(-1), want) <= 2e-3, (s, step_rows)
            row0 += per[s]
            a, b = caches[s].read_raw(0), pcaches[s].read_raw(0)
            assert a[0].tobytes() == b[0].tobytes() and a[1].tobytes() == b[1].tobytes(), (s, step_rows)
            assert caches[s].next_position(0) == refs[s].next_position(0)
    pool.close()
    plain.close()


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(8))
def test_random_blocks_match_the_oracle_across_groups_windows_and_softcap(seed):
    """Seeded blocks of 9 to 200 rows over contexts of 64 to 6000 positions, GQA groups 8, 4, 1
    and 2, every fourth on a sliding-window layer, every third with a softcap: whichever way the
    block kernel cuts them (one or two tiles per wavefront, split or not, either LDS ring), the
    output is the oracle's within the f16-KV bar."""
    import torch

    rng = np.random.default_rng(5000 + seed)
    group, kvh = [(8, 4), (4, 2), (1, 8), (2, 4)][seed % 4]
    qh, d = kvh * group, 128
    ctx, rows = int(rng.integers(64, 6000)), int(rng.integers(9, 200))
    softcap = 20.0 if seed % 3 == 0 else 0.0
    window = int(rng.integers(200, 1500)) if seed % 4 == 3 else 0
    n = ctx + rows
    k, v, q = normal(rng, n, kvh * d), normal(rng, n, kvh * d), normal(rng, rows, qh * d)
    kind = P().LayerKind.windowed(window) if window else P().LayerKind.Global
    okind = oracle.LayerKind.windowed(window) if window else oracle.LayerKind.Global
    pool = P().KvPool([kind], kvh, d, elem="f16", capacity_rows=n + 8,
                      ring_headroom=rows if window else 0)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    ref = oracle.KvCache.new([okind], kvh, d, store_f16=True)
    first = max(0, ctx - window) if window else 0
    cache.restore_bulk(0, first, k[first:ctx], v[first:ctx])
    ref.restore_bulk(0, first, k[first:ctx], v[first:ctx])
    qd, kd, vd = (torch.from_numpy(np.ascontiguousarray(x)).cuda() for x in (q, k[ctx:], v[ctx:]))
    out = torch.empty_like(qd)
    pool.attention_step_device(0, [(cache, rows)], qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                               out.data_ptr(), qh, softcap=softcap)
    pool.synchronize()
    want = oracle.attention_step(ref, 0, q, k[ctx:], v[ctx:], qh, ctx,
                                 oracle.AttentionParams(softcap=softcap), threads=8)
    assert max_abs(out.cpu().numpy().reshape(-1), want) <= 2e-3, (group, ctx, rows, softcap, window)
    pool.close()


@pytest.mark.parametrize("rows", [1, 7])
@pytest.mark.parametrize("q_scale,k_scale", [(3.0, 1.0), (1.0, 3.0), (1.5, 2.0)])
def test_f16_operands_meet_the_bar_up_to_scores_of_deviation_three(rows, q_scale, k_scale):
    # Q and P enter the MFMAs as f16, so the error grows with the size of the scaled scores
    # (Q's rounding is relative). The bar of 2e-3 holds up to scores of standard deviation 3
    # (measured on an MI355X: 3e-5 at deviation 1, the scale of the benchmark's inputs; about
    # 1e-3 to 1.5e-3 at 3; 1.9e-3 at 4; above the bar at 6). This pins the documented limit.
    ctx = 4096
    worst = 0.0
    for seed in range(2):
        rng = np.random.default_rng(1000 + seed)
        k = normal(rng, ctx + rows, 512) * k_scale
        v = normal(rng, ctx + rows, 512)
        q = normal(rng, rows, 32 * 128) * q_scale
        pool = P().KvPool(1, 4, 128, elem="f16", capacity_rows=ctx + rows)
        cache = pool.acquire()
        import torch
        pool.set_stream(torch.cuda.current_stream().cuda_stream)
        kd, vd, qd = (torch.from_numpy(x).cuda() for x in (k, v, q))
        out = torch.empty_like(qd)
        pool.append_device(0, [(cache, ctx)], kd.data_ptr(), vd.data_ptr())
        pool.attention_step_device(0, [(cache, rows)], qd.data_ptr(), kd[ctx:].data_ptr(),
                                   vd[ctx:].data_ptr(), out.data_ptr(), 32)
        pool.synchronize()
        ref = oracle.KvCache.new([oracle.LayerKind.Global], 4, 128, store_f16=True)
        ref.restore_bulk(0, 0, k[:ctx], v[:ctx])
        want = oracle.attention_step(ref, 0, q, k[ctx:], v[ctx:], 32, ctx, threads=8)
        worst = max(worst, max_abs(out.cpu().numpy().reshape(-1), want))
        pool.close()
    assert worst <= F16_ABS, worst


def _worst_error_at_scale(rows, q_scale, k_scale, ctx, slots=1, **pool_args):
    import torch
    worst = 0.0
    for seed in range(2):
        rng = np.random.default_rng(1000 + seed)
        pool_args.setdefault("q_two_halves", False)  # whatever the environment's default says
        pool = P().KvPool(1, 4, 128, elem="f16", max_slots=slots, capacity_rows=ctx + rows, **pool_args)
        pool.set_stream(torch.cuda.current_stream().cuda_stream)
        caches = [pool.acquire() for _ in range(slots)]
        ks = [normal(rng, ctx + rows, 512) * k_scale for _ in range(slots)]
        vs = [normal(rng, ctx + rows, 512) for _ in range(slots)]
        q = normal(rng, slots * rows, 32 * 128) * q_scale
        for c, k, v in zip(caches, ks, vs):
            kd, vd = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
            pool.append_device(0, [(c, ctx)], kd.data_ptr(), vd.data_ptr())
            pool.synchronize()
        kn = torch.from_numpy(np.concatenate([k[ctx:] for k in ks])).cuda()
        vn = torch.from_numpy(np.concatenate([v[ctx:] for v in vs])).cuda()
        qd = torch.from_numpy(q).cuda()
        out = torch.empty_like(qd)
        pool.attention_step_device(0, [(c, rows) for c in caches], qd.data_ptr(), kn.data_ptr(),
                                   vn.data_ptr(), out.data_ptr(), 32)
        pool.synchronize()
        got = out.cpu().numpy().reshape(slots, -1)
        for s in range(slots):
            ref = oracle.KvCache.new([oracle.LayerKind.Global], 4, 128, store_f16=True)
            ref.restore_bulk(0, 0, ks[s][:ctx], vs[s][:ctx])
            want = oracle.attention_step(ref, 0, q[s * rows:(s + 1) * rows], ks[s][ctx:], vs[s][ctx:], 32,
                                         ctx, threads=8)
            worst = max(worst, max_abs(got[s], want))
        pool.close()
    return worst


@pytest.mark.parametrize("rows,slots,ctx", [(1, 1, 4096), (7, 1, 4096), (3, 2, 4096), (1, 6, 9000)])
@pytest.mark.parametrize("q_scale,k_scale", [(3.0, 2.0), (6.0, 1.0), (1.0, 6.0), (2.0, 2.0)])
def test_queries_as_two_halves_hold_the_bar_at_scores_of_deviation_six(rows, slots, ctx, q_scale, k_scale):
    # ITAK_POOL_Q_TWO_HALVES: q = hi + lo, scores K.hi + K.lo, so that the queries' rounding to
    # f16 leaves the scores; what remains is the rounding of the softmax weights. Scaled scores
    # of standard deviation 4 and 6, where the one-half form is at or above the bar (1.9e-3 and
    # 3e-3 to 4.5e-3 measured), over the single-row decode kernel, a 7-row block (four tiles), a
    # two-tile batch and a decode batch on the split-K kernel.
    with_flag = _worst_error_at_scale(rows, q_scale, k_scale, ctx, slots, q_two_halves=True)
    assert with_flag <= F16_ABS, with_flag
    print(f"rows {rows} slots {slots} q x{q_scale} k x{k_scale}: two halves {with_flag:.2e}")


@pytest.mark.parametrize("rows,slots,ctx", [(32, 1, 4096), (300, 1, 3000), (20, 2, 1000), (9, 1, 40)])
@pytest.mark.parametrize("q_scale,k_scale", [(3.0, 2.0), (1.0, 6.0)])
def test_the_block_kernel_takes_the_queries_as_two_halves_too(rows, slots, ctx, q_scale, k_scale):
    # Blocks of more than 8 rows and prefill chunks at head_dim 128: the block kernel's two-tile
    # form with the second halves (blocks that would bring their rows along in the one-tile form
    # are appended by a launch of their own). At these scores the single product is above the bar.
    halves = _worst_error_at_scale(rows, q_scale, k_scale, ctx, slots, q_two_halves=True)
    assert halves <= F16_ABS, halves
    if (rows, slots) == (300, 1):
        plain = _worst_error_at_scale(rows, q_scale, k_scale, ctx, slots)
        assert halves * 2 < plain, (halves, plain)


def test_queries_as_one_half_leave_the_bar_where_two_halves_hold_it():
    # The same step both ways at scores of deviation 6: the flag is what makes the difference.
    plain = _worst_error_at_scale(1, 3.0, 2.0, 4096)
    halves = _worst_error_at_scale(1, 3.0, 2.0, 4096, q_two_halves=True)
    assert halves <= F16_ABS < plain, (halves, plain)
    assert halves * 3 < plain, (halves, plain)


@pytest.mark.parametrize("q_heads,kv_heads,ctx,rows", [(4, 1, 5650, 62), (32, 4, 4096, 1)])
def test_f32_outputs_off_unit_scale_are_held_to_an_f64_evaluation(q_heads, kv_heads, ctx, rows):
    # The 1e-5 bar for f32 KV is a distance between two f32 evaluations that sum in different
    # orders. At unit scale they are 3e-6 to 5e-6 apart. With Q at three and K at two times unit
    # scale (scores of deviation 6) each of the two is 2e-6 to 8e-6 from an f64 evaluation
    # (measured on an MI355X; on a 62-row block at context 5650 the oracle's serial sums 8.3e-6,
    # the device's 3.1e-6), so the distance between them reaches the bar (1.08e-5 seen) without
    # either being wrong. Pinned here: the device within 1e-5 of f64, no more than 1.5 times as
    # far from it as the oracle, and the two within 2e-5 of each other.
    import torch
    d = 128
    rng = np.random.default_rng(104)
    width = kv_heads * d
    k, v = 2.0 * normal(rng, ctx + rows, width), normal(rng, ctx + rows, width)
    q = 3.0 * normal(rng, rows, q_heads * d)
    pool = P().KvPool(1, kv_heads, d, elem="f32", capacity_rows=ctx + rows)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    kd, vd, qd = (torch.from_numpy(x).cuda() for x in (k, v, q))
    out = torch.empty_like(qd)
    pool.append_device(0, [(cache, ctx)], kd.data_ptr(), vd.data_ptr())
    pool.attention_step_device(0, [(cache, rows)], qd.data_ptr(), kd[ctx:].data_ptr(), vd[ctx:].data_ptr(),
                               out.data_ptr(), q_heads)
    pool.synchronize()
    got = out.cpu().numpy().astype(np.float64)
    ref = oracle.KvCache.new([oracle.LayerKind.Global], kv_heads, d, store_f16=False)
    ref.restore_bulk(0, 0, k[:ctx], v[:ctx])
    want = np.asarray(oracle.attention_step(ref, 0, q, k[ctx:], v[ctx:], q_heads, ctx, threads=8),
                      dtype=np.float64).reshape(rows, -1)
    # Softmax attention in f64, straight from the definition (attention.rs:104-215).
    K = k.astype(np.float64).reshape(-1, kv_heads, d)
    V = v.astype(np.float64).reshape(-1, kv_heads, d)
    Q = q.astype(np.float64).reshape(rows, q_heads, d)
    truth = np.zeros((rows, q_heads, d))
    for r in range(rows):
        n = ctx + r + 1
        for h in range(q_heads):
            kvh = h // (q_heads // kv_heads)
            s = K[:n, kvh] @ Q[r, h] / np.sqrt(d)
            w = np.exp(s - s.max())
            truth[r, h] = (w / w.sum()) @ V[:n, kvh]
    truth = truth.reshape(rows, -1)
    top = np.abs(truth).max()
    device, cpu = np.abs(got - truth).max() / top, np.abs(want - truth).max() / top
    assert device <= 1e-5 and device <= 1.5 * cpu, (device, cpu)
    assert np.abs(got - want).max() / top <= 2e-5
    pool.close()


def test_masked_rows_with_non_finite_values_do_not_reach_a_decode_query():
    # The reference never reads the value row of a key a query does not see
    # (attention.rs:160-173): rows of a windowed layer that have just left the window, and
    # storage rows past the sequence's length, may hold anything, NaN and infinity included.
    import torch
    window, ctx = 64, 200
    rng = np.random.default_rng(5)
    k, v = normal(rng, ctx + 1, 512), normal(rng, ctx + 1, 512)
    lo = ctx + 1 - window  # the oldest position the query at `ctx` sees
    v[lo - 1] = np.inf     # just outside the window, in the same 32-row block as visible rows
    v[lo - 2] = np.nan
    q = normal(rng, 1, 32 * 128)
    for in_launch in (False, True):
        pool = P().KvPool([P().LayerKind.windowed(window)], 4, 128, elem="f16", capacity_rows=ctx + 8,
                          ring_headroom=64, merge_in_launch=in_launch)
        pool.set_stream(torch.cuda.current_stream().cuda_stream)
        cache = pool.acquire()
        kd, vd, qd = (torch.from_numpy(x).cuda() for x in (k, v, q))
        out = torch.empty_like(qd)
        for p0 in range(0, ctx, 50):  # the ring keeps the rows just outside the window too
            pool.append_device(0, [(cache, 50)], kd[p0:].data_ptr(), vd[p0:].data_ptr())
        pool.attention_step_device(0, [(cache, 1)], qd.data_ptr(), kd[ctx:].data_ptr(),
                                   vd[ctx:].data_ptr(), out.data_ptr(), 32)
        pool.synchronize()
        ref = oracle.KvCache.new([oracle.LayerKind.windowed(window)], 4, 128, store_f16=True)
        ref.restore_bulk(0, ctx - window, k[ctx - window:ctx], v[ctx - window:ctx])
        want = oracle.attention_step(ref, 0, q, k[ctx:], v[ctx:], 32, ctx, threads=4)
        got = out.cpu().numpy().reshape(-1)
        assert np.isfinite(want).all() and np.isfinite(got).all()
        assert max_abs(got, want) <= F16_ABS
        pool.close()


@pytest.mark.parametrize("elem,ctx,kk", [("f16", 20000, 0), ("f16", 40011, 11), ("f16", 9000, 8), ("f32", 20017, 17)])
def test_long_single_slot_decode_merges_more_splits_than_one_pass_holds(elem, ctx, kk):
    # One slot far beyond 8192 keys: the decode kernel leaves well over 64 partials per head, so the
    # merge kernel folds them in several passes with a running maximum; the new row lands at
    # different places of its 32-row block (kk), a gate rides along on the second step.
    import torch
    assert ctx % 32 == kk
    rng = np.random.default_rng(ctx)
    q_heads, kv_heads, d = 32, 4, 128
    row = kv_heads * d
    pool = P().KvPool(1, kv_heads, d, elem=elem, capacity_rows=ctx + 8)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    k, v = normal(rng, ctx, row), normal(rng, ctx, row)
    kd, vd = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
    pool.append_device(0, [(cache, ctx)], kd.data_ptr(), vd.data_ptr())
    torch.cuda.synchronize()
    ref = oracle.KvCache.new([oracle.LayerKind.Global], kv_heads, d, store_f16=(elem == "f16"))
    ref.restore_bulk(0, 0, k, v)
    for step in range(3):
        q, kn, vn = normal(rng, 1, q_heads * d), normal(rng, 1, row), normal(rng, 1, row)
        qd, knd, vnd = (torch.from_numpy(x).cuda() for x in (q, kn, vn))
        out = torch.empty_like(qd)
        pool.attention_step_device(0, [(cache, 1)], qd.data_ptr(), knd.data_ptr(), vnd.data_ptr(),
                                   out.data_ptr(), q_heads)
        torch.cuda.synchronize()
        want = oracle.attention_step(ref, 0, q, kn, vn, q_heads, ctx + step, threads=8)
        got = out.cpu().numpy().reshape(-1)
        if elem == "f32":
            assert rel_err(got, want) <= 1e-5
        else:
            assert max_abs(got, want) <= 2e-3
    _, gk, gv = cache.read_rows(0, ctx, 3)
    assert gk.shape[0] == 3 and cache.next_position(0) == ctx + 3
    pool.close()
