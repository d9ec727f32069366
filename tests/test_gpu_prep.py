"""The fused attention preparation (per-head RMSNorm + RoPE of Q and K), append, attention
and gate as one device step, against the oracle's composition of the reference's CPU steps
(crates/muse-glimmer/src/model.rs:445-464, crates/cpu-compute/src/cpu.rs:445-475, 586-673).

Bars: prepared K rows in an f32 cache within 1e-6 of the oracle's (the reference pins its own
fused kernel against the unfused chain at 1e-5, crates/wgpu-compute/tests/fused_kernels.rs:
408-431), in an f16 cache within one f16 step or 1e-6, V rows exact; outputs within 1e-5
relative on f32 KV and 2e-3 max-abs on f16 KV."""
import numpy as np
import pytest
import torch

import oracle
from helpers import max_abs, normal, pkg, rel_err

pytestmark = pytest.mark.gpu


def P():
    return pkg()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def run_case(elem, q_heads, kv_heads, d, ctx, rows, norm, rope_base, interleaved, rotary, gate,
             seed=0, slots=1, window=None):
    rng = np.random.default_rng(seed)
    width = kv_heads * d
    kind = P().LayerKind.Global if window is None else P().LayerKind.windowed(window)
    okind = oracle.LayerKind.Global if window is None else oracle.LayerKind.windowed(window)
    pool = P().KvPool([kind], kv_heads, d, elem=elem, max_slots=slots,
                      capacity_rows=ctx + 13 * (slots - 1) + rows + 8)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    qw = (1.0 + 0.1 * normal(rng, d)) if norm else None
    kw = (1.0 + 0.1 * normal(rng, d)) if norm else None
    eps = 1e-6
    caches, refs, qs, ks, vs, gs = [], [], [], [], [], []
    for s in range(slots):
        cache = pool.acquire()
        ref = oracle.KvCache.new([okind], kv_heads, d, store_f16=(elem == "f16"))
        n0 = ctx + 13 * s
        k0 = oracle.attention_prep(normal(rng, n0, width), kv_heads, d, 0, kw, eps, rope_base,
                                   interleaved, rotary or None)
        v0 = normal(rng, n0, width)
        if n0 and window is not None:  # what a prefill leaves in the ring: the last `window` rows
            first = max(0, n0 - window)
            cache.restore_bulk(0, first, k0[first:], v0[first:])
            ref.restore_bulk(0, first, k0[first:], v0[first:])
        elif n0:
            k0d, v0d = dev(k0), dev(v0)
            pool.append_device(0, [(cache, n0)], k0d.data_ptr(), v0d.data_ptr())
            torch.cuda.synchronize()
            ref.restore_bulk(0, 0, k0, v0)
        caches.append(cache); refs.append(ref)
        qs.append(3.0 * normal(rng, rows, q_heads * d)); ks.append(2.0 * normal(rng, rows, width))
        vs.append(normal(rng, rows, width)); gs.append(2.0 * normal(rng, rows, q_heads * d))
    q, k, v, g = (np.concatenate(x) for x in (qs, ks, vs, gs))
    qd, kd, vd, gd = dev(q), dev(k), dev(v), dev(g)
    qwd, kwd = (dev(qw), dev(kw)) if norm else (None, None)  # kept alive across the call
    out = torch.empty_like(qd)
    pool.attention_prep_step_device(
        0, [(c, rows) for c in caches], qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), out.data_ptr(),
        q_heads, q_norm_ptr=qwd.data_ptr() if norm else 0,
        k_norm_ptr=kwd.data_ptr() if norm else 0, eps=eps, rope_base=rope_base,
        interleaved=interleaved, rotary_dim=rotary, gate_ptr=gd.data_ptr() if gate else 0)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    for s in range(slots):
        n0 = ctx + 13 * s
        qp = oracle.attention_prep(qs[s], q_heads, d, n0, qw, eps, rope_base, interleaved, rotary or None)
        kp = oracle.attention_prep(ks[s], kv_heads, d, n0, kw, eps, rope_base, interleaved, rotary or None)
        want = oracle.attention_step(refs[s], 0, qp, kp, vs[s], q_heads, n0, threads=8)
        if gate:
            want = oracle.attn_gate(want, gs[s])
        mine = got[s * rows:(s + 1) * rows].reshape(-1)
        if elem == "f32":
            assert rel_err(mine, want) <= 1e-5
        else:
            assert max_abs(mine, want) <= 2e-3
        # The appended rows: prepared keys, untouched values.
        _, gk, gv = caches[s].read_rows(0, caches[s].stored_len(0) - rows, rows)
        if elem == "f32":
            assert max_abs(gk.reshape(rows, width), kp) <= 1e-6
            assert gv.reshape(rows, width).tobytes() == vs[s].tobytes()
        else:
            # A prepared key that differs from the oracle's in its last f32 bits can round to
            # the neighbouring half: one f16 step at most, except where the rotation cancelled
            # (|x*cos - y*sin| far below |x|), whose result carries the absolute error of the
            # f32 products, a few 1e-7, which near zero is more than one of f16's small steps.
            want_bits = oracle.f32_to_f16_array(kp)
            ulp = np.abs(gk.reshape(rows, width).view(np.int16).astype(np.int32)
                         - want_bits.view(np.int16).astype(np.int32))
            far = np.abs(gk.reshape(rows, width).view(np.float16).astype(np.float64)
                         - want_bits.view(np.float16).astype(np.float64))
            assert np.all((ulp <= 1) | (far <= 1e-6))
            assert np.array_equal(gv.reshape(rows, width), oracle.f32_to_f16_array(vs[s]))
        assert caches[s].next_position(0) == n0 + rows
    pool.close()


@pytest.mark.parametrize("elem", ["f32", "f16"])
def test_decode_step_with_norms_interleaved_rope_and_gate(elem):
    run_case(elem, 32, 4, 128, ctx=300, rows=1, norm=True, rope_base=1e6, interleaved=True,
             rotary=0, gate=True)


def test_long_positions_need_the_f64_angle_law():
    # At position ~100,000 an f32 angle is off by several 1e-3 rad; the f32 cache rows must
    # still be within 1e-6 of the oracle's.
    run_case("f32", 8, 2, 64, ctx=0, rows=3, norm=True, rope_base=1e4, interleaved=True, rotary=0,
             gate=False, seed=1)
    rng = np.random.default_rng(2)
    d, kv_heads, q_heads, pos = 128, 4, 32, 100_000
    pool = P().KvPool(1, kv_heads, d, elem="f32", capacity_rows=pos + 4)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    zeros = torch.zeros(pos, kv_heads * d, device="cuda")
    pool.append_device(0, [(cache, pos)], zeros.data_ptr(), zeros.data_ptr())
    q, k, v = normal(rng, 1, q_heads * d), normal(rng, 1, kv_heads * d), normal(rng, 1, kv_heads * d)
    out = torch.empty(1, q_heads * d, device="cuda")
    qd, kd, vd = dev(q), dev(k), dev(v)
    pool.attention_prep_step_device(0, [(cache, 1)], qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                                    out.data_ptr(), q_heads, rope_base=1e4, interleaved=True)
    torch.cuda.synchronize()
    _, gk, _ = cache.read_rows(0, pos, 1)
    want = oracle.attention_prep(k, kv_heads, d, pos, None, 1e-6, 1e4, True)
    assert max_abs(gk.reshape(1, -1), want) <= 1e-6
    pool.close()


@pytest.mark.parametrize("rows,norm,pos0", [(1, True, 0), (2, False, 50_000), (7, True, 50_000)])
def test_preparation_by_launch_stores_the_oracles_f16_keys_bit_for_bit(rows, norm, pos0):
    # ITAK_POOL_PREP_BY_LAUNCH: decode rows and short blocks at head_dim 128, which otherwise
    # prepare inside the attention launch in f32 (within one f16 step of the reference's chain:
    # a few stored elements in ten thousand differ), go through the f64 preparation launch.
    d, kvh, q_heads, window = 128, 4, 32, 128
    width = kvh * d
    rng = np.random.default_rng(rows + pos0)
    differing = {}
    for by_launch in (True, False):
        data = np.random.default_rng(rows + pos0 + 1)
        pool = P().KvPool([P().LayerKind.windowed(window)], kvh, d, elem="f16", ring_headroom=64,
                          capacity_rows=pos0 + 60 * rows + 200, prep_by_launch=by_launch)
        pool.set_stream(torch.cuda.current_stream().cuda_stream)
        cache = pool.acquire()
        if pos0:
            cache.restore_bulk(0, pos0 - window, normal(data, window, width), normal(data, window, width))
        w = 1.0 + 0.1 * normal(data, d)
        wd = dev(w)
        off = 0
        for rep in range(60):
            q, k, v = normal(data, rows, q_heads * d), normal(data, rows, width), normal(data, rows, width)
            qd, kd, vd = dev(q), dev(k), dev(v)
            out = torch.empty_like(qd)
            pool.attention_prep_step_device(0, [(cache, rows)], qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                                            out.data_ptr(), q_heads, q_norm_ptr=wd.data_ptr() if norm else 0,
                                            k_norm_ptr=wd.data_ptr() if norm else 0, eps=1e-6, rope_base=1e6,
                                            interleaved=True)
            torch.cuda.synchronize()
            kp = oracle.attention_prep(k, kvh, d, pos0 + rep * rows, w if norm else None, 1e-6, 1e6, True, None)
            _, gk, _ = cache.read_rows(0, cache.stored_len(0) - rows, rows)
            want = oracle.f32_to_f16_array(np.asarray(kp, dtype=np.float32).reshape(rows, width))
            off += int((np.asarray(gk).reshape(rows, width).view(np.int16) != want.view(np.int16)).sum())
        differing[by_launch] = off
        pool.close()
    assert differing[True] == 0, differing
    print(f"rows {rows}: stored f16 key elements that differ from the oracle's, folded form {differing[False]}, "
          f"by launch {differing[True]}, of {60 * rows * width}")


@pytest.mark.parametrize("pos,base,interleaved,rotary", [(100_000, 1e4, True, 0), (1_000_000, 1e6, True, 0),
                                                         (1_000_000, 1e4, False, 64)])
def test_rotated_f32_keys_at_long_positions_are_the_oracles_bit_for_bit(pos, base, interleaved, rotary):
    # The angle is position * base^(-2i/d): a last bit of the power is multiplied by the position,
    # and at 10^6 it moved a dozen of 65,536 stored elements by up to 16 units in the last place
    # while the kernel took the power from the device's library. The frequencies come from the
    # host's libm, which is the reference's.
    kvh, d, q_heads, window, rows = 2, 128, 4, 64, 64
    width = kvh * d
    rng = np.random.default_rng(pos + int(base))
    pool = P().KvPool([P().LayerKind.windowed(window)], kvh, d, elem="f32", capacity_rows=pos + 2 * rows + 8)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    cache.restore_bulk(0, pos - window, normal(rng, window, width), normal(rng, window, width))
    for rep in range(2):
        q, k, v = normal(rng, rows, q_heads * d), normal(rng, rows, width), normal(rng, rows, width)
        qd, kd, vd = dev(q), dev(k), dev(v)
        out = torch.empty_like(qd)
        pool.attention_prep_step_device(0, [(cache, rows)], qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                                        out.data_ptr(), q_heads, rope_base=base, interleaved=interleaved,
                                        rotary_dim=rotary)
        torch.cuda.synchronize()
        want = oracle.attention_prep(k, kvh, d, pos + rep * rows, None, 1e-6, base, interleaved, rotary or None)
        _, gk, _ = cache.read_rows(0, cache.stored_len(0) - rows, rows)
        assert np.asarray(gk).reshape(rows, width).tobytes() == np.asarray(want, dtype=np.float32).tobytes()
    pool.close()


@pytest.mark.parametrize("rows,interleaved,rotary,norm,rope_base", [
    (7, True, 0, True, 1e6), (7, False, 0, True, 1e4), (5, False, 64, False, 1e4),
    (5, True, 32, True, 5e5), (1, True, 0, True, 0.0), (200, True, 0, True, 1e6),
    # 9 to 64 rows: the preparation launch, then the block kernel that appends the prepared rows itself
    (20, True, 0, True, 1e6), (40, False, 64, True, 1e4), (64, True, 0, True, 5e5)])
def test_blocks_pairings_partial_rotary_and_nope(rows, interleaved, rotary, norm, rope_base):
    run_case("f16", 32, 4, 128, ctx=150, rows=rows, norm=norm, rope_base=rope_base,
             interleaved=interleaved, rotary=rotary, gate=(rows < 100), seed=rows)


@pytest.mark.parametrize("q_heads,rows,interleaved,rotary,norm,rope_base,ctx,window", [
    (32, 2, True, 0, True, 1e6, 150, None),     # 16 vectors, two positions in one tile
    (32, 2, False, 0, True, 1e4, 150, None),    # half split over the whole head
    (32, 2, False, 64, True, 1e4, 150, None),   # half split, partial rotary
    (32, 1, True, 32, False, 5e5, 150, None),   # partial interleaved, no norm
    (16, 4, True, 0, True, 1e6, 700, None),     # group 4, four rows
    (4, 8, False, 0, True, 1e4, 40, None),      # group 1, eight rows, single split
    (32, 1, True, 0, True, 1e6, 9, None),       # one split: the split kernel writes and gates the output
    (32, 1, False, 0, False, 0.0, 300, None),   # nothing to prepare: the gate alone
    (32, 1, True, 0, True, 1e4, 5000, 1024),    # sliding-window layer, ring wrapped
    (32, 2, True, 0, True, 1e4, 1500, 1024),
])
def test_steps_of_up_to_16_vectors_prepare_inside_the_attention_launch(q_heads, rows, interleaved,
                                                                       rotary, norm, rope_base, ctx,
                                                                       window):
    run_case("f16", q_heads, 4, 128, ctx=ctx, rows=rows, norm=norm, rope_base=rope_base,
             interleaved=interleaved, rotary=rotary, gate=True, seed=ctx + rows, window=window)


def test_folded_preparation_at_a_long_position_keeps_the_f16_bar():
    # Position ~100,000: the angle must be formed and reduced in f64 inside the kernel too.
    rng = np.random.default_rng(9)
    d, kv_heads, q_heads, pos = 128, 4, 32, 100_000
    pool = P().KvPool(1, kv_heads, d, elem="f16", capacity_rows=pos + 4)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    zeros = torch.zeros(pos, kv_heads * d, device="cuda")
    pool.append_device(0, [(cache, pos)], zeros.data_ptr(), zeros.data_ptr())
    q, k, v = normal(rng, 1, q_heads * d), normal(rng, 1, kv_heads * d), normal(rng, 1, kv_heads * d)
    out = torch.empty(1, q_heads * d, device="cuda")
    qd, kd, vd = dev(q), dev(k), dev(v)
    pool.attention_prep_step_device(0, [(cache, 1)], qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                                    out.data_ptr(), q_heads, rope_base=1e4, interleaved=True)
    torch.cuda.synchronize()
    _, gk, _ = cache.read_rows(0, pos, 1)
    want = oracle.f32_to_f16_array(oracle.attention_prep(k, kv_heads, d, pos, None, 1e-6, 1e4, True))
    ulp = np.abs(gk.reshape(-1).view(np.int16).astype(np.int32) - want.reshape(-1).view(np.int16).astype(np.int32))
    far = np.abs(gk.reshape(-1).view(np.float16).astype(np.float64)
                 - want.reshape(-1).view(np.float16).astype(np.float64))
    assert np.all((ulp <= 1) | (far <= 1e-6))
    pool.close()


def test_several_slots_each_at_its_own_position():
    run_case("f16", 32, 4, 128, ctx=90, rows=1, norm=True, rope_base=1e6, interleaved=True, rotary=0,
             gate=True, seed=5, slots=5)
    run_case("f32", 8, 2, 64, ctx=40, rows=3, norm=True, rope_base=1e4, interleaved=False, rotary=0,
             gate=True, seed=6, slots=3)


def test_bad_preparation_parameters_are_refused_by_name():
    pool = P().KvPool(1, 4, 128, elem="f16", capacity_rows=16)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    t = torch.zeros(1, 32 * 128, device="cuda")
    w = torch.ones(128, device="cuda")
    args = (0, [(cache, 1)], t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), 32)
    for kw, text in ((dict(q_norm_ptr=w.data_ptr(), eps=0.0), "eps must be finite and > 0"),
                     (dict(rope_base=1.0), "base must be finite and > 1"),
                     (dict(rope_base=1e4, rotary_dim=130), "rotary_dim must be even"),
                     (dict(rope_base=1e4, rotary_dim=3), "rotary_dim must be even")):
        with pytest.raises(P().StepFailed) as e:
            pool.attention_prep_step_device(*args, **kw)
        assert text in str(e.value)
    assert cache.next_position(0) == 0  # nothing was appended by a refused step
    pool.close()
