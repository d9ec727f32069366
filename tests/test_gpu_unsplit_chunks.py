"""Unsplit causal chunks on the block kernel's two-tile form (a prompt's first chunks, and chunks
with enough row tiles to fill the device without splitting the context): the launch order of
their row tiles is the planner's to choose (longest first, every second run reversed), so the
chunk lengths here leave odd and even numbers of tiles and ragged last tiles, at every group
padding, with several unsplit items in one launch and over prefixes, against the CPU oracle over
the same f16-rounded cache.

Bars as everywhere: outputs within 2e-3 max-abs, stored rows bit-exact."""
import numpy as np
import pytest
import torch

import oracle
from helpers import max_abs, normal, pkg

pytestmark = pytest.mark.gpu

THREADS = 8


def P():
    return pkg()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def new_pool(kv_heads, d, slots, capacity):
    pool = P().KvPool([P().LayerKind.Global], kv_heads, d, elem="f16", max_slots=slots, capacity_rows=capacity)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    return pool


# (q_heads, kv_heads): groups of 8, 1, 3 (padded to 4), 16, 2 and 5 (padded to 8) heads a row.
SHAPES = [(32, 4), (8, 8), (12, 4), (16, 1), (16, 8), (40, 8)]


@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize("q_heads,kv_heads", SHAPES)
@pytest.mark.parametrize("softcap", [0.0, 30.0])
def test_first_chunks_of_a_prompt_on_every_row(d, q_heads, kv_heads, softcap):
    # Lengths chosen per shape so that the context stays under 40 blocks with at least 48
    # (row tile, KV head) units, which the planner leaves unsplit: even and odd numbers of
    # wavefront tiles, and a last one that is not full.
    gp = next(x for x in (1, 2, 4, 8, 16) if x >= q_heads // kv_heads)
    half_rows = 64 // gp
    most = 39 * 32
    lengths = sorted({most, most - half_rows, most - half_rows - 3, (most // half_rows - 4) * half_rows + 1, most // 2 + 5})
    rng = np.random.default_rng(q_heads * 131 + d)
    row = kv_heads * d
    for rows in lengths:
        units = kv_heads * -(-rows // (2 * half_rows))
        if units < 48:
            continue
        pool = new_pool(kv_heads, d, 1, rows)
        cache = pool.acquire()
        q, k, v = normal(rng, rows, q_heads * d), normal(rng, rows, row), normal(rng, rows, row)
        qd, kd, vd = dev(q), dev(k), dev(v)
        out = torch.empty_like(qd)
        pool.attention_step_device(0, [(cache, rows)], qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                                   out.data_ptr(), q_heads, softcap=softcap)
        torch.cuda.synchronize()
        ref = oracle.KvCache.new([oracle.LayerKind.Global], kv_heads, d, store_f16=True)
        want = oracle.attention_step(ref, 0, q, k, v, q_heads, 0, oracle.AttentionParams(softcap=softcap),
                                     threads=THREADS)
        got = out.cpu().numpy().reshape(-1)
        err = max_abs(got, want)
        assert err <= 2e-3, (rows, err)
        _, gk, gv = cache.read_rows(0, 0, rows)
        assert np.array_equal(gk.reshape(rows, row), oracle.f32_to_f16_array(k))
        assert np.array_equal(gv.reshape(rows, row), oracle.f32_to_f16_array(v))
        pool.close()


def test_several_unsplit_chunks_in_one_launch():
    # Three slots, each with a first chunk of its own length, and then a second chunk each over
    # what the first stored (short enough to stay unsplit).
    d, q_heads, kv_heads = 128, 32, 4
    row = kv_heads * d
    rng = np.random.default_rng(11)
    pool = new_pool(kv_heads, d, 3, 1300)
    caches = [pool.acquire() for _ in range(3)]
    refs = [oracle.KvCache.new([oracle.LayerKind.Global], kv_heads, d, store_f16=True) for _ in range(3)]
    for lengths in ((520, 777, 391), (300, 410, 260)):
        total = sum(lengths)
        q, k, v = normal(rng, total, q_heads * d), normal(rng, total, row), normal(rng, total, row)
        qd, kd, vd = dev(q), dev(k), dev(v)
        out = torch.empty_like(qd)
        pool.attention_step_device(0, list(zip(caches, lengths)), qd.data_ptr(), kd.data_ptr(), vd.data_ptr(),
                                   out.data_ptr(), q_heads)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        at = 0
        for ref, n in zip(refs, lengths):
            base = ref.next_position(0)
            want = oracle.attention_step(ref, 0, q[at:at + n], k[at:at + n], v[at:at + n], q_heads, base,
                                         threads=THREADS)
            err = max_abs(got[at:at + n].reshape(-1), want)
            assert err <= 2e-3, (lengths, n, err)
            at += n
    pool.close()


@pytest.mark.parametrize("prefix,chunk", [(1000, 1541), (0, 2048), (4096, 2048)])
def test_long_chunks_over_a_prefix(prefix, chunk):
    # Enough row tiles that the planner leaves the chunk unsplit whatever the context. Rows at
    # and beside every kind of boundary (wavefront tiles of 8 rows, the middle of the chunk where
    # the reversed run meets the first, key blocks of 32) plus a stride through the rest are evaluated by the oracle at their full context.
    d, q_heads, kv_heads = 128, 32, 4
    row = kv_heads * d
    rng = np.random.default_rng(prefix + chunk)
    f16 = lambda a: a.astype(np.float16).astype(np.float32)  # noqa: E731
    k, v = f16(normal(rng, prefix + chunk, row)), f16(normal(rng, prefix + chunk, row))
    q = f16(normal(rng, chunk, q_heads * d))
    pool = new_pool(kv_heads, d, 1, prefix + chunk)
    cache = pool.acquire()
    kd, vd, qd = dev(k), dev(v), dev(q)
    out = torch.empty_like(qd)
    if prefix:
        pool.append_device(0, [(cache, prefix)], kd.data_ptr(), vd.data_ptr())
    pool.attention_step_device(0, [(cache, chunk)], qd.data_ptr(), kd[prefix:].data_ptr(), vd[prefix:].data_ptr(),
                               out.data_ptr(), q_heads)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    ref = oracle.KvCache.new([oracle.LayerKind.Global], kv_heads, d, store_f16=True)
    ref.restore_bulk(0, 0, k, v)
    edges = {0, 1, 7, 8, 9, 15, 16, 31, 32, 33, chunk // 2 - 9, chunk // 2 - 8, chunk // 2 - 1, chunk // 2,
             chunk // 2 + 7, chunk // 2 + 8, chunk - 17, chunk - 9, chunk - 8, chunk - 2, chunk - 1}
    rows = sorted(edges | set(range(3, chunk, 61)))
    want = oracle.gqa_attention(q[rows], len(rows), q_heads, [prefix + r for r in rows], ref.view(0),
                                threads=THREADS).reshape(len(rows), -1)
    err = max_abs(got[rows], want)
    assert err <= 2e-3, err
    _, gk, gv = cache.read_rows(0, prefix, chunk)
    assert np.array_equal(gk.reshape(chunk, row), oracle.f32_to_f16_array(k[prefix:]))
    assert np.array_equal(gv.reshape(chunk, row), oracle.f32_to_f16_array(v[prefix:]))
    pool.close()
