"""itak_attention_device: the attention half of a step alone, over rows the slots already hold
(each item's last `rows` positions are its queries' positions). What bench.py times for the
prefill chunk. Held to the oracle's gqa_attention over the slot's view (attention.rs:104-215) with
those positions as the queries' at drawn shapes: element type, head_dim, groups, slots, contexts
and row counts, global and windowed layers. On a global layer that equals the append-then-attend
step; on a windowed layer it does not, and is not meant to: the view starts at the window of the
newest row, so an earlier query row sees only what of its own window is still in the view.

Bars as everywhere: f16 KV 2e-3 max-abs, f32 KV 1e-5 relative."""
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


@pytest.mark.parametrize("seed", range(36))
def test_attention_over_rows_already_stored(seed):
    rng = np.random.default_rng(seed + 90210)
    elem = "f16" if seed % 4 else "f32"
    d = int(rng.choice([64, 128] if elem == "f32" else [64, 96, 128, 128, 128, 256]))
    kvh = int(rng.choice([1, 2, 4, 8]))
    q_heads = kvh * int(rng.choice([1, 2, 3, 4, 8, 16]))
    window = None if rng.random() < 0.6 else int(rng.integers(8, 600))
    slots = int(rng.choice([1, 1, 2, 4]))
    softcap = float(rng.choice([0.0, 0.0, 30.0]))
    headroom = 256
    contexts = [int(rng.choice([0, rng.integers(1, 100), rng.integers(100, 3000)])) for _ in range(slots)]
    rows = [int(rng.choice([1, rng.integers(2, 9), rng.integers(9, 65), rng.integers(65, 250)])) for _ in range(slots)]
    row = kvh * d
    kind = P().LayerKind.Global if window is None else P().LayerKind.windowed(window)
    okind = oracle.LayerKind.Global if window is None else oracle.LayerKind.windowed(window)
    pool = P().KvPool([kind], kvh, d, elem=elem, max_slots=slots, capacity_rows=max(contexts) + max(rows) + 8,
                      ring_headroom=headroom)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    caches = [pool.acquire() for _ in range(slots)]
    refs = [oracle.KvCache.new([okind], kvh, d, store_f16=(elem == "f16")) for _ in range(slots)]
    for cache, ref, n, r in zip(caches, refs, contexts, rows):
        k, v = normal(rng, n + r, row), normal(rng, n + r, row)
        for first in range(0, n + r, 200):  # in pieces a ring's headroom takes; the last r rows are the step's
            m = min(200, n + r - first)
            kd, vd = dev(k[first:first + m]), dev(v[first:first + m])
            pool.append_device(0, [(cache, m)], kd.data_ptr(), vd.data_ptr())
            pool.synchronize()
        for i in range(n + r):
            ref.append(0, k[i], v[i], i)
    q = normal(rng, sum(rows), q_heads * d)
    qd = dev(q)
    out = torch.full_like(qd, float("nan"))
    # More query rows than the window: the first of them stands before the view's first row and
    # sees nothing. The reference refuses by that position (attention.rs:160-173), and so does the
    # call, before anything is launched.
    blind = [n for n, r in zip(contexts, rows) if window is not None and r > window]
    if blind:
        with pytest.raises(P().AttentionError) as e:
            pool.attention_device(0, list(zip(caches, rows)), qd.data_ptr(), out.data_ptr(), q_heads,
                                  softcap=softcap)
        assert e.value == P().AttentionError("NoVisibleKeys", position=blind[0])
        pool.synchronize()
        assert torch.isnan(out).all()
        pool.close()
        return
    pool.attention_device(0, list(zip(caches, rows)), qd.data_ptr(), out.data_ptr(), q_heads, softcap=softcap)
    pool.synchronize()
    got, at = out.cpu().numpy(), 0
    for ref, n, r in zip(refs, contexts, rows):
        want = oracle.gqa_attention(q[at:at + r], r, q_heads, [n + i for i in range(r)], ref.view(0),
                                    oracle.AttentionParams(softcap=softcap), threads=8)
        mine = got[at:at + r].reshape(-1)
        err = max_abs(mine, want) if elem == "f16" else rel_err(mine, want)
        assert err <= (2e-3 if elem == "f16" else 1e-5), (seed, n, r, err)
        at += r
    for cache, n, r in zip(caches, contexts, rows):
        assert cache.next_position(0) == n + r  # nothing appended, nothing dropped
    pool.close()
