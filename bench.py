"""Benchmark of the decode hot path on one MI355X.

Workload (BASELINE.json configs[1]): 30B-class decode step, batch 1, 48 layers, 32 Q / 4 KV
heads, head_dim 128, f16 KV cache at context 4096, K pre-rotated with RoPE base 1e6. One
step = one token: every layer appends one K/V row (f32 -> f16 RNE) at position 4096 and
runs GQA flash-decode over the 4097 stored positions. All inputs are resident in HBM before
the timed region. After each step the cache is truncated back to 4096 positions (a host-side
length update; nothing is enqueued), so every step does the same work at the same context.

Prints one JSON line: decode-attention KV GB/s over the algorithmic KV bytes
(2 * 4097 * 4 * 128 * 2 B per layer), with the roofline figures of the dominant kernel and
the CPU oracle timed on the host cores beside it.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

LAYERS, Q_HEADS, KV_HEADS, D, CTX = 48, 32, 4, 128, 4096
ROW = KV_HEADS * D
KV_BYTES_PER_LAYER = 2 * (CTX + 1) * KV_HEADS * D * 2  # K and V rows visible after the append
HBM_PEAK_GBS = 8000.0


def rope_on_device(x, base):
    """Half-split RoPE at positions 0..n-1, float64 angles (input generation only)."""
    import torch

    n, heads, d = x.shape
    half = d // 2
    pos = torch.arange(n, dtype=torch.float64, device=x.device)[:, None]
    i = torch.arange(half, dtype=torch.float64, device=x.device)[None, :]
    ang = pos * torch.pow(torch.tensor(base, dtype=torch.float64, device=x.device), -2.0 * i / d)
    s, c = torch.sin(ang)[:, None, :], torch.cos(ang)[:, None, :]
    a, b = x[..., :half].double(), x[..., half:].double()
    return torch.cat([(a * c - b * s).float(), (a * s + b * c).float()], dim=-1)


def cpu_baseline(budget_s: float = 12.0):
    """The CPU oracle (a port of the reference's single-threaded Rust path) on the same
    step: append one row at position 4096, attend over 4097 positions, f16-rounded KV."""
    import numpy as np

    import oracle

    rng = np.random.default_rng(0)
    k = oracle.rope_rows(rng.standard_normal((CTX + 1, KV_HEADS, D), dtype=np.float32), 0, 1e6)
    k = k.reshape(CTX + 1, ROW)
    v = rng.standard_normal((CTX + 1, ROW), dtype=np.float32)
    q = rng.standard_normal((1, Q_HEADS * D), dtype=np.float32)
    cache = oracle.KvCache.new([oracle.LayerKind.Global], KV_HEADS, D, store_f16=True)
    cache.restore_bulk(0, 0, k[:CTX], v[:CTX])
    done, spent = 0, 0.0
    while spent < budget_s or done < 4:
        cp = cache.checkpoint(1)
        t0 = time.perf_counter()
        oracle.attention_step(cache, 0, q, k[CTX:], v[CTX:], Q_HEADS, CTX, threads=1)
        spent += time.perf_counter() - t0
        cache.rewind_to(cp, CTX)
        cache.release(cp)
        done += 1
    per_layer = spent / done
    return {
        "value": round(KV_BYTES_PER_LAYER / per_layer / 1e9, 4),
        "unit": "GB/s",
        "cores": 1,
        "kind": "port",
        "us_per_token": round(per_layer * LAYERS * 1e6, 1),
        "sample": f"{done} layer-steps of the same decode step (append + attend over "
                  f"{CTX + 1} positions), single thread; per-token figure is x{LAYERS} layers",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches only")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (run with --gpus 1)",
              file=sys.stderr)
        sys.exit(2)

    import torch

    from __graft_entry__ import load_package

    pkg = load_package()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.manual_seed(0)

    pool = pkg.KvPool(LAYERS, KV_HEADS, D, elem="f16", max_slots=1, capacity_rows=CTX + 8,
                      scrub_on_truncate=False)
    stream = torch.cuda.current_stream()
    pool.set_stream(stream.cuda_stream)
    cache = pool.acquire()

    # Synthetic inputs, resident in HBM: per-layer prefix K/V, per-layer new K/V row and Q.
    q = torch.randn(LAYERS, 1, Q_HEADS * D, device=dev)
    k_new = torch.randn(LAYERS, 1, ROW, device=dev)
    v_new = torch.randn(LAYERS, 1, ROW, device=dev)
    out = torch.empty_like(q)
    for layer in range(LAYERS):
        k = rope_on_device(torch.randn(CTX, KV_HEADS, D, device=dev), 1e6).reshape(CTX, ROW)
        v = torch.randn(CTX, ROW, device=dev)
        pool.append_device(layer, [(cache, CTX)], k.contiguous().data_ptr(), v.data_ptr())
        torch.cuda.synchronize()
    ptrs = [(q[l].data_ptr(), k_new[l].data_ptr(), v_new[l].data_ptr(), out[l].data_ptr())
            for l in range(LAYERS)]
    item = [(cache, 1)]

    def token_step():
        for layer in range(LAYERS):
            qp, kp, vp, op = ptrs[layer]
            pool.attention_step_device(layer, item, qp, kp, vp, op, Q_HEADS)
        pool.truncate([cache], [CTX])

    def attention_only():
        for layer in range(LAYERS):
            qp, _, _, op = ptrs[layer]
            pool.attention_device(layer, item, qp, op, Q_HEADS)

    def timed(fn, steps):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        start.record(stream)
        for _ in range(steps):
            fn()
        end.record(stream)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        return start.elapsed_time(end) * 1e-3, wall  # seconds on the stream, wall seconds

    for _ in range(max(args.warmup, 1)):
        token_step()
    torch.cuda.synchronize()

    eager_gpu_s, eager_wall_s = timed(token_step, args.steps)

    use_graph = not args.no_graph
    graph_s = None
    attn_launch_s = None
    if use_graph:
        # One token step (48 appends + 48 decode launches) captured once, replayed per step:
        # the launch-bound loop a serving engine would keep in a HIP graph.
        cap = torch.cuda.Stream()
        cap.wait_stream(stream)
        g_step, g_attn = torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()
        with torch.cuda.stream(cap):
            pool.set_stream(cap.cuda_stream)
            with torch.cuda.graph(g_step, stream=cap):
                token_step()
            # Attention launches alone, on a cache that holds 4097 positions.
            pool.append_device(0, item, ptrs[0][1], ptrs[0][2])
            for layer in range(1, LAYERS):
                pool.append_device(layer, item, ptrs[layer][1], ptrs[layer][2])
            with torch.cuda.graph(g_attn, stream=cap):
                attention_only()
        torch.cuda.synchronize()
        pool.set_stream(stream.cuda_stream)
        for _ in range(max(args.warmup, 1)):
            g_step.replay()
        graph_s, _ = timed(g_step.replay, args.steps)
        for _ in range(max(args.warmup, 1)):
            g_attn.replay()
        attn_s, _ = timed(g_attn.replay, args.steps)
        attn_launch_s = attn_s / (args.steps * LAYERS)
        pool.truncate([cache], [CTX])

    step_s = (graph_s if graph_s is not None else eager_gpu_s) / args.steps
    bytes_per_token = KV_BYTES_PER_LAYER * LAYERS
    value = bytes_per_token / step_s / 1e9
    if attn_launch_s is None:
        attn_launch_s = eager_gpu_s / (args.steps * LAYERS)
    achieved = KV_BYTES_PER_LAYER / attn_launch_s / 1e9

    result = {
        "metric": "decode-attn KV GB/s (all layers, ctx 4096)",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32 arithmetic over f16 KV",
        "data": "synthetic",
        "config": {
            "workload": "configs[1]: 30B-class decode step, batch 1, 48 layers, 32 Q / 4 KV "
                        "heads, head_dim 128, f16 KV, context 4096, append 1 token per layer "
                        "then flash-decode",
            "launch": "HIP graph replay of one token step" if graph_s is not None else "eager",
            "kv_bytes_per_token": bytes_per_token,
        },
        "us_per_token": round(step_s * 1e6, 2),
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "eager": {
            "us_per_token_stream": round(eager_gpu_s / args.steps * 1e6, 2),
            "us_per_token_wall": round(eager_wall_s / args.steps * 1e6, 2),
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "decode attention (one launch per layer)",
            "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": None,
            "us_per_launch": round(attn_launch_s * 1e6, 3),
            "bytes_per_launch": KV_BYTES_PER_LAYER,
        },
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))
    pool.close()


if __name__ == "__main__":
    main()
