"""Benchmark of the KV-cache + attention hot path on one MI355X.

Default workload (BASELINE.json configs[1], the one the metric is quoted on): 30B-class decode
step, batch 1, 48 layers, 32 Q / 4 KV heads, head_dim 128, f16 KV cache at context 4096, K
pre-rotated with RoPE base 1e6. One step = one token: every layer appends one K/V row
(f32 -> f16 RNE) at position 4096 and runs GQA flash-decode over the 4097 stored positions.
All inputs are resident in HBM before the timed region. After each step the cache is
truncated back to 4096 positions (a host-side length update; nothing is enqueued), so every
step does the same work at the same context.

Prints one JSON line: decode-attention KV GB/s over the algorithmic KV bytes
(2 * 4097 * 4 * 128 * 2 B per layer), with the roofline figures of the attention launches and
the CPU oracle timed on the host cores beside it.

`--prep` adds a second timing of the same step preceded by the model's Q/K preparation
(per-head RMSNorm, RoPE) and followed by its sigmoid gate (`with_prep` in the JSON line).

`--workload ragged|verify|prefill` measures the other configurations (continuous batching
over 16 ragged slots, the speculative verify block, the chunked causal prefill) with the
same JSON shape; `--workload hybrid` a decode step over the reference model's own layer
pattern (three sliding-window layers of 2048 to one global layer, crates/attention/src/
cache.rs:66-84) at context 32768; `--workload prefill_windowed` a 2048-row prefill chunk on
sliding-window layers; `--workload restore|append` measures the cache-maintenance kernels (the
48-layer prefix-snapshot gather of configs[4]; the append of a 2048-row chunk). They are
secondary measurements, the default line is the contract. `--kv f32` runs the decode or ragged
workload on an f32 cache, the reference's own storage (twice the bytes per row).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

Q_HEADS, KV_HEADS, D = 32, 4, 128
ROW = KV_HEADS * D
HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0

# HBM bytes per layer (all launches of the layer's attention) as rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE counted them in an earlier run, scaled by the same counters on the probe copy of
# known size: (bytes, the summary under profiles/ that holds the run and the scaling factors).
# They are not measured by this run: `traffic_source` says where each came from.
PROFILE_TRAFFIC = {
    ("decode", "f16"): (9_805_775, "profiles/attn_decode_f16_ctx4096_traffic.md"),
    ("ragged", "f16"): (216_797_776, "profiles/attn_splitk_f16_ragged16_traffic.md"),
    ("prefill", "f16"): (201_442_441, "profiles/attn_prefill_f16_chunk2048_prefix30720_traffic.md"),
    ("verify", "f16"): (87_437_369, "profiles/attn_splitk_f16_verify_traffic.md"),
    ("decode", "f32"): (18_240_825, "profiles/attn_splitk_f32_decode_ctx4096_traffic.md"),
}


def host_cpu():
    """Model name and logical CPU count of the host the baseline is timed on."""
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return model, os.cpu_count()


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


def cpu_baseline(ctx: int, kv_bytes_per_layer: int, layers: int, budget_s: float = 12.0,
                 store_f16: bool = True):
    """The CPU oracle (a port of the reference's single-threaded Rust path) on the decode
    step: append one row at position ctx, attend over ctx + 1 positions, f16-rounded KV (or f32
    rows, as the reference stores them, with store_f16=False)."""
    import numpy as np

    import oracle

    rng = np.random.default_rng(0)
    k = oracle.rope_rows(rng.standard_normal((ctx + 1, KV_HEADS, D), dtype=np.float32), 0, 1e6)
    k = k.reshape(ctx + 1, ROW)
    v = rng.standard_normal((ctx + 1, ROW), dtype=np.float32)
    q = rng.standard_normal((1, Q_HEADS * D), dtype=np.float32)
    cache = oracle.KvCache.new([oracle.LayerKind.Global], KV_HEADS, D, store_f16=store_f16)
    cache.restore_bulk(0, 0, k[:ctx], v[:ctx])
    done, spent = 0, 0.0
    while spent < budget_s or done < 4:
        cp = cache.checkpoint(1)
        t0 = time.perf_counter()
        oracle.attention_step(cache, 0, q, k[ctx:], v[ctx:], Q_HEADS, ctx, threads=1)
        spent += time.perf_counter() - t0
        cache.rewind_to(cp, ctx)
        cache.release(cp)
        done += 1
    per_layer = spent / done
    model, logical = host_cpu()
    return {
        "value": round(kv_bytes_per_layer / per_layer / 1e9, 4),
        "unit": "GB/s",
        "cores": 1,
        "kind": "port",
        "cpu_model": model,
        "nproc": logical,
        "us_per_token": round(per_layer * layers * 1e6, 1),
        "sample": f"{done} layer-steps of the decode step (append + attend over {ctx + 1} "
                  f"positions, 32 Q / 4 KV heads, d=128, {'f16-rounded' if store_f16 else 'f32'} KV), single thread; the "
                  f"per-token figure is x{layers} layers",
    }


def cache_maintenance(args, pkg, torch, dev, stream, timed):
    """restore: the 8192-token x 48-layer prefix snapshot of configs[4] gathered into the
    device cache (f16 rows copied raw, f32 rows converted like append), from a source in HBM
    (the kernel's own speed) and from pinned host memory (what a session start pays: the
    host link). append: a 2048-row chunk per layer, f32 -> f16, into a cache of 30720 rows."""
    layers, tokens = 48, 8192
    if args.workload == "append":
        layers, prefix, chunk = 8, 30720, 2048
        pool = pkg.KvPool(layers, KV_HEADS, D, elem="f16", max_slots=1,
                          capacity_rows=prefix + chunk, scrub_on_truncate=False)
        pool.set_stream(stream.cuda_stream)
        cache = pool.acquire()
        k = torch.randn(layers, chunk, ROW, device=dev)
        v = torch.randn(layers, chunk, ROW, device=dev)
        zero = torch.zeros(prefix, ROW, device=dev)
        for layer in range(layers):
            pool.append_device(layer, [(cache, prefix)], zero.data_ptr(), zero.data_ptr())

        def step():
            for layer in range(layers):
                pool.append_device(layer, [(cache, chunk)], k[layer].data_ptr(), v[layer].data_ptr())
            pool.truncate([cache], [prefix])

        for _ in range(max(args.warmup, 1)):
            step()
        graph = capture(torch, pool, stream, step)
        pool.truncate([cache], [prefix])
        graph.replay()
        step_s = timed(graph.replay, args.steps)[0] / args.steps
        bytes_layer = chunk * 2 * ROW * (4 + 2)
        gbs = bytes_layer * layers / step_s / 1e9
        result = {
            "metric": "KV append GB/s (2048-row chunk, f32 -> f16, bytes read + written)",
            "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 5),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
            "data": "synthetic",
            "config": {"workload": "append of a 2048-row chunk per layer into a 30720-row f16 cache, "
                                   "8 layers cycled, HIP graph replay", "layers_per_step": layers},
            "roofline": {"bound": "hbm", "kernel": "kv_append_kernel (rows up to the block boundary) + "
                                                   "kv_restore_blocked (chunk append, per layer)", "achieved": round(gbs, 2),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                         "traffic": None, "us_per_launch": round(step_s / layers * 1e6, 3),
                         "bytes_per_launch": bytes_layer},
        }
        pool.close()
        return result

    pool = pkg.KvPool(layers, KV_HEADS, D, elem="f16", max_slots=1, capacity_rows=tokens,
                      scrub_on_truncate=False)
    pool.set_stream(stream.cuda_stream)
    cache = pool.acquire()
    elems = layers * tokens * ROW
    dev_k = torch.randn(layers, tokens, ROW, device=dev).half()
    dev_v = torch.randn(layers, tokens, ROW, device=dev).half()
    pin_k16, pin_v16 = dev_k.cpu().pin_memory(), dev_v.cpu().pin_memory()
    pin_k32, pin_v32 = dev_k.float().cpu().pin_memory(), dev_v.float().cpu().pin_memory()

    def restore_from(k, v, f16):
        # The layer table is the caller's and built once: indexing 96 tensors for their
        # addresses takes PyTorch longer than the gather takes the device.
        table = cache.snapshot_layer_table([(0, tokens, k[l].data_ptr(), v[l].data_ptr())
                                            for l in range(layers)])

        def run():
            cache.restore_snapshot_ptrs(tokens, table, src_f16=f16)
            pool.truncate([cache], [0])
        run()
        reps = max(3, min(args.steps, 20))
        return timed(run, reps)[0] / reps

    dst_bytes = 2 * elems * 2
    t_dev = restore_from(dev_k, dev_v, True)
    t_pin16 = restore_from(pin_k16, pin_v16, True)
    t_pin32 = restore_from(pin_k32, pin_v32, False)
    gbs = 2 * dst_bytes / t_dev / 1e9  # reads the f16 source and writes the planes

    # The same prefix through the prefix store (entry file in the page cache): lookup with
    # its trust checks, the payload read into the store's pinned buffer, the byte-serial
    # FNV-1a checksum of the format, then the gather. ITKV version 1 (f32 rows, the
    # reference's) against version 2 (the pool's own f16 rows).
    import shutil
    import tempfile
    store_ms = {}
    root = tempfile.mkdtemp(prefix="itak-bench-store-")
    try:
        token_ids = list(range(1, tokens + 1))
        restore_from(dev_k, dev_v, True)  # leaves the slot empty; fill it once more
        cache.restore_snapshot_ptrs(tokens, [(0, tokens, dev_k[l].data_ptr(), dev_v[l].data_ptr())
                                             for l in range(layers)], src_f16=True)
        for elem in ("f32", "f16"):
            store = pkg.PrefixStore.open(os.path.join(root, elem), 1 << 40)
            t0 = time.perf_counter()
            store.capture_and_put(cache, token_ids, "bench-model", now=1, elem=elem)
            put_s = time.perf_counter() - t0
            other = pool  # restore into the same pool: free the slot first
            entry_bytes = store.stats().total_bytes
            pool.truncate([cache], [0])
            t0 = time.perf_counter()
            matched = store.restore_prefix(cache, token_ids + [7], "bench-model", now=2)
            pool.synchronize()
            restore_s = time.perf_counter() - t0
            assert matched == tokens
            store_ms[elem] = {"entry_bytes": entry_bytes, "capture_and_put_ms": round(put_s * 1e3, 1),
                              "lookup_and_restore_ms": round(restore_s * 1e3, 1)}
            store.close()
    finally:
        shutil.rmtree(root, ignore_errors=True)
    result = {
        "metric": "prefix-snapshot restore GB/s (48 layers x 8192 rows, source in HBM, bytes read + written)",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(t_dev * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "configs[4] restore: 8192-token x 48-layer snapshot gathered into the "
                               "f16 device cache", "snapshot_bytes_f16": dst_bytes},
        "from_pinned_host": {
            "f16_rows_ms": round(t_pin16 * 1e3, 3),
            "f16_rows_GBps_over_link": round(dst_bytes / t_pin16 / 1e9, 2),
            "f32_rows_ms": round(t_pin32 * 1e3, 3),
            "f32_rows_GBps_over_link": round(2 * dst_bytes / t_pin32 / 1e9, 2),
        },
        "through_the_prefix_store": store_ms,
        "roofline": {"bound": "hbm", "kernel": "kv_restore_blocked (all layers, one launch)",
                     "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "us_per_launch": round(t_dev * 1e6, 2), "bytes_per_launch": 2 * dst_bytes,
                     "timed": "eager calls one after another with a prebuilt layer table, HIP events "
                              "on the stream: the host's share of a call (an address class per "
                              "source, the launch) hides behind the previous call's kernel"},
    }
    pool.close()
    return result


def timeline(args, pkg, torch, np):
    """Where a decode layer's time goes: the stage timestamps that the measurement build of the
    library records in every wavefront (csrc/timeline.h), read after HIP-graph replays of the
    default workload's step and printed as a table, times in ns from the attention kernel's
    first wavefront's first instruction. The layer shown is the last of the 48."""
    import ctypes as C

    lib_path = os.path.join(os.path.dirname(pkg._native.LIB_PATH), "libitak_hip_kv_timeline.so")
    if not os.path.exists(lib_path):
        print("bench.py --timeline needs the measurement build: run "
              "`python itak-torch-rebuild_amd/build.py --timeline` first", file=sys.stderr)
        sys.exit(2)
    pkg._native.LIB_PATH = lib_path
    pkg._native.load()
    raw = C.CDLL(lib_path)
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream()
    if args.workload in ("verify", "ragged"):
        return timeline_splitk(args, pkg, torch, np, raw, dev, stream)
    layers, ctx = 48, 4096
    pool = pkg.KvPool(layers, KV_HEADS, D, elem="f16", max_slots=1, capacity_rows=ctx + 8,
                      scrub_on_truncate=False, merge_in_launch=args.merge_in_launch)
    pool.set_stream(stream.cuda_stream)
    cache = pool.acquire()
    torch.manual_seed(0)
    for layer in range(layers):
        k = rope_on_device(torch.randn(ctx, KV_HEADS, D, device=dev), 1e6).reshape(ctx, ROW).contiguous()
        v = torch.randn(ctx, ROW, device=dev)
        pool.append_device(layer, [(cache, ctx)], k.data_ptr(), v.data_ptr())
        torch.cuda.synchronize()
    q = torch.randn(layers, 1, Q_HEADS * D, device=dev)
    k_new, v_new = torch.randn(layers, 1, ROW, device=dev), torch.randn(layers, 1, ROW, device=dev)
    out = torch.empty_like(q)

    def step():
        for layer in range(layers):
            pool.attention_step_device(layer, [(cache, 1)], q[layer].data_ptr(), k_new[layer].data_ptr(),
                                       v_new[layer].data_ptr(), out[layer].data_ptr(), Q_HEADS,
                                       softcap=args.softcap)
        pool.truncate([cache], [ctx])

    for _ in range(3):
        step()
    graph = capture(torch, pool, stream, step)
    marks, waves = 12, 8192
    buf = np.zeros(waves * marks, dtype=np.uint64)
    decode_rows, merge_rows = [], []
    for _ in range(max(args.steps // 10, 8)):
        graph.replay()
        torch.cuda.synchronize()
        t0 = None
        for reader, second_half in (("itak_timeline_read_decode", False), ("itak_timeline_read_splitk", True)):
            rc = getattr(raw, reader)(buf.ctypes.data_as(C.c_void_p), C.c_ulonglong(buf.size))
            assert rc == 0, f"{reader} failed with HIP error {rc}"
            t = buf.reshape(waves, marks).astype(np.int64)
            t = t[waves // 2:] if second_half else t[:waves // 2]
            t = t[t[:, 0] > 0]
            if not second_half:
                if len(t) == 0:
                    print("no decode kernel records: the step did not take attn_decode_f16_kernel",
                          file=sys.stderr)
                    sys.exit(1)
                t0 = t[:, 0].min()
                decode_rows.append((t - t0) * 10)
            elif len(t):
                merge_rows.append((t - t0) * 10)
    step_s = Timer(torch, stream)(graph.replay, 50)[0] / 50

    def table(title, rows, names):
        print(title)
        allr = np.concatenate(rows)
        for i, name in names:
            col = allr[:, i]
            col = col[col > -10**9]
            if len(col) == 0 or col.max() <= 0 and i:
                continue
            print(f"  {name:44s} min {col.min():6d}  p50 {int(np.median(col)):6d}  "
                  f"p90 {int(np.percentile(col, 90)):6d}  max {col.max():6d} ns")

    print(f"decode layer timeline: batch 1, context {ctx}, 48 layers as one HIP graph, "
          f"{'splits merged inside the launch' if args.merge_in_launch else 'merge launch'}; "
          f"{step_s / layers * 1e6:.2f} us per layer with the timestamps compiled in")
    table(f"attn_decode_f16_kernel ({decode_rows[0].shape[0]} wavefronts per launch)", decode_rows, [
        (0, "first instruction"), (1, "kernel arguments in, addresses known"),
        (2, "every load issued"), (3, "scores done (keys and queries arrived)"),
        (4, "O^T written to LDS (values arrived)"), (5, "past the workgroup barrier"),
        (6, "partials / exchange words issued"), (7, "every exchange word gathered"),
        (11, "everything in flight done (stores acknowledged)")])
    if merge_rows:
        table(f"attn_combine128_kernel ({merge_rows[0].shape[0]} wavefronts per launch)", merge_rows, [
            (0, "first instruction"), (1, "kernel arguments in, addresses known"),
            (2, "every load issued"), (7, "sums done (partials arrived)"),
            (8, "split lanes joined"), (9, "output issued"),
            (11, "everything in flight done (stores acknowledged)")])
    pool.close()


def timeline_splitk(args, pkg, torch, np, raw, dev, stream):
    """The same for the split-K kernel on the verify block or the ragged batch (--workload),
    merge launch or die form (--die-merge): stage times of every wavefront over ten replays,
    and the last replay's stages by compute die (workgroup index mod 8)."""
    import ctypes as C

    die = bool(getattr(args, "die_merge", False))
    if args.workload == "ragged":
        layers, slots, rows = 4, 16, 1
        lengths = np.random.default_rng(3).integers(256, 16384, size=slots, endpoint=True).tolist()
    else:
        layers, slots, rows, lengths = 4, 4, 7, [8192] * 4
    pool = pkg.KvPool(layers, KV_HEADS, D, elem="f16", max_slots=slots, capacity_rows=max(lengths) + 16,
                      scrub_on_truncate=False, die_merge=die)
    pool.set_stream(stream.cuda_stream)
    caches = [pool.acquire() for _ in range(slots)]
    torch.manual_seed(0)
    for layer in range(layers):
        for s_, n in enumerate(lengths):
            k, v = torch.randn(n, ROW, device=dev), torch.randn(n, ROW, device=dev)
            pool.append_device(layer, [(caches[s_], n)], k.data_ptr(), v.data_ptr())
            torch.cuda.synchronize()
    total = slots * rows
    q = torch.randn(layers, total, Q_HEADS * D, device=dev)
    kn, vn = torch.randn(layers, total, ROW, device=dev), torch.randn(layers, total, ROW, device=dev)
    out = torch.empty_like(q)
    items = [(c, rows) for c in caches]

    def step():
        for layer in range(layers):
            pool.attention_step_device(layer, items, q[layer].data_ptr(), kn[layer].data_ptr(),
                                       vn[layer].data_ptr(), out[layer].data_ptr(), Q_HEADS)
        pool.truncate(caches, lengths)

    for _ in range(3):
        step()
    form = merge_form_of(pkg, pool, step)
    pool.truncate(caches, lengths)
    graph = capture(torch, pool, stream, step)
    marks, waves = 12, 8192
    buf = np.zeros(waves * marks, dtype=np.uint64)
    reader = "itak_timeline_read_splitk_die" if form == "on_die" else "itak_timeline_read_splitk"
    replays, groups = [], None
    for _ in range(10):
        graph.replay()
        torch.cuda.synchronize()
        rc = getattr(raw, reader)(buf.ctypes.data_as(C.c_void_p), C.c_ulonglong(buf.size))
        assert rc == 0, f"{reader} failed with HIP error {rc}"
        t = buf.reshape(waves, marks).astype(np.int64)
        if form != "on_die":
            t = t[:waves // 2]  # the second half holds the merge launch's records
        keep = t[:, 0] > 0
        groups = (np.arange(t.shape[0]) // 8)[keep]
        t = t[keep]
        replays.append((t - t[:, 0].min()) * 10)
    step_s = Timer(torch, stream)(graph.replay, 50)[0] / 50
    print(f"split-K timeline, {args.workload} (the last of {layers} layers in a HIP graph), split partials "
          f"merged by: {form}; {step_s / layers * 1e6:.2f} us per layer with the timestamps compiled in; "
          f"{replays[0].shape[0]} wavefronts per launch; ns from the launch's first instruction")
    allr = np.concatenate(replays)
    names = ["first instruction", "kernel arguments in, addresses known", "first block's loads issued",
             "mask and epilogue bookkeeping done", "Q^T (and new rows) staged in LDS", "query operands in registers (past the barrier)",
             "the wavefront's blocks done", "O^T written to LDS", "past the workgroup barrier",
             "partials issued", "arrival ticket drawn (die form)", "everything in flight done"]
    for i, name in enumerate(names):
        col = allr[:, i]
        col = col[col > 0] if i else col
        if len(col):
            print(f"  {name:42s} min {col.min():6d}  p50 {int(np.median(col)):6d}  "
                  f"p90 {int(np.percentile(col, 90)):6d}  max {col.max():6d}")
    last, die_of = replays[-1], groups % 8
    print("  by compute die (workgroup index mod 8), last replay: loads issued p50 / blocks done p50 / "
          "blocks done max / all done max")
    for d in range(8):
        r = last[die_of == d]
        if len(r):
            print(f"    die {d}: {int(np.median(r[:, 2])):6d} {int(np.median(r[:, 6])):6d} "
                  f"{r[:, 6].max():6d} {r[:, 11].max():6d}")
    pool.close()


class Timer:
    def __init__(self, torch, stream):
        self.torch, self.stream = torch, stream

    def __call__(self, fn, reps):
        torch = self.torch
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        start.record(self.stream)
        for _ in range(reps):
            fn()
        end.record(self.stream)
        torch.cuda.synchronize()
        return start.elapsed_time(end) * 1e-3, time.perf_counter() - t0


def capture(torch, pool, stream, fn):
    """One call of fn captured into a HIP graph on a side stream."""
    cap = torch.cuda.Stream()
    cap.wait_stream(stream)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(cap):
        pool.set_stream(cap.cuda_stream)
        with torch.cuda.graph(graph, stream=cap):
            fn()
    torch.cuda.synchronize()
    pool.set_stream(stream.cuda_stream)
    return graph


def probes(torch, pool, timed, dev):
    """Launch floor (empty kernel) and a streaming copy of known size on this device."""
    n = 256 << 20
    src = torch.empty(n, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    pool.probe_copy_device(src.data_ptr(), dst.data_ptr(), n)
    copy_s, _ = timed(lambda: pool.probe_copy_device(src.data_ptr(), dst.data_ptr(), n), 5)
    pool.probe_read_device(src.data_ptr(), n)
    read_s, _ = timed(lambda: pool.probe_read_device(src.data_ptr(), n), 5)
    for _ in range(50):
        pool.probe_empty_launch()
    empty_s, _ = timed(pool.probe_empty_launch, 2000)
    return {
        "empty_kernel_us_per_launch": round(empty_s / 2000 * 1e6, 3),
        "copy_256MiB_GBps_read_plus_write": round(2 * n * 5 / copy_s / 1e9, 1),
        "read_256MiB_GBps": round(n * 5 / read_s / 1e9, 1),
    }


def mfma_alone(torch, pool, timed, dev):
    """What the matrix pipe sustains by itself on this device (itak_probe_mfma: 32 f16 MFMAs a
    trip, operands in registers, two wavefronts a SIMD), on constant and on random operands, with
    the clock it held: the prefill kernel's data is random, and the second figure is the most any
    kernel built on this instruction could show for it here."""
    out = {}
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)
    for name, random_operands in (("constant_operands", False), ("random_operands", True)):
        trips = 20000
        flops = pool.probe_mfma(random_operands, 2000)  # warm-up
        best = None
        for _ in range(3):
            s, _ = timed(lambda: pool.probe_mfma(random_operands, trips, clocks.data_ptr()), 1)
            best = s if best is None else min(best, s)
        flops = flops // 2000 * trips
        ticks = clocks.cpu().tolist()
        out[name] = {"tflops": round(flops / best / 1e12, 1),
                     "clock_ghz": round(ticks[0] / max(1, ticks[1]) * 0.1, 2)}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", choices=["decode", "ragged", "verify", "prefill", "hybrid",
                                           "prefill_windowed", "restore", "append", "chunk64", "sweep"],
                    default="decode")
    ap.add_argument("--softcap", type=float, default=0.0)
    ap.add_argument("--kv", choices=["f16", "f32"], default="f16",
                    help="element type of the cache: f16 (the metric's) or f32, the reference's "
                         "own storage (decode and ragged workloads only; a secondary figure)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--merge-in-launch", action="store_true",
                    help="merge split partials inside the attention launch (workgroups exchange "
                         "them through a buffer) instead of with a launch of its own")
    ap.add_argument("--die-merge", action="store_true",
                    help="merge each unit's splits on its compute die inside the split-K launch "
                         "(ITAK_POOL_DIE_MERGE) where the batch suits it, instead of with a launch "
                         "of its own")
    ap.add_argument("--q-two-halves", action="store_true",
                    help="queries as two f16 halves in the split-K kernels' score products "
                         "(ITAK_POOL_Q_TWO_HALVES): the 2e-3 bar then holds off unit scale")
    ap.add_argument("--prep-by-launch", action="store_true",
                    help="with --prep: the preparation always as a launch of its own, the reference's "
                         "f64 chain (ITAK_POOL_PREP_BY_LAUNCH)")
    ap.add_argument("--prep", action="store_true",
                    help="also time the step with the fused Q/K preparation (per-head RMSNorm + "
                         "RoPE) before it and the sigmoid gate after it, reported as 'with_prep'")
    ap.add_argument("--timeline", action="store_true",
                    help="print where a decode layer's time goes: stage timestamps from the "
                         "measurement build of the library (python itak-torch-rebuild_amd/build.py "
                         "--timeline), a table instead of the JSON line; with --workload verify or "
                         "ragged the split-K kernel's stages, by compute die too")
    ap.add_argument("--only", action="store_true",
                    help="measure the named workload alone (the default decode run otherwise "
                         "adds short runs of the other configurations under 'workloads')")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (run with --gpus 1)",
              file=sys.stderr)
        sys.exit(2)
    if args.kv == "f32" and args.workload not in ("decode", "ragged"):
        print("--kv f32 is measured on the decode and ragged workloads only", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from __graft_entry__ import load_package

    pkg = load_package()
    if args.timeline:
        timeline(args, pkg, torch, np)
        return
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    stream = torch.cuda.current_stream()
    timed = Timer(torch, stream)

    if args.workload == "sweep":
        print(json.dumps(decode_sweep(args, pkg, torch, stream, full=True)))
        return
    result = run_workload(args, pkg, torch, np, dev, stream, timed)
    primary = (args.workload == "decode" and args.kv == "f16" and args.softcap == 0.0
               and not args.only and not args.merge_in_launch and not args.die_merge
               and not args.q_two_halves and not args.prep_by_launch)
    if primary:
        # The other configurations in short runs of their own, so that one line carries every
        # kernel's figure; `metric`, `value` and `config` stay those of the decode step.
        import copy
        workloads = {"decode": summary_of(result)}
        for wl in ("ragged", "verify", "prefill", "restore", "chunk64"):
            sub = copy.copy(args)
            sub.workload, sub.no_cpu_baseline, sub.prep = wl, True, False
            sub.steps, sub.warmup = max(10, args.steps // 4), max(3, args.warmup // 4)
            try:
                torch.cuda.empty_cache()
                workloads[wl] = summary_of(run_workload(sub, pkg, torch, np, dev, stream, timed))
            except Exception as e:  # a secondary figure must not take the contract line down
                workloads[wl] = {"error": f"{type(e).__name__}: {e}"}
        result["workloads"] = workloads
        # The same decode step over context and batch, a coarse grid: where the 70 % of the HBM
        # peak that the headline asks for is met (`--workload sweep` prints the whole table).
        try:
            torch.cuda.empty_cache()
            sweep = decode_sweep(args, pkg, torch, stream, full=False)
            result["decode_sweep"] = {k: sweep[k] for k in ("summary", "seventy_pct_met_from_mb_per_launch",
                                                            "points")}
        except Exception as e:
            result["decode_sweep"] = {"error": f"{type(e).__name__}: {e}"}
    print(json.dumps(result))


def decode_sweep(args, pkg, torch, stream, full):
    """One decode row per slot (fused append + attention, 32 Q / 4 KV heads, f16) over a grid of
    context lengths and slot counts: us per layer and KV bytes / time as a fraction of the HBM
    peak, 4 layers cycled 12 times in a HIP graph. Also the smallest launch (MB of KV) from which every
    larger launch of the grid meets 70 % of the peak."""
    layers, cycles = 4, 12
    if full:
        contexts = [512, 1024, 2048, 4096, 8192, 16384, 32768, 65536, 131072]
        batches = [1, 2, 4, 8, 16, 32, 64]
    else:
        contexts, batches = [1024, 4096, 16384, 65536], [1, 4, 16, 64]
    points = []
    for ctx in contexts:
        for batch in batches:
            if batch * ctx * 2 * ROW * 2 * layers > 24e9:
                continue
            pool = pkg.KvPool(layers, KV_HEADS, D, elem="f16", max_slots=batch, capacity_rows=ctx + 9,
                              scrub_on_truncate=False, die_merge=getattr(args, "die_merge", False))
            pool.set_stream(stream.cuda_stream)
            caches = [pool.acquire() for _ in range(batch)]
            k = torch.randn(ctx, ROW, device="cuda")
            v = torch.randn(ctx, ROW, device="cuda")
            for layer in range(layers):
                for c in caches:
                    pool.append_device(layer, [(c, ctx)], k.data_ptr(), v.data_ptr())
            torch.cuda.synchronize()
            q = torch.randn(layers, batch, Q_HEADS * D, device="cuda")
            kn = torch.randn(layers, batch, ROW, device="cuda")
            vn = torch.randn(layers, batch, ROW, device="cuda")
            out = torch.empty_like(q)
            items = [(c, 1) for c in caches]

            def step():
                # As many layer steps in a graph as the headline's step has (48): a graph of a few
                # launches would show its own start in every small point.
                for _ in range(cycles):
                    for layer in range(layers):
                        pool.attention_step_device(layer, items, q[layer].data_ptr(), kn[layer].data_ptr(),
                                                   vn[layer].data_ptr(), out[layer].data_ptr(), Q_HEADS)
                    pool.truncate(caches, [ctx] * batch)

            for _ in range(3):
                step()
            torch.cuda.synchronize()
            graph = capture(torch, pool, stream, step)
            for _ in range(3):
                graph.replay()
            reps = 8 if full else 4
            us = Timer(torch, stream)(graph.replay, reps)[0] / reps / (layers * cycles) * 1e6
            kv_bytes = 2 * batch * (ctx + 1) * ROW * 2
            points.append({"context": ctx, "slots": batch, "us_per_layer": round(us, 2),
                           "kv_mb_per_launch": round(kv_bytes / 1e6, 1),
                           "frac": round(kv_bytes / us / 1e3 / HBM_PEAK_GBS, 3)})
            pool.close()
            del pool, caches, graph
            torch.cuda.empty_cache()
    # The smallest size from which every launch of the grid at least as large meets 70 %.
    by_size = sorted(points, key=lambda p: p["kv_mb_per_launch"])
    met_from = None
    for i, p in enumerate(by_size):
        if all(r["frac"] >= 0.70 for r in by_size[i:]):
            met_from = p["kv_mb_per_launch"]
            break
    summary = ("70 % of the HBM peak is not met on this grid" if met_from is None else
               f"70 % of the HBM peak is met from {met_from:.0f} MB of KV per launch")
    return {"metric": "decode-attn KV GB/s over context and batch", "unit": "fraction of 8 TB/s",
            "layers_cycled": layers, "layer_steps_per_graph": layers * cycles, "summary": summary,
            "seventy_pct_met_from_mb_per_launch": met_from, "points": points}


def merge_form_of(pkg, pool, step):
    """How the step's split partials are merged ("launch", "on_die", "in_launch", "none"), read
    from the library's diagnostic line for the step's first attention launch."""
    import re
    import tempfile

    with tempfile.TemporaryFile(mode="w+b") as tmp:
        sys.stderr.flush()
        saved = os.dup(2)
        os.dup2(tmp.fileno(), 2)
        try:
            pkg.set_debug_enabled(True)
            step()
            pool.synchronize()
        finally:
            pkg.set_debug_enabled(False)
            os.dup2(saved, 2)
            os.close(saved)
        tmp.seek(0)
        forms = re.findall(r"merge=(\w+)", tmp.read().decode(errors="replace"))
    return forms[0] if forms else None


def summary_of(result):
    """The few figures of a workload's result that the one-line summary carries."""
    r = result["roofline"]
    out = {"metric": result["metric"], "value": result["value"], "unit": result["unit"],
           "ms_per_step": result["ms_per_step"], "bound": r["bound"], "frac": r["frac"],
           "us_per_launch": r.get("us_per_launch"), "kernel": r.get("kernel")}
    for key in ("step_frac", "frac_of_streaming_read", "mfma_alone", "frac_of_mfma_alone_on_random_operands"):
        if key in r:
            out[key] = r[key]
    return out


def run_workload(args, pkg, torch, np, dev, stream, timed):
    """Measures one workload and returns its JSON object."""
    # ---- workload shapes -------------------------------------------------------------
    wl = args.workload
    elem_bytes = 4 if args.kv == "f32" else 2
    if wl in ("restore", "append"):
        return cache_maintenance(args, pkg, torch, dev, stream, timed)
    if wl == "decode":
        layers, slots, rows, lengths = 48, 1, 1, [4096]
        name = ("configs[1]: 30B-class decode step, batch 1, 48 layers, 32 Q / 4 KV heads, "
                "head_dim 128, f16 KV, context 4096, append 1 token per layer then flash-decode")
    elif wl == "ragged":
        layers, slots, rows = 8, 16, 1
        lengths = np.random.default_rng(3).integers(256, 16384, size=slots, endpoint=True).tolist()
        name = ("configs[2]: continuous-batching decode, 16 slots, ragged context 256..16384 "
                f"(sum {sum(lengths)}), 30B-class heads, f16 KV, 8 of the 48 layers cycled")
    elif wl == "verify":
        layers, slots, rows, lengths = 16, 4, 7, [8192] * 4
        name = ("configs[3]: speculative verify block, 4 slots at context 8192, 7 query rows "
                "appended and attended causally, 30B-class heads, f16 KV, 16 layers cycled")
    elif wl == "chunk64":
        layers, slots, rows, lengths = 16, 1, 64, [4096]
        name = ("the reference's own prefill chunk (crates/wgpu-compute/src/session.rs:186-195): 64 rows "
                "appended and attended causally at context 4096, 30B-class heads, f16 KV, 16 layers "
                "cycled; the block kernel splits the context, appends the rows itself and a merge "
                "launch follows")
    elif wl == "hybrid":
        layers, slots, rows, lengths = 8, 1, 1, [32768]
        name = ("hybrid decode step: sliding-window layers (window 2048) and global layers 3:1, "
                "the pattern of the reference's 52-layer model, batch 1, context 32768, 30B-class "
                "heads, f16 KV, 8 layers cycled (6 windowed, 2 global)")
    elif wl == "prefill_windowed":
        layers, slots, rows, lengths = 4, 1, 2048, [30720]
        name = ("chunked causal prefill on sliding-window layers (window 2048, three of four layers "
                "of the reference's model): 2048-row chunk at position 30720, each row over its "
                "last 2048 keys, 30B-class heads, f16 KV, f32 accumulate, 4 layers cycled")
    else:
        layers, slots, rows, lengths = 4, 1, 2048, [30720]
        name = ("configs[4]: chunked causal prefill, 2048-row chunk over a 30720-token prefix, "
                "30B-class heads, f16 KV, f32 accumulate, 4 layers cycled")
    max_len = max(lengths)
    window = 2048
    pattern = [pkg.LayerKind.Global] * layers
    if wl == "prefill_windowed":
        pattern = [pkg.LayerKind.windowed(window)] * layers
    if wl == "hybrid":  # glimmer_layer_pattern: every fourth layer global
        pattern = [pkg.LayerKind.Global if (i + 1) % 4 == 0 else pkg.LayerKind.windowed(window)
                   for i in range(layers)]
    # Rows a layer's attention reads per slot: everything stored, or the window.
    visible = [[min(n + rows, window + rows - 1) if kind.is_windowed else n + rows for n in lengths]
               for kind in pattern]
    kv_bytes_layer = sum(sum(2 * r * KV_HEADS * D * elem_bytes for r in per) for per in visible) // layers
    flops_layer = sum(4 * D * Q_HEADS * (rows * n + rows * (rows + 1) // 2) for n in lengths)
    if wl == "prefill_windowed":  # row i at position n + i sees min(window, n + i + 1) keys
        flops_layer = sum(4 * D * Q_HEADS * sum(min(window, n + i + 1) for i in range(rows))
                          for n in lengths)

    if args.kv == "f32":
        name = name.replace("f16 KV", "f32 KV (the reference's storage; the metric is quoted on f16)")
    pool = pkg.KvPool(pattern, KV_HEADS, D, elem=args.kv, max_slots=slots,
                      capacity_rows=max_len + rows + 8, scrub_on_truncate=False,
                      ring_headroom=rows if wl == "prefill_windowed" else 0,
                      merge_in_launch=args.merge_in_launch,
                      die_merge=getattr(args, "die_merge", False),
                      q_two_halves=getattr(args, "q_two_halves", False),
                      prep_by_launch=getattr(args, "prep_by_launch", False))
    pool.set_stream(stream.cuda_stream)
    caches = [pool.acquire() for _ in range(slots)]

    # Synthetic inputs, resident in HBM: prefix K/V per layer and slot, new K/V rows and Q.
    total_rows = slots * rows
    q = torch.randn(layers, total_rows, Q_HEADS * D, device=dev)
    k_new = torch.randn(layers, total_rows, ROW, device=dev)
    v_new = torch.randn(layers, total_rows, ROW, device=dev)
    if wl.startswith("prefill") or wl == "chunk64":  # f16-valued Q/K/V
        q, k_new, v_new = q.half().float(), k_new.half().float(), v_new.half().float()
    out = torch.empty_like(q)
    for layer in range(layers):
        for s, n in enumerate(lengths):
            k = rope_on_device(torch.randn(n, KV_HEADS, D, device=dev), 1e6).reshape(n, ROW)
            k = k.contiguous()
            v = torch.randn(n, ROW, device=dev)
            if pattern[layer].is_windowed:  # the last `window` rows, where a prefill leaves them
                first = max(0, n - window)
                caches[s].restore_bulk_ptr(layer, first, k[first:].data_ptr(), v[first:].data_ptr(),
                                           (n - first) * ROW, src_f16=False)
            else:
                pool.append_device(layer, [(caches[s], n)], k.data_ptr(), v.data_ptr())
            torch.cuda.synchronize()
    items = [(c, rows) for c in caches]
    ptrs = [(q[l].data_ptr(), k_new[l].data_ptr(), v_new[l].data_ptr(), out[l].data_ptr())
            for l in range(layers)]

    def step():
        for layer in range(layers):
            qp, kp, vp, op = ptrs[layer]
            pool.attention_step_device(layer, items, qp, kp, vp, op, Q_HEADS,
                                       softcap=args.softcap)
        pool.truncate(caches, lengths)

    def attention_only():
        for layer in range(layers):
            qp, _, _, op = ptrs[layer]
            pool.attention_device(layer, items, qp, op, Q_HEADS, softcap=args.softcap)

    for _ in range(max(args.warmup, 1)):
        step()
    torch.cuda.synchronize()
    merge_form = merge_form_of(pkg, pool, step)
    probe = probes(torch, pool, timed, dev)

    eager_s, eager_wall_s = timed(step, args.steps)

    # One step (all layers) captured once and replayed: the launch-bound loop a serving
    # engine keeps in a HIP graph. The attention launches alone are timed the same way on
    # a cache that already holds the new rows.
    g_step = capture(torch, pool, stream, step)
    for layer in range(layers):
        pool.append_device(layer, items, ptrs[layer][1], ptrs[layer][2])
    g_attn = capture(torch, pool, stream, attention_only)
    for _ in range(max(args.warmup, 1)):
        g_step.replay()
    step_s = timed(g_step.replay, args.steps)[0] / args.steps
    for _ in range(max(args.warmup, 1)):
        g_attn.replay()
    attn_s = timed(g_attn.replay, args.steps)[0] / (args.steps * layers)
    pool.truncate(caches, lengths)
    if wl == "prefill_windowed":
        # On a sliding-window layer a chunk attended after its append sees only what the ring
        # still promises (the last `window` rows: the chunk's first rows would see almost
        # nothing), so the attention launch is timed as the step minus its append.
        def append_only():
            for layer in range(layers):
                pool.append_device(layer, items, ptrs[layer][1], ptrs[layer][2])
            pool.truncate(caches, lengths)

        g_append = capture(torch, pool, stream, append_only)
        for _ in range(max(args.warmup, 1)):
            g_append.replay()
        append_s = timed(g_append.replay, args.steps)[0] / args.steps
        attn_s = (step_s - append_s) / layers

    host_call = None
    if wl == "decode":
        # The same layer step through the host-pointer entry point (what a Compute::attention
        # call with host slices costs): inputs and output cross the host link and the call
        # waits for its result. A secondary figure, never `value`.
        import ctypes as C

        lib = pkg._native.load()
        hq = q[0, :1].cpu().numpy().copy()
        hk = k_new[0, :1].cpu().numpy().copy()
        hv = v_new[0, :1].cpu().numpy().copy()
        ho = np.empty_like(hq)
        pos = lengths[0]
        calls = 0

        def host_step():
            st = lib.itak_compute_attention(pool._h, caches[0].slot, 0, hq.ctypes.data, hq.size,
                                            hk.ctypes.data, hk.size, hv.ctypes.data, hv.size,
                                            Q_HEADS, pos, C.c_float(args.softcap), C.c_float(0.0),
                                            ho.ctypes.data)
            assert st == 0, lib.itak_last_error(pool._h)
            pool.truncate(caches[:1], lengths[:1])

        for _ in range(20):
            host_step()
        t0 = time.perf_counter()
        for _ in range(200):
            host_step()
        per_call = (time.perf_counter() - t0) / 200
        host_call = {
            "entry_point": "itak_compute_attention (host q/k/v in, host output out, one layer)",
            "us_per_layer": round(per_call * 1e6, 2),
            "kv_GBps": round(kv_bytes_layer / per_call / 1e9, 1),
        }

    with_prep = None
    if args.prep and not wl.startswith("prefill"):
        # The model's own sequence around the step (muse-glimmer/src/model.rs:445-464): raw
        # projections -> per-head RMSNorm -> interleaved RoPE on sliding-window layers (global
        # layers carry no rotation) -> append + attention -> out * sigmoid(gate).
        qw, kw = torch.rand(D, device=dev) + 0.5, torch.rand(D, device=dev) + 0.5
        gate = torch.randn(layers, total_rows, Q_HEADS * D, device=dev)

        def prep_step():
            for layer in range(layers):
                qp, kp, vp, op = ptrs[layer]
                pool.attention_prep_step_device(
                    layer, items, qp, kp, vp, op, Q_HEADS, q_norm_ptr=qw.data_ptr(),
                    k_norm_ptr=kw.data_ptr(), eps=1e-6,
                    rope_base=1e4 if pattern[layer].is_windowed else 0.0, interleaved=True,
                    gate_ptr=gate[layer].data_ptr(), softcap=args.softcap)
            pool.truncate(caches, lengths)

        for _ in range(max(args.warmup, 1)):
            prep_step()
        g_prep = capture(torch, pool, stream, prep_step)
        for _ in range(max(args.warmup, 1)):
            g_prep.replay()
        prep_s = timed(g_prep.replay, args.steps)[0] / args.steps
        folded = rows * (Q_HEADS // KV_HEADS) <= 64 and rows <= 8 and not args.prep_by_launch
        with_prep = {
            "us_per_layer": round(prep_s / layers * 1e6, 3),
            "added_us_per_layer": round((prep_s - step_s) / layers * 1e6, 3),
            "launches_added_per_layer": 0 if folded else 1,
            "what": ("RMSNorm + RoPE of Q and of the new K row inside the split-K kernel, the gate "
                     "in the kernel that writes the output: the step's own two launches"
                     if folded else
                     "attn_prep_kernel (RMSNorm + RoPE of Q and K, one launch) before the fused "
                     "append + attention; the gate in the merge kernel"),
        }

    if wl == "chunk64":
        # Neither roofline describes this shape (4.3 GFLOP and 8 MB of KV per layer, 5 us of
        # either): the figure is the layer's time; TFLOP/s and the MFMA fraction go with it.
        metric, unit = "prefill attention TFLOP/s (64-row chunk at context 4096)", "TFLOP/s"
        value = flops_layer * layers / step_s / 1e12
        roofline = {
            "bound": "mfma",
            "kernel": "attn_prefill_f16_kernel (one tile per wavefront, appends the chunk's rows) + "
                      "attn_combine128_wave_kernel",
            "achieved": round(value, 2),
            "peak": MFMA_F16_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(value / MFMA_F16_PEAK_TFLOPS, 4),
            "traffic": None,
            "us_per_launch": round(step_s / layers * 1e6, 2),
            "flops_per_launch": flops_layer,
            "timed": "one layer of the timed step (HIP graph replay of all layers): append + "
                     "attention in the block kernel's launch, then the merge launch",
            "attention_only_us_per_launch": round(attn_s * 1e6, 2),
        }
    elif wl.startswith("prefill"):
        metric, unit = "prefill attention TFLOP/s (2048-row chunk over 30720 prefix)", "TFLOP/s"
        if wl == "prefill_windowed":
            metric = "prefill attention TFLOP/s (2048-row chunk, window 2048)"
        value = flops_layer * layers / step_s / 1e12
        roofline = {
            "bound": "mfma",
            "kernel": "attn_prefill_f16_kernel (one launch per layer)" +
                      (": the step's time less its append's" if wl == "prefill_windowed" else ""),
            "achieved": round(flops_layer / attn_s / 1e12, 2),
            "peak": MFMA_F16_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(flops_layer / attn_s / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
            "traffic": PROFILE_TRAFFIC.get((wl, args.kv), (None, None))[0],
            "traffic_source": PROFILE_TRAFFIC.get((wl, args.kv), (None, None))[1],
            "us_per_launch": round(attn_s * 1e6, 2),
            "flops_per_launch": flops_layer,
            # The same over the whole timed step (the chunk's append launches included).
            "step_frac": round(value / MFMA_F16_PEAK_TFLOPS, 4),
            "timed": "the attention launch of a layer, event-timed in a graph of its own on a "
                     "cache that already holds the chunk",
        }
        # Beside the published peak: the instruction alone on this device, in this run.
        alone = mfma_alone(torch, pool, timed, dev)
        roofline["mfma_alone"] = alone
        roofline["frac_of_mfma_alone_on_random_operands"] = round(
            flops_layer / attn_s / 1e12 / alone["random_operands"]["tflops"], 4)
    else:
        metric, unit = "decode-attn KV GB/s (all layers, ctx 4096)", "GB/s"
        if wl != "decode":
            metric = f"decode-attn KV GB/s ({wl})"
        if args.kv == "f32":
            metric += " on an f32 cache"
        value = kv_bytes_layer * layers / step_s / 1e9
        # The layer's launches as the timed step runs them (fused append + attention, then the
        # merge): achieved = algorithmic KV bytes of a layer / the step's time per layer.
        layer_s = step_s / layers
        lean = args.kv == "f16" and rows == 1 and wl in ("decode", "hybrid")
        roofline = {
            "bound": "hbm",
            "kernel": (("attn_decode_f16_kernel" if lean else f"attn_splitk_{args.kv}_kernel") +
                       (" (splits merged inside the launch)" if args.merge_in_launch else
                        " (each unit's splits merged on its compute die by the unit's last "
                        "workgroup: one launch per layer)" if merge_form == "on_die" else
                        " + attn_combine128_kernel (the two launches of one layer's attention)")),
            "achieved": round(kv_bytes_layer / layer_s / 1e9, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(kv_bytes_layer / layer_s / 1e9 / HBM_PEAK_GBS, 4),
            "traffic": PROFILE_TRAFFIC.get((wl, args.kv), (None, None))[0],
            "traffic_source": PROFILE_TRAFFIC.get((wl, args.kv), (None, None))[1],
            "us_per_launch": round(layer_s * 1e6, 3),
            "bytes_per_launch": kv_bytes_layer,
            # Beside the published peak: what a kernel that only reads gets from this device
            # (itak_probe_read_device, 256 MiB), in this run.
            "frac_of_streaming_read": round(kv_bytes_layer / layer_s / 1e9 / probe["read_256MiB_GBps"], 4),
            "timed": "one layer of the timed step (HIP graph replay of all layers), HIP events on "
                     "the stream the kernels run on",
            # The attention launches alone, on a cache that already holds the new rows.
            "attention_only_us_per_launch": round(attn_s * 1e6, 3),
        }

    result = {
        "metric": metric,
        "value": round(value, 2),
        "unit": unit,
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.kv,
        "data": "synthetic",
        "config": {
            "workload": name,
            "launch": "HIP graph replay of one step (all layers)",
            "layers_per_step": layers,
            "kv_bytes_per_step": kv_bytes_layer * layers,
            "softcap": args.softcap,
            "arithmetic": ("f16 KV and MFMA operands, f32 scores, softmax and accumulation"
                           if args.kv == "f16" else "f32 KV, f32 MFMA operands and accumulation"),
        },
        "us_per_token": round(step_s * 1e6 * ((52 if wl == "hybrid" else 48) / layers), 2),
        "pct_of_hbm_peak": round(100.0 * kv_bytes_layer * layers / step_s / 1e9 / HBM_PEAK_GBS, 2),
        "eager": {
            "us_per_step_stream": round(eager_s / args.steps * 1e6, 2),
            "us_per_step_wall": round(eager_wall_s / args.steps * 1e6, 2),
        },
        "device_probes": probe,
        "roofline": roofline,
    }
    if merge_form is not None:
        result["config"]["split_merge"] = merge_form
    if with_prep is not None:
        result["with_prep"] = with_prep
    if host_call is not None:
        result["host_pointer_call"] = host_call
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(4096, 2 * 4097 * KV_HEADS * D * elem_bytes, 48,
                                              store_f16=args.kv == "f16")
    pool.close()
    return result


if __name__ == "__main__":
    main()
