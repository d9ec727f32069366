"""Host-side mirror of the reference's API for the KV-cache + attention path, on top of the
C ABI in include/itak_hip_kv.h.

Names, argument meaning and refusals follow the Rust:
  KvCache / CacheView / Checkpoint / LayerKind  crates/attention/src/cache.rs
  gqa_attention / AttentionParams               crates/attention/src/attention.rs
  AttentionError                                crates/attention/src/error.rs
  HipCompute (the CpuCompute twin)              crates/cpu-compute/src/cpu.rs:246-339,506-655
  AttentionRequest / PositionCache              crates/muse-glimmer/src/{compute,cache}.rs
KvPool has no reference counterpart: it owns the device memory of several sequences so
that one launch can serve all of them.
"""
from __future__ import annotations

import ctypes as C
import os
import math
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple, Union

import numpy as np

from . import _native as N

# ---------------------------------------------------------------------------- errors

_FIELDS = {
    "ZeroDimension": ("what",),
    "InvalidWindow": ("window",),
    "SizeOverflow": ("what",),
    "ShapeMismatch": ("what", "expected", "actual"),
    "InvalidLayer": ("layer", "layer_count"),
    "OutOfOrderPosition": ("layer", "expected", "actual"),
    "NonDivisibleHeads": ("num_q_heads", "num_kv_heads"),
    "NoVisibleKeys": ("position",),
    "CheckpointBusy": (),
    "StaleCheckpoint": ("checkpoint",),
    "CheckpointTooDeep": ("max_round_tokens", "window"),
    "CheckpointRangeExceeded": ("layer", "position", "limit"),
    "BulkRestoreNotFresh": ("layer", "appended"),
    "RewindOutOfRange": ("layer", "base", "appended", "target"),
}


class AttentionError(Exception):
    """attention::AttentionError: `variant` names the Rust variant, `fields` its fields.
    Library-only refusals (HipError, CapacityExceeded, ...) use the same class."""

    def __init__(self, variant: str, message: str = "", **fields):
        self.variant = variant
        self.fields = fields
        self.message = message
        super().__init__(message or f"{variant} {fields}")

    def __eq__(self, other):
        return (isinstance(other, AttentionError) and self.variant == other.variant
                and self.fields == other.fields)

    def __hash__(self):
        return hash((self.variant, tuple(sorted(self.fields.items()))))

    def __repr__(self):
        inner = ", ".join(f"{k}={v!r}" for k, v in self.fields.items())
        return f"AttentionError.{self.variant}({inner})"


class StepFailed(Exception):
    """muse_glimmer::GlimmerError::StepFailed { step, detail } (error.rs:69-76)."""

    def __init__(self, step: str, detail: str):
        self.step = step
        self.detail = detail
        super().__init__(f"{step}: {detail}")


def _raise_last(handle, step: Optional[str] = None):
    lib = N.load()
    info = N.ErrorInfo()
    lib.itak_last_error_info(handle, C.byref(info))
    message = (lib.itak_last_error(handle) or b"").decode()
    name = N.STATUS_NAMES.get(info.code, f"Status{info.code}")
    if name == "StepFailed":
        raise StepFailed(step or info.what.decode() or "attention", message)
    names = _FIELDS.get(name)
    if names is None:
        raise AttentionError(name, message, what=info.what.decode(), a=int(info.a), b=int(info.b))
    nums = iter((info.a, info.b, info.c, info.d))
    fields = {n: (info.what.decode() if n == "what" else int(next(nums))) for n in names}
    raise AttentionError(name, message, **fields)


def _check(handle, status: int, step: Optional[str] = None):
    if status != N.OK:
        _raise_last(handle, step)


# ------------------------------------------------------------------ kinds and params

@dataclass(frozen=True)
class LayerKind:
    """attention::LayerKind (cache.rs:36-66)."""

    window_size: Optional[int] = None
    is_windowed: bool = False

    @staticmethod
    def windowed(window: int) -> "LayerKind":
        if window == 0:
            raise AttentionError("InvalidWindow", "sliding window must be positive, got 0",
                                 window=0)
        return LayerKind(window, True)

    @staticmethod
    def Windowed(window: int) -> "LayerKind":
        return LayerKind(window, True)

    def window(self) -> Optional[int]:
        return self.window_size if self.is_windowed else None


LayerKind.Global = LayerKind(None, False)
# muse_glimmer::LayerKind::SlidingWindow carries no window of its own (the config does).
LayerKind.SlidingWindow = LayerKind(None, True)


@dataclass(frozen=True)
class AttentionParams:
    """attention::AttentionParams (attention.rs:17-38) plus the logit softcap."""

    scale: Optional[float] = None
    softcap: float = 0.0

    @staticmethod
    def new() -> "AttentionParams":
        return AttentionParams()

    @staticmethod
    def with_scale(scale: float) -> "AttentionParams":
        return AttentionParams(scale=scale)

    def scale_for(self, head_dim: int) -> np.float32:
        if self.scale is not None:
            return np.float32(self.scale)
        return np.float32(1.0) / np.sqrt(np.float32(head_dim))


def kv_head_for_query_head(q_head: int, num_q_heads: int, num_kv_heads: int) -> int:
    """attention.rs:43-72."""
    if num_kv_heads == 0:
        raise AttentionError("ZeroDimension", what="num_kv_heads")
    if num_q_heads == 0:
        raise AttentionError("ZeroDimension", what="num_q_heads")
    if num_q_heads % num_kv_heads != 0:
        raise AttentionError("NonDivisibleHeads", num_q_heads=num_q_heads,
                             num_kv_heads=num_kv_heads)
    if q_head >= num_q_heads:
        raise AttentionError("ShapeMismatch", what="q_head", expected=num_q_heads, actual=q_head)
    return q_head // (num_q_heads // num_kv_heads)


@dataclass
class LayerStats:
    layer: int
    kind: LayerKind
    appended: int
    stored: int


# ------------------------------------------------------------------------------ pool

def set_debug_enabled(enabled: bool) -> None:
    """attention::diag::set_debug_enabled (crates/attention/src/diag.rs:17-19): one stderr line,
    prefixed `[itak_hip_kv::diag]`, per cache and attention event and per refusal; the
    environment variable ITAK_HIP_KV_DEBUG turns the same lines on from outside."""
    N.load().itak_set_debug_enabled(1 if enabled else 0)


def debug_enabled() -> bool:
    """attention::diag::debug_enabled (diag.rs:24-33): the switch or the environment variable."""
    return bool(N.load().itak_debug_enabled())


def _as_f32(x) -> np.ndarray:
    return np.ascontiguousarray(x, dtype=np.float32).reshape(-1)


def _ptr(a: Optional[np.ndarray]):
    return a.ctypes.data if a is not None and a.size else None


class KvPool:
    """Device-resident KV storage for up to `max_slots` sequences (one itak_pool)."""

    def __init__(self, pattern: Union[int, Sequence[LayerKind]], num_kv_heads: int, head_dim: int,
                 *, elem: str = "f16", max_slots: int = 1, capacity_rows: int = 4096,
                 device: int = 0, scrub_on_truncate: bool = True, ring_headroom: int = 0,
                 merge_in_launch: bool = False, die_merge: Optional[bool] = None,
                 q_two_halves: Optional[bool] = None, prep_by_launch: bool = False):
        if isinstance(pattern, int):
            pattern = [LayerKind.Global] * pattern
        self.pattern = list(pattern)
        self.elem = elem
        self.np_elem = np.uint16 if elem == "f16" else np.float32
        self.capacity_rows = capacity_rows
        kinds = np.array([1 if k.is_windowed else 0 for k in self.pattern], dtype=np.uint8)
        windows = np.array([(k.window_size or 0) if k.is_windowed else 0 for k in self.pattern],
                           dtype=np.uint64)
        cfg = N.PoolConfig()
        cfg.layer_count = len(self.pattern)
        cfg.layer_kinds = _ptr(kinds)
        cfg.windows = _ptr(windows)
        cfg.num_kv_heads = num_kv_heads
        cfg.head_dim = head_dim
        cfg.elem = {"f32": N.ELEM_F32, "f16": N.ELEM_F16}[elem]
        cfg.max_slots = max_slots
        cfg.capacity_rows = capacity_rows
        cfg.device = device
        cfg.flags = (N.POOL_SCRUB_ON_TRUNCATE if scrub_on_truncate else 0) | \
                    (N.POOL_MERGE_IN_LAUNCH if merge_in_launch else 0)
        # Split merges on the units' compute dies are opt-in; ITAK_HIP_KV_DIE_MERGE=1 in the
        # environment turns them on for pools that do not say otherwise (how the test suite is
        # run over that form).
        if die_merge is None:
            die_merge = os.environ.get("ITAK_HIP_KV_DIE_MERGE", "0") == "1"
        if die_merge:
            cfg.flags |= N.POOL_DIE_MERGE
        # The same for the queries as two halves: ITAK_HIP_KV_Q_TWO_HALVES=1.
        if q_two_halves is None:
            q_two_halves = os.environ.get("ITAK_HIP_KV_Q_TWO_HALVES", "0") == "1"
        if q_two_halves:
            cfg.flags |= N.POOL_Q_TWO_HALVES
        if prep_by_launch:  # attention_prep_step_device never prepares inside the attention launch
            cfg.flags |= N.POOL_PREP_BY_LAUNCH
        cfg.ring_headroom = ring_headroom
        handle = C.c_void_p()
        self._h = None
        self._lib = N.load()
        status = self._lib.itak_pool_create(C.byref(cfg), C.byref(handle))
        if status != N.OK:
            _raise_last(None)
        self._h = handle
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.row = num_kv_heads * head_dim

    def close(self):
        if self._h:
            self._lib.itak_pool_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def device_bytes(self) -> int:
        return int(self._lib.itak_pool_device_bytes(self._h))

    def set_stream(self, stream_handle: int) -> None:
        _check(self._h, self._lib.itak_pool_set_stream(self._h, stream_handle))

    def synchronize(self) -> None:
        _check(self._h, self._lib.itak_pool_synchronize(self._h))

    def set_merge_spin_limit(self, polls: int) -> None:
        """Bound on the polls a workgroup of an in-launch split merge waits for its group."""
        _check(self._h, self._lib.itak_pool_set_merge_spin_limit(self._h, polls))

    def acquire(self) -> "KvCache":
        slot = C.c_uint32()
        _check(self._h, self._lib.itak_slot_acquire(self._h, C.byref(slot)))
        return KvCache(self, int(slot.value))

    @staticmethod
    def _items(items) -> Tuple[C.Array, int]:
        raw = (N.BatchItem * len(items))()
        for i, (slot, rows) in enumerate(items):
            raw[i].slot = slot.slot if isinstance(slot, KvCache) else int(slot)
            raw[i].rows = int(rows)
        return raw, len(items)

    def attention_step_device(self, layer: int, items, q_ptr: int, k_ptr: int, v_ptr: int,
                              out_ptr: int, num_q_heads: int, scale: Optional[float] = None,
                              softcap: float = 0.0) -> None:
        """Append each item's rows, then attend causally; device pointers, pool's stream."""
        raw, n = self._items(items)
        _check(self._h, self._lib.itak_attention_step_device(
            self._h, layer, raw, n, q_ptr, k_ptr, v_ptr, out_ptr, num_q_heads,
            math.nan if scale is None else scale, softcap))

    def attention_step_device_noalloc(self, layer: int, items, q_ptr: int, k_ptr: int, v_ptr: int,
                                      out_ptr: int, num_q_heads: int, scale: Optional[float] = None,
                                      softcap: float = 0.0) -> None:
        """attention_step_device with its split workspace in the library's static device array:
        allocates nothing; refuses steps that need more than the array holds."""
        raw, n = self._items(items)
        _check(self._h, self._lib.itak_attention_step_device_noalloc(
            self._h, layer, raw, n, q_ptr, k_ptr, v_ptr, out_ptr, num_q_heads,
            math.nan if scale is None else scale, softcap))

    def attention_prep_step_device(self, layer: int, items, q_ptr: int, k_ptr: int, v_ptr: int,
                                   out_ptr: int, num_q_heads: int, *, q_norm_ptr: int = 0,
                                   k_norm_ptr: int = 0, eps: float = 1e-6, rope_base: float = 0.0,
                                   interleaved: bool = True, rotary_dim: int = 0, gate_ptr: int = 0,
                                   scale: float = float("nan"), softcap: float = 0.0) -> None:
        """Per-head RMSNorm + RoPE of the raw Q/K projections, append, attention, gate: the
        steps of muse-glimmer/src/model.rs:445-464 around Compute::attention, device tensors."""
        arr, n = self._items(items)
        prep = N.PrepParams(q_norm_ptr or None, k_norm_ptr or None, eps, rope_base,
                            1 if interleaved else 0, rotary_dim)
        _check(self._h, self._lib.itak_attention_prep_step_device(
            self._h, layer, arr, n, q_ptr, k_ptr, v_ptr, gate_ptr or None, out_ptr, num_q_heads,
            scale, softcap, C.byref(prep)), "attention")

    def attention_device(self, layer: int, items, q_ptr: int, out_ptr: int, num_q_heads: int,
                         scale: Optional[float] = None, softcap: float = 0.0) -> None:
        """Attend with each item's last `rows` stored positions as the queries' positions."""
        raw, n = self._items(items)
        _check(self._h, self._lib.itak_attention_device(
            self._h, layer, raw, n, q_ptr, out_ptr, num_q_heads,
            math.nan if scale is None else scale, softcap))

    def append_device(self, layer: int, items, k_ptr: int, v_ptr: int) -> None:
        raw, n = self._items(items)
        _check(self._h, self._lib.itak_kv_append_device(self._h, layer, raw, n, k_ptr, v_ptr))

    def truncate(self, slots, new_lengths) -> None:
        s = np.array([x.slot if isinstance(x, KvCache) else int(x) for x in slots],
                     dtype=np.uint32)
        n = np.asarray(new_lengths, dtype=np.uint64)
        _check(self._h, self._lib.itak_kv_truncate(self._h, _ptr(s), _ptr(n), len(s)))

    def probe_copy_device(self, src_ptr: int, dst_ptr: int, nbytes: int) -> None:
        """Measurement aid: a plain streaming copy of known size on the pool's stream."""
        _check(self._h, self._lib.itak_probe_copy_device(self._h, src_ptr, dst_ptr, nbytes))

    def probe_read_device(self, src_ptr: int, nbytes: int) -> None:
        """Measurement aid: a plain streaming read of known size on the pool's stream."""
        _check(self._h, self._lib.itak_probe_read_device(self._h, src_ptr, nbytes))

    def probe_empty_launch(self) -> None:
        """Measurement aid: one empty kernel on the pool's stream."""
        _check(self._h, self._lib.itak_probe_empty_launch(self._h))

    def probe_mfma(self, random_operands: bool, trips: int, clocks_ptr: int = 0) -> int:
        """Measurement aid: a loop of f16 MFMAs alone on every compute unit, on the pool's
        stream; returns the launch's floating-point operations (the caller times it)."""
        flops = C.c_uint64(0)
        _check(self._h, self._lib.itak_probe_mfma(self._h, 1 if random_operands else 0, trips,
                                                  C.c_void_p(clocks_ptr or None), C.byref(flops)))
        return int(flops.value)

    def convert_f32_to_f16_device(self, src_ptr: int, dst_ptr: int, count: int) -> None:
        _check(self._h, self._lib.itak_convert_f32_to_f16_device(self._h, src_ptr, dst_ptr, count))


class Checkpoint:
    """attention::Checkpoint (cache.rs:229-273)."""

    def __init__(self, raw: N.CheckpointRaw, bases: List[int]):
        self._raw = raw
        self._bases = bases

    def base(self, layer: int) -> Optional[int]:
        return self._bases[layer] if 0 <= layer < len(self._bases) else None

    def bases(self) -> List[int]:
        return list(self._bases)

    def max_round_tokens(self) -> int:
        return int(self._raw.max_round_tokens)

    def saved_bytes(self) -> int:
        return int(self._raw.saved_bytes)


class KvCache:
    """One sequence's device cache: attention::KvCache (cache.rs:308-834) on a pool slot."""

    def __init__(self, pool: KvPool, slot: int, owns_pool: bool = False):
        self.pool = pool
        self.slot = slot
        self._owns_pool = owns_pool
        self._lib = pool._lib
        self._h = pool._h

    @staticmethod
    def new(pattern: Sequence[LayerKind], num_kv_heads: int, head_dim: int, *, elem: str = "f32",
            capacity_rows: int = 4096, device: int = 0, ring_headroom: int = 0) -> "KvCache":
        """KvCache::new: a private one-slot pool. f32 storage is the reference's."""
        pool = KvPool(pattern, num_kv_heads, head_dim, elem=elem, max_slots=1,
                      capacity_rows=capacity_rows, device=device, ring_headroom=ring_headroom)
        cache = pool.acquire()
        cache._owns_pool = True
        return cache

    def release_slot(self) -> None:
        _check(self._h, self._lib.itak_slot_release(self._h, self.slot))

    def reset(self) -> None:
        _check(self._h, self._lib.itak_slot_reset(self._h, self.slot))

    def layer_count(self) -> int:
        return int(self._lib.itak_kv_layer_count(self._h))

    def num_kv_heads(self) -> int:
        return int(self._lib.itak_kv_num_kv_heads(self._h))

    def head_dim(self) -> int:
        return int(self._lib.itak_kv_head_dim(self._h))

    def layer_kind(self, layer: int) -> LayerKind:
        kind, window = C.c_uint32(), C.c_uint64()
        _check(self._h, self._lib.itak_kv_layer_kind(self._h, layer, C.byref(kind),
                                                     C.byref(window)))
        return self.pool.pattern[layer]

    def stored_len(self, layer: int) -> int:
        out = C.c_uint64()
        _check(self._h, self._lib.itak_kv_stored_len(self._h, self.slot, layer, C.byref(out)))
        return int(out.value)

    def next_position(self, layer: int) -> int:
        out = C.c_uint64()
        _check(self._h, self._lib.itak_kv_next_position(self._h, self.slot, layer, C.byref(out)))
        return int(out.value)

    def append(self, layer: int, k, v, position: int) -> None:
        k, v = _as_f32(k), _as_f32(v)
        _check(self._h, self._lib.itak_kv_append(self._h, self.slot, layer, _ptr(k), k.size,
                                                 _ptr(v), v.size, position))

    def restore_bulk(self, layer: int, first_position: int, keys, values) -> None:
        """keys/values: f32 arrays, or uint16 arrays of f16 bits (f16 pools only)."""
        keys, values = np.ascontiguousarray(keys).reshape(-1), np.ascontiguousarray(values).reshape(-1)
        if keys.dtype == np.uint16 or keys.dtype == np.float16:
            src = N.ELEM_F16
        else:
            keys, values, src = _as_f32(keys), _as_f32(values), N.ELEM_F32
        _check(self._h, self._lib.itak_kv_restore_bulk(
            self._h, self.slot, layer, first_position, _ptr(keys), keys.size, _ptr(values),
            values.size, src))

    def restore_bulk_ptr(self, layer: int, first_position: int, keys_ptr: int, values_ptr: int,
                         elems: int, src_f16: bool) -> None:
        _check(self._h, self._lib.itak_kv_restore_bulk(
            self._h, self.slot, layer, first_position, keys_ptr, elems, values_ptr, elems,
            N.ELEM_F16 if src_f16 else N.ELEM_F32))

    @staticmethod
    def snapshot_layer_table(layers: Sequence[Tuple[int, int, int, int]]):
        """The itak_snapshot_layer array for (first_position, rows, keys_ptr, values_ptr) per
        layer: a caller that restores the same sources again builds it once."""
        raw = (N.SnapshotLayer * len(layers))()
        for i, (first, rows, kp, vp) in enumerate(layers):
            raw[i].first_position, raw[i].rows, raw[i].keys, raw[i].values = first, rows, kp, vp
        return raw

    def restore_snapshot_ptrs(self, token_count: int, layers, src_f16: bool) -> None:
        """layers: (first_position, rows, keys_ptr, values_ptr) per layer, or the array
        `snapshot_layer_table` made of them."""
        raw = layers if isinstance(layers, C.Array) else self.snapshot_layer_table(layers)
        _check(self._h, self._lib.itak_kv_restore_snapshot(
            self._h, self.slot, token_count, raw, len(layers),
            N.ELEM_F16 if src_f16 else N.ELEM_F32), "restore_snapshot")

    def view(self, layer: int) -> "CacheView":
        self.stored_len(layer)
        return CacheView(self, layer)

    def stats(self) -> List[LayerStats]:
        n = self.layer_count()
        raw = (N.LayerStatsRaw * n)()
        _check(self._h, self._lib.itak_kv_stats(self._h, self.slot, raw))
        return [LayerStats(int(s.layer), self.pool.pattern[i], int(s.appended), int(s.stored))
                for i, s in enumerate(raw)]

    def read_rows(self, layer: int, first: int, rows: int):
        """(positions, keys, values): raw storage elements, [rows][kv_heads][head_dim]."""
        shape = (rows, self.pool.num_kv_heads, self.pool.head_dim)
        keys = np.empty(shape, dtype=self.pool.np_elem)
        vals = np.empty(shape, dtype=self.pool.np_elem)
        pos = np.empty(rows, dtype=np.uint64)
        _check(self._h, self._lib.itak_kv_read_rows(self._h, self.slot, layer, first, rows,
                                                    _ptr(keys), _ptr(vals), _ptr(pos)))
        return pos, keys, vals

    def read_raw(self, layer: int):
        """Every storage row of the layer, visible or not: (keys, values)."""
        rows = C.c_uint64()
        _check(self._h, self._lib.itak_kv_storage_rows(self._h, layer, C.byref(rows)))
        shape = (rows.value, self.pool.num_kv_heads, self.pool.head_dim)
        keys = np.empty(shape, dtype=self.pool.np_elem)
        vals = np.empty(shape, dtype=self.pool.np_elem)
        _check(self._h, self._lib.itak_kv_read_raw(self._h, self.slot, layer, _ptr(keys),
                                                   _ptr(vals)))
        return keys, vals

    def checkpoint_active(self) -> bool:
        out = C.c_int32()
        _check(self._h, self._lib.itak_kv_checkpoint_active(self._h, self.slot, C.byref(out)))
        return bool(out.value)

    def _bases(self, raw: N.CheckpointRaw) -> List[int]:
        bases = np.empty(self.layer_count(), dtype=np.uint64)
        _check(self._h, self._lib.itak_kv_checkpoint_bases(self._h, self.slot, C.byref(raw),
                                                           _ptr(bases)))
        return [int(b) for b in bases]

    def checkpoint(self, max_round_tokens: int) -> Checkpoint:
        raw = N.CheckpointRaw()
        _check(self._h, self._lib.itak_kv_checkpoint(self._h, self.slot, max_round_tokens,
                                                     C.byref(raw)))
        return Checkpoint(raw, self._bases(raw))

    def rewind_to(self, cp: Checkpoint, target: int) -> None:
        _check(self._h, self._lib.itak_kv_rewind_to(self._h, self.slot, C.byref(cp._raw), target))

    def release(self, cp: Checkpoint) -> None:
        _check(self._h, self._lib.itak_kv_release(self._h, self.slot, C.byref(cp._raw)))


class CacheView:
    """attention::CacheView (cache.rs:841-904). Rows come back as f32 whatever the storage."""

    def __init__(self, cache: KvCache, layer: int):
        self._c = cache
        self._layer = layer

    def kind(self) -> LayerKind:
        return self._c.layer_kind(self._layer)

    def window(self) -> Optional[int]:
        return self.kind().window()

    def num_kv_heads(self) -> int:
        return self._c.num_kv_heads()

    def head_dim(self) -> int:
        return self._c.head_dim()

    def len(self) -> int:
        return self._c.stored_len(self._layer)

    def __len__(self) -> int:
        return self.len()

    def is_empty(self) -> bool:
        return self.len() == 0

    def position_at(self, visible_index: int) -> Optional[int]:
        if visible_index >= self.len():
            return None
        pos, _, _ = self._c.read_rows(self._layer, visible_index, 1)
        return int(pos[0])

    def _decode(self, raw: np.ndarray) -> np.ndarray:
        return raw.view(np.float16).astype(np.float32) if raw.dtype == np.uint16 else raw

    def key(self, visible_index: int, kv_head: int) -> Optional[np.ndarray]:
        if visible_index >= self.len() or kv_head >= self.num_kv_heads():
            return None
        _, k, _ = self._c.read_rows(self._layer, visible_index, 1)
        return self._decode(k)[0, kv_head]

    def value(self, visible_index: int, kv_head: int) -> Optional[np.ndarray]:
        if visible_index >= self.len() or kv_head >= self.num_kv_heads():
            return None
        _, _, v = self._c.read_rows(self._layer, visible_index, 1)
        return self._decode(v)[0, kv_head]

    def rows(self):
        """(positions, keys, values) of every visible entry; raw storage elements."""
        return self._c.read_rows(self._layer, 0, self.len())


def gqa_attention(q, num_queries: int, num_q_heads: int, query_positions: Sequence[int],
                  view: CacheView, params: AttentionParams = AttentionParams()) -> np.ndarray:
    """attention::gqa_attention (attention.rs:104-215) on the device; flat f32 output."""
    q = _as_f32(q)
    pos = np.asarray(query_positions, dtype=np.uint64).reshape(-1)
    out = np.zeros(q.size, dtype=np.float32)
    c = view._c
    _check(c._h, c._lib.itak_gqa_attention(
        c._h, c.slot, view._layer, _ptr(q), q.size, num_queries, num_q_heads, _ptr(pos), pos.size,
        math.nan if params.scale is None else float(params.scale), float(params.softcap),
        _ptr(out)))
    return out if num_queries else out[:0]


# ------------------------------------------------------- Compute::attention boundary

@dataclass
class GlimmerConfig:
    """The fields of muse_glimmer::GlimmerConfig this path reads (config.rs:249-261)."""

    layers: List[LayerKind]
    q_heads: int
    kv_heads: int
    key_length: int
    value_length: int
    sliding_window: int = 0
    rope_freq_base_swa: float = 10000.0

    def q_width(self) -> int:
        return self.q_heads * self.key_length

    def k_width(self) -> int:
        return self.kv_heads * self.key_length

    def v_width(self) -> int:
        return self.kv_heads * self.value_length

    def layer_kind(self, layer: int) -> Optional[LayerKind]:
        return self.layers[layer] if 0 <= layer < len(self.layers) else None


@dataclass
class AttentionRequest:
    """muse_glimmer::AttentionRequest (compute.rs:29-44)."""

    q: np.ndarray
    k: np.ndarray
    v: np.ndarray
    layer: int
    kind: LayerKind
    cfg: GlimmerConfig


class PositionCache:
    """muse_glimmer::PositionCache (cache.rs:46-75): the position contract only."""

    def __init__(self):
        self._position = 0

    def position(self) -> int:
        return self._position

    def advance(self, tokens: int) -> None:
        self._position += tokens

    def rewind_to(self, position: int) -> None:
        assert position <= self._position
        self._position = position


class HipCompute:
    """The attention half of a muse_glimmer::Compute backend, shaped like CpuCompute
    (cpu.rs:246-339, 506-655): one instance serves one sequence, owns its KV state, builds
    it from the first config it sees and refuses a different shape until reset()."""

    def __init__(self, *, elem: str = "f16", capacity_rows: int = 4096, softcap: float = 0.0,
                 device: int = 0, pool: Optional[KvPool] = None):
        self._elem = elem
        self._capacity = capacity_rows
        self._softcap = softcap
        self._device = device
        self._pool = pool
        self._owns_pool = pool is None
        self._cache: Optional[KvCache] = None
        self._shape = None

    @staticmethod
    def new(**kw) -> "HipCompute":
        return HipCompute(**kw)

    @staticmethod
    def _shape_of(cfg: GlimmerConfig):
        return (tuple(cfg.layers), cfg.kv_heads, cfg.key_length, cfg.value_length,
                cfg.sliding_window)

    def kv_cache(self) -> Optional[KvCache]:
        return self._cache

    def reset(self) -> None:
        """CpuCompute::reset (cpu.rs:264-268)."""
        if self._cache is not None:
            self._cache.reset()
        self._shape = None

    def _build(self, cfg: GlimmerConfig, step: str) -> None:
        pattern = [LayerKind.Global if not k.is_windowed else LayerKind.Windowed(cfg.sliding_window)
                   for k in cfg.layers]
        try:
            if self._pool is None:
                self._pool = KvPool(pattern, cfg.kv_heads, cfg.key_length, elem=self._elem,
                                    max_slots=1, capacity_rows=self._capacity,
                                    device=self._device)
            if self._cache is None:
                self._cache = self._pool.acquire()
        except AttentionError as e:
            raise StepFailed(step, e.message or str(e)) from e
        self._shape = self._shape_of(cfg)

    def attention(self, req: AttentionRequest, cache) -> np.ndarray:
        """Compute::attention (compute.rs:82, cpu.rs:506-655)."""
        step = "attention"
        cfg = req.cfg
        if cfg.key_length != cfg.value_length:
            raise StepFailed(step, f"key_length {cfg.key_length} != value_length "
                                   f"{cfg.value_length}: the KV cache stores keys and values at "
                                   "one head dimension")
        if cfg.layer_kind(req.layer) != req.kind:
            raise StepFailed(step, f"request kind {req.kind} does not match the config's kind for "
                                   f"layer {req.layer}")
        q, k, v = _as_f32(req.q), _as_f32(req.k), _as_f32(req.v)
        if self._shape is None:
            self._build(cfg, step)
        elif self._shape != self._shape_of(cfg):
            raise StepFailed(step, "this HipCompute already serves a model of a different shape; "
                                   "construct a fresh HipCompute per model (or reset this one) "
                                   "instead of retargeting it mid-sequence")
        out = np.zeros(q.size, dtype=np.float32)
        c = self._cache
        _check(c._h, c._lib.itak_compute_attention(
            c._h, c.slot, req.layer, _ptr(q), q.size, _ptr(k), k.size, _ptr(v), v.size,
            cfg.q_heads, cache.position(), self._softcap, cfg.rope_freq_base_swa, _ptr(out)),
            step)
        return out

    def _need_cache(self) -> KvCache:
        if self._cache is None:
            # Route through the library so the refusal text is the library's.
            raise StepFailed("cache_checkpoint",
                             "no KV state exists yet: a speculative round checkpoints after a "
                             "first forward has built the cache (the spec's prefill), not before")
        return self._cache

    def cache_checkpoint(self, max_round_tokens: int) -> Checkpoint:
        c = self._need_cache()
        raw = N.CheckpointRaw()
        _check(c._h, c._lib.itak_compute_cache_checkpoint(c._h, c.slot, max_round_tokens,
                                                          C.byref(raw)), "cache_checkpoint")
        return Checkpoint(raw, c._bases(raw))

    def cache_rewind(self, checkpoint: Checkpoint, target: int) -> None:
        c = self._need_cache()
        _check(c._h, c._lib.itak_compute_cache_rewind(c._h, c.slot, C.byref(checkpoint._raw),
                                                      target), "cache_rewind")

    def cache_release(self, checkpoint: Checkpoint) -> None:
        c = self._need_cache()
        _check(c._h, c._lib.itak_compute_cache_release(c._h, c.slot, C.byref(checkpoint._raw)),
               "cache_release")
