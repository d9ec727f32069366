"""ctypes binding of libitak_hip_kv.so (the C ABI declared in include/itak_hip_kv.h).

There is no fallback: if the library is missing or does not export a declared symbol,
import fails with an error that says how to build it.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libitak_hip_kv.so")

OK = 0
STATUS_NAMES = {
    1: "ZeroDimension", 2: "InvalidWindow", 3: "SizeOverflow", 4: "ShapeMismatch",
    5: "InvalidLayer", 6: "OutOfOrderPosition", 7: "NonDivisibleHeads", 8: "NoVisibleKeys",
    9: "CheckpointBusy", 10: "StaleCheckpoint", 11: "CheckpointTooDeep",
    12: "CheckpointRangeExceeded", 13: "BulkRestoreNotFresh", 14: "RewindOutOfRange",
    15: "StepFailed", 16: "HipError", 17: "InvalidArgument", 18: "NoFreeSlot",
    19: "CapacityExceeded", 20: "Unsupported",
    21: "BadMagic", 22: "UnsupportedVersion", 23: "Truncated", 24: "ChecksumMismatch",
    25: "InconsistentSnapshot", 26: "GeometryMismatch", 27: "FingerprintMismatch",
    28: "IncoherentCache",
    29: "EmptyPrefix", 30: "TokenCountMismatch", 31: "PrefixHashMismatch",
    32: "SnapshotTokenMismatch", 33: "EntryTooLarge", 34: "InvalidConfig", 35: "Io",
}
KV_ERROR_FIRST, KV_ERROR_LAST = 21, 35
ELEM_F32, ELEM_F16 = 0, 1
LAYER_GLOBAL, LAYER_WINDOWED = 0, 1
POOL_SCRUB_ON_TRUNCATE = 1
POOL_MERGE_IN_LAUNCH = 2
POOL_DIE_MERGE = 4
POOL_Q_TWO_HALVES = 8
POOL_PREP_BY_LAUNCH = 16


class PoolConfig(C.Structure):
    _fields_ = [
        ("layer_count", C.c_uint32),
        ("layer_kinds", C.c_void_p),
        ("windows", C.c_void_p),
        ("num_kv_heads", C.c_uint64),
        ("head_dim", C.c_uint64),
        ("elem", C.c_uint32),
        ("max_slots", C.c_uint32),
        ("capacity_rows", C.c_uint64),
        ("device", C.c_int32),
        ("flags", C.c_uint32),
        ("ring_headroom", C.c_uint64),
    ]


class ErrorInfo(C.Structure):
    _fields_ = [("code", C.c_int32), ("what", C.c_char * 96), ("a", C.c_uint64),
                ("b", C.c_uint64), ("c", C.c_uint64), ("d", C.c_uint64)]


class CheckpointRaw(C.Structure):
    _fields_ = [("cache_id", C.c_uint64), ("serial", C.c_uint64),
                ("max_round_tokens", C.c_uint64), ("saved_bytes", C.c_uint64)]


class LayerStatsRaw(C.Structure):
    _fields_ = [("layer", C.c_uint64), ("kind", C.c_uint32), ("reserved", C.c_uint32),
                ("window", C.c_uint64), ("appended", C.c_uint64), ("stored", C.c_uint64)]


class BatchItem(C.Structure):
    _fields_ = [("slot", C.c_uint32), ("rows", C.c_uint32)]


class SnapshotLayer(C.Structure):
    _fields_ = [("first_position", C.c_uint64), ("rows", C.c_uint64), ("keys", C.c_void_p),
                ("values", C.c_void_p)]


class PrepParams(C.Structure):
    _fields_ = [("q_norm_weight", C.c_void_p), ("k_norm_weight", C.c_void_p), ("eps", C.c_float),
                ("rope_base", C.c_float), ("rope_interleaved", C.c_uint32),
                ("rotary_dim", C.c_uint32)]


class ItkvHeader(C.Structure):
    _fields_ = [("token_count", C.c_uint64), ("num_kv_heads", C.c_uint64),
                ("head_dim", C.c_uint64), ("layer_count", C.c_uint64),
                ("fingerprint_len", C.c_uint64), ("fingerprint_offset", C.c_uint64),
                ("encoded_len", C.c_uint64), ("version", C.c_uint32), ("elem", C.c_uint32)]


class ItkvLayer(C.Structure):
    _fields_ = [("kind", C.c_uint32), ("reserved", C.c_uint32), ("window", C.c_uint64),
                ("first_position", C.c_uint64), ("rows", C.c_uint64),
                ("keys_offset", C.c_uint64), ("values_offset", C.c_uint64)]


class StoreEntry(C.Structure):
    _fields_ = [("file_name", C.c_char * 96), ("prefix_hash", C.c_uint64),
                ("token_count", C.c_uint64), ("bytes", C.c_uint64), ("created_unix", C.c_uint64),
                ("last_used_unix", C.c_uint64)]


class StoreStats(C.Structure):
    _fields_ = [("entries", C.c_uint64), ("total_bytes", C.c_uint64), ("max_bytes", C.c_uint64)]


class PrefixHit(C.Structure):
    _fields_ = [("token_count", C.c_uint64), ("snapshot", C.c_void_p),
                ("snapshot_len", C.c_uint64), ("file_name", C.c_char * 96)]


_P = C.c_void_p
_u32, _u64, _f32, _i32 = C.c_uint32, C.c_uint64, C.c_float, C.c_int32

# name -> (restype, argtypes): every symbol include/itak_hip_kv.h declares.
PROTOTYPES = {
    "itak_abi_version": (_u32, []),
    "itak_last_error": (C.c_char_p, [_P]),
    "itak_last_error_info": (_i32, [_P, C.POINTER(ErrorInfo)]),
    "itak_pool_create": (_i32, [C.POINTER(PoolConfig), C.POINTER(_P)]),
    "itak_pool_destroy": (None, [_P]),
    "itak_pool_set_stream": (_i32, [_P, _P]),
    "itak_pool_synchronize": (_i32, [_P]),
    "itak_pool_set_merge_spin_limit": (_i32, [_P, _u32]),
    "itak_pool_device_bytes": (_u64, [_P]),
    "itak_slot_acquire": (_i32, [_P, C.POINTER(_u32)]),
    "itak_slot_release": (_i32, [_P, _u32]),
    "itak_slot_reset": (_i32, [_P, _u32]),
    "itak_kv_layer_count": (_u64, [_P]),
    "itak_kv_num_kv_heads": (_u64, [_P]),
    "itak_kv_head_dim": (_u64, [_P]),
    "itak_kv_layer_kind": (_i32, [_P, _u64, C.POINTER(_u32), C.POINTER(_u64)]),
    "itak_kv_storage_rows": (_i32, [_P, _u64, C.POINTER(_u64)]),
    "itak_kv_stored_len": (_i32, [_P, _u32, _u64, C.POINTER(_u64)]),
    "itak_kv_next_position": (_i32, [_P, _u32, _u64, C.POINTER(_u64)]),
    "itak_kv_append": (_i32, [_P, _u32, _u64, _P, _u64, _P, _u64, _u64]),
    "itak_kv_restore_bulk": (_i32, [_P, _u32, _u64, _u64, _P, _u64, _P, _u64, _u32]),
    "itak_kv_restore_snapshot": (_i32, [_P, _u32, _u64, C.POINTER(SnapshotLayer), _u64, _u32]),
    "itak_kv_prefix_hash": (_u64, [_P, _u64]),
    "itak_kv_prefix_discriminator": (_u64, [_P, _u64]),
    "itak_kv_checksum": (_u64, [_P, _u64]),
    "itak_kv_checksum_blocks": (_u64, [_P, _u64]),
    "itak_itkv_validate": (_i32, [C.POINTER(ItkvHeader), C.POINTER(ItkvLayer), _u64, _P, _P]),
    "itak_itkv_encode": (_i32, [C.POINTER(ItkvHeader), C.c_char_p, C.POINTER(ItkvLayer), _u64, _P,
                                _P, _P, _P, _P, _u64, C.POINTER(_u64)]),
    "itak_itkv_decode": (_i32, [_P, _u64, C.POINTER(ItkvHeader), C.POINTER(ItkvLayer), _u64]),
    "itak_kv_capture_itkv": (_i32, [_P, _u32, C.c_char_p, _u64, _P, _u64, C.POINTER(_u64)]),
    "itak_kv_capture_itkv_f16": (_i32, [_P, _u32, C.c_char_p, _u64, _P, _u64, C.POINTER(_u64)]),
    "itak_kv_restore_itkv": (_i32, [_P, _u32, _P, _u64, C.c_char_p, _u64]),
    "itak_kv_stats": (_i32, [_P, _u32, C.POINTER(LayerStatsRaw)]),
    "itak_kv_read_rows": (_i32, [_P, _u32, _u64, _u64, _u64, _P, _P, _P]),
    "itak_kv_read_raw": (_i32, [_P, _u32, _u64, _P, _P]),
    "itak_kv_checkpoint_active": (_i32, [_P, _u32, C.POINTER(_i32)]),
    "itak_kv_checkpoint": (_i32, [_P, _u32, _u64, C.POINTER(CheckpointRaw)]),
    "itak_kv_checkpoint_bases": (_i32, [_P, _u32, C.POINTER(CheckpointRaw), _P]),
    "itak_kv_rewind_to": (_i32, [_P, _u32, C.POINTER(CheckpointRaw), _u64]),
    "itak_kv_release": (_i32, [_P, _u32, C.POINTER(CheckpointRaw)]),
    "itak_kv_truncate": (_i32, [_P, _P, _P, _u32]),
    "itak_gqa_attention": (_i32, [_P, _u32, _u64, _P, _u64, _u64, _u64, _P, _u64, _f32, _f32, _P]),
    "itak_compute_attention": (_i32, [_P, _u32, _u64, _P, _u64, _P, _u64, _P, _u64, _u64, _u64,
                                      _f32, _f32, _P]),
    "itak_compute_cache_checkpoint": (_i32, [_P, _u32, _u64, C.POINTER(CheckpointRaw)]),
    "itak_compute_cache_rewind": (_i32, [_P, _u32, C.POINTER(CheckpointRaw), _u64]),
    "itak_compute_cache_release": (_i32, [_P, _u32, C.POINTER(CheckpointRaw)]),
    "itak_attention_step_device": (_i32, [_P, _u64, C.POINTER(BatchItem), _u32, _P, _P, _P, _P,
                                          _u64, _f32, _f32]),
    "itak_attention_step_device_noalloc": (_i32, [_P, _u64, C.POINTER(BatchItem), _u32, _P, _P, _P,
                                                  _P, _u64, _f32, _f32]),
    "itak_attention_prep_step_device": (_i32, [_P, _u64, C.POINTER(BatchItem), _u32, _P, _P, _P, _P,
                                               _P, _u64, _f32, _f32, C.POINTER(PrepParams)]),
    "itak_attention_device": (_i32, [_P, _u64, C.POINTER(BatchItem), _u32, _P, _P, _u64, _f32,
                                     _f32]),
    "itak_kv_append_device": (_i32, [_P, _u64, C.POINTER(BatchItem), _u32, _P, _P]),
    "itak_kv_now_unix": (_u64, []),
    "itak_store_open": (_i32, [C.c_char_p, _u64, C.POINTER(_P)]),
    "itak_store_close": (None, [_P]),
    "itak_store_last_error": (C.c_char_p, [_P]),
    "itak_store_last_error_info": (_i32, [_P, C.POINTER(ErrorInfo)]),
    "itak_store_refusals": (C.c_char_p, [_P]),
    "itak_store_clear_refusals": (None, [_P]),
    "itak_store_rescan": (_i32, [_P]),
    "itak_store_get_stats": (_i32, [_P, C.POINTER(StoreStats)]),
    "itak_store_entries": (_i32, [_P, C.POINTER(StoreEntry), _u64, C.POINTER(_u64)]),
    "itak_store_put": (_i32, [_P, _P, _u64, _P, _u64, _u64]),
    "itak_store_lookup": (_i32, [_P, _P, _u64, C.POINTER(ItkvHeader), C.POINTER(ItkvLayer),
                                 C.c_char_p, _u64, _u64, C.POINTER(PrefixHit)]),
    "itak_store_restore_prefix": (_i32, [_P, _P, _u32, _P, _u64, C.c_char_p, _u64, _u64,
                                         C.POINTER(_u64)]),
    "itak_store_capture_and_put": (_i32, [_P, _P, _u32, _P, _u64, C.c_char_p, _u64, _u32, _u64]),
    "itak_convert_f32_to_f16_device": (_i32, [_P, _P, _P, _u64]),
    "itak_probe_copy_device": (_i32, [_P, _P, _P, _u64]),
    "itak_probe_read_device": (_i32, [_P, _P, _u64]),
    "itak_probe_empty_launch": (_i32, [_P]),
    "itak_probe_mfma": (_i32, [_P, _u32, _u32, _P, _P]),
    "itak_set_debug_enabled": (None, [_i32]),
    "itak_debug_enabled": (_i32, []),
}

_lib = None


def load():
    """Load the library and bind every declared symbol; raises if anything is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python {os.path.join(HERE, 'build.py')}` "
            "(hipcc --offload-arch=gfx950). There is no CPU fallback.")
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError names the missing symbol
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib
