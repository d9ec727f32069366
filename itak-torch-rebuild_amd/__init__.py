"""MI355X (gfx950) KV-cache and attention backend: Python front end of the C ABI.

The names mirror the reference's Rust API for this path (attention::KvCache,
attention::gqa_attention, cpu_compute::CpuCompute, muse_glimmer::{AttentionRequest,
PositionCache}); every operation runs in the HIP library, nothing falls back to the CPU.
"""
from .hip_compute import (  # noqa: F401
    AttentionError,
    AttentionParams,
    AttentionRequest,
    CacheView,
    Checkpoint,
    GlimmerConfig,
    HipCompute,
    KvCache,
    KvPool,
    LayerKind,
    LayerStats,
    PositionCache,
    debug_enabled,
    set_debug_enabled,
    StepFailed,
    gqa_attention,
    kv_head_for_query_head,
)
from .itak_kv import (  # noqa: F401
    KvError,
    KvGeometry,
    KvSnapshot,
    LayerSnapshot,
    SNAPSHOT_FORMAT_VERSION,
    capture_bytes,
    checksum,
    checksum_blocks,
    prefix_discriminator,
    prefix_hash,
    restore_bytes,
)
from .prefix_store import (  # noqa: F401
    EntryMeta,
    PrefixHit,
    PrefixStore,
    StoreConfig,
    StoreStats,
    max_bytes_from,
    now_unix,
    prefix_store_enabled,
    prefix_store_enabled_from,
)
from .resident import LayerInputCapture, ResidentTarget, SpecRoundRecord  # noqa: F401
from . import _native  # noqa: F401

__all__ = [
    "AttentionError", "AttentionParams", "AttentionRequest", "CacheView", "Checkpoint",
    "GlimmerConfig", "HipCompute", "KvCache", "KvPool", "LayerKind", "LayerStats",
    "PositionCache", "StepFailed", "gqa_attention", "kv_head_for_query_head",
    "KvError", "KvGeometry", "KvSnapshot", "LayerSnapshot", "SNAPSHOT_FORMAT_VERSION",
    "capture_bytes", "checksum", "checksum_blocks", "prefix_discriminator", "prefix_hash", "restore_bytes",
    "EntryMeta", "PrefixHit", "PrefixStore", "StoreConfig", "StoreStats", "max_bytes_from",
    "now_unix", "prefix_store_enabled", "prefix_store_enabled_from",
    "LayerInputCapture", "ResidentTarget", "SpecRoundRecord",
]
