//! Raw binding of `include/itak_hip_kv.h` (the C ABI of `libitak_hip_kv.so`), written by
//! `gen_bindings.py` from the header: do not edit by hand. The safe wrapper over it is the
//! `safe` module of this crate's sibling `hip-compute`; every `unsafe` of the backend lives
//! behind these declarations (the reference's hot-path crates forbid it, `Cargo.toml:12-43`).
#![allow(non_camel_case_types)]
#![allow(clippy::too_many_arguments)]
#![allow(missing_docs)]

use std::os::raw::{c_char, c_void};

/// Status of every call: 0 is success (`ITAK_OK`), the rest are the `ITAK_*` constants.
pub type itak_status = i32;

pub const ITAK_OK: u32 = 0;
pub const ITAK_ZERO_DIMENSION: u32 = 1;
pub const ITAK_INVALID_WINDOW: u32 = 2;
pub const ITAK_SIZE_OVERFLOW: u32 = 3;
pub const ITAK_SHAPE_MISMATCH: u32 = 4;
pub const ITAK_INVALID_LAYER: u32 = 5;
pub const ITAK_OUT_OF_ORDER_POSITION: u32 = 6;
pub const ITAK_NON_DIVISIBLE_HEADS: u32 = 7;
pub const ITAK_NO_VISIBLE_KEYS: u32 = 8;
pub const ITAK_CHECKPOINT_BUSY: u32 = 9;
pub const ITAK_STALE_CHECKPOINT: u32 = 10;
pub const ITAK_CHECKPOINT_TOO_DEEP: u32 = 11;
pub const ITAK_CHECKPOINT_RANGE_EXCEEDED: u32 = 12;
pub const ITAK_BULK_RESTORE_NOT_FRESH: u32 = 13;
pub const ITAK_REWIND_OUT_OF_RANGE: u32 = 14;
pub const ITAK_STEP_FAILED: u32 = 15;
pub const ITAK_HIP_ERROR: u32 = 16;
pub const ITAK_INVALID_ARGUMENT: u32 = 17;
pub const ITAK_NO_FREE_SLOT: u32 = 18;
pub const ITAK_CAPACITY_EXCEEDED: u32 = 19;
pub const ITAK_UNSUPPORTED: u32 = 20;
pub const ITAK_KV_BAD_MAGIC: u32 = 21;
pub const ITAK_KV_UNSUPPORTED_VERSION: u32 = 22;
pub const ITAK_KV_TRUNCATED: u32 = 23;
pub const ITAK_KV_CHECKSUM_MISMATCH: u32 = 24;
pub const ITAK_KV_INCONSISTENT_SNAPSHOT: u32 = 25;
pub const ITAK_KV_GEOMETRY_MISMATCH: u32 = 26;
pub const ITAK_KV_FINGERPRINT_MISMATCH: u32 = 27;
pub const ITAK_KV_INCOHERENT_CACHE: u32 = 28;
pub const ITAK_KV_EMPTY_PREFIX: u32 = 29;
pub const ITAK_KV_TOKEN_COUNT_MISMATCH: u32 = 30;
pub const ITAK_KV_PREFIX_HASH_MISMATCH: u32 = 31;
pub const ITAK_KV_SNAPSHOT_TOKEN_MISMATCH: u32 = 32;
pub const ITAK_KV_ENTRY_TOO_LARGE: u32 = 33;
pub const ITAK_KV_INVALID_CONFIG: u32 = 34;
pub const ITAK_KV_IO: u32 = 35;
pub const ITAK_ELEM_F32: u32 = 0;
pub const ITAK_ELEM_F16: u32 = 1;
pub const ITAK_LAYER_GLOBAL: u32 = 0;
pub const ITAK_LAYER_WINDOWED: u32 = 1;
pub const ITAK_POOL_SCRUB_ON_TRUNCATE: u32 = 1;
pub const ITAK_POOL_MERGE_IN_LAUNCH: u32 = 2;
pub const ITAK_POOL_DIE_MERGE: u32 = 4;
pub const ITAK_POOL_Q_TWO_HALVES: u32 = 8;
pub const ITAK_POOL_PREP_BY_LAUNCH: u32 = 16;

/// Opaque handle.
#[repr(C)]
pub struct itak_pool {
    _private: [u8; 0],
}

/// Opaque handle.
#[repr(C)]
pub struct itak_store {
    _private: [u8; 0],
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct itak_pool_config {
    pub layer_count: u32,
    pub layer_kinds: *const u8,
    pub windows: *const u64,
    pub num_kv_heads: u64,
    pub head_dim: u64,
    pub elem: u32,
    pub max_slots: u32,
    pub capacity_rows: u64,
    pub device: i32,
    pub flags: u32,
    pub ring_headroom: u64,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct itak_error_info {
    pub code: i32,
    pub what: [c_char; 96],
    pub a: u64,
    pub b: u64,
    pub c: u64,
    pub d: u64,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct itak_checkpoint {
    pub cache_id: u64,
    pub serial: u64,
    pub max_round_tokens: u64,
    pub saved_bytes: u64,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct itak_layer_stats {
    pub layer: u64,
    pub kind: u32,
    pub reserved: u32,
    pub window: u64,
    pub appended: u64,
    pub stored: u64,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct itak_batch_item {
    pub slot: u32,
    pub rows: u32,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct itak_snapshot_layer {
    pub first_position: u64,
    pub rows: u64,
    pub keys: *const c_void,
    pub values: *const c_void,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct itak_itkv_header {
    pub token_count: u64,
    pub num_kv_heads: u64,
    pub head_dim: u64,
    pub layer_count: u64,
    pub fingerprint_len: u64,
    pub fingerprint_offset: u64,
    pub encoded_len: u64,
    pub version: u32,
    pub elem: u32,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct itak_itkv_layer {
    pub kind: u32,
    pub reserved: u32,
    pub window: u64,
    pub first_position: u64,
    pub rows: u64,
    pub keys_offset: u64,
    pub values_offset: u64,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct itak_store_entry {
    pub file_name: [c_char; 96],
    pub prefix_hash: u64,
    pub token_count: u64,
    pub bytes: u64,
    pub created_unix: u64,
    pub last_used_unix: u64,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct itak_store_stats {
    pub entries: u64,
    pub total_bytes: u64,
    pub max_bytes: u64,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct itak_prefix_hit {
    pub token_count: u64,
    pub snapshot: *const c_void,
    pub snapshot_len: u64,
    pub file_name: [c_char; 96],
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct itak_prep_params {
    pub q_norm_weight: *const f32,
    pub k_norm_weight: *const f32,
    pub eps: f32,
    pub rope_base: f32,
    pub rope_interleaved: u32,
    pub rotary_dim: u32,
}

#[link(name = "itak_hip_kv")]
extern "C" {
    pub fn itak_abi_version() -> u32;
    pub fn itak_last_error(pool: *const itak_pool) -> *const c_char;
    pub fn itak_last_error_info(pool: *const itak_pool, out: *mut itak_error_info) -> itak_status;
    pub fn itak_pool_create(config: *const itak_pool_config, out: *mut *mut itak_pool) -> itak_status;
    pub fn itak_pool_destroy(pool: *mut itak_pool);
    pub fn itak_pool_set_stream(pool: *mut itak_pool, hip_stream: *mut c_void) -> itak_status;
    pub fn itak_pool_synchronize(pool: *mut itak_pool) -> itak_status;
    pub fn itak_pool_set_merge_spin_limit(pool: *mut itak_pool, polls: u32) -> itak_status;
    pub fn itak_pool_device_bytes(pool: *const itak_pool) -> u64;
    pub fn itak_slot_acquire(pool: *mut itak_pool, slot: *mut u32) -> itak_status;
    pub fn itak_slot_release(pool: *mut itak_pool, slot: u32) -> itak_status;
    pub fn itak_slot_reset(pool: *mut itak_pool, slot: u32) -> itak_status;
    pub fn itak_kv_layer_count(pool: *const itak_pool) -> u64;
    pub fn itak_kv_num_kv_heads(pool: *const itak_pool) -> u64;
    pub fn itak_kv_head_dim(pool: *const itak_pool) -> u64;
    pub fn itak_kv_layer_kind(pool: *mut itak_pool, layer: u64, kind: *mut u32, window: *mut u64) -> itak_status;
    pub fn itak_kv_storage_rows(pool: *mut itak_pool, layer: u64, out: *mut u64) -> itak_status;
    pub fn itak_kv_stored_len(pool: *mut itak_pool, slot: u32, layer: u64, out: *mut u64) -> itak_status;
    pub fn itak_kv_next_position(pool: *mut itak_pool, slot: u32, layer: u64, out: *mut u64) -> itak_status;
    pub fn itak_kv_append(pool: *mut itak_pool, slot: u32, layer: u64, k: *const f32, k_len: u64, v: *const f32, v_len: u64, position: u64) -> itak_status;
    pub fn itak_kv_restore_bulk(pool: *mut itak_pool, slot: u32, layer: u64, first_position: u64, keys: *const c_void, keys_len: u64, values: *const c_void, values_len: u64, src_elem: u32) -> itak_status;
    pub fn itak_kv_restore_snapshot(pool: *mut itak_pool, slot: u32, token_count: u64, layers: *const itak_snapshot_layer, layer_count: u64, src_elem: u32) -> itak_status;
    pub fn itak_kv_stats(pool: *mut itak_pool, slot: u32, out: *mut itak_layer_stats) -> itak_status;
    pub fn itak_kv_read_rows(pool: *mut itak_pool, slot: u32, layer: u64, first: u64, rows: u64, keys_out: *mut c_void, values_out: *mut c_void, positions_out: *mut u64) -> itak_status;
    pub fn itak_kv_read_raw(pool: *mut itak_pool, slot: u32, layer: u64, keys_out: *mut c_void, values_out: *mut c_void) -> itak_status;
    pub fn itak_kv_checkpoint_active(pool: *mut itak_pool, slot: u32, out: *mut i32) -> itak_status;
    pub fn itak_kv_checkpoint(pool: *mut itak_pool, slot: u32, max_round_tokens: u64, out: *mut itak_checkpoint) -> itak_status;
    pub fn itak_kv_checkpoint_bases(pool: *mut itak_pool, slot: u32, cp: *const itak_checkpoint, out: *mut u64) -> itak_status;
    pub fn itak_kv_rewind_to(pool: *mut itak_pool, slot: u32, cp: *const itak_checkpoint, target: u64) -> itak_status;
    pub fn itak_kv_release(pool: *mut itak_pool, slot: u32, cp: *const itak_checkpoint) -> itak_status;
    pub fn itak_kv_truncate(pool: *mut itak_pool, slots: *const u32, new_lengths: *const u64, count: u32) -> itak_status;
    pub fn itak_kv_prefix_hash(tokens: *const u32, count: u64) -> u64;
    pub fn itak_kv_prefix_discriminator(tokens: *const u32, count: u64) -> u64;
    pub fn itak_kv_checksum(bytes: *const c_void, count: u64) -> u64;
    pub fn itak_kv_checksum_blocks(bytes: *const c_void, count: u64) -> u64;
    pub fn itak_itkv_validate(header: *const itak_itkv_header, layers: *const itak_itkv_layer, blocks: u64, key_floats: *const u64, value_floats: *const u64) -> itak_status;
    pub fn itak_itkv_encode(header: *const itak_itkv_header, fingerprint: *const c_char, layers: *const itak_itkv_layer, blocks: u64, keys: *const *const f32, key_floats: *const u64, values: *const *const f32, value_floats: *const u64, out: *mut c_void, capacity: u64, written: *mut u64) -> itak_status;
    pub fn itak_itkv_decode(bytes: *const c_void, len: u64, header: *mut itak_itkv_header, layers: *mut itak_itkv_layer, layers_capacity: u64) -> itak_status;
    pub fn itak_kv_capture_itkv(pool: *mut itak_pool, slot: u32, fingerprint: *const c_char, fingerprint_len: u64, out: *mut c_void, capacity: u64, written: *mut u64) -> itak_status;
    pub fn itak_kv_capture_itkv_f16(pool: *mut itak_pool, slot: u32, fingerprint: *const c_char, fingerprint_len: u64, out: *mut c_void, capacity: u64, written: *mut u64) -> itak_status;
    pub fn itak_kv_restore_itkv(pool: *mut itak_pool, slot: u32, bytes: *const c_void, len: u64, expected_fingerprint: *const c_char, expected_fingerprint_len: u64) -> itak_status;
    pub fn itak_kv_now_unix() -> u64;
    pub fn itak_store_open(root: *const c_char, max_bytes: u64, out: *mut *mut itak_store) -> itak_status;
    pub fn itak_store_close(store: *mut itak_store);
    pub fn itak_store_last_error(store: *const itak_store) -> *const c_char;
    pub fn itak_store_last_error_info(store: *const itak_store, out: *mut itak_error_info) -> itak_status;
    pub fn itak_store_refusals(store: *const itak_store) -> *const c_char;
    pub fn itak_store_clear_refusals(store: *mut itak_store);
    pub fn itak_store_rescan(store: *mut itak_store) -> itak_status;
    pub fn itak_store_get_stats(store: *mut itak_store, out: *mut itak_store_stats) -> itak_status;
    pub fn itak_store_entries(store: *mut itak_store, out: *mut itak_store_entry, capacity: u64, count: *mut u64) -> itak_status;
    pub fn itak_store_put(store: *mut itak_store, tokens: *const u32, token_count: u64, snapshot: *const c_void, snapshot_len: u64, now: u64) -> itak_status;
    pub fn itak_store_lookup(store: *mut itak_store, query: *const u32, query_len: u64, expected_geometry: *const itak_itkv_header, expected_layers: *const itak_itkv_layer, fingerprint: *const c_char, fingerprint_len: u64, now: u64, hit: *mut itak_prefix_hit) -> itak_status;
    pub fn itak_store_restore_prefix(store: *mut itak_store, pool: *mut itak_pool, slot: u32, tokens: *const u32, token_count: u64, fingerprint: *const c_char, fingerprint_len: u64, now: u64, matched: *mut u64) -> itak_status;
    pub fn itak_store_capture_and_put(store: *mut itak_store, pool: *mut itak_pool, slot: u32, tokens: *const u32, token_count: u64, fingerprint: *const c_char, fingerprint_len: u64, elem: u32, now: u64) -> itak_status;
    pub fn itak_gqa_attention(pool: *mut itak_pool, slot: u32, layer: u64, q: *const f32, q_len: u64, num_queries: u64, num_q_heads: u64, query_positions: *const u64, positions_len: u64, scale: f32, softcap: f32, out: *mut f32) -> itak_status;
    pub fn itak_compute_attention(pool: *mut itak_pool, slot: u32, layer: u64, q: *const f32, q_len: u64, k: *const f32, k_len: u64, v: *const f32, v_len: u64, num_q_heads: u64, cache_position: u64, softcap: f32, rope_freq_base_swa: f32, out: *mut f32) -> itak_status;
    pub fn itak_compute_cache_checkpoint(pool: *mut itak_pool, slot: u32, max_round_tokens: u64, out: *mut itak_checkpoint) -> itak_status;
    pub fn itak_compute_cache_rewind(pool: *mut itak_pool, slot: u32, cp: *const itak_checkpoint, target: u64) -> itak_status;
    pub fn itak_compute_cache_release(pool: *mut itak_pool, slot: u32, cp: *const itak_checkpoint) -> itak_status;
    pub fn itak_attention_step_device(pool: *mut itak_pool, layer: u64, items: *const itak_batch_item, item_count: u32, q_dev: *const f32, k_dev: *const f32, v_dev: *const f32, out_dev: *mut f32, num_q_heads: u64, scale: f32, softcap: f32) -> itak_status;
    pub fn itak_attention_step_device_noalloc(pool: *mut itak_pool, layer: u64, items: *const itak_batch_item, item_count: u32, q_dev: *const f32, k_dev: *const f32, v_dev: *const f32, out_dev: *mut f32, num_q_heads: u64, scale: f32, softcap: f32) -> itak_status;
    pub fn itak_attention_prep_step_device(pool: *mut itak_pool, layer: u64, items: *const itak_batch_item, item_count: u32, q_dev: *const f32, k_dev: *const f32, v_dev: *const f32, gate_dev: *const f32, out_dev: *mut f32, num_q_heads: u64, scale: f32, softcap: f32, prep: *const itak_prep_params) -> itak_status;
    pub fn itak_attention_device(pool: *mut itak_pool, layer: u64, items: *const itak_batch_item, item_count: u32, q_dev: *const f32, out_dev: *mut f32, num_q_heads: u64, scale: f32, softcap: f32) -> itak_status;
    pub fn itak_kv_append_device(pool: *mut itak_pool, layer: u64, items: *const itak_batch_item, item_count: u32, k_dev: *const f32, v_dev: *const f32) -> itak_status;
    pub fn itak_convert_f32_to_f16_device(pool: *mut itak_pool, src_dev: *const f32, dst_dev: *mut u16, count: u64) -> itak_status;
    pub fn itak_set_debug_enabled(enabled: i32);
    pub fn itak_debug_enabled() -> i32;
    pub fn itak_probe_copy_device(pool: *mut itak_pool, src_dev: *const c_void, dst_dev: *mut c_void, bytes: u64) -> itak_status;
    pub fn itak_probe_read_device(pool: *mut itak_pool, src_dev: *const c_void, bytes: u64) -> itak_status;
    pub fn itak_probe_empty_launch(pool: *mut itak_pool) -> itak_status;
    pub fn itak_probe_mfma(pool: *mut itak_pool, random_operands: u32, trips: u32, clocks_dev: *mut u64, flops_out: *mut u64) -> itak_status;
}

pub mod safe;
