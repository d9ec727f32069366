//! The safe face of the C ABI: a pool, a slot in it, and the calls the backend crate makes.
//! Every `unsafe` block of the backend is in this file; each one passes pointers and lengths
//! taken from live Rust slices or from handles this module created.

use std::ffi::CStr;
use std::ptr;
use std::rc::Rc;

use crate::{
    itak_attention_step_device, itak_attention_step_device_noalloc, itak_batch_item,
    itak_checkpoint, itak_compute_attention, itak_compute_cache_checkpoint,
    itak_compute_cache_release, itak_compute_cache_rewind, itak_error_info, itak_kv_next_position,
    itak_kv_now_unix, itak_kv_truncate, itak_last_error, itak_last_error_info, itak_pool,
    itak_pool_config, itak_store, itak_store_capture_and_put, itak_store_close,
    itak_store_last_error, itak_store_open, itak_store_restore_prefix,
    itak_pool_create, itak_pool_destroy, itak_pool_set_stream, itak_pool_synchronize,
    itak_slot_acquire, itak_slot_release, itak_slot_reset, itak_status, ITAK_ELEM_F16,
    ITAK_ELEM_F32, ITAK_LAYER_GLOBAL, ITAK_LAYER_WINDOWED, ITAK_OK,
};

/// Storage element type of a pool.
#[derive(Debug, Clone, Copy, PartialEq, Eq)]
pub enum Elem {
    /// The reference's storage.
    F32,
    /// Round-to-nearest-even halves (the rule of `f32_to_f16_bits`,
    /// `crates/wgpu-compute/src/kernels/k1_q4k_gemv.rs:285-329`).
    F16,
}

/// One layer of the pattern (`attention::LayerKind`, `cache.rs:36-48`).
#[derive(Debug, Clone, Copy, PartialEq, Eq)]
pub enum Layer {
    /// Attends over everything stored.
    Global,
    /// Attends over the last `window` positions.
    Windowed(u64),
}

/// A refusal or failure handed back by the library: the status code, the message (for codes
/// 1..=14 the `Display` text of the matching `attention::AttentionError` variant) and the
/// variant's fields.
#[derive(Debug, Clone)]
pub struct HipKvError {
    /// One of the `ITAK_*` status constants.
    pub code: itak_status,
    /// The message, in the failing component's own words.
    pub message: String,
    /// The variant's `what` field, where it has one.
    pub what: String,
    /// The variant's integer fields, in declaration order.
    pub fields: [u64; 4],
}

impl std::fmt::Display for HipKvError {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        f.write_str(&self.message)
    }
}

impl std::error::Error for HipKvError {}

/// What a pool is built from.
#[derive(Debug, Clone)]
pub struct PoolConfig {
    /// The layer pattern.
    pub layers: Vec<Layer>,
    /// KV heads per layer.
    pub num_kv_heads: u64,
    /// Channels per head.
    pub head_dim: u64,
    /// Storage element type.
    pub elem: Elem,
    /// Sequences the pool can hold at once.
    pub max_slots: u32,
    /// Positions one slot can hold per global layer.
    pub capacity_rows: u64,
    /// HIP device ordinal.
    pub device: i32,
    /// `ITAK_POOL_*` flags.
    pub flags: u32,
    /// Rows a windowed layer's ring holds beyond its window (0 = 64).
    pub ring_headroom: u64,
}

struct PoolHandle(*mut itak_pool);

impl Drop for PoolHandle {
    fn drop(&mut self) {
        // SAFETY: the handle came from itak_pool_create and is destroyed exactly once.
        unsafe { itak_pool_destroy(self.0) }
    }
}

/// Device-resident KV storage for up to `max_slots` sequences. Not `Send`: a pool is used from
/// one thread at a time, as one `CpuCompute` is (`cpu.rs:246-253`).
#[derive(Clone)]
pub struct Pool {
    handle: Rc<PoolHandle>,
}

fn last_error(pool: *const itak_pool, code: itak_status) -> HipKvError {
    let mut info = itak_error_info { code: 0, what: [0; 96], a: 0, b: 0, c: 0, d: 0 };
    // SAFETY: `pool` is null (thread-local create error) or a live handle; `info` is a valid
    // out-pointer; the message pointer is read before any further call on the pool.
    let (message, what) = unsafe {
        let _ = itak_last_error_info(pool, &mut info);
        let text = itak_last_error(pool);
        let message = if text.is_null() {
            String::new()
        } else {
            CStr::from_ptr(text).to_string_lossy().into_owned()
        };
        let what = CStr::from_ptr(info.what.as_ptr()).to_string_lossy().into_owned();
        (message, what)
    };
    HipKvError { code, message, what, fields: [info.a, info.b, info.c, info.d] }
}

/// `attention::diag::set_debug_enabled` (`crates/attention/src/diag.rs:17-19`): one stderr line
/// per cache and attention event and per refusal, prefixed `[itak_hip_kv::diag]`. The
/// environment variable `ITAK_HIP_KV_DEBUG` turns the same lines on from outside.
pub fn set_debug_enabled(enabled: bool) {
    // SAFETY: the switch is one atomic flag of the library.
    unsafe { itak_set_debug_enabled(i32::from(enabled)) }
}

/// `attention::diag::debug_enabled` (`diag.rs:24-33`).
pub fn debug_enabled() -> bool {
    // SAFETY: reads the flag and the environment.
    unsafe { itak_debug_enabled() != 0 }
}

impl Pool {
    /// `KvCache::new` for every slot (`cache.rs:327-371`; the same zero-dimension, window and
    /// overflow refusals).
    pub fn create(config: &PoolConfig) -> Result<Pool, HipKvError> {
        let kinds: Vec<u8> = config
            .layers
            .iter()
            .map(|l| match l {
                Layer::Global => ITAK_LAYER_GLOBAL as u8,
                Layer::Windowed(_) => ITAK_LAYER_WINDOWED as u8,
            })
            .collect();
        let windows: Vec<u64> = config
            .layers
            .iter()
            .map(|l| match l {
                Layer::Global => 0,
                Layer::Windowed(w) => *w,
            })
            .collect();
        let raw = itak_pool_config {
            layer_count: u32::try_from(config.layers.len()).unwrap_or(u32::MAX),
            layer_kinds: kinds.as_ptr(),
            windows: windows.as_ptr(),
            num_kv_heads: config.num_kv_heads,
            head_dim: config.head_dim,
            elem: match config.elem {
                Elem::F32 => ITAK_ELEM_F32,
                Elem::F16 => ITAK_ELEM_F16,
            },
            max_slots: config.max_slots,
            capacity_rows: config.capacity_rows,
            device: config.device,
            flags: config.flags,
            ring_headroom: config.ring_headroom,
        };
        let mut out: *mut itak_pool = ptr::null_mut();
        // SAFETY: `raw` and the two arrays it points at outlive the call; `out` is valid.
        let status = unsafe { itak_pool_create(&raw, &mut out) };
        if status != ITAK_OK as itak_status {
            return Err(last_error(ptr::null(), status));
        }
        Ok(Pool { handle: Rc::new(PoolHandle(out)) })
    }

    fn raw(&self) -> *mut itak_pool {
        self.handle.0
    }

    fn check(&self, status: itak_status) -> Result<(), HipKvError> {
        if status == ITAK_OK as itak_status {
            Ok(())
        } else {
            Err(last_error(self.raw(), status))
        }
    }

    /// The HIP stream later calls enqueue on (null = the null stream).
    pub fn set_stream(&self, hip_stream: *mut std::os::raw::c_void) -> Result<(), HipKvError> {
        // SAFETY: the library only stores the handle; the caller keeps the stream alive.
        self.check(unsafe { itak_pool_set_stream(self.raw(), hip_stream) })
    }

    /// Waits for the pool's stream.
    pub fn synchronize(&self) -> Result<(), HipKvError> {
        // SAFETY: live handle.
        self.check(unsafe { itak_pool_synchronize(self.raw()) })
    }

    /// A fresh `KvCache` in a free slot.
    pub fn acquire(&self) -> Result<Slot, HipKvError> {
        let mut slot = 0_u32;
        // SAFETY: live handle, valid out-pointer.
        self.check(unsafe { itak_slot_acquire(self.raw(), &mut slot) })?;
        Ok(Slot { pool: self.clone(), slot })
    }
}

/// One sequence's cache: the device twin of one `attention::KvCache`.
pub struct Slot {
    pool: Pool,
    slot: u32,
}

impl Drop for Slot {
    fn drop(&mut self) {
        // SAFETY: live handle; releasing a slot twice is refused by the library, not undefined.
        let _ = unsafe { itak_slot_release(self.pool.raw(), self.slot) };
    }
}

/// `attention::Checkpoint` (`cache.rs:229-273`) as the library hands it out.
#[derive(Debug, Clone, Copy)]
pub struct Checkpoint(itak_checkpoint);

impl Checkpoint {
    /// The round bound the checkpoint was taken with.
    #[must_use]
    pub fn max_round_tokens(&self) -> u64 {
        self.0.max_round_tokens
    }
}

/// One sequence's share of a batched device step.
#[derive(Debug, Clone, Copy)]
pub struct StepItem<'a> {
    /// The sequence.
    pub slot: &'a Slot,
    /// New positions it appends and queries in this step.
    pub rows: u32,
}

impl Slot {
    /// The pool this slot lives in.
    #[must_use]
    pub fn pool(&self) -> &Pool {
        &self.pool
    }

    /// `CpuCompute::reset` (`cpu.rs:264-268`).
    pub fn reset(&self) -> Result<(), HipKvError> {
        // SAFETY: live handle.
        self.pool.check(unsafe { itak_slot_reset(self.pool.raw(), self.slot) })
    }

    /// `KvCache::next_position` (`cache.rs:413-415`).
    pub fn next_position(&self, layer: u64) -> Result<u64, HipKvError> {
        let mut out = 0_u64;
        // SAFETY: live handle, valid out-pointer.
        self.pool.check(unsafe { itak_kv_next_position(self.pool.raw(), self.slot, layer, &mut out) })?;
        Ok(out)
    }

    /// The body of `Compute::attention` (`cpu.rs:506-655`) with host slices: cross-checks
    /// `cache_position`, rotates Q and K on sliding-window layers, appends each row's K/V and
    /// attends at its position. `out` has `q.len()` elements.
    #[allow(clippy::too_many_arguments)]
    pub fn compute_attention(
        &self,
        layer: u64,
        q: &[f32],
        k: &[f32],
        v: &[f32],
        num_q_heads: u64,
        cache_position: u64,
        softcap: f32,
        rope_freq_base_swa: f32,
        out: &mut [f32],
    ) -> Result<(), HipKvError> {
        assert_eq!(out.len(), q.len(), "attention output has the query's shape");
        // SAFETY: pointers and lengths come from live slices; `out` holds q.len() elements.
        self.pool.check(unsafe {
            itak_compute_attention(
                self.pool.raw(),
                self.slot,
                layer,
                q.as_ptr(),
                q.len() as u64,
                k.as_ptr(),
                k.len() as u64,
                v.as_ptr(),
                v.len() as u64,
                num_q_heads,
                cache_position,
                softcap,
                rope_freq_base_swa,
                out.as_mut_ptr(),
            )
        })
    }

    /// `CpuCompute::cache_checkpoint` (`cpu.rs:270-300`).
    pub fn cache_checkpoint(&self, max_round_tokens: u64) -> Result<Checkpoint, HipKvError> {
        let mut raw = itak_checkpoint { cache_id: 0, serial: 0, max_round_tokens: 0, saved_bytes: 0 };
        // SAFETY: live handle, valid out-pointer.
        self.pool.check(unsafe {
            itak_compute_cache_checkpoint(self.pool.raw(), self.slot, max_round_tokens, &mut raw)
        })?;
        Ok(Checkpoint(raw))
    }

    /// `CpuCompute::cache_rewind` (`cpu.rs:302-323`).
    pub fn cache_rewind(&self, checkpoint: &Checkpoint, target: u64) -> Result<(), HipKvError> {
        // SAFETY: live handle; the checkpoint is a plain value.
        self.pool.check(unsafe {
            itak_compute_cache_rewind(self.pool.raw(), self.slot, &checkpoint.0, target)
        })
    }

    /// `CpuCompute::cache_release` (`cpu.rs:325-339`).
    pub fn cache_release(&self, checkpoint: &Checkpoint) -> Result<(), HipKvError> {
        // SAFETY: live handle; the checkpoint is a plain value.
        self.pool.check(unsafe { itak_compute_cache_release(self.pool.raw(), self.slot, &checkpoint.0) })
    }

    /// Drops every position at or beyond `new_len` on all layers (the global-layer arm of
    /// `KvCache::rewind_to`, `cache.rs:788-791`; `ResidentSession::rewind_to`,
    /// `crates/wgpu-compute/src/session.rs:5397-5428`).
    pub fn truncate(&self, new_len: u64) -> Result<(), HipKvError> {
        // SAFETY: one-element arrays on the stack.
        self.pool.check(unsafe { itak_kv_truncate(self.pool.raw(), &self.slot, &new_len, 1) })
    }
}

/// Device pointers of one batched step: `q`/`out` are `[sum rows][q_heads*head_dim]`, `k`/`v`
/// `[sum rows][kv_heads*head_dim]`, f32, on the pool's device.
#[derive(Debug, Clone, Copy)]
pub struct DeviceStep {
    /// Query rows.
    pub q: *const f32,
    /// New key rows.
    pub k: *const f32,
    /// New value rows.
    pub v: *const f32,
    /// Output rows.
    pub out: *mut f32,
}

/// `itak_attention_step_device` (or, with `no_alloc`, the entry point that takes its split
/// workspace from the library's static device array and allocates nothing): every item
/// appends its rows at its slot's next position and attends causally. Enqueues on the pool's
/// stream and returns.
///
/// # Safety
///
/// The four pointers must be device memory of the pool's device holding the rows the items
/// name, valid until the pool's stream has run the step.
pub unsafe fn attention_step_device(
    pool: &Pool,
    layer: u64,
    items: &[StepItem<'_>],
    tensors: DeviceStep,
    num_q_heads: u64,
    scale: f32,
    softcap: f32,
    no_alloc: bool,
) -> Result<(), HipKvError> {
    let raw: Vec<itak_batch_item> =
        items.iter().map(|i| itak_batch_item { slot: i.slot.slot, rows: i.rows }).collect();
    let count = u32::try_from(raw.len()).unwrap_or(u32::MAX);
    let call = if no_alloc { itak_attention_step_device_noalloc } else { itak_attention_step_device };
    // SAFETY: `raw` outlives the call; the device pointers are the caller's promise.
    pool.check(unsafe {
        call(pool.raw(), layer, raw.as_ptr(), count, tensors.q, tensors.k, tensors.v, tensors.out,
             num_q_heads, scale, softcap)
    })
}

/// `itak_kv::PrefixStore` (`crates/itak-kv/src/store.rs:128-543`) as the library keeps it: the
/// same directory, the same entry files, and the two store halves of a session start against a
/// pool slot.
pub struct Store(*mut itak_store);

impl Drop for Store {
    fn drop(&mut self) {
        // SAFETY: the handle came from itak_store_open and is closed exactly once.
        unsafe { itak_store_close(self.0) }
    }
}

fn store_error(store: *const itak_store, code: itak_status) -> HipKvError {
    // SAFETY: `store` is null (the last failed open on this thread) or a live handle; the
    // message pointer is read before any further call on the store.
    let message = unsafe {
        let text = itak_store_last_error(store);
        if text.is_null() { String::new() } else { CStr::from_ptr(text).to_string_lossy().into_owned() }
    };
    HipKvError { code, message, what: String::new(), fields: [0; 4] }
}

impl Store {
    /// `PrefixStore::open` (`store.rs:147-168`).
    pub fn open(root: &str, max_bytes: u64) -> Result<Store, HipKvError> {
        let root = std::ffi::CString::new(root).map_err(|_| HipKvError {
            code: crate::ITAK_INVALID_ARGUMENT as itak_status,
            message: "store root holds a NUL byte".to_string(),
            what: String::new(),
            fields: [0; 4],
        })?;
        let mut raw: *mut itak_store = ptr::null_mut();
        // SAFETY: `root` is a live C string; `raw` is a valid out-pointer.
        let status = unsafe { itak_store_open(root.as_ptr(), max_bytes, &mut raw) };
        if status == ITAK_OK as itak_status { Ok(Store(raw)) } else { Err(store_error(ptr::null(), status)) }
    }

    /// `itak_kv::now_unix` (`store.rs:120-126`).
    #[must_use]
    pub fn now_unix() -> u64 {
        // SAFETY: reads the clock.
        unsafe { itak_kv_now_unix() }
    }

    /// `ResidentSession::restore_prefix_from_store` (`crates/wgpu-compute/src/session.rs:
    /// 5000-5053`) into a slot that stands at position zero: the tokens restored, 0 when the
    /// cold prefill serves. Only a device failure is an error.
    pub fn restore_prefix(&self, slot: &Slot, tokens: &[u32], fingerprint: &str) -> Result<u64, HipKvError> {
        let mut matched = 0u64;
        // SAFETY: slices and the string outlive the call; lengths are theirs.
        let status = unsafe {
            itak_store_restore_prefix(self.0, slot.pool.raw(), slot.slot, tokens.as_ptr(),
                                      tokens.len() as u64, fingerprint.as_ptr().cast(),
                                      fingerprint.len() as u64, Store::now_unix(), &mut matched)
        };
        if status == ITAK_OK as itak_status { Ok(matched) } else { Err(store_error(self.0, status)) }
    }

    /// `ResidentSession::capture_and_store_prefix` (`session.rs:5056-5094`): the slot must stand
    /// at exactly `tokens.len()` positions.
    pub fn capture_and_put(&self, slot: &Slot, tokens: &[u32], fingerprint: &str, elem: Elem) -> Result<(), HipKvError> {
        let elem = match elem { Elem::F32 => ITAK_ELEM_F32, Elem::F16 => ITAK_ELEM_F16 };
        // SAFETY: as above.
        let status = unsafe {
            itak_store_capture_and_put(self.0, slot.pool.raw(), slot.slot, tokens.as_ptr(),
                                       tokens.len() as u64, fingerprint.as_ptr().cast(),
                                       fingerprint.len() as u64, elem as u32, Store::now_unix())
        };
        if status == ITAK_OK as itak_status { Ok(()) } else { Err(store_error(self.0, status)) }
    }
}
