//! `muse_glimmer::Compute` with the KV cache and the attention step on an MI355X.
//!
//! A third sibling of `cpu-compute` and `wgpu-compute`: one [`HipCompute`] serves one sequence,
//! like one `CpuCompute` (`crates/cpu-compute/src/cpu.rs:246-253`). It owns a slot of a device
//! KV pool, built from the first config it sees (`KvState::build`, `cpu.rs:207-231`), and
//! answers [`Compute::attention`] with one call into `libitak_hip_kv` that does the whole body
//! of `cpu.rs:558-646`: the position cross-check, the interleaved RoPE of Q and K on
//! sliding-window layers, per-row append-then-attend, the output. Every other step of the
//! trait delegates to an inner `CpuCompute` (the wrapper pattern of `SharedCompute`,
//! `crates/itak-spec/src/speculator.rs:32`).
//!
//! Nothing in `attention`, `itak-kv`, `muse-glimmer` or `itak-spec` changes; the engine picks
//! the backend where it builds its `Box<dyn Compute>`
//! (`crates/itak-engine/src/engine.rs:727-733`).
//!
//! The environment switch follows the workspace's fail-closed rule
//! (`crates/itak-kv/src/config.rs:39-47`): `ITAK_HIP_KV_F16` set to exactly `0` stores f32 rows
//! as the reference does; anything else, unset included, stores f16.

#![forbid(unsafe_code)]

use std::cell::RefCell;

use cpu_compute::CpuCompute;
use itak_hip_sys::safe::{Checkpoint, Elem, HipKvError, Layer, Pool, PoolConfig, Slot, Store};
use muse_glimmer::{
    AttentionRequest, Cache, Compute, GlimmerConfig, GlimmerError, LayerKind, LayerWeights,
    Result, TensorView,
};

pub mod target;

pub use target::HipTarget;

/// Positions a sequence may reach unless [`HipCompute::with_capacity`] says otherwise.
pub const DEFAULT_CAPACITY_ROWS: u64 = 32_768;

fn step_failed(step: &'static str, detail: impl Into<String>) -> GlimmerError {
    GlimmerError::StepFailed { step, detail: detail.into() }
}

fn from_hip(step: &'static str, e: &HipKvError) -> GlimmerError {
    step_failed(step, e.message.clone())
}

/// The KV state of the one sequence being served: the pool (one slot) and the shape it was
/// built for (`cpu.rs:178-231`).
struct KvState {
    slot: Slot,
    layers: usize,
    kv_heads: u32,
    head_dim: u32,
}

/// The MI355X [`Compute`] backend.
pub struct HipCompute {
    inner: CpuCompute,
    kv: RefCell<Option<KvState>>,
    elem: Elem,
    capacity_rows: u64,
    softcap: f32,
    device: i32,
}

impl Default for HipCompute {
    fn default() -> Self {
        Self::new()
    }
}

impl HipCompute {
    /// A fresh backend with no KV state, f16 storage unless `ITAK_HIP_KV_F16` is exactly `0`.
    #[must_use]
    pub fn new() -> Self {
        let f32_rows = std::env::var("ITAK_HIP_KV_F16").is_ok_and(|v| v == "0");
        HipCompute {
            inner: CpuCompute::new(),
            kv: RefCell::new(None),
            elem: if f32_rows { Elem::F32 } else { Elem::F16 },
            capacity_rows: DEFAULT_CAPACITY_ROWS,
            softcap: 0.0,
            device: 0,
        }
    }

    /// Positions the sequence may reach on a global layer (the device pool is sized once).
    #[must_use]
    pub fn with_capacity(mut self, rows: u64) -> Self {
        self.capacity_rows = rows;
        self
    }

    /// Cap the scaled attention scores as `cap * tanh(s / cap)`
    /// (`crates/torch-math/src/logits.rs:26-37`); 0 disables it.
    #[must_use]
    pub fn with_softcap(mut self, cap: f32) -> Self {
        self.softcap = cap;
        self
    }

    /// Drop all stored KV state (`CpuCompute::reset`, `cpu.rs:264-268`).
    pub fn reset(&self) {
        *self.kv.borrow_mut() = None;
    }

    /// `CpuCompute::cache_checkpoint` (`cpu.rs:270-300`).
    pub fn cache_checkpoint(&self, max_round_tokens: usize) -> Result<Checkpoint> {
        let step = "cache_checkpoint";
        let guard = self.kv.borrow();
        let state = guard.as_ref().ok_or_else(|| {
            step_failed(
                step,
                "no KV state exists yet: a speculative round checkpoints after a first \
                 forward has built the cache (the spec's prefill), not before",
            )
        })?;
        state.slot.cache_checkpoint(max_round_tokens as u64).map_err(|e| from_hip(step, &e))
    }

    /// `CpuCompute::cache_rewind` (`cpu.rs:302-323`). Pair it with `Cache::rewind_to` on the
    /// model's position cache, same target, same step.
    pub fn cache_rewind(&self, checkpoint: &Checkpoint, target: usize) -> Result<()> {
        let step = "cache_rewind";
        let guard = self.kv.borrow();
        let state = guard.as_ref().ok_or_else(|| {
            step_failed(
                step,
                "no KV state exists: the sequence was reset after the checkpoint was taken",
            )
        })?;
        state.slot.cache_rewind(checkpoint, target as u64).map_err(|e| from_hip(step, &e))
    }

    /// `CpuCompute::cache_release` (`cpu.rs:325-339`).
    pub fn cache_release(&self, checkpoint: &Checkpoint) -> Result<()> {
        let step = "cache_release";
        let guard = self.kv.borrow();
        let state = guard.as_ref().ok_or_else(|| {
            step_failed(
                step,
                "no KV state exists: the sequence was reset after the checkpoint was taken",
            )
        })?;
        state.slot.cache_release(checkpoint).map_err(|e| from_hip(step, &e))
    }

    /// Drops the positions from `new_len` on, on every layer (the device session's rewind,
    /// `crates/wgpu-compute/src/session.rs:5397-5428`: no checkpoint involved).
    pub fn truncate(&self, new_len: usize) -> Result<()> {
        let step = "session";
        let guard = self.kv.borrow();
        let state = guard.as_ref().ok_or_else(|| step_failed(step, "no KV state yet"))?;
        state.slot.truncate(new_len as u64).map_err(|e| from_hip(step, &e))
    }

    /// The read half of a session start (`ResidentSession::restore_prefix_from_store`,
    /// `crates/wgpu-compute/src/session.rs:5000-5053`): with no row stored yet, installs the
    /// longest stored prefix of `tokens` into this backend's slot (built here if the first
    /// attention call has not built it) and returns its length, `None` when the cold prefill
    /// serves. The caller advances its position cache by the same count.
    pub fn restore_prefix_from_store(&self, cfg: &GlimmerConfig, store: &Store, tokens: &[u32],
                                     fingerprint: &str) -> Result<Option<usize>> {
        let step = "prefix_restore";
        let mut guard = self.kv.borrow_mut();
        if guard.is_none() {
            *guard = Some(self.build(cfg)?);
        }
        let state = guard.as_ref().ok_or_else(|| step_failed(step, "no KV state"))?;
        let matched = store.restore_prefix(&state.slot, tokens, fingerprint).map_err(|e| from_hip(step, &e))?;
        Ok(if matched == 0 { None } else { Some(matched as usize) })
    }

    /// The write half (`ResidentSession::capture_and_store_prefix`, `session.rs:5056-5094`):
    /// files the slot's rows under `tokens`, which must be exactly the forwarded prefix.
    pub fn capture_and_store_prefix(&self, store: &Store, tokens: &[u32], fingerprint: &str) -> Result<()> {
        let step = "prefix_store";
        let guard = self.kv.borrow();
        let state = guard.as_ref().ok_or_else(|| step_failed(step, "no KV state yet: nothing was forwarded"))?;
        store.capture_and_put(&state.slot, tokens, fingerprint, self.elem).map_err(|e| from_hip(step, &e))
    }

    /// `KvState::build` (`cpu.rs:207-231`): one pool of one slot in the config's layer pattern.
    fn build(&self, cfg: &GlimmerConfig) -> Result<KvState> {
        let step = "attention";
        let layers: Vec<Layer> = (0..cfg.block_count as usize)
            .map(|l| match cfg.layer_kind(l) {
                Some(LayerKind::SlidingWindow) => Layer::Windowed(u64::from(cfg.sliding_window)),
                _ => Layer::Global,
            })
            .collect();
        let pool = Pool::create(&PoolConfig {
            layers,
            num_kv_heads: u64::from(cfg.kv_heads),
            head_dim: u64::from(cfg.key_length),
            elem: self.elem,
            max_slots: 1,
            capacity_rows: self.capacity_rows,
            device: self.device,
            flags: 0,
            ring_headroom: 0,
        })
        .map_err(|e| from_hip(step, &e))?;
        let slot = pool.acquire().map_err(|e| from_hip(step, &e))?;
        Ok(KvState {
            slot,
            layers: cfg.block_count as usize,
            kv_heads: cfg.kv_heads,
            head_dim: cfg.key_length,
        })
    }
}

impl Compute for HipCompute {
    fn embed(&self, table: &TensorView, tokens: &[u32], cfg: &GlimmerConfig) -> Result<Vec<f32>> {
        self.inner.embed(table, tokens, cfg)
    }

    fn rms_norm(&self, x: &[f32], weight: &TensorView, rows: usize, eps: f32) -> Result<Vec<f32>> {
        self.inner.rms_norm(x, weight, rows, eps)
    }

    fn rms_norm_plain(&self, x: &[f32], rows: usize, eps: f32) -> Result<Vec<f32>> {
        self.inner.rms_norm_plain(x, rows, eps)
    }

    fn proj(&self, x: &[f32], weight: &TensorView, rows: usize) -> Result<Vec<f32>> {
        self.inner.proj(x, weight, rows)
    }

    fn attention(&self, req: &AttentionRequest<'_>, cache: &mut dyn Cache) -> Result<Vec<f32>> {
        let step = "attention";
        let cfg = req.cfg;
        // The refusals of cpu.rs:514-556, in its order; whole rows, the position cross-check,
        // and everything the KV crate refuses come back from the library in the reference's
        // own words.
        if cfg.key_length != cfg.value_length {
            return Err(step_failed(
                step,
                format!(
                    "key length {} and value length {} differ; the KV store holds one row width",
                    cfg.key_length, cfg.value_length
                ),
            ));
        }
        if cfg.layer_kind(req.layer) != Some(req.kind) {
            return Err(step_failed(
                step,
                format!("layer {} is not a {:?} layer in this config", req.layer, req.kind),
            ));
        }
        let mut guard = self.kv.borrow_mut();
        let rebuild = match guard.as_ref() {
            None => true,
            Some(s) => {
                if s.layers != cfg.block_count as usize
                    || s.kv_heads != cfg.kv_heads
                    || s.head_dim != cfg.key_length
                {
                    return Err(step_failed(
                        step,
                        "the config's KV shape changed under a live sequence; reset() first",
                    ));
                }
                false
            }
        };
        if rebuild {
            *guard = Some(self.build(cfg)?);
        }
        let state = guard.as_ref().expect("built above");
        let mut out = vec![0.0_f32; req.q.len()];
        state
            .slot
            .compute_attention(
                req.layer as u64,
                req.q,
                req.k,
                req.v,
                u64::from(cfg.q_heads),
                cache.position() as u64,
                self.softcap,
                cfg.rope_freq_base_swa,
                &mut out,
            )
            .map_err(|e| from_hip(step, &e))?;
        // The model, not the backend, advances the cache, after the head has succeeded
        // (crates/muse-glimmer/src/model.rs:153).
        Ok(out)
    }

    fn attn_gate(&self, attn_out: &[f32], gate: &[f32]) -> Result<Vec<f32>> {
        self.inner.attn_gate(attn_out, gate)
    }

    fn add(&self, a: &[f32], b: &[f32]) -> Result<Vec<f32>> {
        self.inner.add(a, b)
    }

    fn swiglu_ffn(
        &self,
        x: &[f32],
        w: &LayerWeights,
        rows: usize,
        cfg: &GlimmerConfig,
    ) -> Result<Vec<f32>> {
        self.inner.swiglu_ffn(x, w, rows, cfg)
    }

    fn lm_head(&self, x: &[f32], head: &TensorView, cfg: &GlimmerConfig) -> Result<Vec<f32>> {
        self.inner.lm_head(x, head, cfg)
    }
}
