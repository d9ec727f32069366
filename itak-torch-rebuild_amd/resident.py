"""The device-resident target driver of the speculative loop.

`ResidentTarget` is the twin of itak_spec::ResidentTarget
(crates/itak-spec/src/resident.rs:27-105), the `TargetDriver`
(crates/itak-spec/src/driver.rs:42-99) that the reference lays over its GPU-resident session:
one sequence whose KV lives in a pool slot, forwarded layer by layer with every tensor on the
device, so that a speculative round (checkpoint, verify block, rewind to the accepted length,
release; crates/itak-spec/src/session.rs:616-831) makes no host round trip per layer.

As in the reference's resident driver, checkpoint and release are bookkeeping: the KV is
addressed by absolute position (windowed layers by position modulo the ring), every view
derives from the position a block ends at, entries past the position are never read, so
restoring an earlier committed position is the position restore itself
(ResidentSession::rewind_to, crates/wgpu-compute/src/session.rs:5371-5428, with the same two
refusals: a target ahead of the position, and a span longer than the rings' headroom).

Everything between two attention calls is the model's and not this library's (projections,
norms, the MLP, the head: crates/muse-glimmer/src/model.rs:400-520): the driver takes it as a
`layers` object with four methods over device tensors,

    embed(tokens) -> hidden [rows][hidden]                     (token embedding)
    qkv(layer, hidden, position) -> (q, k, v)                  (the attention block's inputs)
    mix(layer, hidden, attn_out) -> hidden                     (output projection, MLP, residuals)
    head(hidden) -> logits [rows][vocab]                       (final norm and LM head)

and runs `KvPool.attention_step_device` between `qkv` and `mix` for every layer.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import sys

from . import itak_kv as _kv
from . import prefix_store as _store
from .hip_compute import GlimmerConfig, KvCache, KvPool, StepFailed, debug_enabled


PREFILL_CHUNK = 64  # rows of a prompt forwarded per block (session.rs:186-195)


@dataclass
class LayerInputCapture:
    """muse_glimmer::LayerInputCapture (crates/muse-glimmer/src/model.rs:66-71): the residual
    rows entering `layer`, `[tokens][hidden]`, as a device tensor."""
    layer: int
    rows: object


@dataclass
class SpecRoundRecord:
    """What note_spec_round keeps of one completed round: a fingerprint of the proposed ids
    (FNV-1a 64 over their little-endian bytes, the hash the reference's capture diag uses,
    crates/itak-kv/src/hash.rs:44-46) and the accepted count."""
    proposed_fingerprint: int
    proposed: int
    accepted: int


class ResidentTarget:
    """TargetDriver over one slot of a KvPool. `layers` supplies the model around the
    attention calls (module docs); tensors are torch tensors on the pool's device."""

    def __init__(self, pool: KvPool, cache: KvCache, config: GlimmerConfig, layers,
                 softcap: float = 0.0, record_rounds: bool = False):
        self._pool, self._cache, self._config, self._layers = pool, cache, config, layers
        self._softcap = softcap
        self._position = 0
        self._records: Optional[List[SpecRoundRecord]] = [] if record_rounds else None
        # Rows a rewind may discard: what the shortest ring holds beyond its window
        # (the chunk_cap of the reference's session, session.rs:235-249); no bound without rings.
        room = None
        for layer, kind in enumerate(config.layers):
            if kind.is_windowed:
                spare = pool_ring_rows(cache, layer) - kind.window_size
                room = spare if room is None else min(room, spare)
        self._rewind_room = room

    # ---- TargetDriver ------------------------------------------------------------------
    def config(self) -> GlimmerConfig:
        return self._config

    def position(self) -> int:
        """The committed position: tokens forwarded and not rewound."""
        return self._position

    def forward(self, tokens: Sequence[int]):
        """Forward `tokens`, returning the last token's logits. A prompt goes through in chunks,
        as the reference's session sends it (64 rows a chunk, crates/wgpu-compute/src/session.rs:
        186-195), and no longer than the rings' headroom lets one block be."""
        tokens = list(tokens)
        if not tokens:
            raise StepFailed("forward", "no tokens to forward")
        chunk = PREFILL_CHUNK if self._rewind_room is None else max(1, min(PREFILL_CHUNK, self._rewind_room))
        logits = None
        for at in range(0, len(tokens), chunk):
            logits, _ = self.forward_block_capturing(tokens[at:at + chunk], [])
        return logits[-1]

    def forward_capturing(self, tokens: Sequence[int], capture_layers: Sequence[int]):
        logits, captures = self.forward_block_capturing(tokens, capture_layers)
        return logits[-1], captures

    def forward_block_capturing(self, tokens: Sequence[int], capture_layers: Sequence[int]
                                ) -> Tuple[object, List[LayerInputCapture]]:
        """Forward `tokens` as one block: every row's logits `[tokens][vocab]` plus the named
        layers' input rows in position order. The position advances by len(tokens) only when
        every layer has gone through (the model advances its cache after the head,
        crates/muse-glimmer/src/model.rs:153)."""
        rows = len(tokens)
        if rows == 0:
            raise StepFailed("forward", "no tokens to forward")
        for layer in capture_layers:  # model.rs validates the list before anything runs
            if layer >= len(self._config.layers):
                raise StepFailed("forward", f"capture layer {layer} out of range, the model has "
                                            f"{len(self._config.layers)} layers")
        hidden = self._layers.embed(tokens)
        captures: List[LayerInputCapture] = []
        for layer in range(len(self._config.layers)):
            if layer in capture_layers:
                captures.append(LayerInputCapture(layer, hidden.clone()))
            q, k, v = self._layers.qkv(layer, hidden, self._position)
            out = q.new_empty(q.shape)
            self._pool.attention_step_device(layer, [(self._cache, rows)], q.data_ptr(), k.data_ptr(),
                                             v.data_ptr(), out.data_ptr(), self._config.q_heads,
                                             softcap=self._softcap)
            hidden = self._layers.mix(layer, hidden, out)
        logits = self._layers.head(hidden)
        self._position += rows
        return logits, captures

    def checkpoint(self, rows: int) -> int:
        """The position at checkpoint time: restoring it is the whole contract on a
        position-addressed KV (resident.rs:85-87)."""
        return self._position

    def rewind(self, checkpoint: int, to: int) -> None:
        """ResidentSession::rewind_to (session.rs:5397-5428): positions `to..` are abandoned and
        the next forward overwrites them."""
        if to > self._position:
            raise StepFailed("session", f"rewind to {to} is ahead of the current position "
                                        f"{self._position}")
        span = self._position - to
        if self._rewind_room is not None and span > self._rewind_room:
            raise StepFailed("session", f"rewind from {self._position} to {to} discards {span} "
                                        f"positions, past the {self._rewind_room}-position ring "
                                        "headroom; reset the session instead")
        if span > 0:
            self._pool.truncate([self._cache], [to])
            self._position = to

    def release(self, checkpoint: int) -> None:
        """Nothing to free (resident.rs:93-95)."""

    def note_spec_round(self, proposed: Sequence[int], accepted: int) -> None:
        """Record only (driver.rs:84-98): never feeds back into the round."""
        if self._records is not None:
            self._records.append(SpecRoundRecord(_kv.prefix_hash(list(proposed)), len(proposed),
                                                 accepted))

    # ---- the prefix store in the loop -------------------------------------------------
    def restore_prefix_from_store(self, store, tokens: Sequence[int], fingerprint: str) -> Optional[int]:
        """ResidentSession::restore_prefix_from_store (session.rs:5000-5053): at position zero
        with the switch on, installs the longest stored prefix of `tokens` and returns its
        length; None when nothing was installed (switch off, a live sequence, no usable hit:
        the cold prefill serves)."""
        if not _store.prefix_store_enabled():
            return None
        if self._position != 0:
            _diag(f"prefix restore skipped: session position is {self._position}, not 0; a restore "
                  "is a session-start act and the live sequence is left alone")
            return None
        matched = store.restore_prefix(self._cache, tokens, fingerprint)
        if matched == 0:
            return None
        self._position = matched
        return matched

    def capture_and_store_prefix(self, store, tokens: Sequence[int], fingerprint: str,
                                 elem: str = "f32") -> None:
        """ResidentSession::capture_and_store_prefix (session.rs:5056-5094): files the slot's rows
        under `tokens`, which must be exactly the forwarded prefix."""
        if not _store.prefix_store_enabled():
            raise StepFailed("prefix_store", f"the prefix store switch {_store.ENABLE_ENV} is off")
        if self._position != len(tokens):
            raise StepFailed("prefix_store",
                             f"session position {self._position} does not equal the {len(tokens)} "
                             "tokens to store under; a snapshot covers exactly the forwarded "
                             "prefix, so any other token list would file one sequence's KV under "
                             "another's key")
        store.capture_and_put(self._cache, tokens, fingerprint, elem=elem)

    def forward_with_prefix_store(self, store, tokens: Sequence[int], fingerprint: str,
                                  elem: str = "f32"):
        """ResidentSession::forward_with_prefix_store (session.rs:5122-5151), the session-level
        flow in one call. With the switch off, or mid-sequence, exactly `forward`. Otherwise the
        longest stored prefix of `tokens` is installed and only the rest is forwarded; a hit that
        covers the whole prompt is rewound by one position and its last token forwarded again,
        because the returned logits are that token's forward product and no snapshot carries
        logits. Afterwards the whole prefix is captured and stored, hit or miss; a failure
        there is named on the diagnostic channel and the forward's result stands."""
        tokens = list(tokens)
        if not _store.prefix_store_enabled() or self._position != 0:
            return self.forward(tokens)
        matched = self.restore_prefix_from_store(store, tokens, fingerprint) or 0
        if matched > 0 and matched == len(tokens):
            self.rewind(self.checkpoint(1), matched - 1)
            logits = self.forward(tokens[matched - 1:])
        else:
            logits = self.forward(tokens[matched:])
        try:
            self.capture_and_store_prefix(store, tokens, fingerprint, elem=elem)
        except Exception as e:  # store and capture refusals alike: the logits are computed
            _diag(f"prefix store: post-forward capture/store failed: {e}; the forward's result stands")
        return logits

    # ---- beyond the trait --------------------------------------------------------------
    def spec_round_records(self) -> List[SpecRoundRecord]:
        return list(self._records or [])

    def reset(self) -> None:
        """ResidentSession::reset: drop the sequence, positions restart at 0."""
        self._cache.reset()
        self._position = 0


def _diag(line: str) -> None:
    """One line on the library's diagnostic channel (stderr, its prefix), when it is on."""
    if debug_enabled():
        print(f"[itak_hip_kv::diag] {line}", file=sys.stderr, flush=True)


def pool_ring_rows(cache: KvCache, layer: int) -> int:
    """Storage rows of a windowed layer's ring (itak_kv_storage_rows)."""
    import ctypes as C

    from . import _native as N
    out = C.c_uint64()
    status = N.load().itak_kv_storage_rows(cache.pool._h, layer, C.byref(out))
    if status != N.OK:
        raise StepFailed("session", "storage rows of a layer could not be read")
    return int(out.value)
