/*
 * itak_hip_kv: MI355X (gfx950) KV cache and attention backend, C ABI.
 *
 * One itak_pool owns the device-resident KV storage of up to max_slots independent
 * sequences. A slot is one sequence's cache: the device twin of one
 * attention::KvCache (crates/attention/src/cache.rs:308-834) and, through the
 * itak_compute_* calls, of one cpu_compute::CpuCompute
 * (crates/cpu-compute/src/cpu.rs:246-339). A Rust backend crate binds these
 * symbols and implements muse_glimmer::Compute::attention
 * (crates/muse-glimmer/src/compute.rs:82), the inherent cache_checkpoint /
 * cache_rewind / cache_release / reset calls and itak_spec::TargetDriver
 * (crates/itak-spec/src/driver.rs:42-99) on top of them.
 *
 * Conventions
 *   - Every call returns an itak_status. 0 is success; 1..14 are the variants of
 *     attention::AttentionError in declaration order
 *     (crates/attention/src/error.rs:9-127); 15 is a cpu-compute StepFailed
 *     refusal; the rest are this library's own.
 *   - Nothing aborts or throws across the boundary. After a failure,
 *     itak_last_error() returns the message (AttentionError's Display text for
 *     codes 1..14) and itak_last_error_info() the variant's fields.
 *   - "host" pointers are ordinary process memory; "device" pointers are HIP
 *     device memory on the pool's device. Calls taking host pointers return
 *     after the result is in host memory. Calls taking device pointers only
 *     enqueue work on the pool's stream (itak_pool_set_stream).
 *   - Rows are [kv_heads][head_dim] flat, queries and outputs
 *     [query][q_heads][head_dim] flat, exactly as in the reference
 *     (cache.rs:11-15, attention.rs:94-103).
 *   - A pool is not thread-safe; use it from one thread at a time, as one
 *     CpuCompute is (cpu.rs:246-253).
 */
#ifndef ITAK_HIP_KV_H
#define ITAK_HIP_KV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int32_t itak_status;

enum {
    ITAK_OK = 0,
    ITAK_ZERO_DIMENSION = 1,
    ITAK_INVALID_WINDOW = 2,
    ITAK_SIZE_OVERFLOW = 3,
    ITAK_SHAPE_MISMATCH = 4,
    ITAK_INVALID_LAYER = 5,
    ITAK_OUT_OF_ORDER_POSITION = 6,
    ITAK_NON_DIVISIBLE_HEADS = 7,
    ITAK_NO_VISIBLE_KEYS = 8,
    ITAK_CHECKPOINT_BUSY = 9,
    ITAK_STALE_CHECKPOINT = 10,
    ITAK_CHECKPOINT_TOO_DEEP = 11,
    ITAK_CHECKPOINT_RANGE_EXCEEDED = 12,
    ITAK_BULK_RESTORE_NOT_FRESH = 13,
    ITAK_REWIND_OUT_OF_RANGE = 14,
    ITAK_STEP_FAILED = 15,      /* GlimmerError::StepFailed (muse-glimmer/src/error.rs:69-76) */
    ITAK_HIP_ERROR = 16,        /* a HIP runtime call failed; message carries hipGetErrorString */
    ITAK_INVALID_ARGUMENT = 17, /* null pointer, unknown slot, unknown enum value */
    ITAK_NO_FREE_SLOT = 18,     /* every slot of the pool is in use */
    ITAK_CAPACITY_EXCEEDED = 19,/* a slot would outgrow the pool's per-slot row capacity */
    ITAK_UNSUPPORTED = 20,      /* a shape or layer kind this build has no kernel for */
    /* itak_kv::KvError (crates/itak-kv/src/error.rs:13-124), the variants the snapshot path
       raises; messages are its Display text (error.rs:141-188). */
    ITAK_KV_BAD_MAGIC = 21,
    ITAK_KV_UNSUPPORTED_VERSION = 22,   /* a = version */
    ITAK_KV_TRUNCATED = 23,             /* a = expected bytes, b = actual */
    ITAK_KV_CHECKSUM_MISMATCH = 24,     /* a = stored, b = computed */
    ITAK_KV_INCONSISTENT_SNAPSHOT = 25,
    ITAK_KV_GEOMETRY_MISMATCH = 26,
    ITAK_KV_FINGERPRINT_MISMATCH = 27,
    ITAK_KV_INCOHERENT_CACHE = 28,
    /* The variants the prefix store adds (crates/itak-kv/src/store.rs). */
    ITAK_KV_EMPTY_PREFIX = 29,
    ITAK_KV_TOKEN_COUNT_MISMATCH = 30,    /* a = snapshot, b = tokens */
    ITAK_KV_PREFIX_HASH_MISMATCH = 31,    /* a = stored, b = computed */
    ITAK_KV_SNAPSHOT_TOKEN_MISMATCH = 32, /* a = entry, b = snapshot */
    ITAK_KV_ENTRY_TOO_LARGE = 33,         /* a = bytes, b = cap */
    ITAK_KV_INVALID_CONFIG = 34,
    ITAK_KV_IO = 35                       /* what = context, a = errno; message as std::io::Error prints it */
};

/* Storage / source element types.
   An f32 pool computes in f32 throughout. Its outputs are within 1e-5 of the reference's f32
   arithmetic, as the largest deviation over the largest output magnitude, on unit-scale inputs
   (3e-6 to 5e-6 observed). That figure is a distance between two f32 evaluations that sum in
   different orders: with Q at three and K at two times unit scale (scaled scores of standard
   deviation 6) each of the two is 2e-6 to 8e-6 from a float64 evaluation and they have been
   seen 1.08e-5 apart; off unit scale the bar that holds is 1e-5 against float64, not against
   the reference's own rounding.
   An f16 pool rounds the rows it stores to f16 (round to nearest even, as the reference's f16
   session does) and its attention kernels feed Q and the softmax weights to the matrix pipe as
   f16 too (scores, softmax state and accumulators stay f32): outputs are within 2e-3 (max abs)
   of f32 arithmetic over the same rounded rows as long as the scaled scores q.k*scale have a
   standard deviation of at most about 3 (3e-5 at unit scale, 1.5e-3 at 3, above the bar from
   about 4.5 on). Q and K normed per head, as the reference's model norms them, stay at unit
   scale. ITAK_POOL_Q_TWO_HALVES lifts the limit at head_dim 128 (4e-5 to 2.6e-4 observed at
   standard deviation 6).
   Rows that are not finite reach the outputs of exactly the query rows that see their position
   (the reference never reads the key or value row of a masked position), on f32 pools and on
   f16 pools: an infinity or a NaN in a value row the channels it stands in, a key whose score
   is NaN the whole output row. One difference is left on f16 pools: a softmax weight below about
   2^-24 of its row's largest (a scaled score 17 below the row's maximum) is zero as an f16
   operand, and zero times an infinite value is NaN where the reference has an infinity.
   Matrix-pipe kernels exist for f16 pools at head_dim 64, 96, 128 and 256 with up to 16 Q heads per
   KV head and for f32 pools at head_dim 64 and 128; every other shape (any head_dim up to 256)
   runs on a general kernel that is correct and one to two orders of magnitude slower. */
enum { ITAK_ELEM_F32 = 0, ITAK_ELEM_F16 = 1 };

/* Layer kinds (attention::LayerKind, cache.rs:36-48). */
enum { ITAK_LAYER_GLOBAL = 0, ITAK_LAYER_WINDOWED = 1 };

/* itak_pool_config.flags */
enum {
    /* Zero the rows a truncate / rewind drops, so the raw device bytes (not only the
       visible rows) equal those of a cache that never held them. */
    ITAK_POOL_SCRUB_ON_TRUNCATE = 1u,
    /* Merge split partials inside the attention launch instead of with a launch of their own
       (decode steps and speculative blocks of f16 pools at head_dim 128): the workgroups of a KV
       head exchange their partials through a buffer while the launch runs, each polling for the
       others' words (itak_pool_set_merge_spin_limit bounds the wait). One launch per layer
       instead of two; results agree with the default form to rounding. On an MI355X the
       exchange costs what the second launch costs (a round trip through memory between
       compute dies, then the stores that hand the buffer back), so it is not the default. */
    ITAK_POOL_MERGE_IN_LAUNCH = 2u,
    /* Merge split partials on the compute die that produced them, inside the attention launch.
       Split steps of f16 pools at head_dim 128 with at most 32 query vectors per KV head whose
       (sequence, KV head) units deal out evenly over the device's eight compute dies (1, 2, 4 or
       8 KV heads; at least 8 / kv_heads sequences of similar total length) place each unit's
       splits on one die, and the unit's last workgroup to finish merges the unit's partials out
       of that die's L2: no merge launch and no wait inside the launch. Other steps keep the
       merge launch. Pool creation probes that the device deals workgroup i to die i % 8 and
       ignores the flag if it does not; every such launch checks again, and
       itak_pool_synchronize reports ITAK_STEP_FAILED if a workgroup ran elsewhere (seen
       rarely, on small launches between other work; the pool then keeps the merge launch). Results
       agree with the merge launch's to the rounding of another split plan. On an MI355X it is
       2 to 4 % faster than the merge launch on batches of a hundred MB of KV per layer and more,
       level or slower below (the launch's own tail and a slower start cost what the second
       launch costs), so it is not the default. */
    ITAK_POOL_DIE_MERGE = 4u,
    /* f16 pools at head_dim 128, every step (decode rows, blocks, prefill chunks):
       the queries enter the score products as two f16 halves, q = hi + lo, and every score is
       K.hi + K.lo. Without the flag Q is rounded to f16 once, an error relative to each channel
       that grows with the scores: outputs meet the 2e-3 bar up to scaled scores of standard
       deviation 3 (see ITAK_ELEM_F16). With it the queries are good to 2^-22 and what is left is
       the rounding of the softmax weights to f16. The decode and split-K kernels wait for
       memory more than for the matrix pipe: the second product costs 1 % on a decode step or a
       ragged batch and 7 % on a speculative block of 64 query vectors per KV head. Longer
       blocks and prefill chunks (the block kernel, which the matrix pipe bounds) take 22 to
       26 % longer, and blocks of 9 to 64 rows are appended by a launch of their own instead of
       inside the attention launch. Other head dims ignore the flag. One thing it changes for keys
       that are not finite: an infinite channel of a visible key makes the score NaN when the
       channel's two halves have opposite signs (inf - inf), and the output row with it, where
       the single product and the reference have a score of plus or minus infinity. */
    ITAK_POOL_Q_TWO_HALVES = 8u,
    /* itak_attention_prep_step_device always norms and rotates by the launch of its own, with
       the reference's f64 chain, also where the attention kernel could do it inside its own
       launch in f32: the K rows an f16 pool stores are then the reference's prepared rows
       rounded once, bit for bit, where the folded form is within one f16 step of them (3 to 4
       stored elements in 10,000 differ). One launch more per step: a prepared decode step at
       context 4096 takes 10.8 us per layer instead of 8.8. */
    ITAK_POOL_PREP_BY_LAUNCH = 16u
};

typedef struct itak_pool itak_pool;

typedef struct itak_pool_config {
    uint32_t layer_count;
    const uint8_t *layer_kinds; /* [layer_count] ITAK_LAYER_*; NULL = all global */
    const uint64_t *windows;    /* [layer_count], read for windowed layers; may be NULL */
    uint64_t num_kv_heads;
    uint64_t head_dim;
    uint32_t elem;          /* ITAK_ELEM_F32 (reference storage) or ITAK_ELEM_F16 */
    uint32_t max_slots;     /* sequences the pool can hold at once */
    uint64_t capacity_rows; /* positions one slot can hold per global layer */
    int32_t device;         /* HIP device ordinal */
    uint32_t flags;         /* ITAK_POOL_* */
    /* Windowed layers only: rows a layer's device ring holds beyond its window (0 = 64). A
       step appends its whole block before its queries run, so the ring must still hold the
       window of the block's first row after the last row has landed; the same spare rows let
       a rewind drop positions without saved copies. It bounds the rows one device step may
       carry on a windowed layer and how far a truncate may go back (the chunk_cap of the
       reference's resident session, crates/wgpu-compute/src/session.rs:235-249, 5376-5428).
       A ring is window + ring_headroom rows, rounded up to a multiple of 32; the bound that
       blocks and truncates meet is what the rounding leaves, ring - window of the shortest
       such layer, so at least ring_headroom. A checkpoint takes any max_round_tokens up to
       the smallest window, as the reference's cache does (cache.rs:634-651): a round within
       the bound costs nothing, a longer one has the rows it may overwrite copied aside at the
       checkpoint (one small launch, a buffer kept per slot) and copied back by a rewind. */
    uint64_t ring_headroom;
} itak_pool_config;

/* The fields of the last refusal, in the order the Rust variant declares them
   (what, then the integers: e.g. ShapeMismatch = what, a=expected, b=actual). */
typedef struct itak_error_info {
    int32_t code;
    char what[96];
    uint64_t a, b, c, d;
} itak_error_info;

/* attention::Checkpoint (cache.rs:229-273). Per-layer bases: itak_kv_checkpoint_bases. */
typedef struct itak_checkpoint {
    uint64_t cache_id;
    uint64_t serial;
    uint64_t max_round_tokens;
    uint64_t saved_bytes;
} itak_checkpoint;

/* attention::LayerStats (cache.rs:88-98). */
typedef struct itak_layer_stats {
    uint64_t layer;
    uint32_t kind;
    uint32_t reserved;
    uint64_t window;
    uint64_t appended;
    uint64_t stored;
} itak_layer_stats;

/* One sequence's share of a batched device step. */
typedef struct itak_batch_item {
    uint32_t slot;
    uint32_t rows; /* new positions this slot appends and queries in this step */
} itak_batch_item;

/* One layer of a prefix snapshot held in host or device memory
   (itak_kv::LayerSnapshot, crates/itak-kv/src/snapshot.rs:144-151). */
typedef struct itak_snapshot_layer {
    uint64_t first_position;
    uint64_t rows;
    const void *keys;   /* [rows][kv_heads][head_dim], oldest first */
    const void *values; /* same shape */
} itak_snapshot_layer;

/* The fixed part of an ITKV v1 snapshot (crates/itak-kv/src/snapshot.rs:13-29): the
   geometry of itak_kv::KvGeometry (snapshot.rs:57-65) plus token count and fingerprint. */
typedef struct itak_itkv_header {
    uint64_t token_count;
    uint64_t num_kv_heads;
    uint64_t head_dim;
    uint64_t layer_count;
    uint64_t fingerprint_len;
    uint64_t fingerprint_offset; /* decode: byte offset of the UTF-8 fingerprint in the buffer */
    uint64_t encoded_len;        /* decode: bytes consumed, trailing checksum included */
    /* decode: the format version read and the element type of the rows. Version 1 is the
       reference's (f32 rows). Version 2 is this library's: one more u32 after the layer count
       carries the element type (ITAK_ELEM_*), the rows are of that type, and the trailer is
       itak_kv_checksum_blocks of the bytes before it instead of itak_kv_checksum. It exists so
       that an f16 cache can be snapshotted in its own bytes (half the size, nothing to convert)
       and verified by several host threads. The reference's reader refuses version 2 by name. */
    uint32_t version;
    uint32_t elem;
} itak_itkv_header;

/* One layer of an ITKV snapshot: its 28-byte header (snapshot.rs:24-26) and where its
   rows sit in the encoded buffer (f32 little-endian, keys then values). */
typedef struct itak_itkv_layer {
    uint32_t kind; /* ITAK_LAYER_* */
    uint32_t reserved;
    uint64_t window; /* 0 for a global layer */
    uint64_t first_position;
    uint64_t rows;
    uint64_t keys_offset;
    uint64_t values_offset;
} itak_itkv_layer;

/* ---- library ------------------------------------------------------------------ */

/* ABI version of this header; bumps on any incompatible change. */
uint32_t itak_abi_version(void);

/* Message of the last failure on this pool (or, with NULL, of the last failed
   itak_pool_create on this thread). Valid until the next call on the same pool. */
const char *itak_last_error(const itak_pool *pool);
itak_status itak_last_error_info(const itak_pool *pool, itak_error_info *out);

/* ---- pool and slots ------------------------------------------------------------- */

/* Allocates and zero-fills the device KV storage: KvCache::new for every slot
   (cache.rs:327-371; same zero-dimension / window / overflow refusals). */
itak_status itak_pool_create(const itak_pool_config *config, itak_pool **out);
void itak_pool_destroy(itak_pool *pool);

/* Stream every later call on this pool enqueues on (a hipStream_t; NULL = the
   null stream). The pool never creates streams of its own and does not wait for the
   previous stream: ordering between the two is the caller's to arrange. The stream
   may be one that is being captured into a HIP graph, provided the pool's scratch
   buffers are already large enough (run the same step once uncaptured first). */
itak_status itak_pool_set_stream(itak_pool *pool, void *hip_stream);
itak_status itak_pool_synchronize(itak_pool *pool);
/* No counterpart in the reference. Workgroups of a launch that merges its own splits
   (ITAK_POOL_MERGE_IN_LAUNCH) wait for each other's partials by polling; `polls` bounds that
   wait. The unit is one look at the exchange buffer (default 131072 looks). A kernel keeps
   several looks in flight, four in the single-row decode kernel and one elsewhere, each a round
   trip to memory of 1 to 1.5 microseconds, so the default bounds the wait at about 40 ms in
   the decode kernel and 170 ms in the others. A workgroup that runs out writes NaN into the
   outputs it owns, counts itself, and still hands back to the buffer, as empty, the words it had
   already gathered; the words it was still waiting for stay as they are, and producers that
   arrive late write theirs. itak_pool_synchronize then returns ITAK_STEP_FAILED and refills the
   buffer. Everything launched on the pool between the give-up and that synchronize must be
   taken as invalid, not only the step that gave up: later launches of the same stream read the
   same buffer and may have taken leftover words for published ones. 0 makes every wait a
   single look: for tests of that report. */
itak_status itak_pool_set_merge_spin_limit(itak_pool *pool, uint32_t polls);
/* Bytes of device memory the pool holds for KV rows. */
uint64_t itak_pool_device_bytes(const itak_pool *pool);

/* A slot is one sequence's cache. acquire = a fresh KvCache; reset = CpuCompute::reset
   (cpu.rs:264-268): drop everything, positions restart at 0, outstanding checkpoint
   handles go stale. */
itak_status itak_slot_acquire(itak_pool *pool, uint32_t *slot);
itak_status itak_slot_release(itak_pool *pool, uint32_t slot);
itak_status itak_slot_reset(itak_pool *pool, uint32_t slot);

/* ---- KvCache, per slot (crates/attention/src/cache.rs) ---------------------------- */

uint64_t itak_kv_layer_count(const itak_pool *pool);  /* cache.rs:374-376 */
uint64_t itak_kv_num_kv_heads(const itak_pool *pool); /* cache.rs:379-381 */
uint64_t itak_kv_head_dim(const itak_pool *pool);     /* cache.rs:384-386 */
/* KvCache::layer_kind (cache.rs:403-405). */
itak_status itak_kv_layer_kind(itak_pool *pool, uint64_t layer, uint32_t *kind, uint64_t *window);
/* Storage rows of one layer of one slot: capacity_rows on a global layer, the ring length on
   a windowed one (what itak_kv_read_raw returns). */
itak_status itak_kv_storage_rows(itak_pool *pool, uint64_t layer, uint64_t *out);
/* KvCache::stored_len (cache.rs:408-410). */
itak_status itak_kv_stored_len(itak_pool *pool, uint32_t slot, uint64_t layer, uint64_t *out);
/* KvCache::next_position (cache.rs:413-415). */
itak_status itak_kv_next_position(itak_pool *pool, uint32_t slot, uint64_t layer, uint64_t *out);
/* KvCache::append (cache.rs:423-474): one position's K and V rows, host f32.
   f16 pools store round-to-nearest-even halves (spec:
   crates/wgpu-compute/src/kernels/k1_q4k_gemv.rs:285-329). */
itak_status itak_kv_append(itak_pool *pool, uint32_t slot, uint64_t layer, const float *k,
                           uint64_t k_len, const float *v, uint64_t v_len, uint64_t position);
/* KvCache::restore_bulk (cache.rs:513-577): install rows for positions
   first_position.. into a fresh layer. keys/values may be pinned host memory
   (read in place by the gather kernel), ordinary host memory (staged) or device
   memory; *_len count elements of src_elem type. An f32 source into an f16 pool is
   converted exactly as append converts; an f16 source needs an f16 pool. With host memory
   of either kind the rows are in place when the call returns; rows that all lie in device
   memory are gathered in the order of the pool's stream, like itak_kv_append_device, and the
   call returns with the gather enqueued (the sources stay untouched until the stream has
   passed it). The same holds for itak_kv_restore_snapshot. */
itak_status itak_kv_restore_bulk(itak_pool *pool, uint32_t slot, uint64_t layer,
                                 uint64_t first_position, const void *keys, uint64_t keys_len,
                                 const void *values, uint64_t values_len, uint32_t src_elem);
/* KvSnapshot::restore (crates/itak-kv/src/snapshot.rs:321-334) for a whole snapshot:
   validates every layer against token_count first (snapshot.rs:187-236), then
   gathers all layers into the fresh slot. */
itak_status itak_kv_restore_snapshot(itak_pool *pool, uint32_t slot, uint64_t token_count,
                                     const itak_snapshot_layer *layers, uint64_t layer_count,
                                     uint32_t src_elem);
/* KvCache::stats (cache.rs:588-599); out holds layer_count entries. */
itak_status itak_kv_stats(itak_pool *pool, uint32_t slot, itak_layer_stats *out);
/* CacheView::{position_at,key,value} (cache.rs:878-903) for `rows` visible entries
   starting at visible index `first`: raw storage elements (f32 or f16 bits) in
   [row][kv_head][head_dim] order, plus each row's absolute position. Host outputs;
   any of the three may be NULL. */
itak_status itak_kv_read_rows(itak_pool *pool, uint32_t slot, uint64_t layer, uint64_t first,
                              uint64_t rows, void *keys_out, void *values_out,
                              uint64_t *positions_out);
/* Every storage row of one slot and layer, capacity_rows long, visible or not
   (what the scrub guarantee is checked on). Host outputs. */
itak_status itak_kv_read_raw(itak_pool *pool, uint32_t slot, uint64_t layer, void *keys_out,
                             void *values_out);
/* KvCache::checkpoint_active / checkpoint / rewind_to / release (cache.rs:601-833). */
itak_status itak_kv_checkpoint_active(itak_pool *pool, uint32_t slot, int32_t *out);
itak_status itak_kv_checkpoint(itak_pool *pool, uint32_t slot, uint64_t max_round_tokens,
                               itak_checkpoint *out);
/* Checkpoint::bases (cache.rs:253-255); out holds layer_count entries. */
itak_status itak_kv_checkpoint_bases(itak_pool *pool, uint32_t slot, const itak_checkpoint *cp,
                                     uint64_t *out);
itak_status itak_kv_rewind_to(itak_pool *pool, uint32_t slot, const itak_checkpoint *cp,
                              uint64_t target);
itak_status itak_kv_release(itak_pool *pool, uint32_t slot, const itak_checkpoint *cp);
/* Batched truncation on speculative rejection: slot i drops every position
   >= new_lengths[i] on all layers (the global-layer arm of KvCache::rewind_to,
   cache.rs:788-791,814, without a checkpoint object). Refuses a length ahead of any
   layer (RewindOutOfRange) or a slot with a live checkpoint (CheckpointBusy). */
itak_status itak_kv_truncate(itak_pool *pool, const uint32_t *slots, const uint64_t *new_lengths,
                             uint32_t count);

/* ---- prefix snapshots: itak_kv (crates/itak-kv/src) ------------------------------------ */

/* hash::prefix_hash, prefix_discriminator, checksum (hash.rs:44-61): FNV-1a 64. */
uint64_t itak_kv_prefix_hash(const uint32_t *tokens, uint64_t count);
uint64_t itak_kv_prefix_discriminator(const uint32_t *tokens, uint64_t count);
uint64_t itak_kv_checksum(const void *bytes, uint64_t count);
/* No counterpart in the reference: the trailer of this library's snapshot version 2. FNV-1a 64
   over the FNV-1a 64 sums (each written as 8 little-endian bytes, in order) of consecutive
   1 MiB blocks of `bytes`, the last block as short as it falls; no bytes give the offset basis.
   Same strength per block as itak_kv_checksum, and host threads share the blocks: the
   byte-serial walk of version 1 runs at about 1 GB/s whatever the machine. */
uint64_t itak_kv_checksum_blocks(const void *bytes, uint64_t count);

/* The three calls below take no pool: after a failure itak_last_error(NULL) and
   itak_last_error_info(NULL, ..) return the refusal, per thread. */

/* KvSnapshot::validate (snapshot.rs:187-236) of a snapshot held by the caller: `blocks`
   layer blocks whose key / value arrays hold key_floats[i] / value_floats[i] floats. */
itak_status itak_itkv_validate(const itak_itkv_header *header, const itak_itkv_layer *layers,
                               uint64_t blocks, const uint64_t *key_floats,
                               const uint64_t *value_floats);
/* KvSnapshot::to_bytes (snapshot.rs:381-403): validates, then writes the versioned byte
   format. With out == NULL only *written (the size) is set. */
itak_status itak_itkv_encode(const itak_itkv_header *header, const char *fingerprint,
                             const itak_itkv_layer *layers, uint64_t blocks,
                             const float *const *keys, const uint64_t *key_floats,
                             const float *const *values, const uint64_t *value_floats, void *out,
                             uint64_t capacity, uint64_t *written);
/* KvSnapshot::from_bytes (snapshot.rs:405-509): strict decode. Rows are not copied: each
   layer's keys_offset / values_offset locate its f32 rows inside `bytes`. Fills at most
   layers_capacity entries; a smaller capacity than header->layer_count is refused after the
   header has been filled, so a caller may size its array from a first call with 0. */
itak_status itak_itkv_decode(const void *bytes, uint64_t len, itak_itkv_header *header,
                             itak_itkv_layer *layers, uint64_t layers_capacity);

/* KvSnapshot::capture (snapshot.rs:247-302) of a slot, written straight as ITKV v1 bytes
   into host memory: refuses a slot whose layers disagree on position (IncoherentCache),
   reads every layer's visible rows back as f32 (the rows of an f16 pool widen exactly) and
   appends the checksum. With out == NULL only *written (the size) is set. */
itak_status itak_kv_capture_itkv(itak_pool *pool, uint32_t slot, const char *fingerprint,
                                 uint64_t fingerprint_len, void *out, uint64_t capacity,
                                 uint64_t *written);
/* The same capture of an f16 pool in the pool's own bytes: ITKV version 2 with f16 rows and a
   block-summed trailer, half the size of the version 1 encoding and bit-identical on restore. Refused
   (ITAK_UNSUPPORTED) on an f32 pool: a narrowing capture would drop precision the cache
   holds. No counterpart in the reference, whose format has no element-type field. */
itak_status itak_kv_capture_itkv_f16(itak_pool *pool, uint32_t slot, const char *fingerprint,
                                     uint64_t fingerprint_len, void *out, uint64_t capacity,
                                     uint64_t *written);
/* KvSnapshot::from_bytes followed by restore_checked (snapshot.rs:351-371) into a fresh
   slot (either format version; f16 rows go into an f16 pool as they are and are refused by
   an f32 pool): the snapshot's geometry must be the pool's, and, when expected_fingerprint is not
   NULL, its fingerprint the expected one. The rows are gathered from `bytes` in place when
   the device can read them there (pinned host or device memory, 4-byte aligned payload),
   otherwise staged. An f32 snapshot into an f16 pool converts exactly as append does. */
itak_status itak_kv_restore_itkv(itak_pool *pool, uint32_t slot, const void *bytes, uint64_t len,
                                 const char *expected_fingerprint,
                                 uint64_t expected_fingerprint_len);

/* ---- persistent prefix store (crates/itak-kv/src/store.rs) ------------------------- */

/* itak_kv::PrefixStore (store.rs:128-543): one file per entry under a root directory, keyed by
   token prefix, bounded by a byte cap with LRU eviction. Entry files are the reference's
   byte for byte (store.rs:5-22), so both implementations serve each other's directories.
   Host code: a store works without a device. Not thread-safe, like the reference's. */
typedef struct itak_store itak_store;

/* store.rs:77-91. */
typedef struct itak_store_entry {
    char file_name[96];
    uint64_t prefix_hash;
    uint64_t token_count;
    uint64_t bytes;
    uint64_t created_unix;
    uint64_t last_used_unix;
} itak_store_entry;

/* store.rs:108-116. */
typedef struct itak_store_stats {
    uint64_t entries;
    uint64_t total_bytes;
    uint64_t max_bytes;
} itak_store_stats;

/* store.rs:94-105. token_count == 0 means no stored prefix matched. The matched ids are the
   first token_count ids of the query (verified equal). `snapshot` points at the verified
   ITKV v1 bytes inside the store's staging buffer (pinned host memory when a device is
   present, so itak_kv_restore_itkv gathers from it in place); valid until the next call on
   this store. */
typedef struct itak_prefix_hit {
    uint64_t token_count;
    const void *snapshot;
    uint64_t snapshot_len;
    char file_name[96];
} itak_prefix_hit;

/* itak_kv::now_unix (store.rs:120-126). */
uint64_t itak_kv_now_unix(void);
/* PrefixStore::open (store.rs:147-168): creates the root if needed and indexes every
   well-formed entry; malformed files are named in the refusal log and left alone. */
itak_status itak_store_open(const char *root, uint64_t max_bytes, itak_store **out);
void itak_store_close(itak_store *store);
/* Message / fields of the last failure on this store (NULL: of the last failed open on this
   thread). Messages are KvError's Display text (crates/itak-kv/src/error.rs:141-188). */
const char *itak_store_last_error(const itak_store *store);
itak_status itak_store_last_error_info(const itak_store *store, itak_error_info *out);
/* What the reference writes to its diag channel when it refuses an entry or skips a restore:
   one line per refusal, accumulated until cleared. */
const char *itak_store_refusals(const itak_store *store);
void itak_store_clear_refusals(itak_store *store);
/* PrefixStore::rescan (store.rs:204-224). */
itak_status itak_store_rescan(itak_store *store);
/* PrefixStore::stats (store.rs:185-192). */
itak_status itak_store_get_stats(itak_store *store, itak_store_stats *out);
/* PrefixStore::entries (store.rs:177-182): longest prefix first. With out == NULL only
   *count is set. */
itak_status itak_store_entries(itak_store *store, itak_store_entry *out, uint64_t capacity,
                               uint64_t *count);
/* PrefixStore::put (store.rs:236-300) of an encoded snapshot: strict decode (the refusals of
   KvSnapshot::from_bytes), token count against the ids, the cap, atomic write, LRU eviction. */
itak_status itak_store_put(itak_store *store, const uint32_t *tokens, uint64_t token_count,
                           const void *snapshot, uint64_t snapshot_len, uint64_t now);
/* PrefixStore::lookup (store.rs:314-357): the longest stored prefix of `query` that passes
   every trust check (store.rs:364-452). expected_geometry (num_kv_heads, head_dim, layer_count
   are read) with expected_layers (kind, window) and fingerprint are optional requirements
   (NULL = none). A verified hit is restamped to `now`. */
itak_status itak_store_lookup(itak_store *store, const uint32_t *query, uint64_t query_len,
                              const itak_itkv_header *expected_geometry,
                              const itak_itkv_layer *expected_layers, const char *fingerprint,
                              uint64_t fingerprint_len, uint64_t now, itak_prefix_hit *hit);
/* ResidentSession::restore_prefix_from_store
   (crates/wgpu-compute/src/session.rs:5000-5053): looks `tokens` up under the pool's own
   pattern and the fingerprint and restores the hit into the (fresh) slot. *matched = tokens
   now in the slot, 0 when nothing was restored (no hit, slot not fresh, hit refused by the
   install checks: named in the refusal log, slot untouched). Only a device failure is an
   error. */
itak_status itak_store_restore_prefix(itak_store *store, itak_pool *pool, uint32_t slot,
                                      const uint32_t *tokens, uint64_t token_count,
                                      const char *fingerprint, uint64_t fingerprint_len,
                                      uint64_t now, uint64_t *matched);
/* ResidentSession::capture_and_store_prefix (session.rs:5056-5094): the slot must stand at
   exactly token_count positions; its rows are captured and put under `tokens`. elem =
   ITAK_ELEM_F32 writes the reference's ITKV version 1 (an entry the reference's store serves
   too); ITAK_ELEM_F16 (f16 pools) writes version 2, half the bytes on disk and over the
   host link, which the reference's store refuses by name and walks past. */
itak_status itak_store_capture_and_put(itak_store *store, itak_pool *pool, uint32_t slot,
                                       const uint32_t *tokens, uint64_t token_count,
                                       const char *fingerprint, uint64_t fingerprint_len,
                                       uint32_t elem, uint64_t now);

/* ---- attention over one slot, host pointers ---------------------------------------- */

/* attention::gqa_attention (crates/attention/src/attention.rs:104-215) over the slot's
   view of `layer`. scale = NaN selects 1/sqrt(head_dim) (attention.rs:35-37).
   softcap > 0 caps each scaled score as cap*tanh(s/cap) before the softmax
   (formula: crates/torch-math/src/logits.rs:26-37); 0 disables it. */
itak_status itak_gqa_attention(itak_pool *pool, uint32_t slot, uint64_t layer, const float *q,
                               uint64_t q_len, uint64_t num_queries, uint64_t num_q_heads,
                               const uint64_t *query_positions, uint64_t positions_len,
                               float scale, float softcap, float *out);

/* ---- CpuCompute, per slot (crates/cpu-compute/src/cpu.rs) --------------------------- */

/* Compute::attention (cpu.rs:506-655): checks whole rows, cross-checks cache_position
   against the slot's position for `layer`, then for each row appends its K/V and
   attends at its own position. On a windowed (sliding-window) layer Q and K are first
   rotated with the interleaved RoPE at rope_freq_base_swa, each row at its own position;
   global layers are NoPE and pass through unrotated (cpu.rs:594-622; the base is
   GlimmerConfig::rope_freq_base_swa and is not looked at on a global layer). q is
   [rows][q_heads*head_dim], k and v [rows][kv_heads*head_dim]; out has q_len
   elements. The slot is never advanced past what was appended: a failed call
   leaves it ahead of the caller's position and the next call refuses until
   itak_slot_reset, as the reference does. The rotation uses f64 angles, sines and
   cosines like rope_interleaved.rs:103-114, on every shape: the K rows the call stores
   are the reference's rotated rows, rounded once where the pool is f16. (The frequencies
   rope_base^(-2i/d) are computed on the host, in the libm the reference's own host would use,
   and kept on the device: the device library's pow may differ from it in the last bit, and a
   last bit times the position is what reaches the row. Sine and cosine are the device
   library's; no stored element has been seen to differ for it, up to position 10^6.) */
itak_status itak_compute_attention(itak_pool *pool, uint32_t slot, uint64_t layer, const float *q,
                                   uint64_t q_len, const float *k, uint64_t k_len, const float *v,
                                   uint64_t v_len, uint64_t num_q_heads, uint64_t cache_position,
                                   float softcap, float rope_freq_base_swa, float *out);
/* CpuCompute::cache_checkpoint / cache_rewind / cache_release (cpu.rs:270-339): the
   KvCache calls plus the "no KV state exists yet" refusals before a first forward. */
itak_status itak_compute_cache_checkpoint(itak_pool *pool, uint32_t slot,
                                          uint64_t max_round_tokens, itak_checkpoint *out);
itak_status itak_compute_cache_rewind(itak_pool *pool, uint32_t slot, const itak_checkpoint *cp,
                                      uint64_t target);
itak_status itak_compute_cache_release(itak_pool *pool, uint32_t slot, const itak_checkpoint *cp);

/* ---- batched device-resident step --------------------------------------------------- */

/* The body of Compute::attention (cpu.rs:586-646) for several slots at once with all
   tensors already on the device: item i appends items[i].rows new K/V rows at its
   slot's next position for `layer`, then query row r of that item attends at
   position base+r (the causal mask makes append-all-then-attend equal the
   reference's row-at-a-time order on a global layer). q_dev is
   [sum rows][q_heads*head_dim], k_dev and v_dev [sum rows][kv_heads*head_dim],
   out_dev like q_dev, items in order. rows = 1 is decode, a few rows a speculative
   verify block, many rows a prefill chunk. Enqueues on the pool's stream and
   returns without waiting. No counterpart in the reference, whose slots are
   separate threads (crates/itak-engine/src/engine.rs:336-383). */
itak_status itak_attention_step_device(itak_pool *pool, uint64_t layer,
                                       const itak_batch_item *items, uint32_t item_count,
                                       const float *q_dev, const float *k_dev, const float *v_dev,
                                       float *out_dev, uint64_t num_q_heads, float scale,
                                       float softcap);
/* itak_attention_step_device for callers that cannot allocate device memory (code under HIP
   graph capture, tight serving loops, harnesses that forbid it). No counterpart in the
   reference. Same arguments, results and refusals; but where that call takes the split
   workspace of its launches from buffers the pool allocates and grows, this one takes it from
   a static array of 16 MiB in the library's device image (8 MiB of exchange words for launches
   that merge their own splits, 8 MiB of split partials for the others) and calls no
   hipMalloc, hipFree or other allocating routine. A step whose launches would need more
   (8 MiB of partials = rows x q_heads x splits x 520 bytes summed over the slots) is
   refused with ITAK_CAPACITY_EXCEEDED before anything is changed. Every call on a device
   shares that device's array, whichever pool makes it. Eager calls are kept apart by the
   library: each records an event behind its launches, and a call whose stream is not the
   stream of the device's previous such call makes its stream wait for that event first (a wait
   on the device, nothing the host blocks on). Calls made while their stream is being captured
   are outside that: graphs captured from this entry point on different streams of one device
   must not be replayed at the same time, nor beside eager calls of it; that ordering is the
   caller's. */
itak_status itak_attention_step_device_noalloc(itak_pool *pool, uint64_t layer,
                                               const itak_batch_item *items, uint32_t item_count,
                                               const float *q_dev, const float *k_dev,
                                               const float *v_dev, float *out_dev,
                                               uint64_t num_q_heads, float scale, float softcap);
/* What Q and K go through between their projections and attention in the reference's
   model (crates/muse-glimmer/src/model.rs:445-451, crates/cpu-compute/src/cpu.rs:598-622):
   a per-head RMSNorm under one [head_dim] weight each (torch_math::rms_norm,
   crates/torch-math/src/norm.rs:21-52) and RoPE at the row's position
   (rope_interleaved.rs:65-116 or rope.rs:63-116). */
typedef struct itak_prep_params {
    const float *q_norm_weight; /* device, [head_dim]; NULL = Q is not normed */
    const float *k_norm_weight; /* device, [head_dim]; NULL = K is not normed */
    float eps;                  /* > 0 when a weight is given */
    float rope_base;            /* > 1: rotate Q and K; 0: no rotation (a global, NoPE layer) */
    uint32_t rope_interleaved;  /* 1: adjacent pairs (llama.cpp NORM), 0: half split (NEOX) */
    uint32_t rotary_dim;        /* even, <= head_dim; 0 = head_dim */
} itak_prep_params;

/* itak_attention_step_device preceded by the fused preparation of the resident chain
   (crates/wgpu-compute/src/kernels/k9_attn_prep.rs:1-60: the Q and K norms, the rotations
   and the append as one dispatch) and followed by the attention gate
   (CpuCompute::attn_gate, cpu.rs:657-673): q_dev and k_dev are the raw projections, and with
   gate_dev != NULL ([sum rows][q_heads*head_dim]) out = attention * sigmoid(gate).
   On f16 pools with head_dim 128, steps of up to 64 query vectors per KV head (rows x group:
   decode, speculative blocks) add no launch to the plain step's two: the attention kernel norms and
   rotates the Q rows it stages and the new K row it appends (f64 angle, f32 arithmetic:
   within one f16 step, or 1e-6 where a rotation cancels, of the reference's f64 chain in the
   stored K), and the kernel that
   writes the output applies the gate. Other shapes run norms and rotation as one launch
   before the step, with the numerics of the reference's CPU path (f64 norm, f64 angles),
   not of its f32 shader; f32 pools hold prepared K rows within 1e-6 of that path. */
itak_status itak_attention_prep_step_device(itak_pool *pool, uint64_t layer,
                                            const itak_batch_item *items, uint32_t item_count,
                                            const float *q_dev, const float *k_dev,
                                            const float *v_dev, const float *gate_dev,
                                            float *out_dev, uint64_t num_q_heads, float scale,
                                            float softcap, const itak_prep_params *prep);
/* The attention half alone: query row r of item i attends at position
   len_i - rows_i + r, i.e. over rows the slot already holds (gqa_attention over the
   slot's view, attention.rs:104-215, with the last rows_i positions as queries). On a
   windowed layer the view starts at the window of the newest row: an earlier query row sees
   what of its own window is still in the view, and more rows than the window are refused with
   the reference's NoVisibleKeys for the first of them (attention.rs:160-173). */
itak_status itak_attention_device(itak_pool *pool, uint64_t layer, const itak_batch_item *items,
                                  uint32_t item_count, const float *q_dev, float *out_dev,
                                  uint64_t num_q_heads, float scale, float softcap);
/* The append half alone (K5 APPEND_SHADER's job,
   crates/wgpu-compute/src/kernels/k5_rope_kv.rs:90-123), device tensors. */
itak_status itak_kv_append_device(itak_pool *pool, uint64_t layer, const itak_batch_item *items,
                                  uint32_t item_count, const float *k_dev, const float *v_dev);

/* f32 -> f16 bits on the device with the cache's conversion (for tests of the
   rounding rule over arbitrary inputs). Device pointers, pool's stream. */
itak_status itak_convert_f32_to_f16_device(itak_pool *pool, const float *src_dev,
                                           uint16_t *dst_dev, uint64_t count);

/* ---- debug channel ------------------------------------------------------------------- */

/* attention::diag (crates/attention/src/diag.rs:13-33,71-79): one line per cache and
   attention event and per refusal on stderr, prefix "[itak_hip_kv::diag] ", off by default.
   On when this switch is set or the environment holds ITAK_HIP_KV_DEBUG with a value other
   than "0" or empty (looked up at every event, so a running process can be switched from
   outside through its own setenv). Host code only; nothing in a kernel or a captured graph
   changes. itak_kv_stats returns the same state without any logging. */
void itak_set_debug_enabled(int32_t enabled);
int32_t itak_debug_enabled(void);

/* ---- measurement aids (no counterpart in the reference) ------------------------------ */

/* A plain streaming copy of `bytes` (a multiple of 16) on the pool's stream: the kernel of
   known size that hardware traffic counters are scaled by. */
itak_status itak_probe_copy_device(itak_pool *pool, const void *src_dev, void *dst_dev,
                                   uint64_t bytes);
/* A plain streaming read of `bytes` (a multiple of 16) on the pool's stream, nothing written:
   what the device delivers to a kernel that only reads, which is what a decode step's
   attention does with the cache. */
itak_status itak_probe_read_device(itak_pool *pool, const void *src_dev, uint64_t bytes);
/* One empty kernel on the pool's stream: timing a run of these gives the per-launch floor
   of dependent launches on this device. */
itak_status itak_probe_empty_launch(itak_pool *pool);
/* What the matrix pipe sustains by itself on this device, for the prefill roofline: `trips`
   (1 ..= 2^22) trips of 32 v_mfma_f32_16x16x32_f16 per wavefront, operands held in registers,
   two workgroups of four wavefronts on every compute unit, on the pool's stream. With
   random_operands the operands are pseudo-random halves in (-1, 1), else one constant: the clock
   the chip holds under the instruction, and with it the rate, depends on how many operand bits
   change between products (on an MI355X 2.4 PFLOP/s at 2.39 GHz on constants, 1.85 PFLOP/s at
   1.84 GHz on random halves). *flops_out (may be NULL) receives the launch's floating-point
   operations; clocks_dev (device memory, two words, may be NULL) receives the ticks of the
   shader clock and of the 100 MHz constant clock over the loop of one workgroup. The caller
   times the launch. */
itak_status itak_probe_mfma(itak_pool *pool, uint32_t random_operands, uint32_t trips,
                            uint64_t *clocks_dev, uint64_t *flops_out);

#ifdef __cplusplus
}
#endif
#endif
