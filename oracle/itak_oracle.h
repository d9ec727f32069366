/*
 * CPU oracle for the KV-cache + attention path. TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of the reference's Rust CPU path, written to be
 * read next to the Rust it follows. Only tests, the smoke check and the
 * benchmark's cpu_baseline leg may link or load it; the shipped HIP library
 * never does.
 *
 * Pinning status (what fixes each function without the Rust being runnable):
 *   orc_f32_to_f16_bits / orc_f16_to_f32 : all 63,488 finite halves round-trip,
 *       half-ulp bounds, numpy.float16 cross-check        (pinned)
 *   orc_fnv1a64                           : empty-input offset basis KAT,
 *       published FNV-1a vectors                          (pinned)
 *   orc_cache_* (append/view/restore_bulk/checkpoint/rewind/release):
 *       the reference's cache_tests.rs / checkpoint_tests.rs cases (pinned)
 *   orc_gqa_attention                     : attention_tests.rs hand values,
 *       closed forms, an independent float64 numpy reference (pinned)
 *   softcap and f16-rounded storage are extensions the reference does not
 *       have; softcap is pinned by the reference's own formula KATs
 *       (torch-math/src/logits.rs:65-70) and by its invariants.
 */
#ifndef ITAK_ORACLE_H
#define ITAK_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Error kinds: one per AttentionError variant (crates/attention/src/error.rs:9-127). */
enum orc_code {
    ORC_OK = 0,
    ORC_ZERO_DIMENSION = 1,
    ORC_INVALID_WINDOW = 2,
    ORC_SIZE_OVERFLOW = 3,
    ORC_SHAPE_MISMATCH = 4,
    ORC_INVALID_LAYER = 5,
    ORC_OUT_OF_ORDER_POSITION = 6,
    ORC_NON_DIVISIBLE_HEADS = 7,
    ORC_NO_VISIBLE_KEYS = 8,
    ORC_CHECKPOINT_BUSY = 9,
    ORC_STALE_CHECKPOINT = 10,
    ORC_CHECKPOINT_TOO_DEEP = 11,
    ORC_CHECKPOINT_RANGE_EXCEEDED = 12,
    ORC_BULK_RESTORE_NOT_FRESH = 13,
    ORC_REWIND_OUT_OF_RANGE = 14,
    ORC_STEP_FAILED = 15 /* cpu-compute's GlimmerError::StepFailed refusals */
};

/* The fields of the refusal, in the order the Rust variant declares them. */
typedef struct orc_error {
    int32_t code;
    char what[96];
    uint64_t a, b, c, d;
    char message[512]; /* the Display text (error.rs:129-214) */
} orc_error;

typedef struct orc_cache orc_cache;

typedef struct orc_checkpoint {
    uint64_t cache_id;
    uint64_t serial;
    uint64_t max_round_tokens;
    uint64_t saved_bytes;
    uint64_t layer_count;
    uint64_t *bases; /* owned by the handle; free with orc_checkpoint_free */
} orc_checkpoint;

typedef struct orc_layer_stats {
    uint64_t layer;
    uint64_t window; /* 0 = global */
    uint64_t appended;
    uint64_t stored;
} orc_layer_stats;

/* f32 <-> f16 (k1_q4k_gemv.rs:285-329, gguf/src/dequant.rs:12-34). */
uint16_t orc_f32_to_f16_bits(float x);
float orc_f16_to_f32(uint16_t bits);
void orc_f32_to_f16_array(const float *src, uint16_t *dst, size_t n);
void orc_f16_to_f32_array(const uint16_t *src, float *dst, size_t n);
void orc_round_through_f16(const float *src, float *dst, size_t n);

/* FNV-1a 64 (itak-kv/src/hash.rs:14-61). */
uint64_t orc_fnv1a64(const uint8_t *bytes, size_t n);
uint64_t orc_prefix_hash(const uint32_t *tokens, size_t n);

/* Half-split RoPE with float64 angles (torch-math/src/rope.rs:99-116); input generation only. */
void orc_rope_half_split(const float *in, float *out, size_t head_dim, uint64_t position, float base);
/* cap * tanh(x / cap) in f32 (torch-math/src/logits.rs:26-37). */
void orc_rope_half_split_partial(const float *in, float *out, size_t head_dim, size_t rotary_dim,
                                 uint64_t position, float base);
void orc_rope_interleaved(const float *in, float *out, size_t head_dim, size_t rotary_dim,
                          uint64_t position, float base);
void orc_rms_norm(const float *in, const float *weight, float eps, size_t n, float *out);
float orc_sigmoid(float x);
float orc_logit_softcap(float x, float cap);

/*
 * KvCache (crates/attention/src/cache.rs:308-834). kinds[i] == 0 is a global layer,
 * 1 a windowed ring of windows[i] slots. store_f16 != 0 rounds every
 * appended / restored element through f16 (the f16-KV twin of the f32 reference:
 * f32 math over round-tripped values).
 */
int orc_cache_new(const uint8_t *kinds, const uint64_t *windows, uint64_t layer_count,
                  uint64_t num_kv_heads, uint64_t head_dim, int store_f16, orc_cache **out,
                  orc_error *err);
void orc_cache_free(orc_cache *c);
uint64_t orc_cache_layer_count(const orc_cache *c);
uint64_t orc_cache_num_kv_heads(const orc_cache *c);
uint64_t orc_cache_head_dim(const orc_cache *c);
int orc_cache_layer_window(const orc_cache *c, uint64_t layer, uint64_t *window, orc_error *err);
int orc_cache_stored_len(const orc_cache *c, uint64_t layer, uint64_t *out, orc_error *err);
int orc_cache_next_position(const orc_cache *c, uint64_t layer, uint64_t *out, orc_error *err);
int orc_cache_append(orc_cache *c, uint64_t layer, const float *k, uint64_t k_len, const float *v,
                     uint64_t v_len, uint64_t position, orc_error *err);
int orc_cache_restore_bulk(orc_cache *c, uint64_t layer, uint64_t first_position, const float *keys,
                           uint64_t keys_len, const float *values, uint64_t values_len,
                           orc_error *err);
void orc_cache_stats(const orc_cache *c, orc_layer_stats *out /* [layer_count] */);
int orc_cache_checkpoint_active(const orc_cache *c);
int orc_cache_checkpoint(orc_cache *c, uint64_t max_round_tokens, orc_checkpoint *out,
                         orc_error *err);
int orc_cache_rewind_to(orc_cache *c, const orc_checkpoint *cp, uint64_t target, orc_error *err);
int orc_cache_release(orc_cache *c, const orc_checkpoint *cp, orc_error *err);
void orc_checkpoint_free(orc_checkpoint *cp);

/* CacheView (cache.rs:841-904). Return 1 when the index is in range, 0 for None. */
int orc_view_len(const orc_cache *c, uint64_t layer, uint64_t *out, orc_error *err);
int orc_view_position_at(const orc_cache *c, uint64_t layer, uint64_t visible_index, uint64_t *pos);
int orc_view_key(const orc_cache *c, uint64_t layer, uint64_t visible_index, uint64_t kv_head,
                 const float **row);
int orc_view_value(const orc_cache *c, uint64_t layer, uint64_t visible_index, uint64_t kv_head,
                   const float **row);

/*
 * gqa_attention (crates/attention/src/attention.rs:104-215). a NaN scale selects
 * the default 1/sqrt(head_dim) (attention.rs:35-37). softcap > 0 applies
 * cap * tanh(s / cap) to each scaled score before the max/softmax (extension).
 * threads > 1 spreads (query, head) pairs over OpenMP threads; each pair still runs
 * the reference's strictly sequential arithmetic, so results do not depend on it.
 */
int orc_gqa_attention(const float *q, uint64_t q_len, uint64_t num_queries, uint64_t num_q_heads,
                      const uint64_t *query_positions, uint64_t positions_len, const orc_cache *c,
                      uint64_t layer, float scale, float softcap, int threads, float *out,
                      orc_error *err);

/*
 * The global-layer body of CpuCompute::attention (crates/cpu-compute/src/cpu.rs:558-646):
 * position cross-check, then per row append-then-attend with one query at its own
 * position. q is [rows][q_heads*head_dim], k and v are [rows][kv_heads*head_dim].
 * Windowed layers take q/k already rotated (RoPE is applied by the caller).
 */
int orc_attention_step(orc_cache *c, uint64_t layer, const float *q, const float *k, const float *v,
                       uint64_t rows, uint64_t num_q_heads, uint64_t start_position, float scale,
                       float softcap, int threads, float *out, orc_error *err);

#ifdef __cplusplus
}
#endif
#endif
