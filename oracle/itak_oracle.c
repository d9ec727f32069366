/*
 * CPU oracle for the KV-cache + attention path. TEST INFRASTRUCTURE ONLY: see
 * itak_oracle.h for who may use it and how each function is pinned.
 *
 * Build with -O2 -ffp-contract=off so every f32 product and sum is rounded
 * separately, as rustc does (no FMA contraction).
 */
#include "itak_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ errors */

static int fail(orc_error *err, int code, const char *what, uint64_t a, uint64_t b, uint64_t c,
                uint64_t d) {
    if (err == NULL) {
        return code;
    }
    memset(err, 0, sizeof(*err));
    err->code = code;
    if (what != NULL) {
        snprintf(err->what, sizeof(err->what), "%s", what);
    }
    err->a = a;
    err->b = b;
    err->c = c;
    err->d = d;
    char *m = err->message;
    size_t n = sizeof(err->message);
    /* Display texts: crates/attention/src/error.rs:129-214. */
    switch (code) {
    case ORC_ZERO_DIMENSION:
        snprintf(m, n, "%s must be positive, got 0", what);
        break;
    case ORC_INVALID_WINDOW:
        snprintf(m, n, "sliding window must be positive, got %llu", (unsigned long long)a);
        break;
    case ORC_SIZE_OVERFLOW:
        snprintf(m, n, "%s: element count overflows usize", what);
        break;
    case ORC_SHAPE_MISMATCH: /* a = expected, b = actual */
        snprintf(m, n, "%s: got %llu, expected %llu", what, (unsigned long long)b,
                 (unsigned long long)a);
        break;
    case ORC_INVALID_LAYER: /* a = layer, b = layer_count */
        snprintf(m, n, "layer %llu out of range, cache has %llu layers", (unsigned long long)a,
                 (unsigned long long)b);
        break;
    case ORC_OUT_OF_ORDER_POSITION: /* a = layer, b = expected, c = actual */
        snprintf(m, n, "layer %llu appends must be in order: expected position %llu, got %llu",
                 (unsigned long long)a, (unsigned long long)b, (unsigned long long)c);
        break;
    case ORC_NON_DIVISIBLE_HEADS: /* a = num_q_heads, b = num_kv_heads */
        snprintf(m, n, "%llu query heads do not divide evenly across %llu KV heads",
                 (unsigned long long)a, (unsigned long long)b);
        break;
    case ORC_NO_VISIBLE_KEYS: /* a = position */
        snprintf(m, n, "query at position %llu has no visible keys", (unsigned long long)a);
        break;
    case ORC_CHECKPOINT_BUSY:
        snprintf(m, n,
                 "a checkpoint is already outstanding on this cache; release it before taking "
                 "another");
        break;
    case ORC_STALE_CHECKPOINT: /* a = checkpoint serial */
        snprintf(m, n,
                 "checkpoint %llu is not this cache's live checkpoint (already released or "
                 "foreign)",
                 (unsigned long long)a);
        break;
    case ORC_CHECKPOINT_TOO_DEEP: /* a = max_round_tokens, b = window */
        snprintf(m, n,
                 "checkpoint round bound %llu exceeds the smallest sliding window %llu: a round "
                 "that long would overwrite a ring slot twice and no rewind could be exact",
                 (unsigned long long)a, (unsigned long long)b);
        break;
    case ORC_CHECKPOINT_RANGE_EXCEEDED: /* a = layer, b = position, c = limit */
        snprintf(m, n,
                 "layer %llu append at position %llu is outside the live checkpoint's saved range "
                 "(first unsaved position %llu); refusing so a later rewind cannot meet a slot it "
                 "cannot restore",
                 (unsigned long long)a, (unsigned long long)b, (unsigned long long)c);
        break;
    case ORC_BULK_RESTORE_NOT_FRESH: /* a = layer, b = appended */
        snprintf(m, n,
                 "layer %llu already holds %llu appended positions; bulk restore installs into a "
                 "fresh layer only",
                 (unsigned long long)a, (unsigned long long)b);
        break;
    case ORC_REWIND_OUT_OF_RANGE: /* a = layer, b = base, c = appended, d = target */
        snprintf(m, n, "rewind target %llu is outside layer %llu's checkpoint range [%llu, %llu]",
                 (unsigned long long)d, (unsigned long long)a, (unsigned long long)b,
                 (unsigned long long)c);
        break;
    case ORC_STEP_FAILED:
        snprintf(m, n, "%s", what);
        break;
    default:
        snprintf(m, n, "unknown error %d", code);
        break;
    }
    return code;
}

/* ------------------------------------------------------- f16 conversions */

static uint32_t f32_bits(float x) {
    uint32_t b;
    memcpy(&b, &x, sizeof(b));
    return b;
}

static float bits_f32(uint32_t b) {
    float x;
    memcpy(&x, &b, sizeof(x));
    return x;
}

/* k1_q4k_gemv.rs:285-329: round-to-nearest-even, overflow to inf, NaN to sign|0x7e00. */
uint16_t orc_f32_to_f16_bits(float x) {
    uint32_t bits = f32_bits(x);
    uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
    int32_t exp = (int32_t)((bits >> 23) & 0xffu);
    uint32_t frac = bits & 0x7fffffu;
    if (exp == 0xff) {
        return (uint16_t)(sign | (frac == 0 ? 0x7c00u : 0x7e00u));
    }
    int32_t e = exp - 112; /* the f16 exponent field if the result is normal */
    if (e >= 0x1f) {
        return (uint16_t)(sign | 0x7c00u);
    }
    if (e <= 0) {
        /* Subnormal half or zero: shift the 24-bit significand down, RNE on what drops. */
        if (e < -10) {
            return sign;
        }
        uint32_t m = frac | 0x800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1u);
        uint32_t out = m >> shift;
        if (rem > halfway || (rem == halfway && (out & 1u) == 1u)) {
            out += 1u;
        }
        return (uint16_t)(sign | (uint16_t)out);
    }
    uint32_t kept = frac >> 13;
    uint32_t rem = frac & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (kept & 1u) == 1u)) {
        kept += 1u;
        if (kept == 0x400u) {
            kept = 0;
            e += 1;
            if (e >= 0x1f) {
                return (uint16_t)(sign | 0x7c00u);
            }
        }
    }
    return (uint16_t)(sign | ((uint16_t)e << 10) | (uint16_t)kept);
}

/* gguf/src/dequant.rs:12-34. */
float orc_f16_to_f32(uint16_t bits) {
    uint32_t sign = (uint32_t)(bits >> 15);
    uint32_t exp = (uint32_t)((bits >> 10) & 0x1fu);
    uint32_t frac = (uint32_t)(bits & 0x3ffu);
    if (exp == 0x1f) {
        uint32_t out = frac == 0 ? 0x7f800000u : (0x7fc00000u | (frac << 13));
        return bits_f32((sign << 31) | out);
    }
    if (exp == 0) {
        if (frac == 0) {
            return bits_f32(sign << 31);
        }
        float v = (float)frac * bits_f32(0x33800000u); /* frac * 2^-24, exact */
        return sign == 1 ? -v : v;
    }
    uint32_t out = ((exp + 127u - 15u) << 23) | (frac << 13);
    return bits_f32((sign << 31) | out);
}

void orc_f32_to_f16_array(const float *src, uint16_t *dst, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) {
        dst[i] = orc_f32_to_f16_bits(src[i]);
    }
}

void orc_f16_to_f32_array(const uint16_t *src, float *dst, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) {
        dst[i] = orc_f16_to_f32(src[i]);
    }
}

void orc_round_through_f16(const float *src, float *dst, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) {
        dst[i] = orc_f16_to_f32(orc_f32_to_f16_bits(src[i]));
    }
}

/* ----------------------------------------------------------------- hashes */

/* itak-kv/src/hash.rs:14-30,59-61. */
uint64_t orc_fnv1a64(const uint8_t *bytes, size_t n) {
    uint64_t hash = 0xcbf29ce484222325ull;
    for (size_t i = 0; i < n; i++) {
        hash ^= (uint64_t)bytes[i];
        hash *= 0x00000100000001b3ull;
    }
    return hash;
}

/* itak-kv/src/hash.rs:34-47: little-endian token bytes fed through FNV-1a. */
uint64_t orc_prefix_hash(const uint32_t *tokens, size_t n) {
    uint64_t hash = 0xcbf29ce484222325ull;
    for (size_t i = 0; i < n; i++) {
        uint32_t t = tokens[i];
        for (int b = 0; b < 4; b++) {
            hash ^= (uint64_t)((t >> (8 * b)) & 0xffu);
            hash *= 0x00000100000001b3ull;
        }
    }
    return hash;
}

/* ------------------------------------------------------------ input maths */

/* torch-math/src/rope.rs:99-116 with rotary_dim == head_dim. */
void orc_rope_half_split(const float *in, float *out, size_t head_dim, uint64_t position,
                         float base) {
    size_t half = head_dim / 2;
    double pos = (double)position;
    double base64 = (double)base;
    for (size_t i = 0; i < head_dim; i++) {
        out[i] = in[i];
    }
    for (size_t i = 0; i < half; i++) {
        double exponent = -((double)(2 * i)) / (double)head_dim;
        double angle = pos * pow(base64, exponent);
        double s = sin(angle), c = cos(angle);
        double x = (double)in[i], y = (double)in[i + half];
        out[i] = (float)(x * c - y * s);
        out[i + half] = (float)(x * s + y * c);
    }
}

/* torch-math/src/rope.rs:63-116 (half-split pairing: channel i with i + rotary_dim/2) with a
   rotary_dim that may be smaller than head_dim; the tail passes through. */
void orc_rope_half_split_partial(const float *in, float *out, size_t head_dim, size_t rotary_dim,
                                 uint64_t position, float base) {
    size_t half = rotary_dim / 2;
    double pos = (double)position;
    double base64 = (double)base;
    for (size_t i = 0; i < head_dim; i++) {
        out[i] = in[i];
    }
    for (size_t i = 0; i < half; i++) {
        double exponent = -((double)(2 * i)) / (double)rotary_dim;
        double angle = pos * pow(base64, exponent);
        double s = sin(angle), c = cos(angle);
        double x = (double)in[i], y = (double)in[i + half];
        out[i] = (float)(x * c - y * s);
        out[i + half] = (float)(x * s + y * c);
    }
}

/* torch-math/src/rope_interleaved.rs:65-116 (adjacent pairing: channels 2i and 2i+1). */
void orc_rope_interleaved(const float *in, float *out, size_t head_dim, size_t rotary_dim,
                          uint64_t position, float base) {
    double pos = (double)position;
    double base64 = (double)base;
    for (size_t i = 0; i < head_dim; i++) {
        out[i] = in[i];
    }
    for (size_t i = 0; i < rotary_dim / 2; i++) {
        double exponent = -((double)(2 * i)) / (double)rotary_dim;
        double angle = pos * pow(base64, exponent);
        double s = sin(angle), c = cos(angle);
        double x = (double)in[2 * i], y = (double)in[2 * i + 1];
        out[2 * i] = (float)(x * c - y * s);
        out[2 * i + 1] = (float)(x * s + y * c);
    }
}

/* torch-math/src/norm.rs:21-52: mean of squares and the scaled product in f64, one rounding
   to f32 per element. */
void orc_rms_norm(const float *in, const float *weight, float eps, size_t n, float *out) {
    double sum = 0.0;
    for (size_t i = 0; i < n; i++) {
        sum += (double)in[i] * (double)in[i];
    }
    double mean_sq = sum / (double)n;
    double inv_rms = 1.0 / sqrt(mean_sq + (double)eps);
    for (size_t i = 0; i < n; i++) {
        out[i] = (float)((double)in[i] * inv_rms * (double)weight[i]);
    }
}

/* cpu-compute/src/cpu.rs:162-169. */
float orc_sigmoid(float x) {
    if (x >= 0.0f) {
        return 1.0f / (1.0f + expf(-x));
    }
    float e = expf(x);
    return e / (1.0f + e);
}

/* torch-math/src/logits.rs:36. */
float orc_logit_softcap(float x, float cap) { return cap * tanhf(x / cap); }

/* ------------------------------------------------------------------ cache */

typedef struct layer_cache {
    int windowed;    /* LayerKind (cache.rs:36-48) */
    uint64_t window; /* ring capacity when windowed, else 0 */
    uint64_t appended;
    float *keys; /* global: grows; windowed: window*row zeros at construction */
    float *values;
    uint64_t rows_cap;      /* global only: allocated rows */
    int64_t *slot_position; /* windowed only: -1 = None */
} layer_cache;

typedef struct saved_slot {
    uint64_t slot;
    int64_t position;
    float *keys;
    float *values;
} saved_slot;

typedef struct layer_checkpoint {
    saved_slot *saved;
    uint64_t count;
} layer_checkpoint;

struct orc_cache {
    layer_cache *layers;
    uint64_t layer_count;
    uint64_t num_kv_heads;
    uint64_t head_dim;
    uint64_t row;
    int store_f16;
    uint64_t id;
    uint64_t next_serial;
    int live;
    uint64_t live_serial;
    uint64_t live_max_round_tokens;
    uint64_t *live_bases;
    layer_checkpoint *live_layers;
};

static uint64_t g_next_cache_id = 1; /* cache.rs:32 */

static uint64_t layer_stored(const layer_cache *lc) { /* cache.rs:154-159 */
    if (!lc->windowed) {
        return lc->appended;
    }
    return lc->appended < lc->window ? lc->appended : lc->window;
}

static uint64_t layer_first_visible(const layer_cache *lc) { /* cache.rs:162-164 */
    return lc->appended - layer_stored(lc);
}

static uint64_t layer_slot_of(const layer_cache *lc, uint64_t position) { /* cache.rs:168-173 */
    return lc->windowed ? position % lc->window : position;
}

static void store_row(const orc_cache *c, float *dst, const float *src) {
    if (c->store_f16) {
        for (uint64_t i = 0; i < c->row; i++) {
            dst[i] = orc_f16_to_f32(orc_f32_to_f16_bits(src[i]));
        }
    } else {
        memcpy(dst, src, c->row * sizeof(float));
    }
}

static int grow_global(layer_cache *lc, uint64_t row, uint64_t need_rows) {
    if (need_rows <= lc->rows_cap) {
        return 0;
    }
    uint64_t cap = lc->rows_cap == 0 ? 64 : lc->rows_cap;
    while (cap < need_rows) {
        cap *= 2;
    }
    float *k = (float *)realloc(lc->keys, cap * row * sizeof(float));
    if (k == NULL) {
        return -1;
    }
    lc->keys = k;
    float *v = (float *)realloc(lc->values, cap * row * sizeof(float));
    if (v == NULL) {
        return -1;
    }
    lc->values = v;
    lc->rows_cap = cap;
    return 0;
}

static void free_live(orc_cache *c) {
    if (c->live_layers != NULL) {
        for (uint64_t li = 0; li < c->layer_count; li++) {
            for (uint64_t i = 0; i < c->live_layers[li].count; i++) {
                free(c->live_layers[li].saved[i].keys);
                free(c->live_layers[li].saved[i].values);
            }
            free(c->live_layers[li].saved);
        }
        free(c->live_layers);
        c->live_layers = NULL;
    }
    free(c->live_bases);
    c->live_bases = NULL;
    c->live = 0;
}

/* cache.rs:327-371 with LayerCache::new :125-151. */
int orc_cache_new(const uint8_t *kinds, const uint64_t *windows, uint64_t layer_count,
                  uint64_t num_kv_heads, uint64_t head_dim, int store_f16, orc_cache **out,
                  orc_error *err) {
    *out = NULL;
    if (layer_count == 0) {
        return fail(err, ORC_ZERO_DIMENSION, "layer pattern", 0, 0, 0, 0);
    }
    if (num_kv_heads == 0) {
        return fail(err, ORC_ZERO_DIMENSION, "num_kv_heads", 0, 0, 0, 0);
    }
    if (head_dim == 0) {
        return fail(err, ORC_ZERO_DIMENSION, "head_dim", 0, 0, 0, 0);
    }
    for (uint64_t i = 0; i < layer_count; i++) { /* cache.rs:345-351 */
        if (kinds[i] != 0 && windows[i] == 0) {
            return fail(err, ORC_INVALID_WINDOW, NULL, 0, 0, 0, 0);
        }
    }
    orc_cache *c = (orc_cache *)calloc(1, sizeof(orc_cache));
    c->layers = (layer_cache *)calloc(layer_count, sizeof(layer_cache));
    c->layer_count = layer_count;
    c->num_kv_heads = num_kv_heads;
    c->head_dim = head_dim;
    c->store_f16 = store_f16;
    for (uint64_t i = 0; i < layer_count; i++) {
        uint64_t row;
        if (__builtin_mul_overflow(num_kv_heads, head_dim, &row)) {
            orc_cache_free(c);
            return fail(err, ORC_SIZE_OVERFLOW, "kv row length", 0, 0, 0, 0);
        }
        c->row = row;
        layer_cache *lc = &c->layers[i];
        lc->windowed = kinds[i] != 0;
        lc->window = lc->windowed ? windows[i] : 0;
        if (lc->windowed) {
            uint64_t slots, bytes;
            if (__builtin_mul_overflow(lc->window, row, &slots) ||
                __builtin_mul_overflow(slots, (uint64_t)sizeof(float), &bytes)) {
                orc_cache_free(c);
                return fail(err, ORC_SIZE_OVERFLOW, "windowed layer storage", 0, 0, 0, 0);
            }
            lc->keys = (float *)calloc(slots, sizeof(float));
            lc->values = (float *)calloc(slots, sizeof(float));
            lc->slot_position = (int64_t *)malloc(lc->window * sizeof(int64_t));
            if (lc->keys == NULL || lc->values == NULL || lc->slot_position == NULL) {
                orc_cache_free(c);
                return fail(err, ORC_SIZE_OVERFLOW, "windowed layer storage", 0, 0, 0, 0);
            }
            for (uint64_t s = 0; s < lc->window; s++) {
                lc->slot_position[s] = -1;
            }
        }
    }
    c->id = __atomic_fetch_add(&g_next_cache_id, 1, __ATOMIC_RELAXED);
    *out = c;
    return ORC_OK;
}

void orc_cache_free(orc_cache *c) {
    if (c == NULL) {
        return;
    }
    free_live(c);
    if (c->layers != NULL) {
        for (uint64_t i = 0; i < c->layer_count; i++) {
            free(c->layers[i].keys);
            free(c->layers[i].values);
            free(c->layers[i].slot_position);
        }
        free(c->layers);
    }
    free(c);
}

uint64_t orc_cache_layer_count(const orc_cache *c) { return c->layer_count; }
uint64_t orc_cache_num_kv_heads(const orc_cache *c) { return c->num_kv_heads; }
uint64_t orc_cache_head_dim(const orc_cache *c) { return c->head_dim; }

static int check_layer(const orc_cache *c, uint64_t layer, orc_error *err) { /* cache.rs:388-400 */
    if (layer >= c->layer_count) {
        return fail(err, ORC_INVALID_LAYER, NULL, layer, c->layer_count, 0, 0);
    }
    return ORC_OK;
}

int orc_cache_layer_window(const orc_cache *c, uint64_t layer, uint64_t *window, orc_error *err) {
    int rc = check_layer(c, layer, err);
    if (rc != ORC_OK) {
        return rc;
    }
    *window = c->layers[layer].window; /* 0 for a global layer */
    return ORC_OK;
}

int orc_cache_stored_len(const orc_cache *c, uint64_t layer, uint64_t *out, orc_error *err) {
    int rc = check_layer(c, layer, err);
    if (rc != ORC_OK) {
        return rc;
    }
    *out = layer_stored(&c->layers[layer]);
    return ORC_OK;
}

int orc_cache_next_position(const orc_cache *c, uint64_t layer, uint64_t *out, orc_error *err) {
    int rc = check_layer(c, layer, err);
    if (rc != ORC_OK) {
        return rc;
    }
    *out = c->layers[layer].appended;
    return ORC_OK;
}

/* cache.rs:423-474 then LayerCache::write :181-203. */
int orc_cache_append(orc_cache *c, uint64_t layer, const float *k, uint64_t k_len, const float *v,
                     uint64_t v_len, uint64_t position, orc_error *err) {
    uint64_t expected_len = c->num_kv_heads * c->head_dim;
    if (k_len != expected_len) {
        return fail(err, ORC_SHAPE_MISMATCH, "k", expected_len, k_len, 0, 0);
    }
    if (v_len != expected_len) {
        return fail(err, ORC_SHAPE_MISMATCH, "v", expected_len, v_len, 0, 0);
    }
    if (c->live && layer < c->layer_count) {
        uint64_t limit = c->live_bases[layer] + c->live_max_round_tokens;
        if (position >= limit) {
            return fail(err, ORC_CHECKPOINT_RANGE_EXCEEDED, NULL, layer, position, limit, 0);
        }
    }
    int rc = check_layer(c, layer, err);
    if (rc != ORC_OK) {
        return rc;
    }
    layer_cache *lc = &c->layers[layer];
    if (position != lc->appended) {
        return fail(err, ORC_OUT_OF_ORDER_POSITION, NULL, layer, lc->appended, position, 0);
    }
    if (!lc->windowed) {
        if (grow_global(lc, c->row, lc->appended + 1) != 0) {
            return fail(err, ORC_SIZE_OVERFLOW, "global layer storage", 0, 0, 0, 0);
        }
        store_row(c, lc->keys + lc->appended * c->row, k);
        store_row(c, lc->values + lc->appended * c->row, v);
    } else {
        uint64_t slot = layer_slot_of(lc, position);
        store_row(c, lc->keys + slot * c->row, k);
        store_row(c, lc->values + slot * c->row, v);
        lc->slot_position[slot] = (int64_t)position;
    }
    lc->appended += 1;
    return ORC_OK;
}

/* cache.rs:513-577. */
int orc_cache_restore_bulk(orc_cache *c, uint64_t layer, uint64_t first_position, const float *keys,
                           uint64_t keys_len, const float *values, uint64_t values_len,
                           orc_error *err) {
    uint64_t row = c->num_kv_heads * c->head_dim;
    if (keys_len != values_len || keys_len % row != 0) {
        return fail(err, ORC_SHAPE_MISMATCH, "bulk restore rows", values_len, keys_len, 0, 0);
    }
    uint64_t rows = keys_len / row;
    int rc = check_layer(c, layer, err);
    if (rc != ORC_OK) {
        return rc;
    }
    layer_cache *lc = &c->layers[layer];
    if (lc->appended != 0) {
        return fail(err, ORC_BULK_RESTORE_NOT_FRESH, NULL, layer, lc->appended, 0, 0);
    }
    if (!lc->windowed) {
        if (first_position != 0) {
            return fail(err, ORC_SHAPE_MISMATCH, "bulk restore first position (global layer)", 0,
                        first_position, 0, 0);
        }
        if (grow_global(lc, row, rows) != 0) {
            return fail(err, ORC_SIZE_OVERFLOW, "global layer storage", 0, 0, 0, 0);
        }
        for (uint64_t r = 0; r < rows; r++) {
            store_row(c, lc->keys + r * row, keys + r * row);
            store_row(c, lc->values + r * row, values + r * row);
        }
    } else {
        if (rows > lc->window) {
            return fail(err, ORC_SHAPE_MISMATCH, "bulk restore rows (windowed layer)", lc->window,
                        rows, 0, 0);
        }
        for (uint64_t r = 0; r < rows; r++) {
            uint64_t position = first_position + r;
            uint64_t slot = position % lc->window;
            store_row(c, lc->keys + slot * row, keys + r * row);
            store_row(c, lc->values + slot * row, values + r * row);
            lc->slot_position[slot] = (int64_t)position;
        }
    }
    lc->appended = first_position + rows;
    return ORC_OK;
}

void orc_cache_stats(const orc_cache *c, orc_layer_stats *out) { /* cache.rs:588-599 */
    for (uint64_t i = 0; i < c->layer_count; i++) {
        out[i].layer = i;
        out[i].window = c->layers[i].window;
        out[i].appended = c->layers[i].appended;
        out[i].stored = layer_stored(&c->layers[i]);
    }
}

int orc_cache_checkpoint_active(const orc_cache *c) { return c->live; }

/* cache.rs:634-717. */
int orc_cache_checkpoint(orc_cache *c, uint64_t max_round_tokens, orc_checkpoint *out,
                         orc_error *err) {
    if (c->live) {
        return fail(err, ORC_CHECKPOINT_BUSY, NULL, 0, 0, 0, 0);
    }
    if (max_round_tokens == 0) {
        return fail(err, ORC_ZERO_DIMENSION, "max_round_tokens", 0, 0, 0, 0);
    }
    uint64_t smallest = 0;
    int have_window = 0;
    for (uint64_t i = 0; i < c->layer_count; i++) {
        uint64_t w = c->layers[i].window;
        if (c->layers[i].windowed && (!have_window || w < smallest)) {
            smallest = w;
            have_window = 1;
        }
    }
    if (have_window && max_round_tokens > smallest) {
        return fail(err, ORC_CHECKPOINT_TOO_DEEP, NULL, max_round_tokens, smallest, 0, 0);
    }
    c->next_serial += 1;
    uint64_t serial = c->next_serial;
    uint64_t row = c->row;
    c->live_bases = (uint64_t *)malloc(c->layer_count * sizeof(uint64_t));
    c->live_layers = (layer_checkpoint *)calloc(c->layer_count, sizeof(layer_checkpoint));
    uint64_t saved_bytes = 0;
    for (uint64_t li = 0; li < c->layer_count; li++) {
        layer_cache *lc = &c->layers[li];
        c->live_bases[li] = lc->appended;
        if (!lc->windowed) {
            continue; /* global layers save nothing: rewind truncates */
        }
        layer_checkpoint *lcp = &c->live_layers[li];
        lcp->count = max_round_tokens;
        lcp->saved = (saved_slot *)calloc(max_round_tokens, sizeof(saved_slot));
        for (uint64_t i = 0; i < max_round_tokens; i++) {
            uint64_t slot = (lc->appended + i) % lc->window;
            saved_slot *e = &lcp->saved[i];
            e->slot = slot;
            e->position = lc->slot_position[slot];
            e->keys = (float *)malloc(row * sizeof(float));
            e->values = (float *)malloc(row * sizeof(float));
            memcpy(e->keys, lc->keys + slot * row, row * sizeof(float));
            memcpy(e->values, lc->values + slot * row, row * sizeof(float));
            saved_bytes += (row + row) * 4;
        }
    }
    c->live = 1;
    c->live_serial = serial;
    c->live_max_round_tokens = max_round_tokens;
    out->cache_id = c->id;
    out->serial = serial;
    out->max_round_tokens = max_round_tokens;
    out->saved_bytes = saved_bytes;
    out->layer_count = c->layer_count;
    out->bases = (uint64_t *)malloc(c->layer_count * sizeof(uint64_t));
    memcpy(out->bases, c->live_bases, c->layer_count * sizeof(uint64_t));
    return ORC_OK;
}

void orc_checkpoint_free(orc_checkpoint *cp) {
    if (cp != NULL) {
        free(cp->bases);
        cp->bases = NULL;
    }
}

static int live_data(const orc_cache *c, const orc_checkpoint *cp, orc_error *err) { /* :721-728 */
    if (c->live && c->live_serial == cp->serial && cp->cache_id == c->id) {
        return ORC_OK;
    }
    return fail(err, ORC_STALE_CHECKPOINT, NULL, cp->serial, 0, 0, 0);
}

/* cache.rs:758-818. */
int orc_cache_rewind_to(orc_cache *c, const orc_checkpoint *cp, uint64_t target, orc_error *err) {
    int rc = live_data(c, cp, err);
    if (rc != ORC_OK) {
        return rc;
    }
    uint64_t row = c->row;
    for (uint64_t li = 0; li < c->layer_count; li++) {
        uint64_t base = c->live_bases[li];
        if (target < base || target > c->layers[li].appended) {
            return fail(err, ORC_REWIND_OUT_OF_RANGE, NULL, li, base, c->layers[li].appended,
                        target);
        }
    }
    for (uint64_t li = 0; li < c->layer_count; li++) {
        layer_cache *lc = &c->layers[li];
        uint64_t base = c->live_bases[li];
        if (lc->windowed) {
            layer_checkpoint *lcp = &c->live_layers[li];
            for (uint64_t i = 0; i < lcp->count; i++) {
                saved_slot *s = &lcp->saved[i];
                int64_t p = lc->slot_position[s->slot];
                int keep = p >= 0 && (uint64_t)p >= base && (uint64_t)p < target;
                if (!keep) {
                    memcpy(lc->keys + s->slot * row, s->keys, row * sizeof(float));
                    memcpy(lc->values + s->slot * row, s->values, row * sizeof(float));
                    lc->slot_position[s->slot] = s->position;
                }
            }
        }
        /* Global: Vec::truncate; the rows past target simply stop being visible. */
        lc->appended = target;
    }
    return ORC_OK;
}

/* cache.rs:824-833. */
int orc_cache_release(orc_cache *c, const orc_checkpoint *cp, orc_error *err) {
    int rc = live_data(c, cp, err);
    if (rc != ORC_OK) {
        return rc;
    }
    free_live(c);
    return ORC_OK;
}

/* ------------------------------------------------------------------- view */

int orc_view_len(const orc_cache *c, uint64_t layer, uint64_t *out, orc_error *err) {
    return orc_cache_stored_len(c, layer, out, err);
}

int orc_view_position_at(const orc_cache *c, uint64_t layer, uint64_t visible_index,
                         uint64_t *pos) { /* cache.rs:878-883 */
    if (layer >= c->layer_count) {
        return 0;
    }
    const layer_cache *lc = &c->layers[layer];
    if (visible_index >= layer_stored(lc)) {
        return 0;
    }
    *pos = layer_first_visible(lc) + visible_index;
    return 1;
}

int orc_view_key(const orc_cache *c, uint64_t layer, uint64_t visible_index, uint64_t kv_head,
                 const float **row) { /* cache.rs:887-893 with :175-177,205-211 */
    uint64_t position;
    if (!orc_view_position_at(c, layer, visible_index, &position)) {
        return 0;
    }
    if (kv_head >= c->num_kv_heads) {
        return 0;
    }
    const layer_cache *lc = &c->layers[layer];
    *row = lc->keys + (layer_slot_of(lc, position) * c->num_kv_heads + kv_head) * c->head_dim;
    return 1;
}

int orc_view_value(const orc_cache *c, uint64_t layer, uint64_t visible_index, uint64_t kv_head,
                   const float **row) { /* cache.rs:897-903 */
    uint64_t position;
    if (!orc_view_position_at(c, layer, visible_index, &position)) {
        return 0;
    }
    if (kv_head >= c->num_kv_heads) {
        return 0;
    }
    const layer_cache *lc = &c->layers[layer];
    *row = lc->values + (layer_slot_of(lc, position) * c->num_kv_heads + kv_head) * c->head_dim;
    return 1;
}

/* -------------------------------------------------------------- attention */

static int attends(uint64_t kp, uint64_t p, int windowed, uint64_t window) { /* attention.rs:77-85 */
    if (kp > p) {
        return 0;
    }
    if (!windowed) {
        return 1;
    }
    return (int64_t)kp > (int64_t)p - (int64_t)window;
}

static float dot(const float *a, const float *b, uint64_t n) { /* attention.rs:87-89 */
    float s = 0.0f;
    for (uint64_t i = 0; i < n; i++) {
        s += a[i] * b[i];
    }
    return s;
}

/* One (query, head) pair: attention.rs:175-211. scores is scratch of n_visible floats. */
static void attend_head(const orc_cache *c, const layer_cache *lc, const float *qh,
                        uint64_t kv_head, const uint64_t *visible, uint64_t n_visible, float scale,
                        float softcap, float *scores, float *out) {
    uint64_t d = c->head_dim;
    uint64_t first = layer_first_visible(lc);
    float max = -INFINITY;
    for (uint64_t i = 0; i < n_visible; i++) {
        uint64_t position = first + visible[i];
        const float *k = lc->keys + (layer_slot_of(lc, position) * c->num_kv_heads + kv_head) * d;
        float s = dot(qh, k, d) * scale;
        if (softcap > 0.0f) {
            s = softcap * tanhf(s / softcap);
        }
        if (s > max) {
            max = s;
        }
        scores[i] = s;
    }
    float sum = 0.0f;
    for (uint64_t i = 0; i < n_visible; i++) {
        scores[i] = expf(scores[i] - max);
        sum += scores[i];
    }
    for (uint64_t i = 0; i < n_visible; i++) {
        float w = scores[i] / sum;
        uint64_t position = first + visible[i];
        const float *v =
            lc->values + (layer_slot_of(lc, position) * c->num_kv_heads + kv_head) * d;
        for (uint64_t e = 0; e < d; e++) {
            out[e] += w * v[e];
        }
    }
}

int orc_gqa_attention(const float *q, uint64_t q_len, uint64_t num_queries, uint64_t num_q_heads,
                      const uint64_t *query_positions, uint64_t positions_len, const orc_cache *c,
                      uint64_t layer, float scale, float softcap, int threads, float *out,
                      orc_error *err) {
    int rc = check_layer(c, layer, err);
    if (rc != ORC_OK) {
        return rc;
    }
    const layer_cache *lc = &c->layers[layer];
    uint64_t head_dim = c->head_dim;
    uint64_t num_kv_heads = c->num_kv_heads;
    if (positions_len != num_queries) {
        return fail(err, ORC_SHAPE_MISMATCH, "query_positions", num_queries, positions_len, 0, 0);
    }
    uint64_t expected_q = num_queries * num_q_heads * head_dim;
    if (q_len != expected_q) {
        return fail(err, ORC_SHAPE_MISMATCH, "q", expected_q, q_len, 0, 0);
    }
    if (num_queries == 0) {
        return ORC_OK;
    }
    if (num_q_heads == 0) {
        return fail(err, ORC_ZERO_DIMENSION, "num_q_heads", 0, 0, 0, 0);
    }
    if (num_q_heads % num_kv_heads != 0) {
        return fail(err, ORC_NON_DIVISIBLE_HEADS, NULL, num_q_heads, num_kv_heads, 0, 0);
    }
    uint64_t group = num_q_heads / num_kv_heads;
    if (isnan(scale)) {
        scale = 1.0f / sqrtf((float)head_dim); /* AttentionParams { scale: None }, attention.rs:35-37 */
    }
    uint64_t view_len = layer_stored(lc);
    uint64_t first = layer_first_visible(lc);

    /* The mask depends only on the query position (attention.rs:160-173). */
    uint64_t *visible = (uint64_t *)malloc((view_len + 1) * num_queries * sizeof(uint64_t));
    uint64_t *n_visible = (uint64_t *)calloc(num_queries, sizeof(uint64_t));
    for (uint64_t qi = 0; qi < num_queries; qi++) {
        uint64_t p = query_positions[qi];
        uint64_t *vis = visible + qi * (view_len + 1);
        uint64_t n = 0;
        for (uint64_t vi = 0; vi < view_len; vi++) {
            if (attends(first + vi, p, lc->windowed, lc->window)) {
                vis[n++] = vi;
            }
        }
        if (n == 0) {
            free(visible);
            free(n_visible);
            return fail(err, ORC_NO_VISIBLE_KEYS, NULL, p, 0, 0, 0);
        }
        n_visible[qi] = n;
    }
    memset(out, 0, q_len * sizeof(float));
    int64_t pairs = (int64_t)(num_queries * num_q_heads);
    if (threads < 1) {
        threads = 1;
    }
#pragma omp parallel num_threads(threads)
    {
        float *scores = (float *)malloc((view_len + 1) * sizeof(float));
#pragma omp for schedule(dynamic, 1)
        for (int64_t pair = 0; pair < pairs; pair++) {
            uint64_t qi = (uint64_t)pair / num_q_heads;
            uint64_t h = (uint64_t)pair % num_q_heads;
            uint64_t off = (qi * num_q_heads + h) * head_dim;
            attend_head(c, lc, q + off, h / group, visible + qi * (view_len + 1), n_visible[qi],
                        scale, softcap, scores, out + off);
        }
        free(scores);
    }
    free(visible);
    free(n_visible);
    return ORC_OK;
}

int orc_attention_step(orc_cache *c, uint64_t layer, const float *q, const float *k, const float *v,
                       uint64_t rows, uint64_t num_q_heads, uint64_t start_position, float scale,
                       float softcap, int threads, float *out, orc_error *err) {
    uint64_t appended;
    int rc = orc_cache_next_position(c, layer, &appended, err);
    if (rc != ORC_OK) {
        return rc;
    }
    if (appended != start_position) { /* cpu.rs:569-581 */
        char text[96];
        snprintf(text, sizeof(text), "KV state for layer %llu is at position %llu, cache at %llu",
                 (unsigned long long)layer, (unsigned long long)appended,
                 (unsigned long long)start_position);
        return fail(err, ORC_STEP_FAILED, text, layer, appended, start_position, 0);
    }
    uint64_t q_width = num_q_heads * c->head_dim;
    uint64_t kv_width = c->num_kv_heads * c->head_dim;
    for (uint64_t i = 0; i < rows; i++) { /* cpu.rs:592-646 */
        uint64_t position = start_position + i;
        rc = orc_cache_append(c, layer, k + i * kv_width, kv_width, v + i * kv_width, kv_width,
                              position, err);
        if (rc != ORC_OK) {
            return rc;
        }
        rc = orc_gqa_attention(q + i * q_width, q_width, 1, num_q_heads, &position, 1, c, layer,
                               scale, softcap, threads, out + i * q_width, err);
        if (rc != ORC_OK) {
            return rc;
        }
    }
    return ORC_OK;
}
