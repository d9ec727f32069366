/* A client of the C ABI written in C alone: what a foreign-function binding (the cgo-free,
   torch-free way the reference's Rust crate would link the library) sees. It includes the
   public header as a C99 translation unit, links the shared library, and checks results
   against arithmetic done here in double precision, independent of the Python oracle.

     kv_client host <dir>    hashes, snapshot codec and prefix store: no device needed
     kv_client device <dir>  pool, append, attention, speculative round, snapshot, store

   Prints "<mode> ok" and exits 0, or names the first failed check and exits 1. */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "itak_hip_kv.h"

#define CHECK(cond)                                                              \
    do {                                                                         \
        if (!(cond)) {                                                           \
            fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
            exit(1);                                                             \
        }                                                                        \
    } while (0)
#define OK(pool, call)                                                                        \
    do {                                                                                      \
        itak_status st_ = (call);                                                             \
        if (st_ != ITAK_OK) {                                                                 \
            fprintf(stderr, "%s:%d: %s -> %d: %s\n", __FILE__, __LINE__, #call, (int)st_,     \
                    itak_last_error(pool));                                                   \
            exit(1);                                                                          \
        }                                                                                     \
    } while (0)

/* xorshift64*: the inputs need no statistical quality, only to be the same every run. */
static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static float rnd(void) {
    rng_state ^= rng_state >> 12;
    rng_state ^= rng_state << 25;
    rng_state ^= rng_state >> 27;
    return (float)((double)((rng_state * 2685821657736338717ull) >> 11) / 9007199254740992.0 * 2.0 - 1.0);
}

/* f32 -> f16 -> f32, round to nearest even (normal range; the inputs here stay inside it). */
static float through_f16(float x) {
    union { float f; uint32_t u; } v;
    uint32_t sign, mant, rest;
    int32_t exp;
    v.f = x;
    sign = v.u & 0x80000000u;
    exp = (int32_t)((v.u >> 23) & 0xff) - 127;
    if (x == 0.0f) return x;
    CHECK(exp >= -14 && exp <= 14);
    mant = v.u & 0x7fffffu;
    rest = mant & 0x1fffu;
    mant >>= 13;
    if (rest > 0x1000u || (rest == 0x1000u && (mant & 1u))) mant += 1;
    v.u = sign | (uint32_t)((exp + 127) << 23);
    v.u += mant << 13; /* a carry out of the mantissa moves the exponent up, as it should */
    return v.f;
}

static void host_checks(const char *dir) {
    CHECK(itak_abi_version() == 1);
    /* FNV-1a 64 test vectors (the published ones for "", "a", "foobar"). */
    CHECK(itak_kv_checksum("", 0) == 0xcbf29ce484222325ull);
    CHECK(itak_kv_checksum("a", 1) == 0xaf63dc4c8601ec8cull);
    CHECK(itak_kv_checksum("foobar", 6) == 0x85944171f73967e8ull);
    {
        const uint32_t tokens[3] = {1, 2, 0x01020304u};
        const uint8_t bytes[12] = {1, 0, 0, 0, 2, 0, 0, 0, 4, 3, 2, 1};
        CHECK(itak_kv_prefix_hash(tokens, 3) == itak_kv_checksum(bytes, 12));
        CHECK(itak_kv_prefix_discriminator(tokens, 3) != itak_kv_prefix_hash(tokens, 3));
    }
    {
        /* The discriminator's basis (hash.rs:21) and two values folded by hand. */
        const uint32_t one[1] = {1}, two[2] = {0xdeadbeefu, 7};
        CHECK(itak_kv_prefix_discriminator(one, 0) == 0x84222325cbf29ce4ull);
        CHECK(itak_kv_prefix_discriminator(one, 1) == 0xb61d2746190c09b5ull);
        CHECK(itak_kv_prefix_discriminator(two, 2) == 0x393db72d40db1afdull);
        CHECK(itak_kv_prefix_hash(one, 1) == 0xad2aca7747985764ull);
    }
    {
        /* One block: the sum of one sum. */
        const uint64_t inner = itak_kv_checksum("foobar", 6);
        uint8_t le[8];
        int b;
        for (b = 0; b < 8; ++b) le[b] = (uint8_t)(inner >> (8 * b));
        CHECK(itak_kv_checksum_blocks("foobar", 6) == itak_kv_checksum(le, 8));
        CHECK(itak_kv_checksum_blocks("", 0) == 0xcbf29ce484222325ull);
    }
    {
        /* Snapshot codec: 3 tokens, 2 KV heads of dim 4, one global layer. */
        float keys[24], values[24];
        const float *kp[1], *vp[1];
        uint64_t kf[1] = {24}, vf[1] = {24}, written = 0, need = 0;
        itak_itkv_header h, back;
        itak_itkv_layer layer, got;
        uint8_t *buf;
        int i;
        itak_store *store = NULL;
        itak_prefix_hit hit;
        itak_store_stats stats;
        const uint32_t tokens[3] = {7, 8, 9}, query[4] = {7, 8, 9, 10};
        for (i = 0; i < 24; ++i) {
            keys[i] = rnd();
            values[i] = rnd();
        }
        kp[0] = keys;
        vp[0] = values;
        memset(&h, 0, sizeof(h));
        memset(&layer, 0, sizeof(layer));
        h.token_count = 3;
        h.num_kv_heads = 2;
        h.head_dim = 4;
        h.layer_count = 1;
        h.fingerprint_len = 2;
        layer.kind = ITAK_LAYER_GLOBAL;
        layer.rows = 3;
        OK(NULL, itak_itkv_validate(&h, &layer, 1, kf, vf));
        OK(NULL, itak_itkv_encode(&h, "fp", &layer, 1, kp, kf, vp, vf, NULL, 0, &need));
        /* magic, version, fingerprint length + bytes, token count, three geometry words,
           one 28-byte layer header, the rows, the checksum (snapshot.rs:13-29). */
        CHECK(need == 4 + 4 + 4 + 2 + 8 + 12 + 28 + 2 * 24 * 4 + 8);
        buf = (uint8_t *)malloc(need);
        OK(NULL, itak_itkv_encode(&h, "fp", &layer, 1, kp, kf, vp, vf, buf, need, &written));
        CHECK(written == need && memcmp(buf, "ITKV", 4) == 0 && buf[4] == 1);
        OK(NULL, itak_itkv_decode(buf, need, &back, &got, 1));
        CHECK(back.token_count == 3 && back.num_kv_heads == 2 && back.head_dim == 4);
        CHECK(back.version == 1 && back.elem == ITAK_ELEM_F32 && back.encoded_len == need);
        CHECK(memcmp(buf + back.fingerprint_offset, "fp", 2) == 0);
        CHECK(got.rows == 3 && got.first_position == 0 && got.kind == ITAK_LAYER_GLOBAL);
        CHECK(memcmp(buf + got.keys_offset, keys, sizeof(keys)) == 0);
        CHECK(memcmp(buf + got.values_offset, values, sizeof(values)) == 0);
        buf[got.values_offset + 5] ^= 0x20;
        CHECK(itak_itkv_decode(buf, need, &back, &got, 1) == ITAK_KV_CHECKSUM_MISMATCH);
        CHECK(strstr(itak_last_error(NULL), "snapshot checksum mismatch") != NULL);
        buf[got.values_offset + 5] ^= 0x20;
        /* Prefix store: put, then the longest stored prefix of a longer query. */
        OK(NULL, itak_store_open(dir, 1u << 20, &store));
        CHECK(itak_store_put(store, tokens, 3, buf, need, 100) == ITAK_OK);
        CHECK(itak_store_lookup(store, query, 4, NULL, NULL, "fp", 2, 200, &hit) == ITAK_OK);
        CHECK(hit.token_count == 3 && hit.snapshot_len == need);
        CHECK(memcmp(hit.snapshot, buf, need) == 0);
        CHECK(itak_store_lookup(store, query, 4, NULL, NULL, "other", 5, 300, &hit) == ITAK_OK);
        CHECK(hit.token_count == 0);
        CHECK(strstr(itak_store_refusals(store), "model fingerprint mismatch") != NULL);
        CHECK(itak_store_get_stats(store, &stats) == ITAK_OK && stats.entries == 1);
        CHECK(itak_store_put(store, tokens, 0, buf, need, 100) == ITAK_KV_EMPTY_PREFIX);
        itak_store_close(store);
        free(buf);
    }
}

enum { KVH = 2, D = 128, QH = 8, ROW = KVH * D, WINDOW = 16, N0 = 70 };

/* gqa_attention as attention.rs:104-215 states it, in double, over f16-rounded rows. */
static void reference_attention(const float *k, const float *v, int n, int lowest, int position,
                                const float *q, double *out) {
    int h, p, c;
    for (h = 0; h < QH; ++h) {
        const int kvh = h / (QH / KVH);
        double m = -1e300, l = 0.0, acc[D];
        static double score[N0 + 16];
        for (p = lowest; p <= position && p < n; ++p) {
            double s = 0.0;
            for (c = 0; c < D; ++c) s += (double)q[h * D + c] * (double)k[p * ROW + kvh * D + c];
            score[p] = s / sqrt((double)D);
            if (score[p] > m) m = score[p];
        }
        for (c = 0; c < D; ++c) acc[c] = 0.0;
        for (p = lowest; p <= position && p < n; ++p) {
            const double w = exp(score[p] - m);
            l += w;
            for (c = 0; c < D; ++c) acc[c] += w * (double)v[p * ROW + kvh * D + c];
        }
        for (c = 0; c < D; ++c) out[h * D + c] = acc[c] / l;
    }
}

static void device_checks(const char *dir) {
    const uint8_t kinds[2] = {ITAK_LAYER_GLOBAL, ITAK_LAYER_WINDOWED};
    const uint64_t windows[2] = {0, WINDOW};
    static float k[2][(N0 + 8) * ROW], v[2][(N0 + 8) * ROW], q[QH * D], out[QH * D], out2[QH * D];
    static double want[QH * D];
    itak_pool_config cfg;
    itak_pool *pool = NULL;
    uint32_t slot = 0, twin = 0, third = 0, none = 0;
    uint64_t position = 0, stored = 0, bytes = 0, written = 0, matched = 0;
    itak_checkpoint cp;
    itak_store *store = NULL;
    uint32_t tokens[N0 + 1];
    uint8_t *snap;
    int layer, p, i;

    memset(&cfg, 0, sizeof(cfg));
    cfg.layer_count = 2;
    cfg.layer_kinds = kinds;
    cfg.windows = windows;
    cfg.num_kv_heads = KVH;
    cfg.head_dim = D;
    cfg.elem = ITAK_ELEM_F16;
    cfg.max_slots = 3;
    cfg.capacity_rows = 256;
    cfg.flags = ITAK_POOL_SCRUB_ON_TRUNCATE;
    OK(NULL, itak_pool_create(&cfg, &pool));
    CHECK(itak_kv_layer_count(pool) == 2 && itak_kv_head_dim(pool) == D);
    OK(pool, itak_slot_acquire(pool, &slot));

    for (layer = 0; layer < 2; ++layer)
        for (i = 0; i < (N0 + 8) * ROW; ++i) {
            /* Kept inside f16's normal range, which is all through_f16 rounds. */
            float a = rnd(), b = rnd();
            if (fabsf(a) < 1e-3f) a = 0.25f;
            if (fabsf(b) < 1e-3f) b = -0.5f;
            k[layer][i] = through_f16(a);
            v[layer][i] = through_f16(b);
        }
    for (i = 0; i < QH * D; ++i) q[i] = rnd();
    for (i = 0; i <= N0; ++i) tokens[i] = 1000u + (uint32_t)i;

    /* One position at a time, as KvCache::append is called; attention after each tenth. */
    for (p = 0; p < N0; ++p) {
        for (layer = 0; layer < 2; ++layer)
            OK(pool, itak_kv_append(pool, slot, (uint64_t)layer, k[layer] + p * ROW, ROW,
                                    v[layer] + p * ROW, ROW, (uint64_t)p));
        if (p % 10 != 9) continue;
        for (layer = 0; layer < 2; ++layer) {
            const uint64_t at = (uint64_t)p;
            const int lowest = (layer == 1 && p + 1 > WINDOW) ? p + 1 - WINDOW : 0;
            double worst = 0.0;
            OK(pool, itak_gqa_attention(pool, slot, (uint64_t)layer, q, QH * D, 1, QH, &at, 1,
                                        (float)NAN, 0.0f, out));
            reference_attention(k[layer], v[layer], p + 1, lowest, p, q, want);
            for (i = 0; i < QH * D; ++i)
                if (fabs((double)out[i] - want[i]) > worst) worst = fabs((double)out[i] - want[i]);
            if (worst > 2e-3) {
                fprintf(stderr, "attention off by %g at position %d layer %d\n", worst, p, layer);
                exit(1);
            }
        }
    }
    OK(pool, itak_kv_next_position(pool, slot, 1, &position));
    OK(pool, itak_kv_stored_len(pool, slot, 1, &stored));
    CHECK(position == N0 && stored == WINDOW);

    /* A speculative round: checkpoint, four rows, keep one, release. */
    OK(pool, itak_kv_checkpoint(pool, slot, 4, &cp));
    for (p = N0; p < N0 + 4; ++p)
        for (layer = 0; layer < 2; ++layer)
            OK(pool, itak_kv_append(pool, slot, (uint64_t)layer, k[layer] + p * ROW, ROW,
                                    v[layer] + p * ROW, ROW, (uint64_t)p));
    CHECK(itak_kv_rewind_to(pool, slot, &cp, N0 + 5) == ITAK_REWIND_OUT_OF_RANGE);
    OK(pool, itak_kv_rewind_to(pool, slot, &cp, N0 + 1));
    OK(pool, itak_kv_release(pool, slot, &cp));
    CHECK(itak_kv_release(pool, slot, &cp) == ITAK_STALE_CHECKPOINT);
    OK(pool, itak_kv_next_position(pool, slot, 0, &position));
    CHECK(position == N0 + 1);

    /* Snapshot out, into a second slot, and the two answer alike bit for bit. */
    OK(pool, itak_kv_capture_itkv(pool, slot, "model", 5, NULL, 0, &bytes));
    snap = (uint8_t *)malloc(bytes);
    OK(pool, itak_kv_capture_itkv(pool, slot, "model", 5, snap, bytes, &written));
    CHECK(written == bytes);
    OK(pool, itak_slot_acquire(pool, &twin));
    CHECK(itak_kv_restore_itkv(pool, twin, snap, bytes, "another", 7) == ITAK_KV_FINGERPRINT_MISMATCH);
    OK(pool, itak_kv_restore_itkv(pool, twin, snap, bytes, "model", 5));
    for (layer = 0; layer < 2; ++layer) {
        const uint64_t at = N0;
        OK(pool, itak_gqa_attention(pool, slot, (uint64_t)layer, q, QH * D, 1, QH, &at, 1,
                                    (float)NAN, 0.0f, out));
        OK(pool, itak_gqa_attention(pool, twin, (uint64_t)layer, q, QH * D, 1, QH, &at, 1,
                                    (float)NAN, 0.0f, out2));
        CHECK(memcmp(out, out2, sizeof(out)) == 0);
    }

    /* Through the prefix store into a third slot. */
    OK(NULL, itak_store_open(dir, 1u << 26, &store));
    CHECK(itak_store_capture_and_put(store, pool, slot, tokens, N0 + 1, "model", 5, ITAK_ELEM_F16,
                                     50) == ITAK_OK);
    OK(pool, itak_slot_acquire(pool, &third));
    CHECK(itak_store_restore_prefix(store, pool, third, tokens, N0 + 1, "model", 5, 60, &matched) ==
          ITAK_OK);
    CHECK(matched == N0 + 1);
    {
        const uint64_t at = N0;
        OK(pool, itak_gqa_attention(pool, third, 1, q, QH * D, 1, QH, &at, 1, (float)NAN, 0.0f, out2));
        CHECK(memcmp(out, out2, sizeof(out)) == 0);
    }
    itak_store_close(store);

    /* Truncate (a rejected round with no checkpoint held): the length moves back, on the
       windowed layer inside what its ring still holds. */
    {
        const uint64_t shorter = N0 - 3;
        OK(pool, itak_kv_truncate(pool, &slot, &shorter, 1));
        OK(pool, itak_kv_next_position(pool, slot, 1, &position));
        OK(pool, itak_kv_stored_len(pool, slot, 1, &stored));
        CHECK(position == N0 - 3 && stored == WINDOW);
    }
    CHECK(itak_slot_acquire(pool, &none) == ITAK_NO_FREE_SLOT);
    free(snap);
    itak_pool_destroy(pool);
}

int main(int argc, char **argv) {
    if (argc != 3 || (strcmp(argv[1], "host") != 0 && strcmp(argv[1], "device") != 0)) {
        fprintf(stderr, "usage: kv_client host|device <empty directory>\n");
        return 2;
    }
    if (strcmp(argv[1], "host") == 0)
        host_checks(argv[2]);
    else
        device_checks(argv[2]);
    printf("%s ok\n", argv[1]);
    return 0;
}
