// ITKV v1 snapshot codec and FNV-1a hashes, host side: crates/itak-kv/src/snapshot.rs:381-604
// and crates/itak-kv/src/hash.rs. Every size read from the byte stream is bounds-checked with
// checked arithmetic before it is trusted; a refusal is returned by name, nothing aborts.
#include "itkv.h"

#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/itak_hip_kv.h"

namespace itak {

uint64_t fnv1a64(const uint8_t *bytes, uint64_t count, uint64_t basis) {
    uint64_t hash = basis;
    for (uint64_t i = 0; i < count; ++i) {
        hash ^= uint64_t(bytes[i]);
        hash *= kFnvPrime;
    }
    return hash;
}

uint64_t fnv1a64_tokens(const uint32_t *tokens, uint64_t count, uint64_t basis) {
    uint64_t hash = basis;
    for (uint64_t i = 0; i < count; ++i) {
        const uint32_t t = tokens[i];
        for (int b = 0; b < 4; ++b) {  // little-endian bytes, the on-disk token encoding
            hash ^= uint64_t((t >> (8 * b)) & 0xffu);
            hash *= kFnvPrime;
        }
    }
    return hash;
}

unsigned host_threads() {
    static const unsigned threads = [] {
        unsigned limit = 8;
        if (const char *text = getenv("ITAK_HOST_THREADS")) {
            char *end = nullptr;
            const long asked = strtol(text, &end, 10);
            if (end != text && *end == 0 && asked >= 1 && asked <= 64) limit = unsigned(asked);
        }
        const unsigned machine = std::thread::hardware_concurrency();
        return std::max(1u, machine ? std::min(machine, limit) : limit);
    }();
    return threads;
}

uint64_t fnv1a64_of_sums(const uint64_t *sums, uint64_t blocks) {
    uint64_t hash = kFnvOffset;
    for (uint64_t k = 0; k < blocks; ++k)
        for (int b = 0; b < 8; ++b) {
            hash ^= (sums[k] >> (8 * b)) & 0xffu;
            hash *= kFnvPrime;
        }
    return hash;
}

void fnv1a64_block_group(const uint8_t *bytes, uint64_t count, uint64_t first, uint64_t n, uint64_t *sums) {
    const uint8_t *p[kItkvSumGroup];
    uint64_t len[kItkvSumGroup], h[kItkvSumGroup];
    uint64_t common = kItkvSumBlock;
    for (uint64_t j = 0; j < kItkvSumGroup; ++j) {
        const uint64_t k = first + std::min(j, n - 1);  // short groups walk their last block again
        const uint64_t at = k * kItkvSumBlock;
        p[j] = bytes + at;
        len[j] = std::min(kItkvSumBlock, count - at);
        h[j] = kFnvOffset;
        common = std::min(common, len[j]);
    }
    uint64_t a = h[0], b = h[1], c = h[2], d = h[3];
    const uint8_t *pa = p[0], *pb = p[1], *pc = p[2], *pd = p[3];
    for (uint64_t i = 0; i < common; ++i) {
        a ^= pa[i];
        b ^= pb[i];
        c ^= pc[i];
        d ^= pd[i];
        a *= kFnvPrime;
        b *= kFnvPrime;
        c *= kFnvPrime;
        d *= kFnvPrime;
    }
    h[0] = a, h[1] = b, h[2] = c, h[3] = d;
    for (uint64_t j = 0; j < n; ++j)  // only the snapshot's last block can be longer than the others are short
        sums[first + j] = len[j] > common ? fnv1a64(p[j] + common, len[j] - common, h[j]) : h[j];
}

uint64_t fnv1a64_blocks(const uint8_t *bytes, uint64_t count) {
    const uint64_t blocks = count / kItkvSumBlock + (count % kItkvSumBlock ? 1 : 0);
    std::vector<uint64_t> sums(blocks);
    const uint64_t groups = (blocks + kItkvSumGroup - 1) / kItkvSumGroup;
    for_each_index(groups, [&](uint64_t g) {
        const uint64_t first = g * kItkvSumGroup;
        fnv1a64_block_group(bytes, count, first, std::min(kItkvSumGroup, blocks - first), sums.data());
    });
    return fnv1a64_of_sums(sums.data(), blocks);
}

namespace {

bool refuse(ItkvError &err, int32_t code, uint64_t a, uint64_t b, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    err.code = code;
    err.message = buf;
    err.a = a;
    err.b = b;
    return false;
}

#define ULL(x) static_cast<unsigned long long>(x)

bool inconsistent(ItkvError &err, const char *fmt, ...) {
    char detail[400];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(detail, sizeof(detail), fmt, ap);
    va_end(ap);
    return refuse(err, ITAK_KV_INCONSISTENT_SNAPSHOT, 0, 0, "inconsistent snapshot: %s", detail);
}

bool checked_mul(uint64_t a, uint64_t b, uint64_t *out) { return !__builtin_mul_overflow(a, b, out); }

// The Debug text of attention::LayerKind, as the reference's messages print it.
std::string kind_debug(const ItkvLayer &l) {
    if (l.kind == ITAK_LAYER_GLOBAL) return "Global";
    char buf[64];
    snprintf(buf, sizeof(buf), "Windowed { window: %llu }", ULL(l.window));
    return buf;
}

// Well-formed UTF-8 as String::from_utf8 accepts it: no overlong forms, no surrogates,
// nothing above U+10FFFF.
bool valid_utf8(const uint8_t *s, uint64_t n) {
    uint64_t i = 0;
    while (i < n) {
        const uint8_t c = s[i];
        if (c < 0x80) {
            ++i;
        } else if (c >= 0xc2 && c <= 0xdf) {
            if (i + 1 >= n || (s[i + 1] & 0xc0) != 0x80) return false;
            i += 2;
        } else if (c >= 0xe0 && c <= 0xef) {
            if (i + 2 >= n) return false;
            const uint8_t c1 = s[i + 1], c2 = s[i + 2];
            const uint8_t lo = c == 0xe0 ? 0xa0 : 0x80, hi = c == 0xed ? 0x9f : 0xbf;
            if (c1 < lo || c1 > hi || (c2 & 0xc0) != 0x80) return false;
            i += 3;
        } else if (c >= 0xf0 && c <= 0xf4) {
            if (i + 3 >= n) return false;
            const uint8_t c1 = s[i + 1], c2 = s[i + 2], c3 = s[i + 3];
            const uint8_t lo = c == 0xf0 ? 0x90 : 0x80, hi = c == 0xf4 ? 0x8f : 0xbf;
            if (c1 < lo || c1 > hi || (c2 & 0xc0) != 0x80 || (c3 & 0xc0) != 0x80) return false;
            i += 4;
        } else {
            return false;
        }
    }
    return true;
}

// The strict little-endian cursor of snapshot.rs:520-604.
struct Reader {
    const uint8_t *bytes;
    uint64_t len, at = 0;
    ItkvError &err;

    uint64_t remaining() const { return len - at; }
    const uint8_t *take(uint64_t n) {
        if (remaining() < n) {
            uint64_t need = at + n;
            if (need < at) need = UINT64_MAX;
            refuse(err, ITAK_KV_TRUNCATED, need, len,
                   "snapshot: truncated, needs %llu bytes, has %llu", ULL(need), ULL(len));
            return nullptr;
        }
        const uint8_t *p = bytes + at;
        at += n;
        return p;
    }
    bool u32(uint32_t *out) {
        const uint8_t *p = take(4);
        if (!p) return false;
        *out = uint32_t(p[0]) | uint32_t(p[1]) << 8 | uint32_t(p[2]) << 16 | uint32_t(p[3]) << 24;
        return true;
    }
    bool u64(uint64_t *out) {
        const uint8_t *p = take(8);
        if (!p) return false;
        uint64_t v = 0;
        for (int i = 7; i >= 0; --i) v = (v << 8) | p[i];
        *out = v;
        return true;
    }
};

void put_u32(uint8_t *&p, uint32_t v) {
    for (int i = 0; i < 4; ++i) *p++ = uint8_t(v >> (8 * i));
}
void put_u64(uint8_t *&p, uint64_t v) {
    for (int i = 0; i < 8; ++i) *p++ = uint8_t(v >> (8 * i));
}

}  // namespace

bool itkv_validate(const ItkvHeader &h, const ItkvLayer *layers, uint64_t blocks,
                   const uint64_t *key_floats, const uint64_t *value_floats, ItkvError &err) {
    if (blocks != h.layer_count)
        return inconsistent(err, "snapshot carries %llu layer blocks but its geometry has %llu layers",
                            ULL(blocks), ULL(h.layer_count));
    if (h.num_kv_heads == 0 || h.head_dim == 0)
        return inconsistent(err, "geometry has a zero KV head count or head dimension");
    uint64_t row = 0;
    if (!checked_mul(h.num_kv_heads, h.head_dim, &row))
        return inconsistent(err, "KV row width overflows: %llu heads of dim %llu have no usize product",
                            ULL(h.num_kv_heads), ULL(h.head_dim));
    for (uint64_t i = 0; i < h.layer_count; ++i) {
        const ItkvLayer &l = layers[i];
        const uint64_t expected_rows = l.kind == ITAK_LAYER_GLOBAL
                                           ? h.token_count
                                           : (h.token_count < l.window ? h.token_count : l.window);
        const uint64_t expected_first = h.token_count - expected_rows;
        if (l.first_position != expected_first)
            return inconsistent(err,
                                "layer %llu: first stored position is %llu but %llu follows from "
                                "token count %llu and kind %s",
                                ULL(i), ULL(l.first_position), ULL(expected_first),
                                ULL(h.token_count), kind_debug(l).c_str());
        uint64_t expected_floats = 0;
        if (!checked_mul(expected_rows, row, &expected_floats))
            return inconsistent(err, "layer %llu: %llu rows of %llu floats overflow the float count",
                                ULL(i), ULL(expected_rows), ULL(row));
        if (key_floats[i] != expected_floats || value_floats[i] != expected_floats)
            return inconsistent(err,
                                "layer %llu: holds %llu key and %llu value floats but %llu rows of "
                                "%llu floats were expected",
                                ULL(i), ULL(key_floats[i]), ULL(value_floats[i]), ULL(expected_rows),
                                ULL(row));
    }
    return true;
}

bool itkv_decode(const uint8_t *bytes, uint64_t len, ItkvHeader &h, std::vector<ItkvLayer> &layers,
                 ItkvError &err, const uint64_t *known_sum) {
    Reader r{bytes, len, 0, err};
    const uint8_t *magic = r.take(4);
    if (!magic) return false;
    if (memcmp(magic, "ITKV", 4) != 0)
        return refuse(err, ITAK_KV_BAD_MAGIC, 0, 0, "snapshot: bad magic");
    uint32_t version = 0;
    if (!r.u32(&version)) return false;
    if (version != kItkvVersion && version != kItkvVersionTyped)
        return refuse(err, ITAK_KV_UNSUPPORTED_VERSION, version, 0,
                      "snapshot: unsupported format version %u", version);
    h.version = version;
    h.elem = 0;
    uint32_t fp_len = 0;
    if (!r.u32(&fp_len)) return false;
    h.fingerprint_offset = r.at;
    const uint8_t *fp = r.take(fp_len);
    if (!fp) return false;
    if (!valid_utf8(fp, fp_len)) return inconsistent(err, "model fingerprint is not valid UTF-8");
    h.fingerprint_len = fp_len;
    uint32_t heads = 0, dim = 0, layer_count = 0;
    if (!r.u64(&h.token_count) || !r.u32(&heads) || !r.u32(&dim) || !r.u32(&layer_count))
        return false;
    h.num_kv_heads = heads;
    h.head_dim = dim;
    h.layer_count = layer_count;
    if (version == kItkvVersionTyped) {
        if (!r.u32(&h.elem)) return false;
        if (h.elem > 1)
            return inconsistent(err, "element type tag %u is not a known type", h.elem);
    }
    // The count is bounded by the bytes that remain before it sizes anything
    // (snapshot.rs:448-462).
    if (layer_count > r.remaining() / kItkvLayerHeaderLen)
        return inconsistent(err,
                            "snapshot declares %u layers but only %llu bytes remain, not enough for "
                            "the layer headers alone",
                            layer_count, ULL(r.remaining()));
    layers.assign(layer_count, ItkvLayer{});
    for (uint32_t i = 0; i < layer_count; ++i) {
        const uint8_t *tag = r.take(1);
        if (!tag) return false;
        const uint8_t *reserved = r.take(3);
        if (!reserved) return false;
        if (reserved[0] | reserved[1] | reserved[2])
            return inconsistent(err, "layer header reserved bytes are not zero");
        ItkvLayer &l = layers[i];
        if (!r.u64(&l.window) || !r.u64(&l.first_position) || !r.u64(&l.rows)) return false;
        if (*tag == 0) {
            l.kind = ITAK_LAYER_GLOBAL;  // the window field of a global layer is not looked at
        } else if (*tag == 1) {
            if (l.window == 0) return inconsistent(err, "windowed layer carries a zero window");
            l.kind = ITAK_LAYER_WINDOWED;
        } else {
            return inconsistent(err, "layer kind tag %u is not a known kind", unsigned(*tag));
        }
    }
    uint64_t row = 0;
    if (!checked_mul(h.num_kv_heads, h.head_dim, &row))
        return inconsistent(err, "KV row width overflows: %llu heads of dim %llu have no usize product",
                            ULL(h.num_kv_heads), ULL(h.head_dim));
    std::vector<uint64_t> floats(layer_count);
    for (uint32_t i = 0; i < layer_count; ++i) {
        uint64_t bytes_per_side = 0;
        if (!checked_mul(layers[i].rows, row, &floats[i]))
            return inconsistent(err, "layer row count overflows the row width");
        if (!checked_mul(floats[i], h.elem_bytes(), &bytes_per_side))
            return inconsistent(err, "float count overflows the byte count");
        layers[i].keys_offset = r.at;
        if (!r.take(bytes_per_side)) return false;
        layers[i].values_offset = r.at;
        if (!r.take(bytes_per_side)) return false;
    }
    uint64_t stored = 0;
    if (!r.u64(&stored)) return false;
    if (r.remaining() != 0)
        return inconsistent(err, "%llu trailing bytes after the checksum", ULL(r.remaining()));
    const uint64_t computed = known_sum ? *known_sum : itkv_trailer(h.version, bytes, len - 8);
    if (stored != computed)
        return refuse(err, ITAK_KV_CHECKSUM_MISMATCH, stored, computed,
                      "snapshot checksum mismatch: stored 0x%016llx, computed 0x%016llx",
                      ULL(stored), ULL(computed));
    h.encoded_len = len;
    // Global layers ignore the window field on the wire; the in-memory kind carries none.
    for (ItkvLayer &l : layers)
        if (l.kind == ITAK_LAYER_GLOBAL) l.window = 0;
    return itkv_validate(h, layers.data(), layers.size(), floats.data(), floats.data(), err);
}

uint64_t itkv_header_len(const ItkvHeader &h) {
    return 4 + 4 + 4 + h.fingerprint_len + 8 + 4 + 4 + 4 + (h.version == kItkvVersionTyped ? 4 : 0) +
           h.layer_count * kItkvLayerHeaderLen;
}

bool itkv_encoded_len(const ItkvHeader &h, const ItkvLayer *layers, uint64_t *out) {
    uint64_t total = itkv_header_len(h), row = 0;
    if (!checked_mul(h.num_kv_heads, h.head_dim, &row)) return false;
    for (uint64_t i = 0; i < h.layer_count; ++i) {
        uint64_t floats = 0, bytes = 0;
        if (!checked_mul(layers[i].rows, row, &floats) ||
            !checked_mul(floats, 2 * h.elem_bytes(), &bytes) ||
            __builtin_add_overflow(total, bytes, &total))
            return false;
    }
    if (__builtin_add_overflow(total, uint64_t(8), &total)) return false;
    *out = total;
    return true;
}

void itkv_write_header(uint8_t *out, const ItkvHeader &h, const char *fingerprint,
                       ItkvLayer *layers) {
    uint8_t *p = out;
    memcpy(p, "ITKV", 4);
    p += 4;
    put_u32(p, h.version);
    put_u32(p, uint32_t(h.fingerprint_len));
    if (h.fingerprint_len) memcpy(p, fingerprint, h.fingerprint_len);
    p += h.fingerprint_len;
    put_u64(p, h.token_count);
    put_u32(p, uint32_t(h.num_kv_heads));
    put_u32(p, uint32_t(h.head_dim));
    put_u32(p, uint32_t(h.layer_count));
    if (h.version == kItkvVersionTyped) put_u32(p, h.elem);
    for (uint64_t i = 0; i < h.layer_count; ++i) {
        *p++ = layers[i].kind == ITAK_LAYER_GLOBAL ? 0 : 1;
        *p++ = 0;
        *p++ = 0;
        *p++ = 0;
        put_u64(p, layers[i].kind == ITAK_LAYER_GLOBAL ? 0 : layers[i].window);
        put_u64(p, layers[i].first_position);
        put_u64(p, layers[i].rows);
    }
    uint64_t at = uint64_t(p - out);
    const uint64_t row = h.num_kv_heads * h.head_dim;
    for (uint64_t i = 0; i < h.layer_count; ++i) {
        layers[i].keys_offset = at;
        at += layers[i].rows * row * h.elem_bytes();
        layers[i].values_offset = at;
        at += layers[i].rows * row * h.elem_bytes();
    }
}

}  // namespace itak
