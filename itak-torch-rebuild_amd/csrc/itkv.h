// The ITKV snapshot wire format (v1: crates/itak-kv/src/snapshot.rs:13-29; v2: the same with
// an element-type word after the layer count and rows of that type, see kItkvVersionF16) and
// the FNV-1a hashes of crates/itak-kv/src/hash.rs, host side. Nothing here touches the device: the
// format fixes a byte-serial checksum over the whole file, so encoding and decoding are
// host work; the rows themselves move between the encoded buffer and the device planes
// through the gather / readback kernels.
#pragma once

#include <stdint.h>

#include <algorithm>
#include <atomic>
#include <string>
#include <thread>
#include <vector>

struct itak_pool;

namespace itak {

constexpr uint64_t kFnvOffset = 0xcbf29ce484222325ull;     // hash.rs:14
constexpr uint64_t kFnvPrime = 0x00000100000001b3ull;      // hash.rs:16
constexpr uint64_t kFnvAltOffset = 0x84222325cbf29ce4ull;  // hash.rs:21
constexpr uint32_t kItkvVersion = 1;                       // snapshot.rs:53
// Version 2 is this library's own: v1 "carries no storage-format field; its rows are f32 by
// definition" (bench/prefix-f16-guard-2026-11-07.md:46-70 names a format field in a later
// version as the way to snapshots of f16 caches). v2 differs from v1 in two places: one more
// u32 after the layer count, the element type of the rows (0 = f32, 1 = f16 bits), with the
// rows in that type; and the trailer, which is FNV-1a over the FNV-1a sums of consecutive
// 1 MiB blocks of the bytes before it (fnv1a64_blocks) instead of over the bytes themselves,
// so that host threads can share the walk. A v1 reader refuses it by name (UnsupportedVersion),
// never misreads it.
constexpr uint32_t kItkvVersionTyped = 2;
constexpr uint64_t kItkvSumBlock = 1u << 20;
constexpr uint64_t kItkvLayerHeaderLen = 28;               // snapshot.rs:51

uint64_t fnv1a64(const uint8_t *bytes, uint64_t count, uint64_t basis);           // hash.rs:24-31
uint64_t fnv1a64_tokens(const uint32_t *tokens, uint64_t count, uint64_t basis);  // hash.rs:35-41

// Host threads this library may use for one call (the caller's included): 8, or what the
// ITAK_HOST_THREADS environment variable says (1..64), never more than the machine has.
unsigned host_threads();

// f(k) for every k in [0, count), shared among host_threads() threads; returns when all are
// done. f must not throw.
template <class F>
void for_each_index(uint64_t count, F f) {
    std::atomic<uint64_t> next{0};
    auto work = [&] {
        for (uint64_t k; (k = next.fetch_add(1, std::memory_order_relaxed)) < count;) f(k);
    };
    std::vector<std::thread> helpers;
    const uint64_t want = std::min<uint64_t>(host_threads(), count);
    for (uint64_t i = 1; i < want; ++i) {
        try {
            helpers.emplace_back(work);
        } catch (...) {  // no more threads to be had: the ones there share the rest
            break;
        }
    }
    work();
    for (std::thread &t : helpers) t.join();
}

// Version 2's trailer. sums[k] = FNV-1a of block k (kItkvSumBlock bytes, the last one shorter);
// the result is FNV-1a over the sums written little-endian one after another. No bytes: the
// offset basis. fnv1a64_of_sums is the second half alone, for a caller that made the block
// sums itself.
uint64_t fnv1a64_blocks(const uint8_t *bytes, uint64_t count);
uint64_t fnv1a64_of_sums(const uint64_t *sums, uint64_t blocks);
// Block sums of blocks [first, first + n) of `count` bytes, n <= kItkvSumGroup, into sums[first..].
// A sum is a chain of one multiply per byte, each waiting for the last: one thread walks up to
// four blocks side by side, four chains in the multiplier at once (0.7 -> 2.7 GB/s a thread).
constexpr uint64_t kItkvSumGroup = 4;
void fnv1a64_block_group(const uint8_t *bytes, uint64_t count, uint64_t first, uint64_t n, uint64_t *sums);
// The trailer a snapshot of `version` carries for the `count` bytes before it.
inline uint64_t itkv_trailer(uint32_t version, const uint8_t *bytes, uint64_t count) {
    return version == kItkvVersionTyped ? fnv1a64_blocks(bytes, count) : fnv1a64(bytes, count, kFnvOffset);
}

// A refusal of itak_kv::KvError (crates/itak-kv/src/error.rs:13-124); `message` is its
// Display text (error.rs:141-188).
struct ItkvError {
    int32_t code = 0;
    std::string message;
    uint64_t a = 0, b = 0;  // the variant's integers, in declaration order
};

struct ItkvLayer {
    uint32_t kind = 0;  // 0 global, 1 windowed
    uint64_t window = 0;
    uint64_t first_position = 0;
    uint64_t rows = 0;
    uint64_t keys_offset = 0;    // byte offsets into the encoded buffer
    uint64_t values_offset = 0;
};

struct ItkvHeader {
    uint64_t token_count = 0;
    uint64_t num_kv_heads = 0;
    uint64_t head_dim = 0;
    uint64_t layer_count = 0;
    uint64_t fingerprint_len = 0;
    uint64_t fingerprint_offset = 0;
    uint64_t encoded_len = 0;
    uint32_t version = kItkvVersion;
    uint32_t elem = 0;  // 0 = f32 rows, 1 = f16 rows (version 2 only)
    uint64_t elem_bytes() const { return elem ? 2 : 4; }
};

// KvSnapshot::validate (snapshot.rs:187-236). `blocks` is the number of layer blocks the
// snapshot carries (layers.len()); key_floats / value_floats their lengths.
bool itkv_validate(const ItkvHeader &h, const ItkvLayer *layers, uint64_t blocks,
                   const uint64_t *key_floats, const uint64_t *value_floats, ItkvError &err);

// KvSnapshot::from_bytes (snapshot.rs:405-509): strict; fills offsets instead of copying rows.
// `known_sum`, when given, is the checksum of bytes[0, len-8) the caller already computed (while
// the bytes were still arriving, say); the decoder then compares instead of walking them again.
bool itkv_decode(const uint8_t *bytes, uint64_t len, ItkvHeader &h, std::vector<ItkvLayer> &layers,
                 ItkvError &err, const uint64_t *known_sum = nullptr);

// Bytes of everything before the row payload, and of the whole encoding (payload and the
// trailing checksum included), for a header whose layers carry `rows` rows each.
uint64_t itkv_header_len(const ItkvHeader &h);
bool itkv_encoded_len(const ItkvHeader &h, const ItkvLayer *layers, uint64_t *out);
// Writes magic .. layer headers (snapshot.rs:383-403) and fills the payload offsets.
void itkv_write_header(uint8_t *out, const ItkvHeader &h, const char *fingerprint,
                       ItkvLayer *layers);

// Installs an encoding that itkv_decode has already accepted into a fresh slot: `h` and
// `layers` are the decoder's outputs for `bytes`. The geometry and fingerprint checks of
// restore_checked (snapshot.rs:351-371) run; the bytes are not walked a second time. For the
// prefix store, which verifies an entry in its own private buffer and installs from there.
int32_t restore_decoded_itkv(itak_pool *pool, uint32_t slot, const uint8_t *bytes,
                             const ItkvHeader &h, const std::vector<ItkvLayer> &layers,
                             const char *expected_fingerprint, uint64_t expected_fingerprint_len);

// itak_kv_capture_itkv / itak_kv_capture_itkv_f16 with the 8 trailer bytes left zero: for a
// caller that runs the byte-serial checksum itself while it does something else with the bytes
// (the prefix store writes them to disk meanwhile).
int32_t capture_itkv_unsummed(itak_pool *pool, uint32_t slot, const char *fingerprint,
                              uint64_t fingerprint_len, bool f16_rows, void *out, uint64_t capacity,
                              uint64_t *written);

}  // namespace itak
