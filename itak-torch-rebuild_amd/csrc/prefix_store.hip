// The persistent prefix store (crates/itak-kv/src/store.rs): one file per entry under a root
// directory, entries keyed by token prefix, the whole store bounded by a byte cap with LRU
// eviction. Host code; the byte layout of an entry, the trust checks of a lookup and the
// atomic write are the reference's, so either side reads what the other wrote.
//
// What differs is where a hit's snapshot lands: the reference decodes an entry into per-layer
// Vec<f32>s and installs those. Here a candidate's preamble and token ids are read first (a
// few KiB; a candidate on another branch of the prefix tree is dismissed without touching its
// payload, which can be gigabytes), and the payload of a matching candidate is read straight
// into one pinned host buffer that the store keeps. After verification the restore gathers
// the rows from that buffer in place over the host link (itak_kv_restore_itkv), so a hit costs
// one file read and one pass of the gather kernel, with no host copy in between.
#include "../../include/itak_hip_kv.h"

#include <dirent.h>
#include <errno.h>
#include <fcntl.h>
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#include <time.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <string>
#include <thread>
#include <vector>

#include "itkv.h"

using namespace itak;

namespace {

constexpr char kEntryMagic[9] = "ITKVPENT";    // store.rs:63
constexpr uint32_t kEntryFormatVersion = 1;    // store.rs:65
constexpr uint64_t kPreambleLen = 72;          // store.rs:67
constexpr uint64_t kLastUsedOffset = 24;       // store.rs:69
constexpr char kEntrySuffix[] = ".kv";         // store.rs:71
constexpr char kTempPrefix[] = ".tmp-";        // store.rs:73

#define ULL(x) static_cast<unsigned long long>(x)

struct StoreError {
    int32_t code = 0;
    std::string message;
    std::string what;
    uint64_t a = 0, b = 0;
};

struct Entry {  // store.rs:77-91
    std::string file_name;
    uint64_t prefix_hash = 0, token_count = 0, bytes = 0, created_unix = 0, last_used_unix = 0;
};

struct Preamble {  // store.rs:546-553
    uint64_t created_unix = 0, last_used_unix = 0, prefix_hash = 0, token_count = 0,
             payload_bytes = 0;
};

thread_local StoreError g_open_error;

}  // namespace

struct itak_store {
    std::string root;
    uint64_t max_bytes = 0;
    std::vector<Entry> entries;
    StoreError err;
    std::string refusals;  // what the reference writes to its diag channel, one line each
    // The last hit's payload. Pinned host memory when a device is there to read it in place.
    uint8_t *stage = nullptr;
    uint64_t stage_bytes = 0;
    bool stage_pinned = false;
    // What the decoder made of the payload in `stage` when the last candidate was verified.
    ItkvHeader stage_header;
    std::vector<ItkvLayer> stage_layers;
};

namespace {

itak_status fail(StoreError &e, int32_t code, const char *what, uint64_t a, uint64_t b,
                 const char *fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    e.code = code;
    e.message = buf;
    e.what = what ? what : "";
    e.a = a;
    e.b = b;
    return code;
}

// KvError::io (error.rs:127-133) with std::io::Error's Display text.
itak_status io_error(StoreError &e, int err, const char *fmt, ...) {
    char context[768];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(context, sizeof(context), fmt, ap);
    va_end(ap);
    return fail(e, ITAK_KV_IO, context, uint64_t(err), 0, "%s: %s (os error %d)", context,
                strerror(err), err);
}

itak_status from_itkv(StoreError &e, const ItkvError &err) {
    e.code = err.code;
    e.message = err.message;
    e.what = "snapshot";
    e.a = err.a;
    e.b = err.b;
    return err.code;
}

uint64_t get_u64(const uint8_t *p) {
    uint64_t v = 0;
    for (int i = 0; i < 8; ++i) v |= uint64_t(p[i]) << (8 * i);
    return v;
}
void put_u64(uint8_t *p, uint64_t v) {
    for (int i = 0; i < 8; ++i) p[i] = uint8_t(v >> (8 * i));
}

void encode_preamble(const Preamble &p, uint8_t out[kPreambleLen]) {  // store.rs:555-567
    memset(out, 0, kPreambleLen);
    memcpy(out, kEntryMagic, 8);
    out[8] = uint8_t(kEntryFormatVersion);
    put_u64(out + 16, p.created_unix);
    put_u64(out + 24, p.last_used_unix);
    put_u64(out + 32, p.prefix_hash);
    put_u64(out + 40, p.token_count);
    put_u64(out + 48, p.token_count * 4);
    put_u64(out + 56, p.payload_bytes);
}

itak_status parse_preamble(StoreError &e, const uint8_t *bytes, uint64_t len, Preamble &p) {  // store.rs:569-606
    if (len < kPreambleLen)
        return fail(e, ITAK_KV_TRUNCATED, "entry", kPreambleLen, len,
                    "entry: truncated, needs %llu bytes, has %llu", ULL(kPreambleLen), ULL(len));
    if (memcmp(bytes, kEntryMagic, 8) != 0)
        return fail(e, ITAK_KV_BAD_MAGIC, "entry", 0, 0, "entry: bad magic");
    const uint32_t version = uint32_t(bytes[8]) | uint32_t(bytes[9]) << 8 |
                             uint32_t(bytes[10]) << 16 | uint32_t(bytes[11]) << 24;
    if (version != kEntryFormatVersion)
        return fail(e, ITAK_KV_UNSUPPORTED_VERSION, "entry", version, 0,
                    "entry: unsupported format version %u", version);
    const uint64_t token_count = get_u64(bytes + 40), tokens_bytes = get_u64(bytes + 48);
    uint64_t expected = 0;
    if (__builtin_mul_overflow(token_count, uint64_t(4), &expected)) expected = UINT64_MAX;
    if (tokens_bytes != expected)
        return fail(e, ITAK_KV_INCONSISTENT_SNAPSHOT, "entry", 0, 0,
                    "inconsistent snapshot: entry tokens_bytes is %llu but token count %llu "
                    "implies %llu",
                    ULL(tokens_bytes), ULL(token_count), ULL(expected));
    p.created_unix = get_u64(bytes + 16);
    p.last_used_unix = get_u64(bytes + 24);
    p.prefix_hash = get_u64(bytes + 32);
    p.token_count = token_count;
    p.payload_bytes = get_u64(bytes + 56);
    return ITAK_OK;
}

std::string join(const std::string &root, const std::string &name) { return root + "/" + name; }

// Reads exactly `len` bytes at `offset`; returns the bytes read (short at end of file), or -1.
int64_t read_at(int fd, void *out, uint64_t len, uint64_t offset) {
    uint8_t *dst = static_cast<uint8_t *>(out);
    uint64_t done = 0;
    while (done < len) {
        const ssize_t n = pread(fd, dst + done, size_t(std::min<uint64_t>(len - done, 1u << 30)),
                                off_t(offset + done));
        if (n < 0) {
            if (errno == EINTR) continue;
            return -1;
        }
        if (n == 0) break;
        done += uint64_t(n);
    }
    return int64_t(done);
}

// Reads [offset, offset + len) of the file into `out` on a second thread while this one runs
// the byte-serial checksum over the first `sum_len` bytes behind it, so a large payload costs
// the slower of the two instead of their sum. Returns the bytes read (short at end of file),
// -1 with errno set on a read error.
int64_t read_at_with_checksum(int fd, uint8_t *out, uint64_t len, uint64_t offset, uint64_t sum_len,
                              uint64_t *sum) {
    constexpr uint64_t kPiece = 4u << 20;
    *sum = kFnvOffset;
    if (len <= 2 * kPiece) {
        const int64_t got = read_at(fd, out, len, offset);
        if (got >= 0) *sum = fnv1a64(out, std::min<uint64_t>(sum_len, uint64_t(got)), kFnvOffset);
        return got;
    }
    std::atomic<uint64_t> arrived{0};
    std::atomic<int> state{0};  // 0 reading, 1 done (possibly short), 2 failed
    int read_errno = 0;
    auto read_pieces = [&] {
        uint64_t done = 0;
        while (done < len) {
            const uint64_t want = std::min(kPiece, len - done);
            const int64_t got = read_at(fd, out + done, want, offset + done);
            if (got < 0) {
                read_errno = errno;
                state.store(2, std::memory_order_release);
                return;
            }
            done += uint64_t(got);
            arrived.store(done, std::memory_order_release);
            if (uint64_t(got) < want) break;
        }
        state.store(1, std::memory_order_release);
    };
    std::thread reader;
    try {
        reader = std::thread(read_pieces);
    } catch (...) {  // no thread to be had: read, then sum
        read_pieces();
    }
    uint64_t summed = 0, running = kFnvOffset;
    for (;;) {
        const int st = state.load(std::memory_order_acquire);
        const uint64_t have = std::min(arrived.load(std::memory_order_acquire), sum_len);
        if (have > summed) {
            running = fnv1a64(out + summed, have - summed, running);
            summed = have;
            continue;
        }
        if (st != 0) break;
        std::this_thread::yield();
    }
    if (reader.joinable()) reader.join();
    if (state.load() == 2) {
        errno = read_errno;
        return -1;
    }
    *sum = running;
    return int64_t(arrived.load());
}

// The same for a version 2 payload, whose trailer is a sum of block sums: host threads each
// read whole blocks of the file and sum what they read, so neither the copy out of the page
// cache nor the walk is serial.
int64_t read_blocks_with_checksum(int fd, uint8_t *out, uint64_t len, uint64_t offset,
                                  uint64_t sum_len, uint64_t *sum) {
    const uint64_t blocks = len / kItkvSumBlock + (len % kItkvSumBlock ? 1 : 0);
    const uint64_t summed_blocks = sum_len / kItkvSumBlock + (sum_len % kItkvSumBlock ? 1 : 0);
    std::vector<uint64_t> sums(summed_blocks);
    std::atomic<uint64_t> arrived{0};
    std::atomic<int> read_errno{0};
    // A thread reads a group of blocks and then walks them side by side (fnv1a64_block_group).
    const uint64_t groups = (blocks + kItkvSumGroup - 1) / kItkvSumGroup;
    for_each_index(groups, [&](uint64_t g) {
        const uint64_t first = g * kItkvSumGroup, n = std::min(kItkvSumGroup, blocks - first);
        const uint64_t at = first * kItkvSumBlock, want = std::min(n * kItkvSumBlock, len - at);
        const int64_t got = read_at(fd, out + at, want, offset + at);
        if (got < 0) {
            read_errno.store(errno ? errno : EIO, std::memory_order_relaxed);
            return;
        }
        arrived.fetch_add(uint64_t(got), std::memory_order_relaxed);
        // (A short read ends the file: the caller refuses it by its length, the sums are not used.)
        if (uint64_t(got) == want && first < summed_blocks)
            fnv1a64_block_group(out, sum_len, first, std::min(n, summed_blocks - first), sums.data());
    });
    if (read_errno.load()) {
        errno = read_errno.load();
        return -1;
    }
    *sum = fnv1a64_of_sums(sums.data(), summed_blocks);
    return int64_t(arrived.load());
}

bool write_all(int fd, const void *src, uint64_t len) {
    const uint8_t *p = static_cast<const uint8_t *>(src);
    uint64_t done = 0;
    while (done < len) {
        const ssize_t n = write(fd, p + done, size_t(std::min<uint64_t>(len - done, 1u << 30)));
        if (n < 0) {
            if (errno == EINTR) continue;
            return false;
        }
        done += uint64_t(n);
    }
    return true;
}

void refuse_entry(itak_store *s, const std::string &file_name, const StoreError &e) {
    s->refusals += "prefix store refuses entry " + file_name + ": " + e.message + "\n";
}

// Preamble of an entry file into index metadata (store.rs:609-632).
itak_status read_preamble(StoreError &e, const std::string &path, const std::string &file_name,
                          Entry &out) {
    const int fd = open(path.c_str(), O_RDONLY | O_CLOEXEC);
    if (fd < 0) return io_error(e, errno, "open %s", path.c_str());
    uint8_t head[kPreambleLen];
    const int64_t n = read_at(fd, head, kPreambleLen, 0);
    struct stat st {};
    const int stat_rc = fstat(fd, &st);
    const int stat_errno = errno;
    close(fd);
    if (n < 0) return io_error(e, errno, "read preamble of %s", path.c_str());
    if (uint64_t(n) < kPreambleLen)  // read_exact on a short file
        return fail(e, ITAK_KV_IO, "entry", 0, 0, "read preamble of %s: failed to fill whole buffer",
                    path.c_str());
    Preamble p;
    itak_status status = parse_preamble(e, head, kPreambleLen, p);
    if (status != ITAK_OK) return status;
    if (stat_rc != 0) return io_error(e, stat_errno, "stat %s", path.c_str());
    out.file_name = file_name;
    out.prefix_hash = p.prefix_hash;
    out.token_count = p.token_count;
    out.bytes = uint64_t(st.st_size);
    out.created_unix = p.created_unix;
    out.last_used_unix = p.last_used_unix;
    return ITAK_OK;
}

// An entry's stored token ids (store.rs:635-650). The token region is bounded by the file's
// real size before anything is allocated.
itak_status read_entry_tokens(StoreError &e, const std::string &path, std::vector<uint32_t> &out) {
    const int fd = open(path.c_str(), O_RDONLY | O_CLOEXEC);
    if (fd < 0) return io_error(e, errno, "read %s", path.c_str());
    struct stat st {};
    if (fstat(fd, &st) != 0) {
        const int err = errno;
        close(fd);
        return io_error(e, err, "read %s", path.c_str());
    }
    const uint64_t size = uint64_t(st.st_size);
    uint8_t head[kPreambleLen];
    const int64_t n = read_at(fd, head, std::min(size, kPreambleLen), 0);
    Preamble p;
    itak_status status = n < 0 ? io_error(e, errno, "read %s", path.c_str())
                               : parse_preamble(e, head, uint64_t(n), p);
    if (status == ITAK_OK) {
        uint64_t end = 0;
        if (__builtin_mul_overflow(p.token_count, uint64_t(4), &end) ||
            __builtin_add_overflow(end, kPreambleLen, &end) || size < end)
            status = fail(e, ITAK_KV_TRUNCATED, "entry", end, size,
                          "entry: truncated, needs %llu bytes, has %llu", ULL(end), ULL(size));
    }
    if (status == ITAK_OK) {
        out.resize(p.token_count);
        std::vector<uint8_t> raw(p.token_count * 4);
        if (read_at(fd, raw.data(), raw.size(), kPreambleLen) != int64_t(raw.size()))
            status = io_error(e, errno, "read %s", path.c_str());
        for (uint64_t i = 0; status == ITAK_OK && i < p.token_count; ++i)
            out[i] = uint32_t(raw[4 * i]) | uint32_t(raw[4 * i + 1]) << 8 |
                     uint32_t(raw[4 * i + 2]) << 16 | uint32_t(raw[4 * i + 3]) << 24;
    }
    close(fd);
    return status;
}

uint64_t total_bytes(const itak_store *s) {
    uint64_t sum = 0;
    for (const Entry &e : s->entries) sum += e.bytes;
    return sum;
}

itak_status rescan(itak_store *s, StoreError &e) {  // store.rs:204-224
    std::vector<Entry> entries;
    DIR *dir = opendir(s->root.c_str());
    if (!dir) return io_error(e, errno, "list store root %s", s->root.c_str());
    for (;;) {
        errno = 0;
        struct dirent *item = readdir(dir);
        if (!item) {
            if (errno != 0) {
                const int err = errno;
                closedir(dir);
                return io_error(e, err, "read store root entry");
            }
            break;
        }
        const std::string name = item->d_name;
        const size_t suffix = sizeof(kEntrySuffix) - 1, prefix = sizeof(kTempPrefix) - 1;
        if (name.compare(0, prefix, kTempPrefix) == 0 || name.size() < suffix ||
            name.compare(name.size() - suffix, suffix, kEntrySuffix) != 0)
            continue;
        Entry meta;
        StoreError why;
        if (read_preamble(why, join(s->root, name), name, meta) == ITAK_OK)
            entries.push_back(meta);
        else
            refuse_entry(s, name, why);
    }
    closedir(dir);
    s->entries.swap(entries);
    return ITAK_OK;
}

// create_dir_all.
int make_dirs(const std::string &path) {
    std::string partial;
    size_t at = 0;
    while (at <= path.size()) {
        const size_t next = path.find('/', at);
        partial = next == std::string::npos ? path : path.substr(0, next);
        at = next == std::string::npos ? path.size() + 1 : next + 1;
        if (partial.empty()) continue;
        if (mkdir(partial.c_str(), 0777) != 0 && errno != EEXIST) return errno;
    }
    struct stat st {};
    if (stat(path.c_str(), &st) != 0) return errno;
    return S_ISDIR(st.st_mode) ? 0 : ENOTDIR;
}

// The filename of a put (store.rs:458-503): hash-length-discriminator, with a counter suffix
// when another token list already owns the name.
itak_status pick_file_name(itak_store *s, const uint32_t *tokens, uint64_t count, uint64_t key,
                           std::string &out) {
    const uint64_t disc = fnv1a64_tokens(tokens, count, kFnvAltOffset);
    char base[96];
    snprintf(base, sizeof(base), "%016llx-%llu-%016llx", ULL(key), ULL(count), ULL(disc));
    for (uint32_t counter = 0; counter < 1024; ++counter) {
        char name[128];
        if (counter == 0)
            snprintf(name, sizeof(name), "%s%s", base, kEntrySuffix);
        else
            snprintf(name, sizeof(name), "%s-c%u%s", base, counter, kEntrySuffix);
        const std::string path = join(s->root, name);
        const bool indexed = std::any_of(s->entries.begin(), s->entries.end(),
                                         [&](const Entry &e) { return e.file_name == name; });
        struct stat st {};
        if (!indexed && stat(path.c_str(), &st) != 0) {
            out = name;
            return ITAK_OK;
        }
        std::vector<uint32_t> existing;
        StoreError ignored;
        if (read_entry_tokens(ignored, path, existing) != ITAK_OK) {
            if (indexed) continue;
            out = name;  // a stray unreadable file of that name is overwritten
            return ITAK_OK;
        }
        if (existing.size() == count &&
            (count == 0 || memcmp(existing.data(), tokens, count * 4) == 0)) {
            out = name;
            return ITAK_OK;
        }
    }
    return fail(s->err, ITAK_KV_INVALID_CONFIG, nullptr, key, 0,
                "invalid config: no free filename for prefix hash 0x%llx after 1024 collisions; the "
                "store directory is not behaving like a prefix store",
                ULL(key));
}

itak_status evict_except(itak_store *s, const std::string &keep) {  // store.rs:521-548
    while (total_bytes(s) > s->max_bytes) {
        const Entry *victim = nullptr;
        for (const Entry &e : s->entries) {
            if (e.file_name == keep) continue;
            if (!victim || e.last_used_unix < victim->last_used_unix ||
                (e.last_used_unix == victim->last_used_unix && e.file_name < victim->file_name))
                victim = &e;
        }
        if (!victim) break;  // only the kept entry remains, and it fits by construction
        const std::string name = victim->file_name;
        if (unlink(join(s->root, name).c_str()) != 0)
            return io_error(s->err, errno, "evict entry %s", name.c_str());
        s->entries.erase(std::remove_if(s->entries.begin(), s->entries.end(),
                                        [&](const Entry &e) { return e.file_name == name; }),
                         s->entries.end());
    }
    return ITAK_OK;
}

itak_status touch(itak_store *s, const std::string &file_name, uint64_t now) {  // store.rs:506-517
    const int fd = open(join(s->root, file_name).c_str(), O_WRONLY | O_CLOEXEC);
    if (fd < 0) return io_error(s->err, errno, "open entry %s to restamp", file_name.c_str());
    uint8_t stamp[8];
    put_u64(stamp, now);
    const ssize_t n = pwrite(fd, stamp, 8, off_t(kLastUsedOffset));
    const int err = errno;
    close(fd);
    if (n != 8) return io_error(s->err, err, "restamp entry %s", file_name.c_str());
    return ITAK_OK;
}

itak_status ensure_stage(itak_store *s, uint64_t bytes) {
    if (bytes <= s->stage_bytes) return ITAK_OK;
    if (s->stage) {
        if (s->stage_pinned)
            (void)hipHostFree(s->stage);
        else
            free(s->stage);
    }
    s->stage = nullptr;
    s->stage_bytes = 0;
    const uint64_t want = std::max<uint64_t>(bytes + bytes / 4, 1u << 16);
    void *p = nullptr;
    if (hipHostMalloc(&p, want, hipHostMallocDefault) == hipSuccess) {
        s->stage_pinned = true;
    } else {
        (void)hipGetLastError();  // no device: ordinary memory holds the bytes just as well
        p = malloc(want);
        s->stage_pinned = false;
        if (!p) return fail(s->err, ITAK_KV_IO, "stage", ENOMEM, 0, "allocate %llu bytes for an entry payload: %s (os error %d)", ULL(want), strerror(ENOMEM), ENOMEM);
    }
    s->stage = static_cast<uint8_t *>(p);
    s->stage_bytes = want;
    return ITAK_OK;
}

// Reads and fully verifies one candidate against the query (store.rs:364-452). *is_hit false
// with ITAK_OK means a well-formed entry on another branch of the prefix tree; a failure
// status means the entry failed a trust check (text in `why`).
itak_status verify_candidate(itak_store *s, StoreError &why, const Entry &meta,
                             const uint32_t *query, const itak_itkv_header *expected_geometry,
                             const itak_itkv_layer *expected_layers, const char *fingerprint,
                             uint64_t fingerprint_len, bool *is_hit, uint64_t *payload_len) {
    *is_hit = false;
    const std::string path = join(s->root, meta.file_name);
    const int fd = open(path.c_str(), O_RDONLY | O_CLOEXEC);
    if (fd < 0) return io_error(why, errno, "read entry %s", meta.file_name.c_str());
    struct Closer {
        int fd;
        ~Closer() { close(fd); }
    } closer{fd};
    struct stat st {};
    if (fstat(fd, &st) != 0) return io_error(why, errno, "read entry %s", meta.file_name.c_str());
    const uint64_t size = uint64_t(st.st_size);
    uint8_t head[kPreambleLen];
    const int64_t got = read_at(fd, head, std::min(size, kPreambleLen), 0);
    if (got < 0) return io_error(why, errno, "read entry %s", meta.file_name.c_str());
    Preamble p;
    itak_status status = parse_preamble(why, head, uint64_t(got), p);
    if (status != ITAK_OK) return status;
    if (p.prefix_hash != meta.prefix_hash || p.token_count != meta.token_count)
        return fail(why, ITAK_KV_INCONSISTENT_SNAPSHOT, "entry", 0, 0,
                    "inconsistent snapshot: entry %s changed between scan and read (index hash "
                    "0x%llx / %llu tokens, file hash 0x%llx / %llu tokens)",
                    meta.file_name.c_str(), ULL(meta.prefix_hash), ULL(meta.token_count),
                    ULL(p.prefix_hash), ULL(p.token_count));
    uint64_t tokens_end = 0;
    if (__builtin_mul_overflow(p.token_count, uint64_t(4), &tokens_end) ||
        __builtin_add_overflow(tokens_end, kPreambleLen, &tokens_end) || size < tokens_end)
        return fail(why, ITAK_KV_TRUNCATED, "entry", tokens_end, size,
                    "entry: truncated, needs %llu bytes, has %llu", ULL(tokens_end), ULL(size));
    std::vector<uint8_t> raw(p.token_count * 4);
    if (read_at(fd, raw.data(), raw.size(), kPreambleLen) != int64_t(raw.size()))
        return io_error(why, errno, "read entry %s", meta.file_name.c_str());
    // Trust check 1: the stored ids must hash back to the key. (The ids are little-endian on
    // disk, which is also the byte order the hash walks them in.)
    const uint64_t computed = fnv1a64(raw.data(), raw.size(), kFnvOffset);
    if (computed != p.prefix_hash)
        return fail(why, ITAK_KV_PREFIX_HASH_MISMATCH, nullptr, p.prefix_hash, computed,
                    "stored token ids hash to 0x%016llx, not the entry key 0x%016llx; entry refused",
                    ULL(computed), ULL(p.prefix_hash));
    // Prefix check: not an error, just not this query's branch.
    for (uint64_t i = 0; i < p.token_count; ++i) {
        const uint32_t t = uint32_t(raw[4 * i]) | uint32_t(raw[4 * i + 1]) << 8 |
                           uint32_t(raw[4 * i + 2]) << 16 | uint32_t(raw[4 * i + 3]) << 24;
        if (t != query[i]) return ITAK_OK;
    }
    // Trust check 2: the payload must decode whole and agree with the preamble.
    const uint64_t payload = size - tokens_end;
    if (payload != p.payload_bytes)
        return fail(why, ITAK_KV_TRUNCATED, "entry payload", p.payload_bytes, payload,
                    "entry payload: truncated, needs %llu bytes, has %llu", ULL(p.payload_bytes),
                    ULL(payload));
    status = ensure_stage(s, payload);
    if (status != ITAK_OK) {
        why = s->err;
        return status;
    }
    // Magic and version lead the payload (snapshot.rs:13-16); the version says how the trailer
    // is summed, and so how the bytes are best brought in. Anything the decoder will refuse
    // anyway takes the version 1 way.
    uint8_t lead[8] = {0};
    const bool typed = payload >= 8 && read_at(fd, lead, 8, tokens_end) == 8 &&
                       (uint32_t(lead[4]) | uint32_t(lead[5]) << 8 | uint32_t(lead[6]) << 16 |
                        uint32_t(lead[7]) << 24) == kItkvVersionTyped;
    uint64_t sum = 0;
    const uint64_t sum_len = payload >= 8 ? payload - 8 : 0;
    const int64_t arrived =
        typed ? read_blocks_with_checksum(fd, s->stage, payload, tokens_end, sum_len, &sum)
              : read_at_with_checksum(fd, s->stage, payload, tokens_end, sum_len, &sum);
    if (arrived < 0) return io_error(why, errno, "read entry %s", meta.file_name.c_str());
    if (uint64_t(arrived) != payload)  // the file shrank after it was measured
        return fail(why, ITAK_KV_TRUNCATED, "entry payload", payload, uint64_t(arrived),
                    "entry payload: truncated, needs %llu bytes, has %llu", ULL(payload),
                    ULL(uint64_t(arrived)));
    ItkvHeader &h = s->stage_header;
    std::vector<ItkvLayer> &layers = s->stage_layers;
    ItkvError decode_error;
    if (!itkv_decode(s->stage, payload, h, layers, decode_error, payload >= 8 ? &sum : nullptr))
        return from_itkv(why, decode_error);
    if (h.token_count != p.token_count)
        return fail(why, ITAK_KV_SNAPSHOT_TOKEN_MISMATCH, nullptr, p.token_count, h.token_count,
                    "entry preamble covers %llu tokens but its snapshot covers %llu",
                    ULL(p.token_count), ULL(h.token_count));
    // Trust check 3: caller-required geometry and fingerprint.
    if (expected_geometry) {
        bool same = h.layer_count == expected_geometry->layer_count &&
                    h.num_kv_heads == expected_geometry->num_kv_heads &&
                    h.head_dim == expected_geometry->head_dim;
        for (uint64_t i = 0; same && i < h.layer_count; ++i)
            same = layers[i].kind == expected_layers[i].kind &&
                   (layers[i].kind == ITAK_LAYER_GLOBAL || layers[i].window == expected_layers[i].window);
        if (!same)
            return fail(why, ITAK_KV_GEOMETRY_MISMATCH, nullptr, 0, 0,
                        "geometry mismatch: entry %s snapshot geometry differs from the required "
                        "geometry",
                        meta.file_name.c_str());
    }
    if (fingerprint &&
        (fingerprint_len != h.fingerprint_len ||
         memcmp(fingerprint, s->stage + h.fingerprint_offset, h.fingerprint_len) != 0))
        return fail(why, ITAK_KV_FINGERPRINT_MISMATCH, nullptr, 0, 0,
                    "model fingerprint mismatch: need %.*s, snapshot carries %.*s",
                    int(std::min<uint64_t>(fingerprint_len, 400)), fingerprint,
                    int(std::min<uint64_t>(h.fingerprint_len, 400)),
                    reinterpret_cast<const char *>(s->stage + h.fingerprint_offset));
    *is_hit = true;
    *payload_len = payload;
    return ITAK_OK;
}

}  // namespace

extern "C" {

uint64_t itak_kv_now_unix(void) {  // store.rs:120-126
    const time_t now = time(nullptr);
    return now < 0 ? 0 : uint64_t(now);
}

const char *itak_store_last_error(const itak_store *store) {
    return store ? store->err.message.c_str() : g_open_error.message.c_str();
}

itak_status itak_store_last_error_info(const itak_store *store, itak_error_info *out) {
    if (!out) return ITAK_INVALID_ARGUMENT;
    const StoreError &e = store ? store->err : g_open_error;
    memset(out, 0, sizeof(*out));
    out->code = e.code;
    snprintf(out->what, sizeof(out->what), "%s", e.what.c_str());
    out->a = e.a;
    out->b = e.b;
    return ITAK_OK;
}

itak_status itak_store_open(const char *root, uint64_t max_bytes, itak_store **out) {  // store.rs:147-168
    StoreError &e = g_open_error;
    if (!out) return fail(e, ITAK_INVALID_ARGUMENT, nullptr, 0, 0, "out is null");
    *out = nullptr;
    if (!root || !*root) return fail(e, ITAK_INVALID_ARGUMENT, nullptr, 0, 0, "root is null or empty");
    if (max_bytes == 0)
        return fail(e, ITAK_KV_INVALID_CONFIG, nullptr, 0, 0,
                    "invalid config: the store byte cap is zero");
    const int err = make_dirs(root);
    if (err != 0) return io_error(e, err, "create store root %s", root);
    itak_store *store = new itak_store();
    store->root = root;
    while (store->root.size() > 1 && store->root.back() == '/') store->root.pop_back();
    store->max_bytes = max_bytes;
    const itak_status status = rescan(store, e);
    if (status != ITAK_OK) {
        delete store;
        return status;
    }
    *out = store;
    return ITAK_OK;
}

void itak_store_close(itak_store *store) {
    if (!store) return;
    if (store->stage) {
        if (store->stage_pinned)
            (void)hipHostFree(store->stage);
        else
            free(store->stage);
    }
    delete store;
}

const char *itak_store_refusals(const itak_store *store) {
    return store ? store->refusals.c_str() : "";
}

void itak_store_clear_refusals(itak_store *store) {
    if (store) store->refusals.clear();
}

itak_status itak_store_rescan(itak_store *store) {
    if (!store) return ITAK_INVALID_ARGUMENT;
    return rescan(store, store->err);
}

itak_status itak_store_get_stats(itak_store *store, itak_store_stats *out) {  // store.rs:185-192
    if (!store) return ITAK_INVALID_ARGUMENT;
    if (!out) return fail(store->err, ITAK_INVALID_ARGUMENT, nullptr, 0, 0, "out is null");
    out->entries = store->entries.size();
    out->total_bytes = total_bytes(store);
    out->max_bytes = store->max_bytes;
    return ITAK_OK;
}

itak_status itak_store_entries(itak_store *store, itak_store_entry *out, uint64_t capacity,
                               uint64_t *count) {  // store.rs:177-182
    if (!store) return ITAK_INVALID_ARGUMENT;
    if (!count) return fail(store->err, ITAK_INVALID_ARGUMENT, nullptr, 0, 0, "count is null");
    *count = store->entries.size();
    if (!out) return ITAK_OK;
    if (capacity < store->entries.size())
        return fail(store->err, ITAK_INVALID_ARGUMENT, nullptr, 0, 0,
                    "entry array is smaller than the index");
    std::vector<const Entry *> order;
    for (const Entry &e : store->entries) order.push_back(&e);
    std::stable_sort(order.begin(), order.end(),
                     [](const Entry *a, const Entry *b) { return a->token_count > b->token_count; });
    for (size_t i = 0; i < order.size(); ++i) {
        memset(&out[i], 0, sizeof(out[i]));
        snprintf(out[i].file_name, sizeof(out[i].file_name), "%s", order[i]->file_name.c_str());
        out[i].prefix_hash = order[i]->prefix_hash;
        out[i].token_count = order[i]->token_count;
        out[i].bytes = order[i]->bytes;
        out[i].created_unix = order[i]->created_unix;
        out[i].last_used_unix = order[i]->last_used_unix;
    }
    return ITAK_OK;
}

// store.rs:236-300. `own_capture` says the bytes were written a moment ago by this library's
// own capture into the store's buffer with the trailer still to come: the strict decode below
// checks the structure only, and the byte-serial checksum (~1 GB/s) then runs once, on a second
// thread, while this one writes the file.
static itak_status put_entry(itak_store *store, const uint32_t *tokens, uint64_t token_count,
                             void *snapshot, uint64_t snapshot_len, uint64_t now,
                             bool own_capture) {
    StoreError &e = store->err;
    if (token_count == 0) return fail(e, ITAK_KV_EMPTY_PREFIX, nullptr, 0, 0, "empty token prefix refused");
    if (!tokens || !snapshot) return fail(e, ITAK_INVALID_ARGUMENT, nullptr, 0, 0, "tokens or snapshot is null");
    // The reference is handed a KvSnapshot and encodes it (which validates it); here the
    // caller brings the encoding, so it is decoded strictly instead: same refusals.
    ItkvHeader h;
    std::vector<ItkvLayer> layers;
    ItkvError decode_error;
    uint8_t *payload = static_cast<uint8_t *>(snapshot);
    uint64_t trailer = 0;
    if (own_capture && snapshot_len >= 8)
        for (int b = 0; b < 8; ++b) trailer |= uint64_t(payload[snapshot_len - 8 + b]) << (8 * b);
    if (!itkv_decode(payload, snapshot_len, h, layers, decode_error,
                     own_capture && snapshot_len >= 8 ? &trailer : nullptr))
        return from_itkv(e, decode_error);
    if (h.token_count != token_count)
        return fail(e, ITAK_KV_TOKEN_COUNT_MISMATCH, nullptr, h.token_count, token_count,
                    "snapshot covers %llu tokens but was offered under %llu token ids",
                    ULL(h.token_count), ULL(token_count));
    const uint64_t key = fnv1a64_tokens(tokens, token_count, kFnvOffset);
    uint64_t entry_bytes = 0;
    if (__builtin_mul_overflow(token_count, uint64_t(4), &entry_bytes) ||
        __builtin_add_overflow(entry_bytes, kPreambleLen, &entry_bytes) ||
        __builtin_add_overflow(entry_bytes, snapshot_len, &entry_bytes))
        entry_bytes = UINT64_MAX;
    if (entry_bytes > store->max_bytes)
        return fail(e, ITAK_KV_ENTRY_TOO_LARGE, nullptr, entry_bytes, store->max_bytes,
                    "entry of %llu bytes exceeds the store cap of %llu bytes", ULL(entry_bytes),
                    ULL(store->max_bytes));
    std::string file_name;
    itak_status status = pick_file_name(store, tokens, token_count, key, file_name);
    if (status != ITAK_OK) return status;
    // Atomic write: temp file in the same directory, sync, rename over the final name.
    char temp_name[192];
    snprintf(temp_name, sizeof(temp_name), "%s%s-%ld", kTempPrefix, file_name.c_str(), long(getpid()));
    const std::string temp_path = join(store->root, temp_name), path = join(store->root, file_name);
    const int fd = open(temp_path.c_str(), O_WRONLY | O_CREAT | O_TRUNC | O_CLOEXEC, 0666);
    if (fd < 0) return io_error(e, errno, "create temp entry %s", temp_name);
    Preamble p;
    p.created_unix = p.last_used_unix = now;
    p.prefix_hash = key;
    p.token_count = token_count;
    p.payload_bytes = snapshot_len;
    uint8_t head[kPreambleLen];
    encode_preamble(p, head);
    std::vector<uint8_t> ids(token_count * 4);
    for (uint64_t i = 0; i < token_count; ++i)
        for (int b = 0; b < 4; ++b) ids[4 * i + b] = uint8_t(tokens[i] >> (8 * b));
    const bool sum_here = own_capture && snapshot_len >= 8;
    const uint64_t body_len = sum_here ? snapshot_len - 8 : snapshot_len;
    uint64_t sum = 0;
    std::thread summer;
    bool summed = false;
    if (sum_here) {
        try {
            summer = std::thread([&] { sum = itkv_trailer(h.version, payload, body_len); });
        } catch (...) {  // no thread to be had: the checksum runs here, before the write
            sum = itkv_trailer(h.version, payload, body_len);
            summed = true;
        }
    }
    bool written = write_all(fd, head, kPreambleLen) && write_all(fd, ids.data(), ids.size()) &&
                   write_all(fd, payload, body_len);
    int write_errno = errno;
    if (sum_here) {
        if (!summed) summer.join();
        for (int b = 0; b < 8; ++b) payload[body_len + b] = uint8_t(sum >> (8 * b));
        if (written) {
            written = write_all(fd, payload + body_len, 8);
            write_errno = errno;
        }
    }
    if (written && fsync(fd) != 0) {
        written = false;
        write_errno = errno;
    }
    close(fd);
    if (!written) {
        (void)unlink(temp_path.c_str());
        return io_error(e, write_errno, "write temp entry %s", temp_name);
    }
    if (rename(temp_path.c_str(), path.c_str()) != 0) {
        const int err = errno;
        (void)unlink(temp_path.c_str());
        return io_error(e, err, "rename entry %s", file_name.c_str());
    }
    store->entries.erase(std::remove_if(store->entries.begin(), store->entries.end(),
                                        [&](const Entry &x) { return x.file_name == file_name; }),
                         store->entries.end());
    Entry meta;
    meta.file_name = file_name;
    meta.prefix_hash = key;
    meta.token_count = token_count;
    meta.bytes = entry_bytes;
    meta.created_unix = meta.last_used_unix = now;
    store->entries.push_back(meta);
    return evict_except(store, file_name);
}

itak_status itak_store_put(itak_store *store, const uint32_t *tokens, uint64_t token_count,
                           const void *snapshot, uint64_t snapshot_len, uint64_t now) {
    if (!store) return ITAK_INVALID_ARGUMENT;
    return put_entry(store, tokens, token_count, const_cast<void *>(snapshot), snapshot_len, now, false);
}

itak_status itak_store_lookup(itak_store *store, const uint32_t *query, uint64_t query_len,
                              const itak_itkv_header *expected_geometry,
                              const itak_itkv_layer *expected_layers, const char *fingerprint,
                              uint64_t fingerprint_len, uint64_t now, itak_prefix_hit *hit) {  // store.rs:314-357
    if (!store) return ITAK_INVALID_ARGUMENT;
    if (!hit) return fail(store->err, ITAK_INVALID_ARGUMENT, nullptr, 0, 0, "hit is null");
    memset(hit, 0, sizeof(*hit));
    if (query_len && !query) return fail(store->err, ITAK_INVALID_ARGUMENT, nullptr, 0, 0, "query is null");
    if (expected_geometry && expected_geometry->layer_count && !expected_layers)
        return fail(store->err, ITAK_INVALID_ARGUMENT, nullptr, 0, 0, "expected_layers is null");
    std::vector<Entry> candidates;
    for (const Entry &e : store->entries)
        if (e.token_count <= query_len) candidates.push_back(e);
    std::stable_sort(candidates.begin(), candidates.end(),
                     [](const Entry &a, const Entry &b) { return a.token_count > b.token_count; });
    for (const Entry &candidate : candidates) {
        StoreError why;
        bool is_hit = false;
        uint64_t payload_len = 0;
        const itak_status status =
            verify_candidate(store, why, candidate, query, expected_geometry, expected_layers,
                             fingerprint, fingerprint_len, &is_hit, &payload_len);
        if (status != ITAK_OK) {
            refuse_entry(store, candidate.file_name, why);
            continue;
        }
        if (!is_hit) continue;
        const itak_status touched = touch(store, candidate.file_name, now);
        if (touched != ITAK_OK) return touched;
        for (Entry &e : store->entries)
            if (e.file_name == candidate.file_name) e.last_used_unix = now;
        hit->token_count = candidate.token_count;
        hit->snapshot = store->stage;
        hit->snapshot_len = payload_len;
        snprintf(hit->file_name, sizeof(hit->file_name), "%s", candidate.file_name.c_str());
        return ITAK_OK;
    }
    return ITAK_OK;
}

// The read half of the session flow (crates/wgpu-compute/src/session.rs:5000-5053): the
// longest stored prefix of `tokens` that matches the pool's pattern and the fingerprint goes
// into the slot. Anything short of a device failure leaves the slot as it was and reports
// *matched = 0 (the caller prefills cold), with the reason in the refusal log.
itak_status itak_store_restore_prefix(itak_store *store, itak_pool *pool, uint32_t slot,
                                      const uint32_t *tokens, uint64_t token_count,
                                      const char *fingerprint, uint64_t fingerprint_len,
                                      uint64_t now, uint64_t *matched) {
    if (!store || !pool) return ITAK_INVALID_ARGUMENT;
    if (!matched) return fail(store->err, ITAK_INVALID_ARGUMENT, nullptr, 0, 0, "matched is null");
    *matched = 0;
    const uint64_t layer_count = itak_kv_layer_count(pool);
    for (uint64_t layer = 0; layer < layer_count; ++layer) {
        uint64_t position = 0;
        const itak_status status = itak_kv_next_position(pool, slot, layer, &position);
        if (status != ITAK_OK)
            return fail(store->err, status, nullptr, 0, 0, "%s", itak_last_error(pool));
        if (position != 0) {
            char line[200];
            snprintf(line, sizeof(line),
                     "prefix restore skipped: session position is %llu, not 0; a restore is a "
                     "session-start act and the live sequence is left alone\n",
                     ULL(position));
            store->refusals += line;
            return ITAK_OK;
        }
    }
    itak_itkv_header geometry{};
    geometry.num_kv_heads = itak_kv_num_kv_heads(pool);
    geometry.head_dim = itak_kv_head_dim(pool);
    geometry.layer_count = layer_count;
    std::vector<itak_itkv_layer> layers(layer_count);
    for (uint64_t layer = 0; layer < layer_count; ++layer) {
        memset(&layers[layer], 0, sizeof(itak_itkv_layer));
        (void)itak_kv_layer_kind(pool, layer, &layers[layer].kind, &layers[layer].window);
    }
    itak_prefix_hit hit{};
    itak_status status = itak_store_lookup(store, tokens, token_count, &geometry, layers.data(),
                                           fingerprint, fingerprint_len, now, &hit);
    if (status != ITAK_OK) {
        store->refusals += "prefix restore skipped: store lookup refused: " + store->err.message +
                           "; cold prefill serves\n";
        return ITAK_OK;
    }
    if (hit.token_count == 0) return ITAK_OK;
    // The hit's bytes lie verified in the store's own buffer: install from there without
    // walking the checksum a second time.
    status = restore_decoded_itkv(pool, slot, store->stage, store->stage_header, store->stage_layers,
                                  fingerprint, fingerprint_len);
    if (status == ITAK_HIP_ERROR)
        return fail(store->err, status, "prefix_restore", 0, 0, "%s", itak_last_error(pool));
    if (status != ITAK_OK) {
        store->refusals += std::string("prefix restore skipped: the store hit fails install "
                                       "validation: ") +
                           itak_last_error(pool) + "; cold prefill serves\n";
        return ITAK_OK;
    }
    *matched = hit.token_count;
    return ITAK_OK;
}

// The write half (session.rs:5056-5094): the slot's rows, captured as ITKV v1, stored under
// the tokens they were computed from.
itak_status itak_store_capture_and_put(itak_store *store, itak_pool *pool, uint32_t slot,
                                       const uint32_t *tokens, uint64_t token_count,
                                       const char *fingerprint, uint64_t fingerprint_len,
                                       uint32_t elem, uint64_t now) {
    if (!store || !pool) return ITAK_INVALID_ARGUMENT;
    if (elem != ITAK_ELEM_F32 && elem != ITAK_ELEM_F16)
        return fail(store->err, ITAK_INVALID_ARGUMENT, nullptr, elem, 0,
                    "elem is neither ITAK_ELEM_F32 nor ITAK_ELEM_F16");
    // f32 rows are the reference's version 1; f16 rows this library's version 2.
    auto capture = elem == ITAK_ELEM_F16 ? itak_kv_capture_itkv_f16 : itak_kv_capture_itkv;
    uint64_t position = 0;
    itak_status status = itak_kv_next_position(pool, slot, 0, &position);
    if (status != ITAK_OK) return fail(store->err, status, nullptr, 0, 0, "%s", itak_last_error(pool));
    if (position != token_count)
        return fail(store->err, ITAK_STEP_FAILED, "prefix_store", position, token_count,
                    "session position %llu does not equal the %llu tokens to store under; a "
                    "snapshot covers exactly the forwarded prefix, so any other token list would "
                    "file one sequence's KV under another's key",
                    ULL(position), ULL(token_count));
    uint64_t bytes = 0;
    status = capture(pool, slot, fingerprint, fingerprint_len, nullptr, 0, &bytes);
    if (status == ITAK_OK) status = ensure_stage(store, bytes) == ITAK_OK ? ITAK_OK : store->err.code;
    if (status == ITAK_OK)  // the trailer is left for put_entry, which sums while it writes
        status = capture_itkv_unsummed(pool, slot, fingerprint, fingerprint_len,
                                       elem == ITAK_ELEM_F16, store->stage, store->stage_bytes, &bytes);
    if (status != ITAK_OK) {
        if (store->err.code != status)
            return fail(store->err, status, "prefix_store", 0, 0, "%s", itak_last_error(pool));
        return status;
    }
    return put_entry(store, tokens, token_count, store->stage, bytes, now, true);
}

}  // extern "C"
