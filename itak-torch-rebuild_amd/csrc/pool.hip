// Host side of the C ABI: the pool, its slots, the per-slot bookkeeping that mirrors
// attention::KvCache (crates/attention/src/cache.rs) and cpu_compute::CpuCompute
// (crates/cpu-compute/src/cpu.rs), and the launch logic for the kernels in this directory.
// All validation happens here, in the reference's order, before anything is enqueued.
#include "../../include/itak_hip_kv.h"
#include "internal.h"
#include "itkv.h"

#include <algorithm>
#include <atomic>
#include <mutex>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <ctime>
#include <string>
#include <vector>

using namespace itak;

// Split workspace of itak_attention_step_device_noalloc: see the notes at g_scratch_of_device.
// Host code never passes this name to a kernel or a memory call: it is a host-side handle,
// the device address comes from hipGetSymbolAddress.
static __device__ __align__(256) unsigned char scratch[16ull << 20];

namespace {

// One windowed layer's rows set aside by a checkpoint whose round is longer than the ring's
// headroom (the saved slots of cache.rs:678-697): `rows` positions from the layer's base on.
struct RingSave {
    uint32_t layer = 0;      // pool layer
    uint32_t rows = 0;
    uint64_t saved_off = 0;  // elements into the slot's side buffer
    uint64_t high0 = 0;      // the layer's high-water mark when the checkpoint was taken
};

struct LiveCheckpoint {
    bool live = false;
    uint64_t serial = 0;
    uint64_t max_round_tokens = 0;
    std::vector<uint64_t> bases;
    std::vector<RingSave> ring_saves;  // empty when the headroom covers the round
};

struct Slot {
    bool in_use = false;
    bool built = false;  // CpuCompute's KvState exists (cpu.rs:560-564)
    uint64_t cache_id = 0;
    uint64_t next_serial = 0;
    std::vector<uint64_t> appended;  // per layer: positions appended == next position
    // Per layer: one past the highest position ever written into the storage since it was
    // last fresh. Positions in [appended, high) were dropped by a rewind; on a windowed layer
    // their rows still sit in the ring and alias the positions one ring length below them.
    std::vector<uint64_t> high;
    // Per layer: the oldest position the storage was ever given. 0 for a sequence appended
    // from its start; the first restored position of a windowed layer filled from a snapshot,
    // which carries only the last `window` rows: nothing below it can come back into view.
    std::vector<uint64_t> floor;
    LiveCheckpoint cp;
};

// One layer of the pattern (attention::LayerKind, cache.rs:36-48) and where it lives.
struct LayerInfo {
    bool windowed = false;
    uint32_t index = 0;   // among the layers of its kind, which are stored together
    uint64_t window = 0;  // attention window; 0 on a global layer
    uint32_t ring = 0;    // storage rows of the ring (a multiple of 32); 0 on a global layer
};

struct ErrorState {
    std::string message;
    itak_error_info info{};
};

thread_local ErrorState g_create_error;

// ---- the split workspace of the allocation-free entry point --------------------------------
// itak_attention_step_device_noalloc may not allocate, so its split workspace is this array:
// every device the library runs on holds a copy until the process ends. The first part holds
// exchange words for launches that merge their own splits (all empty between launches, like
// the pool's own exchange buffer); the rest takes the partials of launches that leave the
// merge to a second launch. In host code the array's name is only a handle: the address the
// kernels get is looked up once per device (bind_scratch) and kept here.
constexpr uint64_t kScratchBytes = sizeof(scratch);
constexpr uint64_t kScratchExchangeBytes = 8ull << 20;
constexpr int kMaxDevices = 64;
unsigned char *g_scratch_of_device[kMaxDevices];
std::mutex g_scratch_mutex;
// Every pool and stream of a device shares the device's copy of the array. Eager calls are kept
// apart by an event (made with the address, at set-up): recorded behind every allocation-free
// step on the stream it ran on, and waited for, on the device, by the next such step when that
// one runs on another stream. Calls made while their stream is being captured into a graph are
// outside this guard: nothing runs at the call, and when the replays run is the caller's matter.
struct ScratchGuard {
    hipEvent_t done = nullptr;     // behind the last eager allocation-free step of the device
    hipStream_t stream = nullptr;  // the stream that step ran on
    bool recorded = false;
};
ScratchGuard g_scratch_guard[kMaxDevices];
std::atomic<uint64_t> g_next_cache_id{1};  // cache.rs:32

}  // namespace

// rope_base^(-2i/rotary_dim), i < rotary_dim/2, computed on the host and kept on the device.
struct RopeFreqTable {
    float base;
    uint32_t rotary;
    double *dev;
};

struct itak_pool {
    itak_pool_config cfg{};
    std::vector<RopeFreqTable> rope_tables;
    // Global layers and windowed layers are two groups of planes with their own row capacity:
    // `g` (capacity_rows per plane) and `gw` (the longest ring per plane). Within a group the
    // layers are consecutive, so the kernels that walk several layers take (group base,
    // group geometry, index within the group).
    PoolGeom g{};
    PoolGeom gw{};
    std::vector<LayerInfo> layers;
    uint32_t global_layers = 0, windowed_layers = 0;
    // Rows a windowed layer's ring holds beyond its window: the longest block one step may
    // append there and the deepest rewind (crates/wgpu-compute/src/session.rs:235-249,
    // 5376-5428 give the algebra).
    uint64_t headroom = 0;
    int elem_f16 = 0;
    uint32_t elem_bytes = 4;
    uint64_t row = 0;         // kv_heads * head_dim
    uint64_t rows_limit = 0;  // positions a slot may hold on a global layer (the configured capacity)
    unsigned char *base = nullptr;    // global layers
    unsigned char *base_w = nullptr;  // windowed layers (inside the same allocation)
    uint64_t bytes = 0;
    hipStream_t stream = nullptr;
    std::vector<Slot> slots;
    // Device scratch, grown on demand and reused: staging for host-pointer calls and
    // split partials.
    unsigned char *stage = nullptr;
    uint64_t stage_bytes = 0;
    float *ws = nullptr;
    uint64_t ws_floats = 0;
    float *prep = nullptr;  // prepared Q and K rows of a prep step
    uint64_t prep_floats = 0;
    // Exchange buffer of split-K launches that merge their splits themselves: 64-bit words,
    // every one holding the empty pattern whenever no such launch is running; word 0 counts
    // the consumers that gave up waiting (checked by itak_pool_synchronize).
    unsigned long long *xws = nullptr;
    uint64_t xws_words = 0;
    uint32_t spin_limit = 1u << 17;  // looks at the buffer a consumer makes before it gives up
    // This device's copy of the static split workspace, and whether the call in progress must
    // use it instead of the pool's own buffers (itak_attention_step_device_noalloc).
    unsigned char *scratch_dev = nullptr;
    bool no_alloc_call = false;
    bool scratch_exchange_used = false;  // its give-up counter is then looked at too
    bool merge_in_launch = false;
    // ITAK_POOL_DIE_MERGE: split-K launches whose units deal out evenly over the compute dies
    // merge each unit's splits on its die (attn_splitk_f16_die.hip): one ticket word per unit, then the count of
    // workgroups that found themselves on another die than planned.
    bool die_merge = false;
    uint32_t *die_words = nullptr;
    bool q_two_halves = false;  // ITAK_POOL_Q_TWO_HALVES
    bool prep_by_launch = false;  // ITAK_POOL_PREP_BY_LAUNCH
    // Per slot: the side buffer of a deep checkpoint's ring rows, kept for the next one
    // (cache.rs:620-625: allocated once per cache, not once per round).
    std::vector<void *> ring_saved;
    std::vector<uint64_t> ring_saved_bytes;
    // Pinned host memory for the host-pointer attention call: its small inputs are packed here
    // and go up in one copy; its kernels write the output here directly.
    unsigned char *hstage = nullptr;
    uint64_t hstage_bytes = 0;
    uint32_t call_number = 0;  // what the last host-pointer call asked to be told when done
    mutable ErrorState err;
};

namespace {

// ------------------------------------------------------------------------------ debug channel
// attention::diag (crates/attention/src/diag.rs:13-33,71-79): off by default; the switch or
// ITAK_HIP_KV_DEBUG in the environment (any value but "0" or empty, looked up at every event as
// the reference looks its variable up) turns one stderr line per event on.
std::atomic<bool> g_debug_enabled{false};

bool diag_enabled() {
    if (g_debug_enabled.load(std::memory_order_relaxed)) return true;
    const char *v = getenv("ITAK_HIP_KV_DEBUG");
    return v && v[0] != '\0' && !(v[0] == '0' && v[1] == '\0');
}

__attribute__((format(printf, 1, 2))) void diag_emit(const char *fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    fprintf(stderr, "[itak_hip_kv::diag] %s\n", buf);
}

#define ITAK_DIAG(...)                          \
    do {                                        \
        if (diag_enabled()) diag_emit(__VA_ARGS__); \
    } while (0)

// ------------------------------------------------------------------------------ errors

itak_status set_error(ErrorState &e, int32_t code, const char *what, uint64_t a, uint64_t b,
                      uint64_t c, uint64_t d, const char *fmt, ...) {
    e.info = itak_error_info{};
    e.info.code = code;
    if (what) snprintf(e.info.what, sizeof(e.info.what), "%s", what);
    e.info.a = a;
    e.info.b = b;
    e.info.c = c;
    e.info.d = d;
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    e.message = buf;
    ITAK_DIAG("refused code=%d: %s", int(code), buf);  // every refusal says why
    return code;
}

#define ULL(x) static_cast<unsigned long long>(x)

// The Display texts of AttentionError (crates/attention/src/error.rs:129-214).
itak_status zero_dimension(ErrorState &e, const char *what) {
    return set_error(e, ITAK_ZERO_DIMENSION, what, 0, 0, 0, 0, "%s must be positive, got 0", what);
}
itak_status invalid_window(ErrorState &e, uint64_t window) {
    return set_error(e, ITAK_INVALID_WINDOW, nullptr, window, 0, 0, 0,
                     "sliding window must be positive, got %llu", ULL(window));
}
itak_status size_overflow(ErrorState &e, const char *what) {
    return set_error(e, ITAK_SIZE_OVERFLOW, what, 0, 0, 0, 0, "%s: element count overflows usize",
                     what);
}
itak_status shape_mismatch(ErrorState &e, const char *what, uint64_t expected, uint64_t actual) {
    return set_error(e, ITAK_SHAPE_MISMATCH, what, expected, actual, 0, 0,
                     "%s: got %llu, expected %llu", what, ULL(actual), ULL(expected));
}
itak_status invalid_layer(ErrorState &e, uint64_t layer, uint64_t layer_count) {
    return set_error(e, ITAK_INVALID_LAYER, nullptr, layer, layer_count, 0, 0,
                     "layer %llu out of range, cache has %llu layers", ULL(layer),
                     ULL(layer_count));
}
itak_status out_of_order(ErrorState &e, uint64_t layer, uint64_t expected, uint64_t actual) {
    return set_error(e, ITAK_OUT_OF_ORDER_POSITION, nullptr, layer, expected, actual, 0,
                     "layer %llu appends must be in order: expected position %llu, got %llu",
                     ULL(layer), ULL(expected), ULL(actual));
}
itak_status non_divisible(ErrorState &e, uint64_t q_heads, uint64_t kv_heads) {
    return set_error(e, ITAK_NON_DIVISIBLE_HEADS, nullptr, q_heads, kv_heads, 0, 0,
                     "%llu query heads do not divide evenly across %llu KV heads", ULL(q_heads),
                     ULL(kv_heads));
}
itak_status no_visible_keys(ErrorState &e, uint64_t position) {
    return set_error(e, ITAK_NO_VISIBLE_KEYS, nullptr, position, 0, 0, 0,
                     "query at position %llu has no visible keys", ULL(position));
}
itak_status checkpoint_busy(ErrorState &e) {
    return set_error(e, ITAK_CHECKPOINT_BUSY, nullptr, 0, 0, 0, 0,
                     "a checkpoint is already outstanding on this cache; release it before "
                     "taking another");
}
itak_status stale_checkpoint(ErrorState &e, uint64_t serial) {
    return set_error(e, ITAK_STALE_CHECKPOINT, nullptr, serial, 0, 0, 0,
                     "checkpoint %llu is not this cache's live checkpoint (already released or "
                     "foreign)",
                     ULL(serial));
}
itak_status range_exceeded(ErrorState &e, uint64_t layer, uint64_t position, uint64_t limit) {
    return set_error(e, ITAK_CHECKPOINT_RANGE_EXCEEDED, nullptr, layer, position, limit, 0,
                     "layer %llu append at position %llu is outside the live checkpoint's saved "
                     "range (first unsaved position %llu); refusing so a later rewind cannot meet "
                     "a slot it cannot restore",
                     ULL(layer), ULL(position), ULL(limit));
}
itak_status not_fresh(ErrorState &e, uint64_t layer, uint64_t appended) {
    return set_error(e, ITAK_BULK_RESTORE_NOT_FRESH, nullptr, layer, appended, 0, 0,
                     "layer %llu already holds %llu appended positions; bulk restore installs "
                     "into a fresh layer only",
                     ULL(layer), ULL(appended));
}
itak_status rewind_range(ErrorState &e, uint64_t layer, uint64_t base, uint64_t appended,
                         uint64_t target) {
    return set_error(e, ITAK_REWIND_OUT_OF_RANGE, nullptr, layer, base, appended, target,
                     "rewind target %llu is outside layer %llu's checkpoint range [%llu, %llu]",
                     ULL(target), ULL(layer), ULL(base), ULL(appended));
}
itak_status hip_error(ErrorState &e, hipError_t code, const char *doing) {
    return set_error(e, ITAK_HIP_ERROR, doing, uint64_t(code), 0, 0, 0, "%s: HIP error %d (%s)",
                     doing, int(code), hipGetErrorString(code));
}
itak_status invalid_argument(ErrorState &e, const char *what) {
    return set_error(e, ITAK_INVALID_ARGUMENT, what, 0, 0, 0, 0, "invalid argument: %s", what);
}
itak_status capacity_exceeded(ErrorState &e, uint64_t layer, uint64_t need, uint64_t capacity) {
    return set_error(e, ITAK_CAPACITY_EXCEEDED, nullptr, layer, need, capacity, 0,
                     "layer %llu would hold %llu positions but the pool's slots hold %llu",
                     ULL(layer), ULL(need), ULL(capacity));
}
itak_status unsupported(ErrorState &e, const char *what) {
    return set_error(e, ITAK_UNSUPPORTED, what, 0, 0, 0, 0, "unsupported: %s", what);
}

#define HIP_TRY(pool, call, doing)                                   \
    do {                                                             \
        hipError_t _e = (call);                                      \
        if (_e != hipSuccess) return hip_error((pool)->err, _e, doing); \
    } while (0)

// ------------------------------------------------------------------------------ helpers

Slot *find_slot(itak_pool *pool, uint32_t slot) {
    if (slot >= pool->slots.size() || !pool->slots[slot].in_use) return nullptr;
    return &pool->slots[slot];
}

const PoolGeom &geom_of(const itak_pool *pool, uint64_t layer) {
    return pool->layers[layer].windowed ? pool->gw : pool->g;
}

void *layer_base(itak_pool *pool, uint64_t layer) {
    const LayerInfo &L = pool->layers[layer];
    return (L.windowed ? pool->base_w : pool->base) +
           L.index * geom_of(pool, layer).layer_stride * pool->elem_bytes;
}

// Positions stored and visible (cache.rs:154-159) and the oldest of them (cache.rs:162-164).
uint64_t stored_of(const itak_pool *pool, const Slot &s, uint64_t layer) {
    const LayerInfo &L = pool->layers[layer];
    return L.windowed ? std::min(s.appended[layer], L.window) : s.appended[layer];
}
uint64_t first_visible(const itak_pool *pool, const Slot &s, uint64_t layer) {
    return s.appended[layer] - stored_of(pool, s, layer);
}

void advance(Slot &s, uint64_t layer, uint64_t rows) {
    s.appended[layer] += rows;
    s.high[layer] = std::max(s.high[layer], s.appended[layer]);
}

itak_status ensure_stage(itak_pool *pool, uint64_t bytes) {
    if (bytes <= pool->stage_bytes) return ITAK_OK;
    HIP_TRY(pool, hipStreamSynchronize(pool->stream), "synchronize before growing staging");
    if (pool->stage) HIP_TRY(pool, hipFree(pool->stage), "free staging");
    pool->stage = nullptr;
    pool->stage_bytes = 0;
    uint64_t want = std::max<uint64_t>(bytes + bytes / 2, 1u << 20);
    HIP_TRY(pool, hipMalloc(reinterpret_cast<void **>(&pool->stage), want), "allocate staging");
    pool->stage_bytes = want;
    return ITAK_OK;
}

// The rotation frequencies of (base, rotary_dim) in device memory, made on first use: the same
// expression, in the same f64 libm, as rope.rs:99-116 and rope_interleaved.rs:103-114 evaluate
// on the host. Null when the table does not exist yet and cannot be made now (the stream is
// being captured, or the allocation failed): the preparation kernel then takes the powers itself.
const double *rope_freq_table(itak_pool *pool, float base, uint32_t rotary) {
    if (!(base > 1.0f) || rotary < 2) return nullptr;
    for (const RopeFreqTable &t : pool->rope_tables)
        if (t.base == base && t.rotary == rotary) return t.dev;
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(pool->stream, &status) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    if (status != hipStreamCaptureStatusNone || pool->rope_tables.size() >= 64) return nullptr;
    std::vector<double> host(rotary / 2);
    for (uint32_t i = 0; i < rotary / 2; ++i)
        host[i] = std::pow(double(base), -double(2 * i) / double(rotary));
    double *dev = nullptr;
    if (hipMalloc(reinterpret_cast<void **>(&dev), host.size() * sizeof(double)) != hipSuccess ||
        hipMemcpy(dev, host.data(), host.size() * sizeof(double), hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipGetLastError();
        if (dev) (void)hipFree(dev);
        return nullptr;
    }
    pool->rope_tables.push_back(RopeFreqTable{base, rotary, dev});
    return dev;
}

itak_status ensure_workspace(itak_pool *pool, uint64_t floats) {
    if (floats > pool->ws_floats) {
        HIP_TRY(pool, hipStreamSynchronize(pool->stream), "synchronize before growing workspace");
        if (pool->ws) HIP_TRY(pool, hipFree(pool->ws), "free workspace");
        pool->ws = nullptr;
        pool->ws_floats = 0;
        uint64_t want = std::max<uint64_t>(floats + floats / 2, 1u << 18);
        HIP_TRY(pool, hipMalloc(reinterpret_cast<void **>(&pool->ws), want * sizeof(float)),
                "allocate split workspace");
        pool->ws_floats = want;
    }
    return ITAK_OK;
}

// (Re)fills the exchange buffer with the empty pattern and zeroes its give-up counter.
itak_status clean_exchange(itak_pool *pool) {
    HIP_TRY(pool, launch_fill_words(pool->xws, pool->xws_words, kExchangeEmptyWord, pool->stream),
            "fill the split exchange buffer");
    HIP_TRY(pool, launch_fill_words(pool->xws, 1, 0, pool->stream), "zero the give-up counter");
    return ITAK_OK;
}

itak_status ensure_exchange(itak_pool *pool, uint64_t words) {
    if (words > pool->xws_words) {
        HIP_TRY(pool, hipStreamSynchronize(pool->stream), "synchronize before growing the exchange buffer");
        if (pool->xws) HIP_TRY(pool, hipFree(pool->xws), "free the exchange buffer");
        pool->xws = nullptr;
        pool->xws_words = 0;
        const uint64_t want = std::max<uint64_t>(words + words / 2, 1u << 17);
        HIP_TRY(pool, hipMalloc(reinterpret_cast<void **>(&pool->xws), want * 8),
                "allocate the split exchange buffer");
        pool->xws_words = want;
        return clean_exchange(pool);
    }
    return ITAK_OK;
}

itak_status ensure_prep(itak_pool *pool, uint64_t floats) {
    if (floats > pool->prep_floats) {
        HIP_TRY(pool, hipStreamSynchronize(pool->stream), "synchronize before growing prep scratch");
        if (pool->prep) HIP_TRY(pool, hipFree(pool->prep), "free prep scratch");
        pool->prep = nullptr;
        pool->prep_floats = 0;
        uint64_t want = std::max<uint64_t>(floats + floats / 2, 1u << 16);
        HIP_TRY(pool, hipMalloc(reinterpret_cast<void **>(&pool->prep), want * sizeof(float)),
                "allocate prep scratch");
        pool->prep_floats = want;
    }
    return ITAK_OK;
}

constexpr uint64_t kHostWord = 256;  // bytes at the head of the pinned staging kept for the completion word
itak_status ensure_hstage(itak_pool *pool, uint64_t bytes) {
    if (bytes <= pool->hstage_bytes) return ITAK_OK;
    HIP_TRY(pool, hipStreamSynchronize(pool->stream), "synchronize before growing pinned staging");
    if (pool->hstage) HIP_TRY(pool, hipHostFree(pool->hstage), "free pinned staging");
    pool->hstage = nullptr;
    pool->hstage_bytes = 0;
    const uint64_t want = std::max<uint64_t>(bytes + bytes / 2, 1u << 18);
    HIP_TRY(pool, hipHostMalloc(reinterpret_cast<void **>(&pool->hstage), want, hipHostMallocDefault),
            "allocate pinned staging");
    memset(pool->hstage, 0, want);  // the completion word of a call must not start out matching
    pool->hstage_bytes = want;
    return ITAK_OK;
}

uint64_t align_up(uint64_t x, uint64_t a) { return (x + a - 1) / a * a; }

// The address of this device's copy of `scratch`, looked up on first use with the device
// current; the exchange part is filled with the empty pattern then (a kernel on the null
// stream, waited for). Later calls return the kept address.
hipError_t bind_scratch(int device, unsigned char **out) {
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_of_device[device]) {
        unsigned char *ptr = nullptr;
        hipError_t e = hipGetSymbolAddress(reinterpret_cast<void **>(&ptr), HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!ptr) return hipErrorInvalidSymbol;
        e = launch_fill_words(reinterpret_cast<unsigned long long *>(ptr), kScratchExchangeBytes / 8,
                              kExchangeEmptyWord, nullptr);
        if (e == hipSuccess) e = launch_fill_words(reinterpret_cast<unsigned long long *>(ptr), 1, 0, nullptr);
        if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
        if (e != hipSuccess) return e;
        e = hipEventCreateWithFlags(&g_scratch_guard[device].done, hipEventDisableTiming);
        if (e != hipSuccess) return e;
        g_scratch_of_device[device] = ptr;
    }
    *out = g_scratch_of_device[device];
    return hipSuccess;
}

// Before an allocation-free step is enqueued on `stream`: if the device's last such step ran on
// another stream, this one waits for it on the device. Returns whether the stream is being
// captured (the guard then stands aside).
hipError_t scratch_guard_enter(int device, hipStream_t stream, bool *capturing) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    hipError_t e = hipStreamIsCapturing(stream, &status);
    if (e != hipSuccess) return e;
    *capturing = status != hipStreamCaptureStatusNone;
    if (*capturing) return hipSuccess;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    ScratchGuard &g = g_scratch_guard[device];
    if (g.recorded && g.stream != stream) return hipStreamWaitEvent(stream, g.done, 0);
    return hipSuccess;
}
// After it: the event now stands behind this step.
hipError_t scratch_guard_leave(int device, hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    ScratchGuard &g = g_scratch_guard[device];
    const hipError_t e = hipEventRecord(g.done, stream);
    if (e == hipSuccess) {
        g.stream = stream;
        g.recorded = true;
    }
    return e;
}

// What the launches of one attention call need beyond their inputs and outputs.
struct WorkspaceNeed {
    uint64_t partial_floats = 0;   // split partials for a merge launch
    uint64_t exchange_words = 0;   // exchange words of launches that merge their own splits
};

// One item's query rows against its slot; fills the split plan.
struct PlanInput {
    uint32_t slot;
    uint32_t rows;
    uint32_t pos0;
    uint32_t kv_len;
    uint32_t kv_lo;  // oldest position the item's queries may see
};

// Builds the work list and launches the attention kernels. q/out are device pointers.
// f16 pools at head_dim 128 with up to 64 query vectors per KV head (decode and
// speculative blocks) take the MFMA split-K kernel; everything else the generic kernel.
// Either way a second small launch merges the split partials.
// True when a batch takes the MFMA split-K kernel (which can also fuse the append).
bool takes_splitk_f16(const itak_pool *pool, const PlanInput *in, uint32_t n, uint64_t q_heads,
                      const uint32_t *q_pos_dev) {
    const uint32_t group = uint32_t(q_heads / pool->g.kv_heads);
    uint32_t max_rows = 0;
    for (uint32_t i = 0; i < n; ++i) max_rows = std::max(max_rows, in[i].rows);
    // Decode and speculative blocks (up to 64 query vectors per KV head, up to 8 new rows):
    // the split-K kernel, which also appends the new rows. Its 64-vector variant and the
    // block kernel (wavefronts split the query vectors, K/V shared through LDS) attend at the
    // same speed on a 7-row block; the fused append decides (one launch less per layer).
    constexpr uint32_t max_vec = 64;
    return pool->elem_f16 && q_pos_dev == nullptr && max_rows * group <= max_vec &&
           attn_splitk_f16_supports(pool->g, group, max_rows);  // g and gw differ in capacity only
}

// k_new / v_new non-null = the rows are not in the cache yet and the kernel appends them
// (only valid when takes_splitk_f16 holds).
itak_status run_attention(itak_pool *pool, uint64_t layer, const PlanInput *in, uint32_t n,
                          const float *q_dev, float *out_dev, const uint32_t *q_pos_dev,
                          uint64_t q_heads, float scale, float softcap,
                          const float *k_new = nullptr, const float *v_new = nullptr,
                          const FoldedParams *folded = nullptr, WorkspaceNeed *need_only = nullptr) {
    const uint32_t group = uint32_t(q_heads / pool->g.kv_heads);
    uint32_t max_rows = 0;
    for (uint32_t i = 0; i < n; ++i) max_rows = std::max(max_rows, in[i].rows);
    const bool mfma = takes_splitk_f16(pool, in, n, q_heads, q_pos_dev);
    // Blocks of many rows (prefill chunks) on the same pools take the MFMA prefill kernel.
    const bool prefill = !mfma && pool->elem_f16 && q_pos_dev == nullptr &&
                         attn_prefill_f16_supports(pool->g, group);
    // Decode steps and short blocks on f32 pools of head_dim 128: the f32 MFMA split-K kernel.
    const bool f32fast = !pool->elem_f16 && q_pos_dev == nullptr &&
                         attn_splitk_f32_supports(pool->g, group, max_rows);
    const uint32_t rpb =
        (mfma || prefill || f32fast) ? 0 : attn_generic_rows_per_block(group, pool->g.head_dim);
    if (!mfma && !prefill && !f32fast && rpb == 0)
        return unsupported(pool->err, "head_dim above 256 or GQA group too wide");
    const uint32_t tile = attn_generic_tile(pool->g.head_dim);
    constexpr uint64_t kTargetBlocks = 1024;  // about four workgroups per CU
    const LayerInfo &L = pool->layers[layer];
    const PoolGeom &geom = geom_of(pool, layer);
    const uint32_t window = uint32_t(std::min<uint64_t>(L.window, 0xffffffffu));

    uint32_t q_row0 = 0;
    for (uint32_t first = 0; first < n; first += kMaxBatchItems) {
        const uint32_t count = std::min<uint32_t>(kMaxBatchItems, n - first);
        AttnBatch b{};
        b.n = count;
        b.two_halves = prefill && pool->q_two_halves && pool->g.head_dim == 128 ? 1 : 0;
        uint32_t total_rows = 0;
        for (uint32_t i = 0; i < count; ++i) {
            const PlanInput &pi = in[first + i];
            AttnItem &it = b.item[i];
            it.slot = pi.slot;
            it.rows = pi.rows;
            it.pos0 = pi.pos0;
            it.q_row0 = q_row0;
            it.kv_len = pi.kv_len;
            it.kv_lo = pi.kv_lo;
            q_row0 += pi.rows;
            total_rows += pi.rows;
        }
        uint32_t partials = 0;
        if (mfma) {
            partials = attn_splitk_f16_plan(geom, b, uint32_t(q_heads));
        } else if (prefill) {
            partials = attn_prefill_f16_plan(geom, b, group, uint32_t(q_heads), window, k_new != nullptr);
        } else if (f32fast) {
            partials = attn_splitk_f32_plan(geom, b, uint32_t(q_heads));
        } else {
            b.rows_per_block = rpb;
            uint64_t key_work = 0;
            for (uint32_t i = 0; i < count; ++i) {
                const uint64_t qblocks = (b.item[i].rows + rpb - 1) / rpb;
                key_work += qblocks * pool->g.kv_heads * (b.item[i].kv_len - b.item[i].kv_lo);
            }
            const uint64_t kps = align_up(
                std::max<uint64_t>((key_work + kTargetBlocks - 1) / kTargetBlocks, tile), tile);
            uint32_t block0 = 0;
            for (uint32_t i = 0; i < count; ++i) {
                AttnItem &it = b.item[i];
                const uint32_t keys = it.kv_len - it.kv_lo;
                it.keys_per_split = uint32_t(kps);
                it.splits = uint32_t((keys + kps - 1) / kps);
                if (it.splits == 0) it.splits = 1;
                if (it.splits > 1024) {  // the merge kernel holds at most 1024 weights
                    it.keys_per_split = uint32_t(align_up((keys + 1023) / 1024, tile));
                    it.splits = (keys + it.keys_per_split - 1) / it.keys_per_split;
                }
                const uint32_t qblocks = (it.rows + rpb - 1) / rpb;
                it.block0 = block0;
                it.ws0 = partials;
                block0 += qblocks * pool->g.kv_heads * it.splits;
                if (it.splits > 1) partials += it.rows * uint32_t(q_heads) * it.splits;
            }
            b.total_blocks = block0;
        }
        // Split-K launches merge their splits themselves where the plan allows it (the gate,
        // when there is one, must then be applied by that kernel: its preparing variants).
        const float *gate = folded ? folded->gate : nullptr;
        const bool prepares = folded && folded->prep_on && mfma;
        uint64_t exchange_words = 0;
        if (mfma && pool->merge_in_launch && (!gate || prepares))
            exchange_words = attn_splitk_f16_plan_exchange(geom, b, uint32_t(q_heads));
        // Or on the units' compute dies, when the batch deals out evenly over them and is not
        // one the single-row decode kernel takes.
        AttnBatch bd{};
        DieMap dm{};
        uint32_t die_partials = 0;
        if (mfma && pool->die_merge && !exchange_words && !pool->q_two_halves) {
            AttnParams probe{};
            probe.g = geom;
            probe.group = group;
            if (prepares || !attn_decode_f16_takes(probe, b))
                die_partials = attn_splitk_f16_plan_die(geom, b, uint32_t(q_heads), bd, dm);
        }
        const bool on_die = die_partials != 0;
        if (on_die) partials = die_partials;
        const AttnBatch &bl = on_die ? bd : b;  // the batch the attention launch takes
        const uint64_t partial_floats = uint64_t(partials) * (pool->g.head_dim + 2);
        if (need_only) {  // planning only: nothing is allocated, launched or changed
            need_only->exchange_words = std::max(need_only->exchange_words, exchange_words);
            if (!exchange_words)
                need_only->partial_floats = std::max(need_only->partial_floats, partial_floats);
            continue;
        }
        float *ws = nullptr;
        if (pool->no_alloc_call) {
            // The caller has checked the need against the static workspace's two parts.
            ws = reinterpret_cast<float *>(exchange_words ? pool->scratch_dev
                                                          : pool->scratch_dev + kScratchExchangeBytes);
        } else {
            itak_status st = exchange_words ? ensure_exchange(pool, exchange_words)
                                            : ensure_workspace(pool, partial_floats);
            if (st != ITAK_OK) return st;
            ws = exchange_words ? reinterpret_cast<float *>(pool->xws) : pool->ws;
        }
        // The reference's line (attention.rs:147-155) plus which kernel takes the launch.
        if (diag_enabled()) {
            uint32_t splits = 0;
            uint64_t view_len = 0;
            for (uint32_t i = 0; i < count; ++i) {
                splits = std::max(splits, bl.item[i].splits);
                view_len = std::max<uint64_t>(view_len, b.item[i].kv_len - b.item[i].kv_lo);
            }
            diag_emit("gqa_attention layer=%llu items=%u queries=%u q_heads=%llu kv_heads=%llu "
                      "view_len=%llu window=%u scale=%g softcap=%g kernel=%s workgroups=%u splits=%u "
                      "fused_append=%d merge=%s",
                      ULL(layer), count, total_rows, ULL(q_heads), ULL(pool->g.kv_heads), ULL(view_len),
                      window, double(scale), double(softcap),
                      mfma ? "splitk_f16" : prefill ? "prefill_f16" : f32fast ? "splitk_f32" : "generic",
                      bl.total_blocks, splits, int(k_new != nullptr && (mfma || f32fast || prefill)),
                      partials == 0 ? "none" : on_die ? "on_die" : exchange_words ? "in_launch" : "launch");
        }
        AttnParams p{};
        p.layer_base = layer_base(pool, layer);
        p.g = geom;
        p.window = window;
        p.ring_blocks = L.ring / kVBlock;
        p.q = q_dev;
        p.out = out_dev;
        p.q_pos = q_pos_dev;
        p.ws = ws;
        p.exchange = exchange_words ? 1 : 0;
        p.fold_units = prefill ? b.fold_units : 0;
        {
            uint64_t rows_read = 0;
            for (uint32_t i = 0; i < count; ++i) rows_read += b.item[i].kv_len - b.item[i].kv_lo;
            const uint64_t layer_bytes = rows_read * 2 * pool->g.kv_heads * pool->g.head_dim *
                                         (pool->elem_f16 ? 2 : 4);
            p.kv_streams = layer_bytes * pool->layers.size() > (uint64_t(512) << 20) ? 1 : 0;  // twice the cache: well clear of it
        }
        p.spin_limit = pool->spin_limit;
        p.k_new = (mfma || f32fast || prefill) ? k_new : nullptr;  // the caller passes them only to
        p.v_new = (mfma || f32fast || prefill) ? v_new : nullptr;  // launches that append themselves
        p.q_heads = uint32_t(q_heads);
        p.group = group;
        p.group_magic = (65536u + group - 1) / group;
        p.scale = scale;
        p.softcap = softcap;
        // The gate is applied by whoever writes the output: the merge for items of several
        // splits; for items of one split the split-K kernel, which only its preparing
        // variants can; otherwise a launch of its own over the chunk's rows.
        bool merged_only = mfma || prefill;
        for (uint32_t i = 0; i < count; ++i) merged_only = merged_only && bl.item[i].splits > 1;
        const bool gate_folded = gate && (prepares || (mfma && merged_only));
        if (on_die) {
            dm.tickets = pool->die_words;
            dm.faults = pool->die_words + kDieTicketBytes / sizeof(uint32_t);
            dm.gate = gate_folded ? gate : nullptr;
            HIP_TRY(pool,
                    launch_attn_splitk_f16_die(p, bd, dm, partials, pool->stream,
                                               prepares ? folded : nullptr),
                    "launch split-K attention");
        } else if (mfma) {
            HIP_TRY(pool,
                    launch_attn_splitk_f16(p, b, partials, max_rows, pool->stream,
                                           prepares ? folded : nullptr, pool->q_two_halves),
                    "launch split-K attention");
        } else if (prefill) {
            HIP_TRY(pool, launch_attn_prefill_f16(p, b, partials, pool->stream),
                    "launch block attention");
        } else if (f32fast) {
            HIP_TRY(pool, launch_attn_splitk_f32(p, b, partials, pool->stream),
                    "launch f32 split-K attention");
        } else {
            HIP_TRY(pool, launch_attn_generic(pool->elem_f16, p, b, partials, pool->stream),
                    "launch attention");
        }
        if (!exchange_words && !on_die)
            HIP_TRY(pool, launch_attn_combine(p, b, partials, total_rows, (mfma || prefill || f32fast) ? 1 : 0,
                                              pool->stream, gate_folded ? gate : nullptr),
                    "launch split merge");
        if (gate && !gate_folded) {
            const uint64_t q_width = q_heads * pool->g.head_dim;
            const uint64_t at = uint64_t(q_row0 - total_rows) * q_width;
            HIP_TRY(pool, launch_attn_gate(out_dev + at, gate + at, total_rows * q_width, pool->stream),
                    "launch attention gate");
        }
    }
    return ITAK_OK;
}

float default_scale(uint64_t head_dim) {  // attention.rs:35-37
    return 1.0f / std::sqrt(static_cast<float>(head_dim));
}

// Appends `rows` rows per item from device sources; the caller has validated everything.
itak_status run_append(itak_pool *pool, uint64_t layer, const itak_batch_item *items, uint32_t n,
                       const float *k_dev, const float *v_dev) {
    // A long run of rows into blocked planes (a prefill chunk) goes in two parts: the rows up
    // to the next 32-row boundary through the row kernel, the block-aligned rest through the
    // gather kernels of the snapshot restore, which transpose whole value blocks in LDS and
    // store 16 bytes per thread instead of 2. The rows after the run inside its last block
    // are beyond the slot's length; the gather writes zeros there, which is what they hold.
    constexpr uint32_t kChunkRows = 4 * kVBlock;
    const LayerInfo &L = pool->layers[layer];
    const PoolGeom &geom = geom_of(pool, layer);
    if (n == 1 && !L.windowed && pool->elem_f16 && pool->g.v_block != 0 &&
        items[0].rows >= kChunkRows) {
        const uint32_t slot = items[0].slot, rows = items[0].rows;
        const uint32_t pos0 = uint32_t(pool->slots[slot].appended[layer]);
        const uint32_t head_rows = (kVBlock - pos0 % kVBlock) % kVBlock;
        if (head_rows) {
            AppendBatch b{};
            b.n = 1;
            b.total_rows = head_rows;
            b.item[0] = AppendItem{slot, head_rows, pos0, 0};
            HIP_TRY(pool, launch_append(layer_base(pool, layer), 1, pool->g, b, k_dev, v_dev,
                                        pool->stream),
                    "launch append");
        }
        RestoreBatch rb{};
        rb.n = 1;
        rb.max_rows = rows - head_rows;
        rb.slot = slot;
        rb.layer[0] = RestoreLayer{k_dev + uint64_t(head_rows) * pool->row,
                                   v_dev + uint64_t(head_rows) * pool->row, L.index,
                                   rows - head_rows, pos0 + head_rows, 0};
        HIP_TRY(pool, launch_restore(pool->base, 1, 0, pool->g, rb, pool->stream),
                "launch chunk append");
        advance(pool->slots[slot], layer, rows);
        return ITAK_OK;
    }
    // The same on a ring whose length is a whole number of blocks: the rows before the first
    // block boundary and those after the last one go through the row kernel in one launch,
    // the whole blocks between them through the gather, in two pieces where they wrap. Nothing
    // beyond the run is written: on a ring the rows behind it are older positions that a
    // rewind may still need.
    if (n == 1 && L.windowed && pool->elem_f16 && pool->gw.v_block != 0 &&
        L.ring % kVBlock == 0 && items[0].rows >= kChunkRows && items[0].rows <= L.ring) {
        const uint32_t slot = items[0].slot, rows = items[0].rows;
        const uint32_t pos0 = uint32_t(pool->slots[slot].appended[layer]);
        const uint32_t head_rows = (kVBlock - pos0 % kVBlock) % kVBlock;
        const uint32_t body = (rows - head_rows) / kVBlock * kVBlock;
        const uint32_t tail_rows = rows - head_rows - body;
        if (head_rows + tail_rows) {
            AppendBatch b{};
            b.ring = uint32_t(L.ring);
            b.total_rows = head_rows + tail_rows;
            b.gap_at = head_rows;
            b.gap_rows = body;
            if (head_rows) b.item[b.n++] = AppendItem{slot, head_rows, pos0, 0};
            if (tail_rows)
                b.item[b.n++] = AppendItem{slot, tail_rows, pos0 + head_rows + body, head_rows + body};
            HIP_TRY(pool, launch_append(layer_base(pool, layer), 1, pool->gw, b, k_dev, v_dev,
                                        pool->stream),
                    "launch append");
        }
        const uint32_t at = uint32_t((pos0 + head_rows) % L.ring);
        const uint32_t first_piece = std::min<uint32_t>(body, uint32_t(L.ring) - at);
        RestoreBatch rb{};
        rb.slot = slot;
        rb.max_rows = std::max(first_piece, body - first_piece);
        const float *ks = k_dev + uint64_t(head_rows) * pool->row, *vs = v_dev + uint64_t(head_rows) * pool->row;
        rb.layer[rb.n++] = RestoreLayer{ks, vs, L.index, first_piece, at, 0};
        if (body > first_piece)
            rb.layer[rb.n++] = RestoreLayer{ks + uint64_t(first_piece) * pool->row,
                                            vs + uint64_t(first_piece) * pool->row, L.index,
                                            body - first_piece, 0, 0};
        HIP_TRY(pool, launch_restore(pool->base_w, 1, 0, pool->gw, rb, pool->stream),
                "launch chunk append");
        advance(pool->slots[slot], layer, rows);
        return ITAK_OK;
    }
    uint32_t src_row = 0;
    for (uint32_t first = 0; first < n; first += kMaxBatchItems) {
        const uint32_t count = std::min<uint32_t>(kMaxBatchItems, n - first);
        AppendBatch b{};
        b.n = count;
        b.ring = L.ring;
        const uint32_t chunk_row0 = src_row;
        for (uint32_t i = 0; i < count; ++i) {
            const itak_batch_item &bi = items[first + i];
            b.item[i].slot = bi.slot;
            b.item[i].rows = bi.rows;
            b.item[i].pos0 = uint32_t(pool->slots[bi.slot].appended[layer]);
            b.item[i].src_row0 = src_row - chunk_row0;
            src_row += bi.rows;
        }
        b.total_rows = src_row - chunk_row0;
        HIP_TRY(pool,
                launch_append(layer_base(pool, layer), pool->elem_f16, geom, b,
                              k_dev + uint64_t(chunk_row0) * pool->row,
                              v_dev + uint64_t(chunk_row0) * pool->row, pool->stream),
                "launch append");
    }
    for (uint32_t i = 0; i < n; ++i) {
        advance(pool->slots[items[i].slot], layer, items[i].rows);
        ITAK_DIAG("append layer=%llu slot=%u rows=%u kind=%s stored=%llu", ULL(layer), items[i].slot,
                  items[i].rows, L.windowed ? "windowed" : "global",
                  ULL(pool->slots[items[i].slot].appended[layer]));
    }
    return ITAK_OK;
}

// The append preconditions of KvCache::append (cache.rs:445-471) for `rows` consecutive
// positions starting at the layer's next one; returns how many rows may be appended
// before a refusal (rows if none) and leaves that refusal in the error state.
// Positions a slot may hold on a layer: the configured capacity on a global layer; a ring
// never fills, its positions only have to stay well inside 32 bits.
uint64_t position_limit(const itak_pool *pool, uint64_t layer) {
    return pool->layers[layer].windowed ? 0xfff00000ull : pool->rows_limit;
}

itak_status check_append_rows(itak_pool *pool, Slot &s, uint64_t layer, uint64_t rows,
                              uint64_t *ok_rows) {
    uint64_t ok = rows;
    itak_status st = ITAK_OK;
    const uint64_t start = s.appended[layer];
    if (s.cp.live) {
        const uint64_t limit = s.cp.bases[layer] + s.cp.max_round_tokens;
        if (start + rows > limit) {
            ok = limit > start ? limit - start : 0;
            st = range_exceeded(pool->err, layer, start + ok, limit);
        }
    }
    const uint64_t rows_limit = position_limit(pool, layer);
    if (start + ok > rows_limit) {
        ok = rows_limit > start ? rows_limit - start : 0;
        st = capacity_exceeded(pool->err, layer, start + ok + 1, rows_limit);
    }
    *ok_rows = ok;
    return st;
}

// A block of a device step lands in a windowed layer's ring before its queries run, so it
// may be at most as long as the ring's headroom over the window.
itak_status check_block_rows(itak_pool *pool, uint64_t layer, uint64_t rows) {
    const LayerInfo &L = pool->layers[layer];
    if (!L.windowed || rows <= L.ring - L.window) return ITAK_OK;
    return set_error(pool->err, ITAK_CAPACITY_EXCEEDED, nullptr, layer, rows, L.ring - L.window, 0,
                     "a block of %llu rows does not fit the %llu rows of ring headroom of windowed "
                     "layer %llu; split the block or build the pool with a larger ring_headroom",
                     ULL(rows), ULL(L.ring - L.window), ULL(layer));
}

// Zero fill of rows [row_from, row_to) of every global layer of the listed slots.
itak_status scrub_rows(itak_pool *pool, const ZeroBatch &zb) {
    HIP_TRY(pool,
            launch_zero_rows(pool->base, pool->elem_f16, pool->g, 0, pool->global_layers, zb,
                             pool->stream),
            "launch row scrub");
    return ITAK_OK;
}

// Pointer kinds for restore sources. For memory the device can read in place, `usable`
// is the address a kernel should dereference.
enum class PtrKind { Device, PinnedHost, PlainHost };
PtrKind classify(const void *p, const void **usable) {
    *usable = p;
    hipPointerAttribute_t attr{};
    hipError_t e = hipPointerGetAttributes(&attr, p);
    if (e != hipSuccess) {
        (void)hipGetLastError();  // an unknown pointer is ordinary host memory, not a failure
        return PtrKind::PlainHost;
    }
    if (attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged)
        return PtrKind::Device;
    if (attr.type == hipMemoryTypeHost) {
        if (attr.devicePointer) *usable = attr.devicePointer;
        return PtrKind::PinnedHost;
    }
    return PtrKind::PlainHost;
}

// The same for the many sources of one restore: a snapshot's layers usually lie in one or two
// device allocations, and the runtime's lookup costs microseconds a pointer (two lookups a
// layer and side were more host time than the gather of a 48-layer prefix takes the device).
// The extent of the last device allocation seen answers for every pointer inside it.
struct PtrClassifier {
    uintptr_t lo = 0, hi = 0;  // a device allocation already looked up
    PtrKind operator()(const void *p, const void **usable) {
        const uintptr_t a = reinterpret_cast<uintptr_t>(p);
        if (a >= lo && a < hi) {
            *usable = p;
            return PtrKind::Device;
        }
        const PtrKind kind = classify(p, usable);
        if (kind == PtrKind::Device) {
            hipDeviceptr_t base = nullptr;
            size_t size = 0;
            if (hipMemGetAddressRange(&base, &size, const_cast<void *>(p)) == hipSuccess && size) {
                lo = reinterpret_cast<uintptr_t>(base);
                hi = lo + size;
            } else {
                (void)hipGetLastError();
            }
        }
        return kind;
    }
};

// Rows the gather kernel cannot read where they lie: ordinary host memory, or a source that
// is not aligned to its element size (the payload of an encoded snapshot starts wherever
// its fingerprint ends).
bool must_stage(PtrClassifier &kind_of, const void *p, uint64_t elem_bytes) {
    const void *usable;
    return kind_of(p, &usable) == PtrKind::PlainHost ||
           reinterpret_cast<uintptr_t>(p) % elem_bytes != 0;
}

itak_status set_itkv_error(ErrorState &e, const ItkvError &err) {
    return set_error(e, err.code, "snapshot", err.a, err.b, 0, 0, "%s", err.message.c_str());
}

ItkvHeader to_internal(const itak_itkv_header &h) {
    ItkvHeader r;
    r.token_count = h.token_count;
    r.num_kv_heads = h.num_kv_heads;
    r.head_dim = h.head_dim;
    r.layer_count = h.layer_count;
    r.fingerprint_len = h.fingerprint_len;
    return r;
}
std::vector<ItkvLayer> to_internal(const itak_itkv_layer *layers, uint64_t n) {
    std::vector<ItkvLayer> r(n);
    for (uint64_t i = 0; i < n; ++i) {
        r[i].kind = layers[i].kind;
        r[i].window = layers[i].window;
        r[i].first_position = layers[i].first_position;
        r[i].rows = layers[i].rows;
    }
    return r;
}

}  // namespace

// ======================================================================== public ABI

namespace itak {

int32_t restore_decoded_itkv(itak_pool *pool, uint32_t slot, const uint8_t *b8, const ItkvHeader &h,
                             const std::vector<ItkvLayer> &ls, const char *expected_fingerprint,
                             uint64_t expected_fingerprint_len) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (!find_slot(pool, slot)) return invalid_argument(pool->err, "slot is not in use");
    // restore_checked (snapshot.rs:351-371): geometry first, then the fingerprint.
    bool same = h.layer_count == pool->cfg.layer_count && h.num_kv_heads == pool->g.kv_heads &&
                h.head_dim == pool->g.head_dim;
    for (size_t i = 0; same && i < ls.size(); ++i)
        same = pool->layers[i].windowed
                   ? (ls[i].kind == ITAK_LAYER_WINDOWED && ls[i].window == pool->layers[i].window)
                   : ls[i].kind == ITAK_LAYER_GLOBAL;
    if (!same)
        return set_error(pool->err, ITAK_KV_GEOMETRY_MISMATCH, "snapshot", 0, 0, 0, 0,
                         "geometry mismatch: snapshot geometry (%llu layers, %llu KV heads, head "
                         "dim %llu) differs from the required geometry (%llu layers, %llu KV "
                         "heads, head dim %llu)",
                         ULL(h.layer_count), ULL(h.num_kv_heads), ULL(h.head_dim),
                         ULL(pool->cfg.layer_count), ULL(pool->g.kv_heads), ULL(pool->g.head_dim));
    if (expected_fingerprint &&
        (expected_fingerprint_len != h.fingerprint_len ||
         memcmp(expected_fingerprint, b8 + h.fingerprint_offset, h.fingerprint_len) != 0))
        return set_error(pool->err, ITAK_KV_FINGERPRINT_MISMATCH, "snapshot", 0, 0, 0, 0,
                         "model fingerprint mismatch: need %.*s, snapshot carries %.*s",
                         int(std::min<uint64_t>(expected_fingerprint_len, 400)), expected_fingerprint,
                         int(std::min<uint64_t>(h.fingerprint_len, 400)),
                         reinterpret_cast<const char *>(b8 + h.fingerprint_offset));
    std::vector<itak_snapshot_layer> layers(ls.size());
    for (size_t i = 0; i < ls.size(); ++i)
        layers[i] = itak_snapshot_layer{ls[i].first_position, ls[i].rows, b8 + ls[i].keys_offset,
                                        b8 + ls[i].values_offset};
    return itak_kv_restore_snapshot(pool, slot, h.token_count, layers.data(), layers.size(),
                                    h.elem ? ITAK_ELEM_F16 : ITAK_ELEM_F32);
}

}  // namespace itak

static itak_status capture_itkv(itak_pool *pool, uint32_t slot, const char *fingerprint,
                                uint64_t fingerprint_len, bool f16_rows, void *out,
                                uint64_t capacity, uint64_t *written, bool with_checksum);

namespace itak {

int32_t capture_itkv_unsummed(itak_pool *pool, uint32_t slot, const char *fingerprint,
                              uint64_t fingerprint_len, bool f16_rows, void *out, uint64_t capacity,
                              uint64_t *written) {
    if (pool && f16_rows && !pool->elem_f16)
        return unsupported(pool->err,
                           "an f16 snapshot of an f32 pool would drop precision the cache holds");
    return capture_itkv(pool, slot, fingerprint, fingerprint_len, f16_rows, out, capacity, written,
                        false);
}

}  // namespace itak

extern "C" {

uint32_t itak_abi_version(void) { return 1; }

const char *itak_last_error(const itak_pool *pool) {
    return pool ? pool->err.message.c_str() : g_create_error.message.c_str();
}

itak_status itak_last_error_info(const itak_pool *pool, itak_error_info *out) {
    if (!out) return ITAK_INVALID_ARGUMENT;
    *out = pool ? pool->err.info : g_create_error.info;
    return ITAK_OK;
}

itak_status itak_pool_create(const itak_pool_config *config, itak_pool **out) {
    ErrorState &e = g_create_error;
    if (!out) return invalid_argument(e, "out is null");
    *out = nullptr;
    if (!config) return invalid_argument(e, "config is null");
    // KvCache::new (cache.rs:327-351) and LayerCache::new (cache.rs:125-141).
    if (config->layer_count == 0) return zero_dimension(e, "layer pattern");
    if (config->num_kv_heads == 0) return zero_dimension(e, "num_kv_heads");
    if (config->head_dim == 0) return zero_dimension(e, "head_dim");
    bool any_windowed = false;
    for (uint32_t i = 0; i < config->layer_count; ++i) {
        if (config->layer_kinds && config->layer_kinds[i] == ITAK_LAYER_WINDOWED) {
            any_windowed = true;
            const uint64_t w = config->windows ? config->windows[i] : 0;
            if (w == 0) return invalid_window(e, 0);
        } else if (config->layer_kinds && config->layer_kinds[i] != ITAK_LAYER_GLOBAL) {
            return invalid_argument(e, "unknown layer kind");
        }
    }
    uint64_t row = 0;
    if (__builtin_mul_overflow(config->num_kv_heads, config->head_dim, &row))
        return size_overflow(e, "kv row length");
    for (uint32_t i = 0; any_windowed && i < config->layer_count; ++i) {
        if (config->layer_kinds[i] != ITAK_LAYER_WINDOWED) continue;
        uint64_t slots = 0;
        if (__builtin_mul_overflow(config->windows[i], row, &slots))  // cache.rs:131-137
            return size_overflow(e, "windowed layer storage");
    }
    if (config->elem != ITAK_ELEM_F32 && config->elem != ITAK_ELEM_F16)
        return invalid_argument(e, "elem is neither ITAK_ELEM_F32 nor ITAK_ELEM_F16");
    if (config->max_slots == 0) return zero_dimension(e, "max_slots");
    if (config->capacity_rows == 0) return zero_dimension(e, "capacity_rows");
    if (config->capacity_rows > (1ull << 30) || config->head_dim > (1u << 16) ||
        config->num_kv_heads > (1u << 16))
        return size_overflow(e, "global layer storage");
    const uint64_t headroom = config->ring_headroom ? config->ring_headroom : 64;
    if (headroom > (1ull << 20)) return size_overflow(e, "windowed layer storage");
    const uint64_t elem_bytes = config->elem == ITAK_ELEM_F16 ? 2 : 4;
    // f16 pools whose head_dim suits the MFMA kernels keep value planes in transposed
    // 32-row blocks; their planes are padded to whole blocks.
    const bool v_blocked = config->elem == ITAK_ELEM_F16 && config->head_dim % 16 == 0;

    // The pattern: global layers share one group of planes, windowed layers another whose
    // planes hold the longest ring. A ring is window + headroom rows rounded up to whole
    // 32-row blocks, so that a 32-position block is also a 32-row block of the ring.
    std::vector<LayerInfo> layers(config->layer_count);
    uint32_t n_global = 0, n_windowed = 0;
    uint64_t max_ring = 0;
    for (uint32_t i = 0; i < config->layer_count; ++i) {
        LayerInfo &L = layers[i];
        L.windowed = config->layer_kinds && config->layer_kinds[i] == ITAK_LAYER_WINDOWED;
        if (!L.windowed) {
            L.index = n_global++;
            continue;
        }
        L.index = n_windowed++;
        L.window = config->windows[i];
        if (L.window > (1ull << 30)) return size_overflow(e, "windowed layer storage");
        L.ring = uint32_t(align_up(L.window + headroom, kVBlock));
        max_ring = std::max<uint64_t>(max_ring, L.ring);
    }
    auto make_geom = [&](uint64_t plane_rows, uint64_t layer_count, PoolGeom &g,
                         uint64_t &bytes) -> bool {
        uint64_t head_stride, side_stride, slot_stride, layer_stride, total;
        if (__builtin_mul_overflow(plane_rows, config->head_dim, &head_stride) ||
            __builtin_mul_overflow(head_stride, config->num_kv_heads, &side_stride) ||
            __builtin_mul_overflow(side_stride, uint64_t(2), &slot_stride) ||
            __builtin_mul_overflow(slot_stride, uint64_t(config->max_slots), &layer_stride) ||
            __builtin_mul_overflow(layer_stride, layer_count, &total) ||
            __builtin_mul_overflow(total, elem_bytes, &bytes))
            return false;
        g.kv_heads = uint32_t(config->num_kv_heads);
        g.head_dim = uint32_t(config->head_dim);
        g.capacity = uint32_t(plane_rows);
        g.max_slots = config->max_slots;
        g.v_block = v_blocked ? kVBlock : 0;
        g.head_stride = head_stride;
        g.side_stride = side_stride;
        g.slot_stride = slot_stride;
        g.layer_stride = layer_stride;
        return true;
    };
    // Planes whose size in bytes is a multiple of 1 MiB + 8 KiB or of 1 MiB - 8 KiB put the
    // streams of a multi-slot launch (one per slot, head and side, a plane apart, all advancing
    // together) onto few memory channels: measured on an MI355X, 32 slots at context 4096 decode
    // in 69 us per layer with planes of 129 blocks of 8 KiB and in 51 us with 128 or 130 (127,
    // 254, 258, 387 and 516 blocks likewise 60 to 66 us against 52). Such a plane gets one more
    // block; the rows are never addressed (a ring's length is its own).
    // The distance between two slots' planes of a head (2 * kv_heads planes) is held to the same
    // rule: that is the spacing of a batch's streams.
    auto spread = [&](uint64_t rows) -> uint64_t {
        const uint64_t step = kVBlock;
        auto bad = [](uint64_t bytes) {
            return bytes != 0 && (bytes % ((1u << 20) + (1u << 13)) == 0 ||
                                  bytes % ((1u << 20) - (1u << 13)) == 0);
        };
        for (int guard = 0; guard < 8; ++guard) {
            const uint64_t plane_bytes = rows * config->head_dim * elem_bytes;
            if (!bad(plane_bytes) && !bad(plane_bytes * 2 * config->num_kv_heads)) break;
            rows += step;
        }
        return rows;
    };
    const uint64_t plane_rows =
        spread(v_blocked ? align_up(config->capacity_rows, kVBlock) : config->capacity_rows);
    PoolGeom g{}, gw{};
    uint64_t bytes_g = 0, bytes_w = 0, bytes = 0;
    if (!make_geom(plane_rows, n_global, g, bytes_g))
        return size_overflow(e, "global layer storage");
    if (!make_geom(spread(max_ring), n_windowed, gw, bytes_w))
        return size_overflow(e, "windowed layer storage");
    bytes_g = align_up(bytes_g, 256);
    if (__builtin_add_overflow(bytes_g, bytes_w, &bytes) || bytes == 0)
        return size_overflow(e, "global layer storage");

    hipError_t he = hipSetDevice(config->device);
    if (he != hipSuccess) return hip_error(e, he, "select device");
    itak_pool *pool = new itak_pool();
    pool->cfg = *config;
    pool->cfg.layer_kinds = nullptr;  // the caller's arrays are not retained: see `layers`
    pool->cfg.windows = nullptr;
    pool->layers = std::move(layers);
    pool->global_layers = n_global;
    pool->windowed_layers = n_windowed;
    pool->headroom = headroom;
    pool->elem_f16 = config->elem == ITAK_ELEM_F16;
    pool->elem_bytes = uint32_t(elem_bytes);
    pool->row = row;
    pool->g = g;
    pool->gw = gw;
    pool->rows_limit = config->capacity_rows;
    pool->bytes = bytes;
    he = hipMalloc(reinterpret_cast<void **>(&pool->base), bytes);
    if (he != hipSuccess) {
        delete pool;
        return hip_error(e, he, "allocate KV pool");
    }
    pool->base_w = pool->base + bytes_g;
    // Fresh storage is all zero bytes, as the reference's ring storage is
    // (cache.rs:139) and as the scrub guarantee needs.
    he = hipMemset(pool->base, 0, bytes);
    if (he != hipSuccess) {
        (void)hipFree(pool->base);
        delete pool;
        return hip_error(e, he, "zero KV pool");
    }
    pool->slots.resize(config->max_slots);
    pool->ring_saved.assign(config->max_slots, nullptr);
    pool->ring_saved_bytes.assign(config->max_slots, 0);
    pool->merge_in_launch = (config->flags & ITAK_POOL_MERGE_IN_LAUNCH) != 0;
    pool->q_two_halves = pool->elem_f16 && (config->flags & ITAK_POOL_Q_TWO_HALVES) != 0;
    pool->prep_by_launch = (config->flags & ITAK_POOL_PREP_BY_LAUNCH) != 0;
    if (pool->elem_f16 && !pool->merge_in_launch && (config->flags & ITAK_POOL_DIE_MERGE) &&
        die_layout_ok(config->device)) {
        he = hipMalloc(reinterpret_cast<void **>(&pool->die_words), kDieTicketBytes + 256);
        if (he == hipSuccess) he = hipMemset(pool->die_words, 0, kDieTicketBytes + 256);
        if (he != hipSuccess) {
            if (pool->die_words) (void)hipFree(pool->die_words);
            (void)hipFree(pool->base);
            delete pool;
            return hip_error(e, he, "allocate the split tickets");
        }
        pool->die_merge = true;
    }
    he = bind_scratch(config->device, &pool->scratch_dev);
    if (he != hipSuccess) {
        (void)hipFree(pool->base);
        delete pool;
        return hip_error(e, he, "look up the static split workspace");
    }
    ITAK_DIAG("kv pool built layers=%u kv_heads=%llu head_dim=%llu elem=%s slots=%u capacity_rows=%llu "
              "device_bytes=%llu",
              config->layer_count, ULL(config->num_kv_heads), ULL(config->head_dim),
              pool->elem_f16 ? "f16" : "f32", config->max_slots, ULL(config->capacity_rows),
              ULL(pool->bytes));
    *out = pool;
    return ITAK_OK;
}

void itak_pool_destroy(itak_pool *pool) {
    if (!pool) return;
    (void)hipStreamSynchronize(pool->stream);
    if (pool->base) (void)hipFree(pool->base);
    if (pool->stage) (void)hipFree(pool->stage);
    if (pool->ws) (void)hipFree(pool->ws);
    if (pool->prep) (void)hipFree(pool->prep);
    if (pool->xws) (void)hipFree(pool->xws);
    if (pool->die_words) (void)hipFree(pool->die_words);
    for (const RopeFreqTable &t : pool->rope_tables)
        if (t.dev) (void)hipFree(t.dev);
    for (void *buf : pool->ring_saved)
        if (buf) (void)hipFree(buf);
    if (pool->hstage) (void)hipHostFree(pool->hstage);
    delete pool;
}

itak_status itak_pool_set_stream(itak_pool *pool, void *hip_stream) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    pool->stream = static_cast<hipStream_t>(hip_stream);
    return ITAK_OK;
}

itak_status itak_pool_synchronize(itak_pool *pool) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    HIP_TRY(pool, hipStreamSynchronize(pool->stream), "synchronize");
    // Consumers of an in-launch merge that gave up waiting counted themselves in their
    // buffer's first word; their outputs are NaN and the buffer may hold words nobody took,
    // so it is made clean again.
    unsigned long long *buffers[2] = {pool->xws,
                                      pool->scratch_exchange_used
                                          ? reinterpret_cast<unsigned long long *>(pool->scratch_dev)
                                          : nullptr};
    const uint64_t words[2] = {pool->xws_words, kScratchExchangeBytes / 8};
    uint32_t total = 0;
    for (int i = 0; i < 2; ++i) {
        if (!buffers[i]) continue;
        uint32_t gave_up = 0;
        HIP_TRY(pool, hipMemcpy(&gave_up, buffers[i], sizeof(gave_up), hipMemcpyDeviceToHost),
                "read the split merge's give-up counter");
        if (!gave_up) continue;
        total += gave_up;
        HIP_TRY(pool, launch_fill_words(buffers[i], words[i], kExchangeEmptyWord, pool->stream),
                "fill the split exchange buffer");
        HIP_TRY(pool, launch_fill_words(buffers[i], 1, 0, pool->stream), "zero the give-up counter");
        HIP_TRY(pool, hipStreamSynchronize(pool->stream), "synchronize");
    }
    if (total)
        return set_error(pool->err, ITAK_STEP_FAILED, "attention", total, 0, 0, 0,
                         "attention: %u workgroups of a split merge gave up waiting for their "
                         "group; their outputs are NaN and every step launched on this pool since "
                         "the last successful synchronize is invalid",
                         total);
    if (pool->die_words) {
        // A launch that merges on the units' compute dies relies on where the device runs each
        // workgroup; every workgroup checks, and one that ran elsewhere has counted itself.
        uint32_t strays = 0;
        uint32_t *faults = pool->die_words + kDieTicketBytes / sizeof(uint32_t);
        HIP_TRY(pool, hipMemcpy(&strays, faults, sizeof(strays), hipMemcpyDeviceToHost),
                "read the die check's counter");
        if (strays) {
            pool->die_merge = false;  // the ordinary merge launch from here on
            HIP_TRY(pool, hipMemset(pool->die_words, 0, kDieTicketBytes + 256), "clear the split tickets");
            return set_error(pool->err, ITAK_STEP_FAILED, "attention", strays, 0, 0, 0,
                             "attention: %u workgroups of a split merge ran on another compute die "
                             "than their index names; outputs of the steps since the last "
                             "synchronize may be wrong (later steps use the merge launch)",
                             strays);
        }
    }
    return ITAK_OK;
}

itak_status itak_pool_set_merge_spin_limit(itak_pool *pool, uint32_t polls) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    pool->spin_limit = polls;
    return ITAK_OK;
}

uint64_t itak_pool_device_bytes(const itak_pool *pool) { return pool ? pool->bytes : 0; }

itak_status itak_slot_acquire(itak_pool *pool, uint32_t *slot) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (!slot) return invalid_argument(pool->err, "slot is null");
    for (uint32_t i = 0; i < pool->slots.size(); ++i) {
        Slot &s = pool->slots[i];
        if (s.in_use) continue;
        s = Slot{};
        s.in_use = true;
        s.cache_id = g_next_cache_id++;
        s.appended.assign(pool->cfg.layer_count, 0);
        s.high.assign(pool->cfg.layer_count, 0);
        s.floor.assign(pool->cfg.layer_count, 0);
        *slot = i;
        return ITAK_OK;
    }
    return set_error(pool->err, ITAK_NO_FREE_SLOT, nullptr, pool->slots.size(), 0, 0, 0,
                     "all %llu slots of the pool are in use", ULL(pool->slots.size()));
}

itak_status itak_slot_reset(itak_pool *pool, uint32_t slot) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    uint64_t max_rows = 0;
    bool ring_used = false;
    for (uint64_t l = 0; l < s->high.size(); ++l) {
        if (pool->layers[l].windowed)
            ring_used = ring_used || s->high[l] > 0;
        else
            max_rows = std::max(max_rows, s->high[l]);
    }
    if (max_rows > 0) {
        ZeroBatch zb{};
        zb.n = 1;
        zb.max_rows = uint32_t(max_rows);
        zb.item[0] = ZeroItem{slot, 0, uint32_t(max_rows), 0};
        itak_status st = scrub_rows(pool, zb);
        if (st != ITAK_OK) return st;
    }
    if (ring_used) {  // the whole ring of every windowed layer
        ZeroBatch zb{};
        zb.n = 1;
        zb.max_rows = pool->gw.capacity;
        zb.item[0] = ZeroItem{slot, 0, pool->gw.capacity, 0};
        HIP_TRY(pool,
                launch_zero_rows(pool->base_w, pool->elem_f16, pool->gw, 0, pool->windowed_layers,
                                 zb, pool->stream),
                "launch ring scrub");
    }
    std::fill(s->appended.begin(), s->appended.end(), 0);
    std::fill(s->high.begin(), s->high.end(), 0);
    std::fill(s->floor.begin(), s->floor.end(), 0);
    s->built = false;
    s->cp = LiveCheckpoint{};
    s->next_serial = 0;
    s->cache_id = g_next_cache_id++;  // outstanding handles go stale (cache.rs:721-728)
    return ITAK_OK;
}

itak_status itak_slot_release(itak_pool *pool, uint32_t slot) {
    itak_status st = itak_slot_reset(pool, slot);
    if (st != ITAK_OK) return st;
    pool->slots[slot].in_use = false;
    return ITAK_OK;
}

uint64_t itak_kv_layer_count(const itak_pool *pool) { return pool ? pool->cfg.layer_count : 0; }
uint64_t itak_kv_num_kv_heads(const itak_pool *pool) { return pool ? pool->g.kv_heads : 0; }
uint64_t itak_kv_head_dim(const itak_pool *pool) { return pool ? pool->g.head_dim : 0; }

itak_status itak_kv_layer_kind(itak_pool *pool, uint64_t layer, uint32_t *kind, uint64_t *window) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (layer >= pool->cfg.layer_count) return invalid_layer(pool->err, layer, pool->cfg.layer_count);
    if (kind) *kind = pool->layers[layer].windowed ? ITAK_LAYER_WINDOWED : ITAK_LAYER_GLOBAL;
    if (window) *window = pool->layers[layer].window;
    return ITAK_OK;
}

itak_status itak_kv_storage_rows(itak_pool *pool, uint64_t layer, uint64_t *out) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (layer >= pool->cfg.layer_count) return invalid_layer(pool->err, layer, pool->cfg.layer_count);
    if (!out) return invalid_argument(pool->err, "out is null");
    *out = pool->layers[layer].windowed ? pool->layers[layer].ring : pool->rows_limit;
    return ITAK_OK;
}

itak_status itak_kv_stored_len(itak_pool *pool, uint32_t slot, uint64_t layer, uint64_t *out) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (!out) return invalid_argument(pool->err, "out is null");
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    if (layer >= pool->cfg.layer_count) return invalid_layer(pool->err, layer, pool->cfg.layer_count);
    *out = stored_of(pool, *s, layer);  // cache.rs:154-159
    return ITAK_OK;
}

itak_status itak_kv_next_position(itak_pool *pool, uint32_t slot, uint64_t layer, uint64_t *out) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (!out) return invalid_argument(pool->err, "out is null");
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    if (layer >= pool->cfg.layer_count) return invalid_layer(pool->err, layer, pool->cfg.layer_count);
    *out = s->appended[layer];
    return ITAK_OK;
}

itak_status itak_kv_append(itak_pool *pool, uint32_t slot, uint64_t layer, const float *k,
                           uint64_t k_len, const float *v, uint64_t v_len, uint64_t position) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    // cache.rs:430-471, in order.
    if (k_len != pool->row) return shape_mismatch(pool->err, "k", pool->row, k_len);
    if (v_len != pool->row) return shape_mismatch(pool->err, "v", pool->row, v_len);
    if (s->cp.live && layer < pool->cfg.layer_count) {
        const uint64_t limit = s->cp.bases[layer] + s->cp.max_round_tokens;
        if (position >= limit) return range_exceeded(pool->err, layer, position, limit);
    }
    if (layer >= pool->cfg.layer_count) return invalid_layer(pool->err, layer, pool->cfg.layer_count);
    if (position != s->appended[layer])
        return out_of_order(pool->err, layer, s->appended[layer], position);
    if (position >= position_limit(pool, layer))
        return capacity_exceeded(pool->err, layer, position + 1, position_limit(pool, layer));
    if (!k || !v) return invalid_argument(pool->err, "k or v is null");
    const uint64_t bytes = pool->row * sizeof(float);
    itak_status st = ensure_stage(pool, 2 * bytes);
    if (st != ITAK_OK) return st;
    float *kd = reinterpret_cast<float *>(pool->stage);
    float *vd = kd + pool->row;
    HIP_TRY(pool, hipMemcpyAsync(kd, k, bytes, hipMemcpyHostToDevice, pool->stream), "upload k");
    HIP_TRY(pool, hipMemcpyAsync(vd, v, bytes, hipMemcpyHostToDevice, pool->stream), "upload v");
    itak_batch_item item{slot, 1};
    st = run_append(pool, layer, &item, 1, kd, vd);
    if (st != ITAK_OK) return st;
    HIP_TRY(pool, hipStreamSynchronize(pool->stream), "synchronize after append");
    return ITAK_OK;
}

itak_status itak_kv_append_device(itak_pool *pool, uint64_t layer, const itak_batch_item *items,
                                  uint32_t item_count, const float *k_dev, const float *v_dev) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (layer >= pool->cfg.layer_count) return invalid_layer(pool->err, layer, pool->cfg.layer_count);
    if (item_count && (!items || !k_dev || !v_dev))
        return invalid_argument(pool->err, "items, k_dev or v_dev is null");
    std::vector<uint8_t> seen(pool->slots.size(), 0);
    for (uint32_t i = 0; i < item_count; ++i) {
        Slot *s = find_slot(pool, items[i].slot);
        if (!s) return invalid_argument(pool->err, "slot is not in use");
        if (seen[items[i].slot]++) return invalid_argument(pool->err, "slot listed twice in one step");
        uint64_t ok = 0;
        itak_status st = check_append_rows(pool, *s, layer, items[i].rows, &ok);
        if (st != ITAK_OK) return st;
        st = check_block_rows(pool, layer, items[i].rows);
        if (st != ITAK_OK) return st;
    }
    return run_append(pool, layer, items, item_count, k_dev, v_dev);
}

static itak_status restore_layers(itak_pool *pool, uint32_t slot, Slot &s,
                                  const itak_snapshot_layer *layers, const uint64_t *layer_ids,
                                  uint64_t count, uint32_t src_elem) {
    if (src_elem != ITAK_ELEM_F32 && src_elem != ITAK_ELEM_F16)
        return invalid_argument(pool->err, "src_elem is neither ITAK_ELEM_F32 nor ITAK_ELEM_F16");
    if (src_elem == ITAK_ELEM_F16 && !pool->elem_f16)
        return unsupported(pool->err, "an f16 snapshot restores only into an f16 pool");
    const uint64_t src_bytes_per_elem = src_elem == ITAK_ELEM_F16 ? 2 : 4;
    // Sources the device cannot read in place are staged through one temporary buffer.
    uint64_t stage_need = 0;
    PtrClassifier kind_of;
    // Rows that all lie in device memory are gathered in stream order, like a device append: the
    // call returns with the gather enqueued. Host memory of either kind is the caller's to free
    // when the call returns, so the call waits for the stream then.
    bool all_device = true;
    for (uint64_t i = 0; i < count; ++i) {
        if (layers[i].rows == 0) continue;
        const uint64_t bytes = layers[i].rows * pool->row * src_bytes_per_elem;
        if (must_stage(kind_of, layers[i].keys, src_bytes_per_elem)) stage_need += align_up(bytes, 256);
        if (must_stage(kind_of, layers[i].values, src_bytes_per_elem)) stage_need += align_up(bytes, 256);
        const void *usable;
        if (kind_of(layers[i].keys, &usable) != PtrKind::Device ||
            kind_of(layers[i].values, &usable) != PtrKind::Device)
            all_device = false;
    }
    unsigned char *temp = nullptr;
    if (stage_need) HIP_TRY(pool, hipMalloc(reinterpret_cast<void **>(&temp), stage_need), "allocate restore staging");
    uint64_t temp_off = 0;
    itak_status st = ITAK_OK;
    // One gather batch per group of planes (global, windowed), launched when it fills up. A
    // windowed layer's rows go to storage rows position % ring: one run, or two when the
    // positions wrap past the end of the ring (session.rs:320-346 states the same split).
    RestoreBatch batch[2] = {};
    batch[0].slot = batch[1].slot = slot;
    // A ring that was filled and then rewound to empty still holds the old rows; a restore
    // that writes fewer rows than the window must find zeros around them, as in a fresh cache.
    for (uint64_t i = 0; i < count; ++i) {
        const uint64_t layer = layer_ids ? layer_ids[i] : i;
        const LayerInfo &info = pool->layers[layer];
        if (!info.windowed || s.high[layer] == 0) continue;
        ZeroBatch zb{};
        zb.n = 1;
        zb.max_rows = info.ring;
        zb.item[0] = ZeroItem{slot, 0, info.ring, 0};
        hipError_t e = launch_zero_rows(pool->base_w, pool->elem_f16, pool->gw, info.index,
                                        info.index + 1, zb, pool->stream);
        if (e != hipSuccess) {
            if (temp) (void)hipFree(temp);
            return hip_error(pool->err, e, "launch ring scrub");
        }
    }
    auto flush = [&](int w) -> itak_status {
        if (batch[w].n == 0) return ITAK_OK;
        hipError_t e = launch_restore(w ? pool->base_w : pool->base, pool->elem_f16,
                                      src_elem == ITAK_ELEM_F16, w ? pool->gw : pool->g, batch[w],
                                      pool->stream);
        batch[w].n = 0;
        batch[w].max_rows = 0;
        return e == hipSuccess ? ITAK_OK : hip_error(pool->err, e, "launch restore gather");
    };
    for (uint64_t i = 0; i < count && st == ITAK_OK; ++i) {
        const itak_snapshot_layer &L = layers[i];
        if (L.rows == 0) continue;
        const uint64_t layer = layer_ids ? layer_ids[i] : i;
        const LayerInfo &info = pool->layers[layer];
        const uint64_t bytes = L.rows * pool->row * src_bytes_per_elem;
        const void *src[2] = {L.keys, L.values};
        for (int side = 0; side < 2; ++side) {
            const void *usable;
            if (!must_stage(kind_of, src[side], src_bytes_per_elem)) {
                kind_of(src[side], &usable);
                src[side] = usable;
                continue;
            }
            hipError_t he = hipMemcpyAsync(temp + temp_off, src[side], bytes, hipMemcpyHostToDevice,
                                           pool->stream);
            if (he != hipSuccess) {
                st = hip_error(pool->err, he, "stage snapshot rows");
                break;
            }
            src[side] = temp + temp_off;
            temp_off += align_up(bytes, 256);
        }
        if (st != ITAK_OK) break;
        const int w = info.windowed ? 1 : 0;
        uint64_t done = 0;
        while (done < L.rows && st == ITAK_OK) {
            const uint64_t position = L.first_position + done;
            const uint64_t row = info.windowed ? position % info.ring : position;
            const uint64_t run =
                info.windowed ? std::min<uint64_t>(L.rows - done, info.ring - row) : L.rows - done;
            if (batch[w].n == kMaxRestoreLayers) st = flush(w);
            if (st != ITAK_OK) break;
            RestoreLayer &R = batch[w].layer[batch[w].n++];
            const uint64_t skip = done * pool->row * src_bytes_per_elem;
            R.keys = static_cast<const unsigned char *>(src[0]) + skip;
            R.values = static_cast<const unsigned char *>(src[1]) + skip;
            R.layer = info.index;
            R.rows = uint32_t(run);
            R.first_row = uint32_t(row);
            batch[w].max_rows = std::max(batch[w].max_rows, R.rows);
            done += run;
        }
    }
    for (int w = 0; w < 2 && st == ITAK_OK; ++w) st = flush(w);
    if (!all_device || stage_need || st != ITAK_OK) {
        hipError_t he = hipStreamSynchronize(pool->stream);
        if (st == ITAK_OK && he != hipSuccess) st = hip_error(pool->err, he, "synchronize after restore");
    }
    if (temp) (void)hipFree(temp);
    if (st != ITAK_OK) return st;
    for (uint64_t i = 0; i < count; ++i) {
        const uint64_t layer = layer_ids ? layer_ids[i] : i;
        s.appended[layer] = layers[i].first_position + layers[i].rows;  // cache.rs:568
        s.high[layer] = s.appended[layer];
        s.floor[layer] = layers[i].first_position;
        ITAK_DIAG("bulk restore slot=%u layer=%llu first_position=%llu rows=%llu appended=%llu", slot,
                  ULL(layer), ULL(layers[i].first_position), ULL(layers[i].rows),
                  ULL(s.appended[layer]));
    }
    return ITAK_OK;
}

itak_status itak_kv_restore_bulk(itak_pool *pool, uint32_t slot, uint64_t layer,
                                 uint64_t first_position, const void *keys, uint64_t keys_len,
                                 const void *values, uint64_t values_len, uint32_t src_elem) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    // cache.rs:520-546, in order.
    if (keys_len != values_len || keys_len % pool->row != 0)
        return shape_mismatch(pool->err, "bulk restore rows", values_len, keys_len);
    const uint64_t rows = keys_len / pool->row;
    if (layer >= pool->cfg.layer_count) return invalid_layer(pool->err, layer, pool->cfg.layer_count);
    if (s->appended[layer] != 0) return not_fresh(pool->err, layer, s->appended[layer]);
    if (pool->layers[layer].windowed) {
        if (rows > pool->layers[layer].window)
            return shape_mismatch(pool->err, "bulk restore rows (windowed layer)",
                                  pool->layers[layer].window, rows);
    } else if (first_position != 0) {
        return shape_mismatch(pool->err, "bulk restore first position (global layer)", 0,
                              first_position);
    }
    if (first_position > position_limit(pool, layer) ||
        rows > position_limit(pool, layer) - first_position)
        return capacity_exceeded(pool->err, layer, first_position + rows,
                                 position_limit(pool, layer));
    if (rows && (!keys || !values)) return invalid_argument(pool->err, "keys or values is null");
    itak_snapshot_layer L{first_position, rows, keys, values};
    return restore_layers(pool, slot, *s, &L, &layer, 1, src_elem);
}

itak_status itak_kv_restore_snapshot(itak_pool *pool, uint32_t slot, uint64_t token_count,
                                     const itak_snapshot_layer *layers, uint64_t layer_count,
                                     uint32_t src_elem) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    if (!layers) return invalid_argument(pool->err, "layers is null");
    // KvSnapshot::validate (snapshot.rs:187-236) against the pool's own pattern.
    if (layer_count != pool->cfg.layer_count)
        return set_error(pool->err, ITAK_STEP_FAILED, "restore_snapshot", layer_count,
                         pool->cfg.layer_count, 0, 0,
                         "snapshot carries %llu layer blocks but its geometry has %llu layers",
                         ULL(layer_count), ULL(pool->cfg.layer_count));
    for (uint64_t i = 0; i < layer_count; ++i) {
        const LayerInfo &info = pool->layers[i];
        const uint64_t expected_rows =
            info.windowed ? std::min(token_count, info.window) : token_count;
        const uint64_t expected_first = token_count - expected_rows;
        if (layers[i].first_position != expected_first) {
            char kind[64] = "Global";
            if (info.windowed)
                snprintf(kind, sizeof(kind), "Windowed { window: %llu }", ULL(info.window));
            return set_error(pool->err, ITAK_STEP_FAILED, "restore_snapshot", i,
                             layers[i].first_position, expected_first, 0,
                             "layer %llu: first stored position is %llu but %llu follows from token "
                             "count %llu and kind %s",
                             ULL(i), ULL(layers[i].first_position), ULL(expected_first),
                             ULL(token_count), kind);
        }
        if (layers[i].rows != expected_rows)
            return set_error(pool->err, ITAK_STEP_FAILED, "restore_snapshot", i, layers[i].rows,
                             expected_rows, 0,
                             "layer %llu: holds %llu rows but %llu rows were expected", ULL(i),
                             ULL(layers[i].rows), ULL(expected_rows));
        if (expected_rows && (!layers[i].keys || !layers[i].values))
            return invalid_argument(pool->err, "a layer's keys or values is null");
    }
    // KvSnapshot::restore builds a fresh cache (snapshot.rs:321-334): every layer must be
    // fresh here, checked for all layers before any is touched.
    for (uint64_t i = 0; i < layer_count; ++i)
        if (s->appended[i] != 0) return not_fresh(pool->err, i, s->appended[i]);
    for (uint64_t i = 0; i < layer_count; ++i)
        if (token_count > position_limit(pool, i))
            return capacity_exceeded(pool->err, i, token_count, position_limit(pool, i));
    return restore_layers(pool, slot, *s, layers, nullptr, layer_count, src_elem);
}

// ---- itak_kv: hashes, the ITKV codec, capture and restore of encoded snapshots ----------

uint64_t itak_kv_prefix_hash(const uint32_t *tokens, uint64_t count) {  // hash.rs:44-46
    return fnv1a64_tokens(tokens, tokens ? count : 0, kFnvOffset);
}
uint64_t itak_kv_prefix_discriminator(const uint32_t *tokens, uint64_t count) {  // hash.rs:52-54
    return fnv1a64_tokens(tokens, tokens ? count : 0, kFnvAltOffset);
}
uint64_t itak_kv_checksum(const void *bytes, uint64_t count) {  // hash.rs:59-61
    return fnv1a64(static_cast<const uint8_t *>(bytes), bytes ? count : 0, kFnvOffset);
}
uint64_t itak_kv_checksum_blocks(const void *bytes, uint64_t count) {
    return fnv1a64_blocks(static_cast<const uint8_t *>(bytes), bytes ? count : 0);
}

itak_status itak_itkv_validate(const itak_itkv_header *header, const itak_itkv_layer *layers,
                               uint64_t blocks, const uint64_t *key_floats,
                               const uint64_t *value_floats) {
    ErrorState &e = g_create_error;
    if (!header || (blocks && (!layers || !key_floats || !value_floats)))
        return invalid_argument(e, "header, layers or the float counts are null");
    ItkvError err;
    const std::vector<ItkvLayer> ls = to_internal(layers, blocks);
    if (!itkv_validate(to_internal(*header), ls.data(), blocks, key_floats, value_floats, err))
        return set_itkv_error(e, err);
    return ITAK_OK;
}

itak_status itak_itkv_encode(const itak_itkv_header *header, const char *fingerprint,
                             const itak_itkv_layer *layers, uint64_t blocks,
                             const float *const *keys, const uint64_t *key_floats,
                             const float *const *values, const uint64_t *value_floats, void *out,
                             uint64_t capacity, uint64_t *written) {
    ErrorState &e = g_create_error;
    itak_status st = itak_itkv_validate(header, layers, blocks, key_floats, value_floats);
    if (st != ITAK_OK) return st;
    if (!written) return invalid_argument(e, "written is null");
    if (header->fingerprint_len && !fingerprint) return invalid_argument(e, "fingerprint is null");
    if (header->version > 1 || header->elem != 0)
        return unsupported(e, "itak_itkv_encode writes version 1 (f32 rows); version 2 comes from "
                              "itak_kv_capture_itkv_f16");
    if (header->num_kv_heads > UINT32_MAX || header->head_dim > UINT32_MAX ||
        header->layer_count > UINT32_MAX || header->fingerprint_len > UINT32_MAX)
        return invalid_argument(e, "a header field does not fit the 32-bit wire field");
    ItkvHeader h = to_internal(*header);
    std::vector<ItkvLayer> ls = to_internal(layers, blocks);
    uint64_t total = 0;
    if (!itkv_encoded_len(h, ls.data(), &total)) return size_overflow(e, "encoded snapshot");
    *written = total;
    if (!out) return ITAK_OK;
    if (capacity < total) return invalid_argument(e, "output buffer is smaller than the encoding");
    uint8_t *bytes = static_cast<uint8_t *>(out);
    itkv_write_header(bytes, h, fingerprint, ls.data());
    for (uint64_t i = 0; i < blocks; ++i) {
        if (key_floats[i] && (!keys || !keys[i] || !values || !values[i]))
            return invalid_argument(e, "a layer's keys or values is null");
        if (key_floats[i]) {  // f32 little-endian is this host's own representation
            memcpy(bytes + ls[i].keys_offset, keys[i], key_floats[i] * 4);
            memcpy(bytes + ls[i].values_offset, values[i], value_floats[i] * 4);
        }
    }
    const uint64_t sum = fnv1a64(bytes, total - 8, kFnvOffset);
    for (int b = 0; b < 8; ++b) bytes[total - 8 + b] = uint8_t(sum >> (8 * b));
    return ITAK_OK;
}

itak_status itak_itkv_decode(const void *bytes, uint64_t len, itak_itkv_header *header,
                             itak_itkv_layer *layers, uint64_t layers_capacity) {
    ErrorState &e = g_create_error;
    if (!bytes || !header) return invalid_argument(e, "bytes or header is null");
    ItkvHeader h;
    std::vector<ItkvLayer> ls;
    ItkvError err;
    if (!itkv_decode(static_cast<const uint8_t *>(bytes), len, h, ls, err))
        return set_itkv_error(e, err);
    *header = itak_itkv_header{h.token_count,     h.num_kv_heads,       h.head_dim,      h.layer_count,
                               h.fingerprint_len, h.fingerprint_offset, h.encoded_len,   h.version,
                               h.elem};
    if (layers_capacity < ls.size())
        return invalid_argument(e, "layers_capacity is smaller than the snapshot's layer count");
    for (size_t i = 0; i < ls.size(); ++i)
        layers[i] = itak_itkv_layer{ls[i].kind, 0, ls[i].window, ls[i].first_position, ls[i].rows,
                                    ls[i].keys_offset, ls[i].values_offset};
    return ITAK_OK;
}

static itak_status capture_itkv(itak_pool *pool, uint32_t slot, const char *fingerprint,
                                uint64_t fingerprint_len, bool f16_rows, void *out,
                                uint64_t capacity, uint64_t *written, bool with_checksum = true);

itak_status itak_kv_capture_itkv(itak_pool *pool, uint32_t slot, const char *fingerprint,
                                 uint64_t fingerprint_len, void *out, uint64_t capacity,
                                 uint64_t *written) {
    return capture_itkv(pool, slot, fingerprint, fingerprint_len, false, out, capacity, written);
}

itak_status itak_kv_capture_itkv_f16(itak_pool *pool, uint32_t slot, const char *fingerprint,
                                     uint64_t fingerprint_len, void *out, uint64_t capacity,
                                     uint64_t *written) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (!pool->elem_f16)
        return unsupported(pool->err,
                           "an f16 snapshot of an f32 pool would drop precision the cache holds");
    return capture_itkv(pool, slot, fingerprint, fingerprint_len, true, out, capacity, written);
}

static itak_status capture_itkv(itak_pool *pool, uint32_t slot, const char *fingerprint,
                                uint64_t fingerprint_len, bool f16_rows, void *out,
                                uint64_t capacity, uint64_t *written, bool with_checksum) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    if (!written) return invalid_argument(pool->err, "written is null");
    if (fingerprint_len && !fingerprint) return invalid_argument(pool->err, "fingerprint is null");
    if (fingerprint_len > UINT32_MAX) return invalid_argument(pool->err, "fingerprint too long");
    // snapshot.rs:249-262: one sequence, every layer at the same position.
    const uint64_t token_count = s->appended[0];
    for (uint64_t i = 0; i < pool->cfg.layer_count; ++i)
        if (s->appended[i] != token_count)
            return set_error(pool->err, ITAK_KV_INCOHERENT_CACHE, "snapshot", token_count,
                             s->appended[i], i, 0,
                             "incoherent cache: layer 0 has appended %llu positions but layer %llu "
                             "has appended %llu; a snapshot is one sequence",
                             ULL(token_count), ULL(i), ULL(s->appended[i]));
    ItkvHeader h;
    h.token_count = token_count;
    h.num_kv_heads = pool->g.kv_heads;
    h.head_dim = pool->g.head_dim;
    h.layer_count = pool->cfg.layer_count;
    h.fingerprint_len = fingerprint_len;
    if (f16_rows) {
        h.version = kItkvVersionTyped;
        h.elem = ITAK_ELEM_F16;
    }
    const uint64_t out_elem = h.elem_bytes();
    // snapshot.rs:264-295: every row of a global layer, the last `window` rows of a windowed
    // one, oldest first.
    std::vector<ItkvLayer> ls(h.layer_count);
    for (uint64_t i = 0; i < h.layer_count; ++i) {
        const LayerInfo &info = pool->layers[i];
        ls[i].kind = info.windowed ? ITAK_LAYER_WINDOWED : ITAK_LAYER_GLOBAL;
        ls[i].window = info.window;
        ls[i].rows = stored_of(pool, *s, i);
        ls[i].first_position = token_count - ls[i].rows;
    }
    uint64_t total = 0;
    if (!itkv_encoded_len(h, ls.data(), &total)) return size_overflow(pool->err, "encoded snapshot");
    *written = total;
    if (!out) return ITAK_OK;
    if (capacity < total)
        return invalid_argument(pool->err, "output buffer is smaller than the encoding");
    uint8_t *bytes = static_cast<uint8_t *>(out);
    itkv_write_header(bytes, h, fingerprint, ls.data());
    // Rows come back through the readback kernel in chunks that bound the staging buffer:
    // planes -> [row][kv_head][d] in the pool's element type, widened to f32 for an f16 pool.
    const uint64_t chunk_rows = std::max<uint64_t>(1, (uint64_t(16) << 20) / (pool->row * 4));
    const uint64_t raw = align_up(chunk_rows * pool->row * pool->elem_bytes, 256);
    const uint64_t wide = align_up(chunk_rows * pool->row * 4, 256);
    itak_status st = ensure_stage(pool, 2 * raw + (pool->elem_f16 ? 2 * wide : 0));
    if (st != ITAK_OK) return st;
    for (uint64_t layer = 0; layer < h.layer_count; ++layer) {
        for (uint64_t first = 0; first < ls[layer].rows; first += chunk_rows) {
            const uint64_t rows = std::min(chunk_rows, ls[layer].rows - first);
            const uint64_t elems = rows * pool->row;
            unsigned char *kd = pool->stage, *vd = pool->stage + raw;
            HIP_TRY(pool,
                    launch_read_rows(layer_base(pool, layer), pool->elem_f16, geom_of(pool, layer),
                                     slot, uint32_t(ls[layer].first_position + first),
                                     uint32_t(rows), pool->layers[layer].ring, kd, vd,
                                     pool->stream),
                    "launch row readback");
            const void *ksrc = kd, *vsrc = vd;
            if (pool->elem_f16 && !f16_rows) {
                float *kw = reinterpret_cast<float *>(pool->stage + 2 * raw);
                float *vw = reinterpret_cast<float *>(pool->stage + 2 * raw + wide);
                HIP_TRY(pool,
                        launch_widen_f16(reinterpret_cast<const uint16_t *>(kd), kw, elems, pool->stream),
                        "launch widening");
                HIP_TRY(pool,
                        launch_widen_f16(reinterpret_cast<const uint16_t *>(vd), vw, elems, pool->stream),
                        "launch widening");
                ksrc = kw;
                vsrc = vw;
            }
            HIP_TRY(pool,
                    hipMemcpyAsync(bytes + ls[layer].keys_offset + first * pool->row * out_elem,
                                   ksrc, elems * out_elem, hipMemcpyDeviceToHost, pool->stream),
                    "download keys");
            HIP_TRY(pool,
                    hipMemcpyAsync(bytes + ls[layer].values_offset + first * pool->row * out_elem,
                                   vsrc, elems * out_elem, hipMemcpyDeviceToHost, pool->stream),
                    "download values");
            // The staging buffer is reused by the next chunk.
            HIP_TRY(pool, hipStreamSynchronize(pool->stream), "synchronize after readback");
        }
    }
    const uint64_t sum = with_checksum ? itkv_trailer(h.version, bytes, total - 8) : 0;
    for (int b = 0; b < 8; ++b) bytes[total - 8 + b] = uint8_t(sum >> (8 * b));
    return ITAK_OK;
}

itak_status itak_kv_restore_itkv(itak_pool *pool, uint32_t slot, const void *bytes, uint64_t len,
                                 const char *expected_fingerprint,
                                 uint64_t expected_fingerprint_len) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    if (!bytes) return invalid_argument(pool->err, "bytes is null");
    // The decoder walks the bytes on the host (header fields, then the checksum over all of
    // them); a device-resident buffer would have to be copied first.
    const void *unused;
    if (classify(bytes, &unused) == PtrKind::Device)
        return invalid_argument(pool->err, "an encoded snapshot is decoded on the host: pass host memory");
    ItkvHeader h;
    std::vector<ItkvLayer> ls;
    ItkvError err;
    const uint8_t *b8 = static_cast<const uint8_t *>(bytes);
    if (!itkv_decode(b8, len, h, ls, err)) return set_itkv_error(pool->err, err);
    return restore_decoded_itkv(pool, slot, b8, h, ls, expected_fingerprint, expected_fingerprint_len);
}

itak_status itak_kv_stats(itak_pool *pool, uint32_t slot, itak_layer_stats *out) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    if (!out) return invalid_argument(pool->err, "out is null");
    for (uint32_t i = 0; i < pool->cfg.layer_count; ++i) {
        const LayerInfo &info = pool->layers[i];
        out[i] = itak_layer_stats{i, uint32_t(info.windowed ? ITAK_LAYER_WINDOWED : ITAK_LAYER_GLOBAL),
                                  0, info.window, s->appended[i], stored_of(pool, *s, i)};
    }
    return ITAK_OK;
}

// `first` is a position (a storage row on a global layer, which is the same thing); `ring`
// maps positions to storage rows on a windowed layer, 0 reads storage rows as they lie.
static itak_status read_rows_common(itak_pool *pool, uint32_t slot, uint64_t layer, uint64_t first,
                                    uint64_t rows, uint32_t ring, void *keys_out,
                                    void *values_out) {
    if (rows == 0 || (!keys_out && !values_out)) return ITAK_OK;
    const uint64_t bytes = rows * pool->row * pool->elem_bytes;
    itak_status st = ensure_stage(pool, 2 * align_up(bytes, 256));
    if (st != ITAK_OK) return st;
    void *kd = keys_out ? pool->stage : nullptr;
    void *vd = values_out ? pool->stage + align_up(bytes, 256) : nullptr;
    HIP_TRY(pool,
            launch_read_rows(layer_base(pool, layer), pool->elem_f16, geom_of(pool, layer), slot,
                             uint32_t(first), uint32_t(rows), ring, kd, vd, pool->stream),
            "launch row readback");
    if (keys_out)
        HIP_TRY(pool, hipMemcpyAsync(keys_out, kd, bytes, hipMemcpyDeviceToHost, pool->stream),
                "download keys");
    if (values_out)
        HIP_TRY(pool, hipMemcpyAsync(values_out, vd, bytes, hipMemcpyDeviceToHost, pool->stream),
                "download values");
    HIP_TRY(pool, hipStreamSynchronize(pool->stream), "synchronize after readback");
    return ITAK_OK;
}

itak_status itak_kv_read_rows(itak_pool *pool, uint32_t slot, uint64_t layer, uint64_t first,
                              uint64_t rows, void *keys_out, void *values_out,
                              uint64_t *positions_out) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    if (layer >= pool->cfg.layer_count) return invalid_layer(pool->err, layer, pool->cfg.layer_count);
    const uint64_t stored = stored_of(pool, *s, layer);
    if (first > stored || rows > stored - first)
        return shape_mismatch(pool->err, "visible rows", stored,
                              rows > UINT64_MAX - first ? UINT64_MAX : first + rows);  // (no wrapped sum in the text)
    const uint64_t oldest = first_visible(pool, *s, layer);
    if (positions_out)
        for (uint64_t i = 0; i < rows; ++i) positions_out[i] = oldest + first + i;  // cache.rs:878-883
    return read_rows_common(pool, slot, layer, oldest + first, rows, pool->layers[layer].ring,
                            keys_out, values_out);
}

itak_status itak_kv_read_raw(itak_pool *pool, uint32_t slot, uint64_t layer, void *keys_out,
                             void *values_out) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    if (layer >= pool->cfg.layer_count) return invalid_layer(pool->err, layer, pool->cfg.layer_count);
    const uint64_t rows = pool->layers[layer].windowed ? pool->layers[layer].ring : pool->rows_limit;
    return read_rows_common(pool, slot, layer, 0, rows, 0, keys_out, values_out);
}

// Moves ring rows of the layers in `saves` between their rings and the slot's side buffer:
// positions [from, to) of each layer that fall inside what its save covers.
static itak_status move_ring_rows(itak_pool *pool, uint32_t slot, const Slot &s,
                                  const std::vector<RingSave> &saves, const uint64_t *bases,
                                  uint64_t from, const uint64_t *to_per_layer, bool to_ring) {
    RingRowsBatch b{};
    b.slot = slot;
    auto flush = [&]() -> itak_status {
        if (b.n == 0) return ITAK_OK;
        hipError_t e = launch_ring_rows(pool->base_w, pool->elem_f16, pool->gw, b,
                                        pool->ring_saved[slot], to_ring, pool->stream);
        b.n = 0;
        b.max_rows = 0;
        return e == hipSuccess ? ITAK_OK : hip_error(pool->err, e, "launch ring row copy");
    };
    (void)s;
    for (const RingSave &rs : saves) {
        const uint64_t base = bases[rs.layer];
        const uint64_t lo = std::max(from, base);
        const uint64_t hi = std::min<uint64_t>(to_per_layer[rs.layer], base + rs.rows);
        if (hi <= lo) continue;
        const LayerInfo &L = pool->layers[rs.layer];
        RingRowsLayer &R = b.layer[b.n++];
        R.layer = L.index;
        R.ring = L.ring;
        R.pos0 = uint32_t(lo);
        R.rows = uint32_t(hi - lo);
        R.saved_row0 = uint32_t(lo - base);
        R.saved_rows = rs.rows;
        R.saved_off = rs.saved_off;
        b.max_rows = std::max(b.max_rows, R.rows);
        if (b.n == kMaxRestoreLayers) {
            itak_status st = flush();
            if (st != ITAK_OK) return st;
        }
    }
    return flush();
}

// The checkpoint's copy of the rows a deep round may overwrite (cache.rs:678-697).
static itak_status save_ring_rows(itak_pool *pool, uint32_t slot, const Slot &s,
                                  const std::vector<RingSave> &saves, uint64_t elems) {
    const uint64_t bytes = elems * pool->elem_bytes;
    if (bytes > pool->ring_saved_bytes[slot]) {
        HIP_TRY(pool, hipStreamSynchronize(pool->stream), "synchronize before growing the checkpoint buffer");
        if (pool->ring_saved[slot]) HIP_TRY(pool, hipFree(pool->ring_saved[slot]), "free the checkpoint buffer");
        pool->ring_saved[slot] = nullptr;
        pool->ring_saved_bytes[slot] = 0;
        HIP_TRY(pool, hipMalloc(&pool->ring_saved[slot], bytes), "allocate the checkpoint buffer");
        pool->ring_saved_bytes[slot] = bytes;
    }
    std::vector<uint64_t> to(pool->layers.size());
    for (const RingSave &rs : saves) to[rs.layer] = s.appended[rs.layer] + rs.rows;
    return move_ring_rows(pool, slot, s, saves, s.appended.data(), 0, to.data(), false);
}

itak_status itak_kv_checkpoint_active(itak_pool *pool, uint32_t slot, int32_t *out) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (!out) return invalid_argument(pool->err, "out is null");
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    *out = s->cp.live ? 1 : 0;
    return ITAK_OK;
}

itak_status itak_kv_checkpoint(itak_pool *pool, uint32_t slot, uint64_t max_round_tokens,
                               itak_checkpoint *out) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    if (!out) return invalid_argument(pool->err, "out is null");
    // cache.rs:635-651, in order.
    if (s->cp.live) return checkpoint_busy(pool->err);
    if (max_round_tokens == 0) return zero_dimension(pool->err, "max_round_tokens");
    uint64_t smallest_window = 0, windowed = 0;
    for (const LayerInfo &L : pool->layers)
        if (L.windowed) {
            smallest_window = windowed ? std::min(smallest_window, L.window) : L.window;
            ++windowed;
        }
    if (windowed && max_round_tokens > smallest_window)
        return set_error(pool->err, ITAK_CHECKPOINT_TOO_DEEP, nullptr, max_round_tokens,
                         smallest_window, 0, 0,
                         "checkpoint round bound %llu exceeds the smallest sliding window %llu: a "
                         "round that long would overwrite a ring slot twice and no rewind could be "
                         "exact",
                         ULL(max_round_tokens), ULL(smallest_window));
    // A round the ring's headroom covers needs no copies: the rows it overwrites are outside
    // every window a rewind can bring back. A longer one (up to the smallest window, as the
    // reference allows) sets the rows it may overwrite aside first, layer by layer where the
    // headroom is too short, exactly the slots the reference saves (cache.rs:678-697).
    std::vector<RingSave> saves;
    uint64_t save_elems = 0;
    for (uint64_t li = 0; li < pool->layers.size(); ++li) {
        const LayerInfo &L = pool->layers[li];
        if (!L.windowed || max_round_tokens <= L.ring - L.window) continue;
        RingSave rs;
        rs.layer = uint32_t(li);
        rs.rows = uint32_t(max_round_tokens);
        rs.saved_off = save_elems;
        rs.high0 = s->high[li];
        save_elems += 2 * max_round_tokens * pool->row;
        saves.push_back(rs);
    }
    if (!saves.empty()) {
        itak_status st = save_ring_rows(pool, slot, *s, saves, save_elems);
        if (st != ITAK_OK) return st;
    }
    s->next_serial += 1;
    s->cp.live = true;
    s->cp.serial = s->next_serial;
    s->cp.max_round_tokens = max_round_tokens;
    s->cp.bases = s->appended;
    s->cp.ring_saves = std::move(saves);
    out->cache_id = s->cache_id;
    out->serial = s->cp.serial;
    out->max_round_tokens = max_round_tokens;
    // What the reference's snapshot of the evictable ring slots holds (cache.rs:678-697), as
    // the reference counts it (f32 rows of every windowed layer); the device sets rows aside
    // only on layers whose headroom the round outgrows, in the pool's element type.
    out->saved_bytes = windowed * max_round_tokens * 2 * pool->row * 4;
    ITAK_DIAG("checkpoint slot=%u serial=%llu max_round_tokens=%llu saved_bytes=%llu", slot,
              ULL(out->serial), ULL(max_round_tokens), ULL(out->saved_bytes));
    return ITAK_OK;
}

static itak_status live_data(itak_pool *pool, Slot &s, const itak_checkpoint *cp) {
    if (!cp) return invalid_argument(pool->err, "checkpoint is null");
    if (s.cp.live && s.cp.serial == cp->serial && cp->cache_id == s.cache_id) return ITAK_OK;
    return stale_checkpoint(pool->err, cp->serial);  // cache.rs:721-728
}

itak_status itak_kv_checkpoint_bases(itak_pool *pool, uint32_t slot, const itak_checkpoint *cp,
                                     uint64_t *out) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (!out || !cp) return invalid_argument(pool->err, "cp or out is null");
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    itak_status st = live_data(pool, *s, cp);
    if (st != ITAK_OK) return st;
    std::copy(s->cp.bases.begin(), s->cp.bases.end(), out);
    return ITAK_OK;
}

// A windowed layer can drop positions only while the rows written above the target have not
// wrapped onto rows the target's view still needs: with H the highest position ever written
// plus one, position x is overwritten once x + ring < H, and the view after the rewind starts
// at target - window, so H - target may be at most ring - window.
static itak_status check_ring_rewind(itak_pool *pool, const Slot &s, uint64_t target,
                                     const std::vector<RingSave> *saves = nullptr) {
    for (uint64_t li = 0; li < s.appended.size(); ++li) {
        const LayerInfo &L = pool->layers[li];
        if (!L.windowed || target >= s.appended[li]) continue;
        bool saved = false;  // a live checkpoint holds this layer's overwritten rows
        if (saves)
            for (const RingSave &rs : *saves) saved = saved || rs.layer == li;
        // A layer restored from a snapshot holds nothing older than the snapshot's first row.
        // The query appended next stands at `target` and sees down to target + 1 - window:
        // that must not reach under the first row. The lowest target that passes, first +
        // window - 1, is the resident session's rewind by one after a stored prefix covered
        // the whole prompt (crates/wgpu-compute/src/session.rs:5138-5143); the view at that
        // length has one row in it, the oldest, that was never written and reads as a fresh
        // ring's zeros, as after the reference's restore of fewer rows than the window.
        if (s.floor[li] > 0 && target + 1 < s.floor[li] + L.window)
            return rewind_range(pool->err, li, s.floor[li] + L.window - 1, s.appended[li], target);
        if (!saved && s.high[li] - target > L.ring - L.window)
            return set_error(pool->err, ITAK_CAPACITY_EXCEEDED, nullptr, li, s.high[li] - target,
                             L.ring - L.window, 0,
                             "dropping windowed layer %llu back to position %llu discards rows up to "
                             "%llu positions ahead of it, past the %llu rows of ring headroom; reset "
                             "the slot instead",
                             ULL(li), ULL(target), ULL(s.high[li] - target), ULL(L.ring - L.window));
    }
    return ITAK_OK;
}

// Drops positions >= target on every layer of the slot (the caller validated the range).
// Global layers truncate (cache.rs:788-791); windowed layers only move their length back: the
// dropped rows stay in the ring's headroom, out of every later query's window, until the
// positions are appended again.
static itak_status truncate_slots(itak_pool *pool, const uint32_t *slots, const uint64_t *targets,
                                  uint32_t count) {
    if ((pool->cfg.flags & ITAK_POOL_SCRUB_ON_TRUNCATE) && pool->global_layers) {
        for (uint32_t first = 0; first < count; first += kMaxBatchItems) {
            const uint32_t n = std::min<uint32_t>(kMaxBatchItems, count - first);
            ZeroBatch zb{};
            for (uint32_t i = 0; i < n; ++i) {
                const Slot &s = pool->slots[slots[first + i]];
                uint64_t max_len = 0;
                for (uint64_t li = 0; li < s.appended.size(); ++li)
                    if (!pool->layers[li].windowed) max_len = std::max(max_len, s.appended[li]);
                if (max_len <= targets[first + i]) continue;
                zb.item[zb.n++] = ZeroItem{slots[first + i], uint32_t(targets[first + i]),
                                           uint32_t(max_len), 0};
                zb.max_rows = std::max<uint32_t>(zb.max_rows, uint32_t(max_len - targets[first + i]));
            }
            itak_status st = scrub_rows(pool, zb);
            if (st != ITAK_OK) return st;
        }
    }
    for (uint32_t i = 0; i < count; ++i) {
        Slot &s = pool->slots[slots[i]];
        for (uint64_t li = 0; li < s.appended.size(); ++li) {
            s.appended[li] = std::min(s.appended[li], targets[i]);  // cache.rs:788-791,814
            // Scrubbed or not, a global layer's dropped rows are never read again.
            if (!pool->layers[li].windowed) s.high[li] = s.appended[li];
        }
    }
    return ITAK_OK;
}

itak_status itak_kv_rewind_to(itak_pool *pool, uint32_t slot, const itak_checkpoint *cp,
                              uint64_t target) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    itak_status st = live_data(pool, *s, cp);
    if (st != ITAK_OK) return st;
    // Validate every layer before touching any (cache.rs:772-783).
    for (uint64_t li = 0; li < s->appended.size(); ++li) {
        const uint64_t base = s->cp.bases[li];
        if (target < base || target > s->appended[li])
            return rewind_range(pool->err, li, base, s->appended[li], target);
    }
    st = check_ring_rewind(pool, *s, target, &s->cp.ring_saves);
    if (st != ITAK_OK) return st;
    ITAK_DIAG("rewind slot=%u serial=%llu target=%llu", slot, ULL(cp->serial), ULL(target));
    if (!s->cp.ring_saves.empty()) {
        // The rows the dropped positions overwrote come back from the checkpoint's copy
        // (cache.rs:792-812); what the ring then holds beyond `target` is what it held when
        // the checkpoint was taken.
        st = move_ring_rows(pool, slot, *s, s->cp.ring_saves, s->cp.bases.data(), target,
                            s->high.data(), true);
        if (st != ITAK_OK) return st;
        for (const RingSave &rs : s->cp.ring_saves)
            s->high[rs.layer] = std::max(target, std::min(rs.high0, s->high[rs.layer]));
    }
    return truncate_slots(pool, &slot, &target, 1);
}

itak_status itak_kv_release(itak_pool *pool, uint32_t slot, const itak_checkpoint *cp) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    itak_status st = live_data(pool, *s, cp);
    if (st != ITAK_OK) return st;
    s->cp.live = false;  // cache.rs:824-833
    s->cp.ring_saves.clear();
    ITAK_DIAG("release slot=%u serial=%llu", slot, ULL(cp->serial));
    return ITAK_OK;
}

itak_status itak_kv_truncate(itak_pool *pool, const uint32_t *slots, const uint64_t *new_lengths,
                             uint32_t count) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (count && (!slots || !new_lengths))
        return invalid_argument(pool->err, "slots or new_lengths is null");
    for (uint32_t i = 0; i < count; ++i) {
        Slot *s = find_slot(pool, slots[i]);
        if (!s) return invalid_argument(pool->err, "slot is not in use");
        if (s->cp.live) return checkpoint_busy(pool->err);
        for (uint64_t li = 0; li < s->appended.size(); ++li)
            if (new_lengths[i] > s->appended[li])
                return rewind_range(pool->err, li, 0, s->appended[li], new_lengths[i]);
        itak_status st = check_ring_rewind(pool, *s, new_lengths[i]);
        if (st != ITAK_OK) return st;
    }
    for (uint32_t i = 0; i < count; ++i)
        ITAK_DIAG("truncate slot=%u new_length=%llu", slots[i], ULL(new_lengths[i]));
    return truncate_slots(pool, slots, new_lengths, count);
}

itak_status itak_gqa_attention(itak_pool *pool, uint32_t slot, uint64_t layer, const float *q,
                               uint64_t q_len, uint64_t num_queries, uint64_t num_q_heads,
                               const uint64_t *query_positions, uint64_t positions_len,
                               float scale, float softcap, float *out) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    if (layer >= pool->cfg.layer_count) return invalid_layer(pool->err, layer, pool->cfg.layer_count);
    // attention.rs:115-146, in order.
    if (positions_len != num_queries)
        return shape_mismatch(pool->err, "query_positions", num_queries, positions_len);
    const uint64_t expected_q = num_queries * num_q_heads * pool->g.head_dim;
    if (q_len != expected_q) return shape_mismatch(pool->err, "q", expected_q, q_len);
    if (num_queries == 0) return ITAK_OK;
    if (num_q_heads == 0) return zero_dimension(pool->err, "num_q_heads");
    if (num_q_heads % pool->g.kv_heads != 0)
        return non_divisible(pool->err, num_q_heads, pool->g.kv_heads);
    if (!q || !out || !query_positions)
        return invalid_argument(pool->err, "q, out or query_positions is null");
    // The view holds positions oldest..appended; a query sees those at or below its own
    // position and inside its window (attention.rs:77-85,160-173).
    const uint64_t appended = s->appended[layer];
    const uint64_t oldest = first_visible(pool, *s, layer);
    const uint64_t window = pool->layers[layer].window;
    for (uint64_t i = 0; i < num_queries; ++i) {
        const uint64_t p = query_positions[i];
        const uint64_t newest_seen = std::min(p + 1, appended);  // exclusive
        const uint64_t oldest_seen =
            std::max(oldest, (window && p + 1 > window) ? p + 1 - window : 0);
        if (newest_seen <= oldest_seen) return no_visible_keys(pool->err, p);
    }
    if (std::isnan(scale)) scale = default_scale(pool->g.head_dim);

    bool consecutive = true;
    for (uint64_t i = 1; i < num_queries; ++i)
        consecutive = consecutive && query_positions[i] == query_positions[0] + i;
    const uint64_t q_bytes = q_len * sizeof(float);
    const uint64_t pos_bytes = align_up(num_queries * sizeof(uint32_t), 256);
    itak_status st = ensure_stage(pool, 2 * align_up(q_bytes, 256) + pos_bytes);
    if (st != ITAK_OK) return st;
    float *qd = reinterpret_cast<float *>(pool->stage);
    float *od = reinterpret_cast<float *>(pool->stage + align_up(q_bytes, 256));
    uint32_t *pd = reinterpret_cast<uint32_t *>(pool->stage + 2 * align_up(q_bytes, 256));
    HIP_TRY(pool, hipMemcpyAsync(qd, q, q_bytes, hipMemcpyHostToDevice, pool->stream), "upload q");
    std::vector<uint32_t> pos32;
    if (!consecutive) {
        pos32.resize(num_queries);
        for (uint64_t i = 0; i < num_queries; ++i)
            pos32[i] = uint32_t(std::min<uint64_t>(query_positions[i], 0xffffffffu));
        HIP_TRY(pool,
                hipMemcpyAsync(pd, pos32.data(), num_queries * 4, hipMemcpyHostToDevice,
                               pool->stream),
                "upload query positions");
    }
    PlanInput pi{slot, uint32_t(num_queries),
                 uint32_t(std::min<uint64_t>(query_positions[0], 0xffffffffu - num_queries)),
                 uint32_t(appended), uint32_t(oldest)};
    st = run_attention(pool, layer, &pi, 1, qd, od, consecutive ? nullptr : pd, num_q_heads, scale,
                       softcap);
    if (st != ITAK_OK) return st;
    HIP_TRY(pool, hipMemcpyAsync(out, od, q_bytes, hipMemcpyDeviceToHost, pool->stream),
            "download attention output");
    HIP_TRY(pool, hipStreamSynchronize(pool->stream), "synchronize after attention");
    return ITAK_OK;
}

// Append + attend for a validated plan. Decode and speculative blocks on f16 pools run as
// one launch that appends and attends (plus the split merge); other shapes append first.
static itak_status step_on_device(itak_pool *pool, uint64_t layer, const itak_batch_item *items,
                                  uint32_t item_count, const std::vector<PlanInput> &plan,
                                  const float *q_dev, const float *k_dev, const float *v_dev,
                                  float *out_dev, uint64_t num_q_heads, float scale,
                                  float softcap, const FoldedParams *folded = nullptr,
                                  bool no_alloc = false) {
    // Rows of zero-row items contribute nothing; q/k/v rows are numbered by walking the
    // items in order, so such items may simply be dropped.
    std::vector<PlanInput> active;
    for (const PlanInput &p : plan)
        if (p.rows) active.push_back(p);
    uint32_t most_rows = 0;
    for (const PlanInput &p : active) most_rows = std::max(most_rows, p.rows);
    // Mid-size blocks on f16 pools: the block kernel in its one-tile form appends too.
    uint32_t most_blocks = 0;
    for (const PlanInput &p : active)
        most_blocks = std::max(most_blocks, (p.kv_len + 31) / 32 - p.kv_lo / 32);
    const bool splitk = takes_splitk_f16(pool, active.data(), uint32_t(active.size()), num_q_heads, nullptr);
    // (With the queries as two halves the block kernel runs its two-tile form, which brings no
    // rows along: the append is a launch of its own.)
    const bool block_fuses =
        !splitk && pool->elem_f16 && !active.empty() && !(pool->q_two_halves && pool->g.head_dim == 128) &&
        attn_prefill_f16_appends(pool->g, uint32_t(num_q_heads / pool->g.kv_heads), most_rows, most_blocks);
    const bool fuse =
        splitk || block_fuses ||
        (!pool->elem_f16 && !active.empty() &&
         attn_splitk_f32_appends(pool->g, uint32_t(num_q_heads / pool->g.kv_heads), most_rows));
    // The allocation-free form plans first and refuses, before anything changes, a step whose
    // launches need more workspace than the static array has.
    struct NoAllocScope {
        itak_pool *pool;
        bool on;
        ~NoAllocScope() { if (on) pool->no_alloc_call = false; }
    } scope{pool, no_alloc};
    if (no_alloc) {
        WorkspaceNeed need;
        itak_status st = run_attention(pool, layer, active.data(), uint32_t(active.size()), q_dev, out_dev,
                                       nullptr, num_q_heads, scale, softcap, nullptr, nullptr, folded,
                                       &need);
        if (st != ITAK_OK) return st;
        const uint64_t partial_bytes = need.partial_floats * sizeof(float);
        const uint64_t exchange_bytes = need.exchange_words * 8;
        if (partial_bytes > kScratchBytes - kScratchExchangeBytes)
            return set_error(pool->err, ITAK_CAPACITY_EXCEEDED, "split workspace", layer, partial_bytes,
                             kScratchBytes - kScratchExchangeBytes, 0,
                             "the step's split partials need %llu bytes of workspace and the "
                             "allocation-free entry point holds %llu: use fewer slots or rows per "
                             "step, or itak_attention_step_device",
                             ULL(partial_bytes), ULL(kScratchBytes - kScratchExchangeBytes));
        if (exchange_bytes > kScratchExchangeBytes)
            return set_error(pool->err, ITAK_CAPACITY_EXCEEDED, "split workspace", layer, exchange_bytes,
                             kScratchExchangeBytes, 0,
                             "the step's split exchange needs %llu bytes of workspace and the "
                             "allocation-free entry point holds %llu: use fewer slots or rows per "
                             "step, or itak_attention_step_device",
                             ULL(exchange_bytes), ULL(kScratchExchangeBytes));
        pool->no_alloc_call = true;
        if (need.exchange_words) pool->scratch_exchange_used = true;
    }
    if (fuse) {
        for (uint32_t i = 0; i < item_count; ++i)
            advance(pool->slots[items[i].slot], layer, items[i].rows);
        return run_attention(pool, layer, active.data(), uint32_t(active.size()), q_dev, out_dev,
                             nullptr, num_q_heads, scale, softcap, k_dev, v_dev, folded);
    }
    itak_status st = run_append(pool, layer, items, item_count, k_dev, v_dev);
    if (st != ITAK_OK) return st;
    return run_attention(pool, layer, active.data(), uint32_t(active.size()), q_dev, out_dev,
                         nullptr, num_q_heads, scale, softcap, nullptr, nullptr, folded);
}

// Validates one batched step and returns the per-item plan (positions before the append).
static itak_status plan_step(itak_pool *pool, uint64_t layer, const itak_batch_item *items,
                             uint32_t item_count, uint64_t num_q_heads,
                             std::vector<PlanInput> &plan) {
    if (layer >= pool->cfg.layer_count) return invalid_layer(pool->err, layer, pool->cfg.layer_count);
    if (num_q_heads == 0) return zero_dimension(pool->err, "num_q_heads");
    if (num_q_heads % pool->g.kv_heads != 0)
        return non_divisible(pool->err, num_q_heads, pool->g.kv_heads);
    std::vector<uint8_t> seen(pool->slots.size(), 0);
    plan.clear();
    for (uint32_t i = 0; i < item_count; ++i) {
        Slot *s = find_slot(pool, items[i].slot);
        if (!s) return invalid_argument(pool->err, "slot is not in use");
        if (seen[items[i].slot]++) return invalid_argument(pool->err, "slot listed twice in one step");
        uint64_t ok = 0;
        itak_status st = check_append_rows(pool, *s, layer, items[i].rows, &ok);
        if (st != ITAK_OK) return st;
        st = check_block_rows(pool, layer, items[i].rows);
        if (st != ITAK_OK) return st;
        const uint64_t base = s->appended[layer];
        // The block's first row still sees its whole window: the rows below the view of the
        // block's end are kept by the ring's headroom.
        const uint64_t window = pool->layers[layer].window;
        const uint64_t lo = (window && base + 1 > window) ? base + 1 - window : 0;
        plan.push_back(PlanInput{items[i].slot, items[i].rows, uint32_t(base),
                                 uint32_t(base + items[i].rows), uint32_t(lo)});
    }
    return ITAK_OK;
}

itak_status itak_attention_step_device(itak_pool *pool, uint64_t layer,
                                       const itak_batch_item *items, uint32_t item_count,
                                       const float *q_dev, const float *k_dev, const float *v_dev,
                                       float *out_dev, uint64_t num_q_heads, float scale,
                                       float softcap) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (item_count == 0) return ITAK_OK;
    if (!items || !q_dev || !k_dev || !v_dev || !out_dev)
        return invalid_argument(pool->err, "items or a device tensor is null");
    std::vector<PlanInput> plan;
    itak_status st = plan_step(pool, layer, items, item_count, num_q_heads, plan);
    if (st != ITAK_OK) return st;
    if (std::isnan(scale)) scale = default_scale(pool->g.head_dim);
    return step_on_device(pool, layer, items, item_count, plan, q_dev, k_dev, v_dev, out_dev,
                          num_q_heads, scale, softcap);
}

itak_status itak_attention_step_device_noalloc(itak_pool *pool, uint64_t layer,
                                               const itak_batch_item *items, uint32_t item_count,
                                               const float *q_dev, const float *k_dev,
                                               const float *v_dev, float *out_dev,
                                               uint64_t num_q_heads, float scale, float softcap) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (item_count == 0) return ITAK_OK;
    if (!items || !q_dev || !k_dev || !v_dev || !out_dev)
        return invalid_argument(pool->err, "items or a device tensor is null");
    std::vector<PlanInput> plan;
    itak_status st = plan_step(pool, layer, items, item_count, num_q_heads, plan);
    if (st != ITAK_OK) return st;
    if (std::isnan(scale)) scale = default_scale(pool->g.head_dim);
    bool capturing = false;
    HIP_TRY(pool, scratch_guard_enter(pool->cfg.device, pool->stream, &capturing),
            "order the step behind the static workspace's last user");
    st = step_on_device(pool, layer, items, item_count, plan, q_dev, k_dev, v_dev, out_dev,
                        num_q_heads, scale, softcap, nullptr, true);
    if (!capturing)
        HIP_TRY(pool, scratch_guard_leave(pool->cfg.device, pool->stream),
                "mark the static workspace's last user");
    return st;
}

itak_status itak_attention_prep_step_device(itak_pool *pool, uint64_t layer,
                                            const itak_batch_item *items, uint32_t item_count,
                                            const float *q_dev, const float *k_dev,
                                            const float *v_dev, const float *gate_dev,
                                            float *out_dev, uint64_t num_q_heads, float scale,
                                            float softcap, const itak_prep_params *prep) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (item_count == 0) return ITAK_OK;
    if (!items || !q_dev || !k_dev || !v_dev || !out_dev || !prep)
        return invalid_argument(pool->err, "items, a device tensor or prep is null");
    const uint32_t D = pool->g.head_dim;
    // torch-math's refusals (norm.rs:32-38, rope_interleaved.rs:72-99), by name.
    if ((prep->q_norm_weight || prep->k_norm_weight) && !(std::isfinite(prep->eps) && prep->eps > 0.0f))
        return set_error(pool->err, ITAK_STEP_FAILED, "rms_norm", 0, 0, 0, 0,
                         "rms_norm: eps must be finite and > 0");
    const bool rotate = prep->rope_base != 0.0f;
    const uint32_t rotary = prep->rotary_dim ? prep->rotary_dim : D;
    if (rotate) {
        if (D < 2 || D % 2 != 0)
            return set_error(pool->err, ITAK_STEP_FAILED, "attention", 0, 0, 0, 0,
                             "rope: head_dim must be even and >= 2");
        if (rotary < 2 || rotary % 2 != 0 || rotary > D)
            return set_error(pool->err, ITAK_STEP_FAILED, "attention", 0, 0, 0, 0,
                             "rope: rotary_dim must be even, >= 2, and <= head_dim");
        if (!std::isfinite(prep->rope_base) || prep->rope_base <= 1.0f)
            return set_error(pool->err, ITAK_STEP_FAILED, "attention", 0, 0, 0, 0,
                             "rope: base must be finite and > 1");
    } else if (D % 2 != 0) {
        return unsupported(pool->err, "attention preparation needs an even head_dim");
    }
    std::vector<PlanInput> plan;
    itak_status st = plan_step(pool, layer, items, item_count, num_q_heads, plan);
    if (st != ITAK_OK) return st;
    uint64_t total_rows = 0;
    for (const PlanInput &p : plan) total_rows += p.rows;
    if (total_rows == 0) return ITAK_OK;
    const uint64_t q_width = num_q_heads * D, k_width = pool->row;
    if (std::isnan(scale)) scale = default_scale(D);
    // Steps the split-K kernel takes (decode, speculative blocks: up to 64 query vectors per KV
    // head) have Q and the new K rows prepared by that kernel and the gate applied by the
    // kernel that writes the output: no launch but the step's own two.
    std::vector<PlanInput> active;
    for (const PlanInput &p : plan)
        if (p.rows) active.push_back(p);
    const bool splitk = takes_splitk_f16(pool, active.data(), uint32_t(active.size()), num_q_heads,
                                         nullptr);
    const bool interleaved = prep->rope_interleaved != 0;
    const bool folds = splitk && !pool->prep_by_launch && (!rotate || interleaved || rotary % 8 == 0);
    FoldedParams folded{};
    folded.gate = gate_dev;
    if (folds) {
        folded.prep_on = 1;
        folded.prep_interleaved = interleaved ? 1 : 0;
        folded.prep_rot = rotate ? rotary : 0;
        folded.prep_eps = prep->eps;
        folded.prep_q_weight = prep->q_norm_weight;
        folded.prep_k_weight = prep->k_norm_weight;
        // Pair i turns at position * base^(-2i/rot) = position * 2^(i * step).
        folded.prep_freq_step = rotate ? -2.0 * std::log2(double(prep->rope_base)) / double(rotary) : 0.0;
        return step_on_device(pool, layer, items, item_count, plan, q_dev, k_dev, v_dev, out_dev,
                              num_q_heads, scale, softcap, &folded);
    }
    st = ensure_prep(pool, total_rows * (q_width + k_width));
    if (st != ITAK_OK) return st;
    float *q_prep = pool->prep, *k_prep = pool->prep + total_rows * q_width;
    uint32_t row = 0;
    for (uint32_t first = 0; first < item_count; first += kMaxBatchItems) {
        const uint32_t count = std::min<uint32_t>(kMaxBatchItems, item_count - first);
        PrepArgs a{};
        a.q_in = q_dev + uint64_t(row) * q_width;
        a.k_in = k_dev + uint64_t(row) * k_width;
        a.q_out = q_prep + uint64_t(row) * q_width;
        a.k_out = k_prep + uint64_t(row) * k_width;
        a.q_weight = prep->q_norm_weight;
        a.k_weight = prep->k_norm_weight;
        a.eps = prep->eps;
        a.rope_base = rotate ? prep->rope_base : 0.0f;
        a.rope_freq = rotate ? rope_freq_table(pool, prep->rope_base, rotary) : nullptr;
        a.interleaved = interleaved ? 1 : 0;
        a.rotary_dim = rotary;
        a.head_dim = D;
        a.q_heads = uint32_t(num_q_heads);
        a.kv_heads = pool->g.kv_heads;
        a.n = count;
        uint32_t chunk_rows = 0;
        for (uint32_t i = 0; i < count; ++i) {
            a.row0[i] = chunk_rows;
            a.pos0[i] = plan[first + i].pos0;
            chunk_rows += plan[first + i].rows;
        }
        a.total_rows = chunk_rows;
        HIP_TRY(pool, launch_attn_prep(a, pool->stream), "launch attention preparation");
        row += chunk_rows;
    }
    return step_on_device(pool, layer, items, item_count, plan, q_prep, k_prep, v_dev, out_dev,
                          num_q_heads, scale, softcap, &folded);
}

itak_status itak_attention_device(itak_pool *pool, uint64_t layer, const itak_batch_item *items,
                                  uint32_t item_count, const float *q_dev, float *out_dev,
                                  uint64_t num_q_heads, float scale, float softcap) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (item_count == 0) return ITAK_OK;
    if (!items || !q_dev || !out_dev)
        return invalid_argument(pool->err, "items or a device tensor is null");
    if (layer >= pool->cfg.layer_count) return invalid_layer(pool->err, layer, pool->cfg.layer_count);
    if (num_q_heads == 0) return zero_dimension(pool->err, "num_q_heads");
    if (num_q_heads % pool->g.kv_heads != 0)
        return non_divisible(pool->err, num_q_heads, pool->g.kv_heads);
    std::vector<PlanInput> plan;
    for (uint32_t i = 0; i < item_count; ++i) {
        Slot *s = find_slot(pool, items[i].slot);
        if (!s) return invalid_argument(pool->err, "slot is not in use");
        const uint64_t len = s->appended[layer];
        if (items[i].rows == 0) continue;
        if (len == 0) return no_visible_keys(pool->err, 0);
        if (items[i].rows > len)
            return shape_mismatch(pool->err, "query rows", len, items[i].rows);
        // The newest `rows` positions query the view as it stands: nothing older than the
        // view's first row is promised to be in the ring. A query that stands before that row
        // (more rows than a windowed layer's window) sees none of the view: the reference's
        // refusal for its position (attention.rs:160-173), the lowest such query first.
        const uint64_t first = first_visible(pool, *s, layer);
        if (len - items[i].rows < first) return no_visible_keys(pool->err, len - items[i].rows);
        plan.push_back(PlanInput{items[i].slot, items[i].rows, uint32_t(len - items[i].rows),
                                 uint32_t(len), uint32_t(first)});
    }
    if (std::isnan(scale)) scale = default_scale(pool->g.head_dim);
    return run_attention(pool, layer, plan.data(), uint32_t(plan.size()), q_dev, out_dev, nullptr,
                         num_q_heads, scale, softcap);
}

itak_status itak_compute_attention(itak_pool *pool, uint32_t slot, uint64_t layer, const float *q,
                                   uint64_t q_len, const float *k, uint64_t k_len, const float *v,
                                   uint64_t v_len, uint64_t num_q_heads, uint64_t cache_position,
                                   float softcap, float rope_freq_base_swa, float *out) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    const char *step = "attention";
    // cpu.rs:529-556: whole rows, matching K/V row counts.
    const uint64_t q_width = num_q_heads * pool->g.head_dim;
    if (q_width == 0 || q_len % q_width != 0)
        return set_error(pool->err, ITAK_STEP_FAILED, step, q_len, q_width, 0, 0,
                         "query projection holds %llu elements, not a whole number of "
                         "%llu-wide rows",
                         ULL(q_len), ULL(q_width));
    const uint64_t rows = q_len / q_width;
    if (k_len != rows * pool->row || v_len != rows * pool->row)
        return set_error(pool->err, ITAK_STEP_FAILED, step, k_len, v_len, rows * pool->row, 0,
                         "key/value projections hold %llu/%llu elements for %llu rows, expected "
                         "%llu/%llu",
                         ULL(k_len), ULL(v_len), ULL(rows), ULL(rows * pool->row),
                         ULL(rows * pool->row));
    if (layer >= pool->cfg.layer_count) {
        invalid_layer(pool->err, layer, pool->cfg.layer_count);
        pool->err.info.code = ITAK_STEP_FAILED;  // forwarded as StepFailed text (cpu.rs:565-568)
        return ITAK_STEP_FAILED;
    }
    s->built = true;  // KvState::build on first use (cpu.rs:560-564)
    const uint64_t appended = s->appended[layer];
    if (appended != cache_position)  // cpu.rs:569-581
        return set_error(pool->err, ITAK_STEP_FAILED, step, layer, appended, cache_position, 0,
                         "KV state for layer %llu is at position %llu but the sequence cache is "
                         "at position %llu: the two disagree, so attending would read the wrong "
                         "history. Pair one Cache with one compute slot per sequence, or reset "
                         "the slot when a sequence is abandoned (a forward that failed midway "
                         "leaves the KV state ahead of the cache and also needs a reset)",
                         ULL(layer), ULL(appended), ULL(cache_position));
    if (rows == 0) return ITAK_OK;
    if (num_q_heads % pool->g.kv_heads != 0) {
        non_divisible(pool->err, num_q_heads, pool->g.kv_heads);
        pool->err.info.code = ITAK_STEP_FAILED;
        return ITAK_STEP_FAILED;
    }
    if (!q || !k || !v || !out) return invalid_argument(pool->err, "q, k, v or out is null");
    // Sliding-window layers rotate Q and K (cpu.rs:594-622); torch_math::rope_interleaved's
    // refusals (rope_interleaved.rs:72-99) surface under the attention step.
    const bool rotate = pool->layers[layer].windowed;
    if (rotate) {
        if (pool->g.head_dim < 2 || pool->g.head_dim % 2 != 0)
            return set_error(pool->err, ITAK_STEP_FAILED, step, 0, 0, 0, 0,
                             "rope: head_dim must be even and >= 2");
        if (!std::isfinite(rope_freq_base_swa) || rope_freq_base_swa <= 1.0f)
            return set_error(pool->err, ITAK_STEP_FAILED, step, 0, 0, 0, 0,
                             "rope: base must be finite and > 1");
    }

    // Row-at-a-time appends stop at the first refusal (cpu.rs:623-631): rows before it are
    // in the cache when the call fails, exactly as in the reference.
    uint64_t ok_rows = rows;
    itak_status refusal = check_append_rows(pool, *s, layer, rows, &ok_rows);
    ErrorState saved = pool->err;

    const uint64_t q_bytes = align_up(q_len * sizeof(float), 256);
    const uint64_t kv_bytes = align_up(k_len * sizeof(float), 256);
    itak_status st = ensure_stage(pool, 2 * q_bytes + 2 * kv_bytes);
    if (st != ITAK_OK) return st;
    float *qd = reinterpret_cast<float *>(pool->stage);
    float *kd = reinterpret_cast<float *>(pool->stage + q_bytes);
    float *vd = reinterpret_cast<float *>(pool->stage + q_bytes + kv_bytes);
    float *od = reinterpret_cast<float *>(pool->stage + q_bytes + 2 * kv_bytes);
    // A call is dominated by its trips over the host link, not by its kernels. Small inputs
    // (a decode row, a speculative block) are packed into pinned memory and go up in one copy,
    // and the kernel that writes the output writes it into pinned memory directly; large ones
    // (a prefill chunk) are copied as they lie.
    const uint64_t in_bytes = q_bytes + 2 * kv_bytes;
    const bool packed = in_bytes <= (1u << 20);
    float *out_pinned = nullptr;
    uint32_t *done_word = nullptr;  // in pinned memory, after the output
    if (packed) {
        // Layout: [completion word, 256 bytes] [q | k | v] [output]. The word sits at a fixed
        // place, so it only ever holds call numbers, which only grow.
        st = ensure_hstage(pool, kHostWord + in_bytes + q_bytes);
        if (st != ITAK_OK) return st;
        unsigned char *hin = pool->hstage + kHostWord;
        memcpy(hin, q, q_len * 4);
        memcpy(hin + q_bytes, k, k_len * 4);
        memcpy(hin + q_bytes + kv_bytes, v, v_len * 4);
        void *mapped = nullptr;
        HIP_TRY(pool, hipHostGetDevicePointer(&mapped, pool->hstage, 0), "map pinned staging");
        unsigned char *pinned_dev = static_cast<unsigned char *>(mapped);
        if (in_bytes <= (64u << 10))
            HIP_TRY(pool, launch_stage_in(pinned_dev + kHostWord, qd, in_bytes, pool->stream),
                    "launch stage-in");
        else
            HIP_TRY(pool, hipMemcpyAsync(qd, hin, in_bytes, hipMemcpyHostToDevice, pool->stream),
                    "upload q, k, v");
        out_pinned = reinterpret_cast<float *>(pinned_dev + kHostWord + in_bytes);
        done_word = reinterpret_cast<uint32_t *>(pinned_dev);
    } else {
        HIP_TRY(pool, hipMemcpyAsync(kd, k, k_len * 4, hipMemcpyHostToDevice, pool->stream), "upload k");
        HIP_TRY(pool, hipMemcpyAsync(vd, v, v_len * 4, hipMemcpyHostToDevice, pool->stream), "upload v");
        HIP_TRY(pool, hipMemcpyAsync(qd, q, q_len * 4, hipMemcpyHostToDevice, pool->stream), "upload q");
    }
    // The reference appends and attends row by row (cpu.rs:586-646). Here a block is appended
    // whole and attended under the causal mask, which is the same thing on a global layer; on
    // a windowed layer a block may be as long as the ring's headroom, so longer inputs go in
    // several blocks.
    const LayerInfo &L = pool->layers[layer];
    const uint64_t block_cap = L.windowed ? L.ring - L.window : std::max<uint64_t>(rows, 1);
    // The rotation of a sliding-window layer (row i at position appended + i): in place on the
    // staged rows, by the preparation launch, whose f64 angles, sines and cosines are the
    // reference's (rope_interleaved.rs:103-114), so that the K rows this call stores are the
    // reference's rounded once. (The split-K kernel can rotate inside its own launch, with the
    // hardware's sine and cosine, within one f16 step of that; the device-resident step uses it,
    // where a launch counts. Here the call already copies its rows in and its output out.)
    auto rotate_block = [&](uint64_t done, uint64_t n, bool with_q) -> itak_status {
        PrepArgs a{};
        a.q_in = a.q_out = qd + done * q_width;
        a.k_in = a.k_out = kd + done * pool->row;
        a.rope_base = rope_freq_base_swa;
        a.rope_freq = rope_freq_table(pool, rope_freq_base_swa, pool->g.head_dim);
        a.interleaved = 1;
        a.rotary_dim = pool->g.head_dim;
        a.head_dim = pool->g.head_dim;
        a.q_heads = with_q ? uint32_t(num_q_heads) : 0;
        a.kv_heads = pool->g.kv_heads;
        a.total_rows = uint32_t(n);
        a.n = 1;
        a.row0[0] = 0;
        a.pos0[0] = uint32_t(appended + done);
        HIP_TRY(pool, launch_attn_prep(a, pool->stream), "launch rope");
        return ITAK_OK;
    };
    if (refusal != ITAK_OK) {
        for (uint64_t done = 0; done < ok_rows; done += block_cap) {
            const uint64_t n = std::min(block_cap, ok_rows - done);
            if (rotate && (st = rotate_block(done, n, false)) != ITAK_OK) return st;
            itak_batch_item item{slot, uint32_t(n)};
            st = run_append(pool, layer, &item, 1, kd + done * pool->row, vd + done * pool->row);
            if (st != ITAK_OK) return st;
        }
        HIP_TRY(pool, hipStreamSynchronize(pool->stream), "synchronize after append");
        pool->err = saved;
        pool->err.info.code = ITAK_STEP_FAILED;
        return ITAK_STEP_FAILED;
    }
    float *out_dev = out_pinned ? out_pinned : od;
    for (uint64_t done = 0; done < rows; done += block_cap) {
        const uint64_t n = std::min(block_cap, rows - done);
        itak_batch_item item{slot, uint32_t(n)};
        const uint64_t base = appended + done;
        const uint64_t lo = (L.window && base + 1 > L.window) ? base + 1 - L.window : 0;
        std::vector<PlanInput> plan{
            PlanInput{slot, uint32_t(n), uint32_t(base), uint32_t(base + n), uint32_t(lo)}};
        if (rotate && (st = rotate_block(done, n, true)) != ITAK_OK) return st;
        st = step_on_device(pool, layer, &item, 1, plan, qd + done * q_width, kd + done * pool->row,
                            vd + done * pool->row, out_dev + done * q_width, num_q_heads,
                            default_scale(pool->g.head_dim),  // AttentionParams::new(), cpu.rs:584
                            softcap, nullptr);
        if (st != ITAK_OK) return st;
    }
    if (!out_pinned) {
        HIP_TRY(pool, hipMemcpyAsync(out, od, q_len * 4, hipMemcpyDeviceToHost, pool->stream),
                "download attention output");
        HIP_TRY(pool, hipStreamSynchronize(pool->stream), "synchronize after attention");
        return ITAK_OK;
    }
    // The last launch of the call writes the call's number where the host can see it; the host
    // watches that word for a short while before it asks the runtime (which also reports a
    // failed launch, and is what a call that takes longer falls back to).
    const uint32_t number = ++pool->call_number ? pool->call_number : ++pool->call_number;
    HIP_TRY(pool, launch_signal_done(done_word, number, pool->stream), "launch completion signal");
    const volatile uint32_t *seen =
        reinterpret_cast<const volatile uint32_t *>(pool->hstage);
    timespec t0{};
    clock_gettime(CLOCK_MONOTONIC, &t0);
    bool arrived = false;
    for (uint32_t spin = 0; !arrived; ++spin) {
        arrived = __atomic_load_n(seen, __ATOMIC_ACQUIRE) == number;
        if (arrived || (spin & 63u) != 63u) {
            __builtin_ia32_pause();
            continue;
        }
        timespec t1{};
        clock_gettime(CLOCK_MONOTONIC, &t1);
        if ((t1.tv_sec - t0.tv_sec) * 1000000000ll + (t1.tv_nsec - t0.tv_nsec) > 300000) break;
    }
    if (!arrived) HIP_TRY(pool, hipStreamSynchronize(pool->stream), "synchronize after attention");
    memcpy(out, pool->hstage + kHostWord + in_bytes, q_len * 4);
    return ITAK_OK;
}

static itak_status no_kv_state(itak_pool *pool, const char *step, const char *detail) {
    return set_error(pool->err, ITAK_STEP_FAILED, step, 0, 0, 0, 0, "%s", detail);
}

static itak_status as_step_failed(itak_pool *pool, itak_status st) {
    if (st == ITAK_OK) return st;
    pool->err.info.code = ITAK_STEP_FAILED;  // map_err(step_failed(...)) in cpu.rs:292-294
    return ITAK_STEP_FAILED;
}

itak_status itak_compute_cache_checkpoint(itak_pool *pool, uint32_t slot,
                                          uint64_t max_round_tokens, itak_checkpoint *out) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    if (!s->built)  // cpu.rs:284-290
        return no_kv_state(pool, "cache_checkpoint",
                           "no KV state exists yet: a speculative round checkpoints after a first "
                           "forward has built the cache (the spec's prefill), not before");
    return as_step_failed(pool, itak_kv_checkpoint(pool, slot, max_round_tokens, out));
}

itak_status itak_compute_cache_rewind(itak_pool *pool, uint32_t slot, const itak_checkpoint *cp,
                                      uint64_t target) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    if (!s->built)  // cpu.rs:311-317
        return no_kv_state(pool, "cache_rewind",
                           "no KV state exists: the sequence was reset after the checkpoint was "
                           "taken");
    return as_step_failed(pool, itak_kv_rewind_to(pool, slot, cp, target));
}

itak_status itak_compute_cache_release(itak_pool *pool, uint32_t slot, const itak_checkpoint *cp) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    Slot *s = find_slot(pool, slot);
    if (!s) return invalid_argument(pool->err, "slot is not in use");
    if (!s->built)  // cpu.rs:327-333
        return no_kv_state(pool, "cache_release",
                           "no KV state exists: the sequence was reset after the checkpoint was "
                           "taken");
    return as_step_failed(pool, itak_kv_release(pool, slot, cp));
}

itak_status itak_convert_f32_to_f16_device(itak_pool *pool, const float *src_dev,
                                           uint16_t *dst_dev, uint64_t count) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (count && (!src_dev || !dst_dev)) return invalid_argument(pool->err, "src or dst is null");
    HIP_TRY(pool, launch_convert_f16(src_dev, dst_dev, count, pool->stream), "launch conversion");
    return ITAK_OK;
}

itak_status itak_probe_copy_device(itak_pool *pool, const void *src_dev, void *dst_dev,
                                   uint64_t bytes) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (bytes && (!src_dev || !dst_dev)) return invalid_argument(pool->err, "src or dst is null");
    if (bytes % 16 != 0) return invalid_argument(pool->err, "bytes is not a multiple of 16");
    HIP_TRY(pool, launch_probe_copy(src_dev, dst_dev, bytes, pool->stream), "launch probe copy");
    return ITAK_OK;
}

itak_status itak_probe_read_device(itak_pool *pool, const void *src_dev, uint64_t bytes) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (bytes && !src_dev) return invalid_argument(pool->err, "src is null");
    if (bytes % 16 != 0) return invalid_argument(pool->err, "bytes is not a multiple of 16");
    HIP_TRY(pool, launch_probe_read(src_dev, bytes, pool->stream), "launch probe read");
    return ITAK_OK;
}

void itak_set_debug_enabled(int32_t enabled) {
    g_debug_enabled.store(enabled != 0, std::memory_order_relaxed);
}
int32_t itak_debug_enabled(void) { return diag_enabled() ? 1 : 0; }

itak_status itak_probe_empty_launch(itak_pool *pool) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    HIP_TRY(pool, launch_probe_empty(pool->stream), "launch empty probe");
    return ITAK_OK;
}

itak_status itak_probe_mfma(itak_pool *pool, uint32_t random_operands, uint32_t trips,
                            uint64_t *clocks_dev, uint64_t *flops_out) {
    if (!pool) return ITAK_INVALID_ARGUMENT;
    if (trips == 0 || trips > (1u << 22)) return invalid_argument(pool->err, "trips is not in 1 ..= 2^22");
    uint32_t workgroups = 0;
    HIP_TRY(pool,
            launch_probe_mfma(random_operands != 0, trips,
                              reinterpret_cast<unsigned long long *>(clocks_dev), &workgroups, pool->stream),
            "launch MFMA probe");
    // 4 wavefronts a workgroup, 32 products a trip, 16 x 16 x 32 multiply-adds a product.
    if (flops_out) *flops_out = uint64_t(workgroups) * 4u * uint64_t(trips) * 32u * 16384u;
    return ITAK_OK;
}

}  // extern "C"
