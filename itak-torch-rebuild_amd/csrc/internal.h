// Shared declarations between the host logic (pool.hip) and the kernel files.
// Nothing here is part of the public ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

namespace itak {

// Device layout of the KV pool, in elements of the storage type. One "plane" is the
// rows of one (layer, slot, side, kv_head): capacity x head_dim elements, contiguous,
// so a workgroup that streams one KV head reads one unbroken run of memory.
//   plane(layer, slot, side, head) =
//     layer*layer_stride + slot*slot_stride + side*side_stride + head*head_stride
// side 0 = keys, 1 = values. With v_block == 0 both are row-major (row*head_dim + d).
// With v_block == 32 (f16 pools whose head_dim is a multiple of 16) both are stored in
// blocks of 32 rows laid out as the MFMA kernels consume them, so that every operand load
// of a wavefront is 64 lanes x 16 bytes of contiguous memory:
//   values: block transposed, element (row, d) at
//       (row/32)*32*head_dim + d*32 + row%32
//     (a lane's 8 consecutive rows of one channel are 16 contiguous bytes);
//   keys: 16-byte pieces of 8 channels, grouped by MFMA tile t and channel chunk c, element
//     (row, d) with kk = row%32, t = (kk/4)%2, i = (kk/8)*4 + kk%4, c = d/8 at
//       (row/32)*32*head_dim + ((t*(head_dim/8) + c)*16 + i)*8 + d%8
//     (tile t holds the 16 rows whose scores one lane group receives as 8 consecutive
//     keys; the lanes (chunk c, row i) of one load instruction are adjacent in memory).
struct PoolGeom {
    uint32_t kv_heads;
    uint32_t head_dim;
    uint32_t capacity;  // rows per plane (a multiple of 32 when v_block != 0)
    uint32_t max_slots;
    uint32_t v_block;   // 0 or 32
    uint32_t pad;
    uint64_t head_stride;   // capacity * head_dim
    uint64_t side_stride;   // kv_heads * head_stride
    uint64_t slot_stride;   // 2 * side_stride
    uint64_t layer_stride;  // max_slots * slot_stride
};

constexpr uint32_t kVBlock = 32;

// Element offset of (row, d) inside a value plane.
__host__ __device__ inline uint64_t v_offset(const PoolGeom &g, uint32_t row, uint32_t d) {
    if (g.v_block == 0) return uint64_t(row) * g.head_dim + d;
    return uint64_t(row / kVBlock) * (kVBlock * g.head_dim) + uint64_t(d) * kVBlock + row % kVBlock;
}

// Element offset of (row, d) inside a key plane.
__host__ __device__ inline uint64_t k_offset(const PoolGeom &g, uint32_t row, uint32_t d) {
    if (g.v_block == 0) return uint64_t(row) * g.head_dim + d;
    const uint32_t kk = row % kVBlock;
    const uint32_t t = (kk >> 2) & 1, i = (kk >> 3) * 4 + (kk & 3);
    return uint64_t(row / kVBlock) * (kVBlock * g.head_dim) +
           ((t * (g.head_dim / 8) + d / 8) * 16 + i) * 8 + d % 8;
}

// Element offset inside a plane of either side.
__host__ __device__ inline uint64_t kv_offset(const PoolGeom &g, uint32_t side, uint32_t row,
                                              uint32_t d) {
    return side ? v_offset(g, row, d) : k_offset(g, row, d);
}

// f32 -> f16 bits, round-to-nearest-even, overflow to infinity, subnormals rounded, and
// every NaN stored as sign|0x7e00: the rule of f32_to_f16_bits in
// crates/wgpu-compute/src/kernels/k1_q4k_gemv.rs:285-329. v_cvt_f16_f32 implements all of
// it except the NaN payload, which is replaced explicitly.
__device__ __forceinline__ uint16_t f32_to_f16_bits(float x) {
    _Float16 h = static_cast<_Float16>(x);
    uint16_t bits = __builtin_bit_cast(uint16_t, h);
    uint32_t in = __builtin_bit_cast(uint32_t, x);
    if ((in & 0x7fffffffu) > 0x7f800000u) {
        bits = static_cast<uint16_t>(((in >> 16) & 0x8000u) | 0x7e00u);
    }
    return bits;
}

constexpr int kMaxBatchItems = 64;

// ---- append ---------------------------------------------------------------------
struct AppendItem {
    uint32_t slot;
    uint32_t rows;
    uint32_t pos0;      // position of the item's first new row
    uint32_t src_row0;  // row offset of the item inside k_src / v_src
};
struct AppendBatch {
    uint32_t n;
    uint32_t total_rows;
    uint32_t ring;      // storage rows of a windowed layer's ring (position p lives in row p % ring); 0 = row p
    // The launch moves total_rows source rows: rows [0, gap_at) and, when gap_rows != 0, the
    // rows from gap_at + gap_rows on (the rows in between go another way).
    uint32_t gap_at;
    uint32_t gap_rows;
    uint32_t pad;
    AppendItem item[kMaxBatchItems];
};
hipError_t launch_append(void *layer_base, int elem_f16, const PoolGeom &g, const AppendBatch &b,
                         const float *k_src, const float *v_src, hipStream_t stream);

// ---- zero fill of dropped rows (truncate scrub, slot reset) ------------------------
struct ZeroItem {
    uint32_t slot;
    uint32_t row_from;
    uint32_t row_to;  // exclusive
    uint32_t pad;
};
struct ZeroBatch {
    uint32_t n;
    uint32_t max_rows;
    ZeroItem item[kMaxBatchItems];
};
hipError_t launch_zero_rows(void *pool_base, int elem_f16, const PoolGeom &g, uint32_t layer_from,
                            uint32_t layer_to, const ZeroBatch &b, hipStream_t stream);

// ---- snapshot restore (gather from [row][kv_head][d] sources into the planes) --------
constexpr int kMaxRestoreLayers = 64;
struct RestoreLayer {
    const void *keys;
    const void *values;
    uint32_t layer;
    uint32_t rows;
    uint32_t first_row;  // destination storage row of source row 0
    uint32_t pad;
};
struct RestoreBatch {
    uint32_t n;
    uint32_t max_rows;
    uint32_t slot;
    uint32_t pad;
    RestoreLayer layer[kMaxRestoreLayers];
};
hipError_t launch_restore(void *pool_base, int dst_f16, int src_f16, const PoolGeom &g,
                          const RestoreBatch &b, hipStream_t stream);

// ---- row readback: planes -> [row][kv_head][d] ---------------------------------------
// Row r of the output is position first_row + r, read from storage row (first_row + r) % ring
// when ring != 0.
hipError_t launch_read_rows(const void *layer_base, int elem_f16, const PoolGeom &g, uint32_t slot,
                            uint32_t first_row, uint32_t rows, uint32_t ring, void *keys_out,
                            void *values_out, hipStream_t stream);

// ---- ring rows aside and back (checkpoints deeper than a ring's headroom) -----------------
// Copies rows of windowed layers between their rings and a side buffer that holds, per entry,
// [side][saved_rows][kv_head][d] elements at saved_off: row saved_row0 + r of the buffer is
// position pos0 + r, storage row (pos0 + r) % ring.
struct RingRowsLayer {
    uint32_t layer;       // index among the windowed layers
    uint32_t ring;
    uint32_t pos0;
    uint32_t rows;
    uint32_t saved_row0;
    uint32_t saved_rows;
    uint64_t saved_off;   // elements
};
struct RingRowsBatch {
    uint32_t n;
    uint32_t slot;
    uint32_t max_rows;
    uint32_t pad;
    RingRowsLayer layer[kMaxRestoreLayers];
};
// to_ring = false: rings -> buffer; true: buffer -> rings.
hipError_t launch_ring_rows(void *pool_base_w, int elem_f16, const PoolGeom &gw,
                            const RingRowsBatch &b, void *saved, bool to_ring, hipStream_t stream);

hipError_t launch_convert_f16(const float *src, uint16_t *dst, uint64_t count, hipStream_t stream);
// f16 bits -> f32, exact (the widening a snapshot capture of an f16 pool needs).
hipError_t launch_widen_f16(const uint16_t *src, float *dst, uint64_t count, hipStream_t stream);
// Host-pointer calls: `bytes` (rounded up to 16) from pinned host memory into device memory by
// a kernel, and a word in pinned host memory set to `value` once everything before it on the
// stream has finished.
hipError_t launch_stage_in(const void *pinned, void *dst, uint64_t bytes, hipStream_t stream);
hipError_t launch_signal_done(uint32_t *pinned_word, uint32_t value, hipStream_t stream);
hipError_t launch_probe_copy(const void *src, void *dst, uint64_t bytes, hipStream_t stream);
hipError_t launch_probe_read(const void *src, uint64_t bytes, hipStream_t stream);
hipError_t launch_probe_empty(hipStream_t stream);
// `iters` trips of 32 f16 MFMAs per wavefront, two workgroups of four wavefronts per compute unit
// (*workgroups receives how many were launched); clocks: two device words or null.
hipError_t launch_probe_mfma(bool random_operands, uint32_t iters, unsigned long long *clocks,
                             uint32_t *workgroups, hipStream_t stream);

// ---- attention preparation (per-head RMSNorm + RoPE of Q and K) and the output gate ------
struct PrepArgs {
    const float *q_in;      // [total_rows][q_heads*head_dim]
    const float *k_in;      // [total_rows][kv_heads*head_dim]
    float *q_out;
    float *k_out;
    const float *q_weight;  // [head_dim] or null: no norm
    const float *k_weight;
    float eps;
    float rope_base;        // > 1 rotates, otherwise no rotation
    // Pair i turns at position * rope_freq[i] radians: rope_base^(-2i/rotary_dim) as the host's
    // libm gives it, which is what the reference's own host computes. Null: the kernel takes
    // the power itself (the device library's may differ in the last bit, and a last bit times
    // the position is what reaches the stored row).
    const double *rope_freq;
    uint32_t interleaved;   // 1: pairs (2i, 2i+1); 0: pairs (i, i + rotary_dim/2)
    uint32_t rotary_dim;
    uint32_t head_dim;
    uint32_t q_heads;
    uint32_t kv_heads;
    uint32_t total_rows;
    uint32_t n;                      // items
    uint32_t row0[kMaxBatchItems];   // first row of item i (rows are laid out item after item)
    uint32_t pos0[kMaxBatchItems];   // position of that row
};
hipError_t launch_attn_prep(const PrepArgs &a, hipStream_t stream);
// out[i] *= sigmoid(gate[i]) (CpuCompute::attn_gate, cpu.rs:657-673).
hipError_t launch_attn_gate(float *out, const float *gate, uint64_t count, hipStream_t stream);

// ---- attention ----------------------------------------------------------------------
// One item = one slot's query rows against that slot's rows of one layer. Query row r
// sits at position pos0 + r unless q_pos is given. A query at position p sees the keys at
// positions max(kv_lo, p + 1 - window) .. min(p, kv_len - 1) (window 0 = no lower bound but
// kv_lo); on a windowed layer position kp lives in storage row kp % (32 * ring_blocks), so
// that 32-position blocks stay whole and in order inside the ring. A workgroup owns (item, row block,
// kv head, split of the key range) and writes either the final output (splits == 1) or
// a partial (m, l, acc[head_dim]) per query vector; a second, small launch merges the
// partials of each (row, Q head). Partials live in `ws`: first total_partials*head_dim
// accumulators, then total_partials (m, l) pairs; the partial of (row, head, split) of
// an item is ws0 + (row*q_heads + head)*splits + split.
struct AttnItem {
    uint32_t slot;
    uint32_t rows;
    uint32_t pos0;
    uint32_t q_row0;        // first row of the item in q / out
    uint32_t kv_len;        // stored rows visible to the item's last query row (exclusive end)
    uint32_t splits;
    uint32_t keys_per_split;
    uint32_t block0;        // first workgroup index of the item
    uint32_t ws0;           // first partial index of the item
    uint32_t splits_magic;  // ceil(2^32 / splits) for splits > 1: x / splits == mulhi(x, magic), x < 2^16
    uint32_t kv_lo;         // oldest position any query of the item may see (0 on global layers)
};
// Key blocks (32 positions) an item's queries can touch: [first, end).
__host__ __device__ inline uint32_t item_first_block(const AttnItem &it) { return it.kv_lo / 32; }
__host__ __device__ inline uint32_t item_block_count(const AttnItem &it) {
    return (it.kv_len + 31) / 32 - it.kv_lo / 32;
}
struct AttnBatch {
    uint32_t n;
    uint32_t total_blocks;
    uint32_t rows_per_block;
    uint32_t deep_ring;  // host side only: the block kernel's plan asks for its deeper LDS ring
    uint32_t fold_units; // host side only: the block kernel's plan for AttnParams::fold_units
    uint32_t two_halves; // host side only: the block kernel multiplies each query as two f16 halves
    AttnItem item[kMaxBatchItems];
};
// The kernel argument form of AttnBatch, sized to the batch: kernel arguments are
// expensive to read on this GPU (a 2.6 KB argument block costs about a microsecond per
// launch, a scan through 40-byte items several), so small batches get a small block and
// the workgroup-to-item search runs over a compact array of first-workgroup indices.
template <int N>
struct AttnBatchT {
    uint32_t n;
    uint32_t total_blocks;
    uint32_t rows_per_block;
    uint32_t base_row;  // q_row0 of item 0
    uint32_t block0[N];
    uint32_t row0[N];   // q_row0 - base_row
    AttnItem item[N];

    explicit AttnBatchT(const AttnBatch &b)
        : n(b.n), total_blocks(b.total_blocks), rows_per_block(b.rows_per_block),
          base_row(b.n ? b.item[0].q_row0 : 0) {
        for (int i = 0; i < N; ++i) {
            const bool live = uint32_t(i) < b.n;
            item[i] = live ? b.item[i] : AttnItem{};
            block0[i] = live ? b.item[i].block0 : 0xffffffffu;
            row0[i] = live ? b.item[i].q_row0 - base_row : 0xffffffffu;
        }
    }
    __device__ __forceinline__ uint32_t find_by_block(uint32_t block) const {
        uint32_t it = 0;
        if (N > 1) {
#pragma unroll 1
            while (it + 1 < n && block >= block0[it + 1]) ++it;
        }
        return it;
    }
    __device__ __forceinline__ uint32_t find_by_row(uint32_t row) const {
        uint32_t it = 0;
        if (N > 1) {
#pragma unroll 1
            while (it + 1 < n && row >= row0[it + 1]) ++it;
        }
        return it;
    }
};

// Runs CALL with `constexpr int N` set to the smallest of {1, 8, 64} that holds n items.
#define ITAK_DISPATCH_BATCH(n, CALL) \
    do {                              \
        if ((n) <= 1) {               \
            constexpr int N = 1;      \
            CALL;                     \
        } else if ((n) <= 8) {        \
            constexpr int N = 8;      \
            CALL;                     \
        } else {                      \
            constexpr int N = 64;     \
            CALL;                     \
        }                             \
    } while (0)

struct AttnParams {
    const void *layer_base;
    PoolGeom g;
    const float *q;
    float *out;
    const uint32_t *q_pos;  // optional explicit positions, [sum rows]
    float *ws;              // partials: (head_dim + 2) floats each
    // Fused append (split-K f16 kernel only): when set, the last `rows` positions of every
    // item are not in the cache yet; their K/V rows are read from here (row q_row0 + r,
    // [kv_heads*head_dim] f32 each), written to the cache by the kernel, and attended to.
    const float *k_new;
    const float *v_new;
    uint32_t q_heads;
    uint32_t group;         // q_heads / kv_heads
    uint32_t group_magic;   // ceil(2^16 / group): j / group == (j * magic) >> 16 for j < 64
    float scale;
    float softcap;
    uint32_t window;        // attention window of the layer (cache.rs:36-48); 0 = global
    uint32_t ring_blocks;   // 32-row blocks of the layer's storage ring; 0 = rows are positions
    // Split-K f16 kernel only: merge the splits inside the launch. `ws` is then the exchange
    // buffer (every word empty between launches) and item.ws0 counts its records; a consumer
    // gives up after spin_limit polls.
    uint32_t exchange;
    uint32_t spin_limit;
    // Block kernel only, unsplit causal launches: workgroups reach the device in runs of this
    // many (one per compute unit); every second run takes its units in reverse, so that the
    // two workgroups that share a compute unit are a long row tile and a short one. 0 = off.
    uint32_t fold_units;
    // The step's keys and values, over all layers of the pool, are more than the last-level cache
    // holds (so the next step will not find them there): kernels that read each row once may ask
    // for them with the streaming hint.
    uint32_t kv_streams;
};
// What the reference's model does around the step (muse-glimmer/src/model.rs:445-464),
// folded into the step's own launches instead of running as launches of their own. `gate`
// (out *= sigmoid(gate), cpu.rs:657-673) is applied by whichever kernel writes the final
// output; `prep_on` makes the split-K kernel norm and rotate the raw Q rows and new K rows it
// reads (its 16-vector variants only). A separate kernel argument, so that launches without
// any of it carry and fetch nothing more.
struct FoldedParams {
    const float *gate;          // [sum rows][q_heads*head_dim] or null
    uint32_t prep_on;
    uint32_t prep_interleaved;  // 1: pairs (2i, 2i+1); 0: pairs (i, i + prep_rot/2)
    uint32_t prep_rot;          // rotary_dim; 0 = no rotation
    float prep_eps;
    const float *prep_q_weight; // [head_dim] or null: no norm
    const float *prep_k_weight;
    double prep_freq_step;      // pair i turns at position * 2^(i * prep_freq_step) radians
};
// sigmoid for the writers of f16-KV attention output, whose bar is 2e-3: one exponential
// and one reciprocal instruction, a few ulp, the same limits at both ends (0 and 1) as the
// reference's two-branch form (cpu.rs:162-169).
__device__ __forceinline__ float sigmoid_fast(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __expf(-x));
}
// sigmoid as the reference writes it (cpu.rs:162-169).
__device__ __forceinline__ float sigmoid_ref(float x) {
    if (x >= 0.0f) return 1.0f / (1.0f + expf(-x));
    const float e = expf(x);
    return e / (1.0f + e);
}
// The oldest position a query at `pos` sees (attention.rs:77-85 and the view's oldest row).
__host__ __device__ inline uint32_t lowest_visible(uint32_t pos, uint32_t window, uint32_t kv_lo) {
    const uint32_t lo = (window != 0 && pos + 1 > window) ? pos + 1 - window : 0;
    return lo > kv_lo ? lo : kv_lo;
}

// Generic VALU path: f32 or f16 storage, any head_dim <= 256, group <= 64. Partials are in
// natural-log domain (combine with base2 = 0).
hipError_t launch_attn_generic(int elem_f16, const AttnParams &p, const AttnBatch &b,
                               uint32_t total_partials, hipStream_t stream);
// Query rows one workgroup of the generic kernel carries (0 = shape not supported).
uint32_t attn_generic_rows_per_block(uint32_t group, uint32_t head_dim);
// Keys per tile of the generic kernel for a head_dim.
uint32_t attn_generic_tile(uint32_t head_dim);

// MFMA split-K path: f16 pools with blocked value planes, head_dim 128, rows*group <= 64.
// Partials are in log2 domain (combine with base2 = 1).
bool attn_splitk_f16_supports(const PoolGeom &g, uint32_t group, uint32_t max_rows);
uint32_t attn_splitk_f16_plan(const PoolGeom &g, AttnBatch &b, uint32_t q_heads);
// After attn_splitk_f16_plan: whether the batch can merge its splits inside the split-K launch
// (AttnParams::exchange). Returns the 64-bit words the exchange buffer must hold and re-bases
// the items' ws0 on it, or 0 (items untouched) when the batch keeps the merge launch.
uint64_t attn_splitk_f16_plan_exchange(const PoolGeom &g, AttnBatch &b, uint32_t q_heads);
// Sets `count` 64-bit words to `value` (the exchange buffer's empty pattern, at set-up).
hipError_t launch_fill_words(unsigned long long *dst, uint64_t count, unsigned long long value,
                             hipStream_t stream);
constexpr unsigned long long kExchangeEmptyWord = 0xffffffffffffffffull;
// `folded` with prep_on set selects the variants that prepare Q and the new K rows themselves
// and gate what they write (every item must then be a 16-vector step); otherwise it is ignored.
// `q_two_halves`: the queries enter the score products as f16 hi + f16 lo (two products per
// score tile), so that their rounding to f16 leaves the scores (ITAK_POOL_Q_TWO_HALVES).
hipError_t launch_attn_splitk_f16(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                  uint32_t max_rows, hipStream_t stream,
                                  const FoldedParams *folded = nullptr, bool q_two_halves = false);
// The two-halves instantiations (attn_splitk_f16_qlo.hip) and the variant a batch takes.
hipError_t launch_attn_splitk_f16_qlo(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                      hipStream_t stream, const FoldedParams *folded);
int attn_splitk_f16_variant(const PoolGeom &g, const AttnBatch &b, uint32_t group);
// ---- the split merge on a unit's compute die (attn_splitk_f16_die.hip) ---------------------
// The device's workgroups are dealt round-robin over its eight compute dies, each with an L2 of
// its own. A launch planned for it puts every split of a unit = (item, KV head, part of the
// query vectors) on one die; the unit's last workgroup to finish merges the partials out of
// that die's L2, so there is neither a merge launch nor a wait.
constexpr uint32_t kDieCount = 8;
constexpr uint32_t kDieTicketStride = 32;  // words from one unit's ticket to the next: a cache line each
constexpr uint32_t kDieMaxUnits = 1024;
constexpr uint64_t kDieTicketBytes = uint64_t(kDieMaxUnits) * kDieTicketStride * 4;
struct DieMap {
    uint32_t *tickets;  // kDieMaxUnits words kDieTicketStride apart, zero whenever no launch runs
    uint32_t *faults;   // workgroups that found themselves on another die than their index names
    const float *gate;  // merged rows are multiplied by sigmoid(gate) as they are written, or null
    uint32_t shift;     // log2(heads a bin's dies share out): die = bin << shift | KV head
    uint32_t pad;
    uint32_t bin_first[kDieCount + 1];  // items of bin i: [bin_first[i], bin_first[i + 1])
    uint32_t bin_count[kDieCount];      // workgroups of a die of bin i
};
// True when the current device deals workgroup i to compute die i % 8 (probed once per device:
// a small launch whose workgroups report the hardware's die number).
bool die_layout_ok(int device);
// Plans `b` (slot, rows, pos0, q_row0, kv_len, kv_lo set) for the die-local merge: `out` gets
// the items in bin order with splits, keys_per_split, block0 (first index on the die), ws0 and
// the unit's first ticket (in splits_magic); `map` the bins. Returns the partials the launch
// writes, 0 when the batch is better served by the ordinary plan (too few or too uneven units,
// a KV head count that does not deal out over eight dies, nothing to split).
uint32_t attn_splitk_f16_plan_die(const PoolGeom &g, const AttnBatch &b, uint32_t q_heads,
                                  AttnBatch &out, DieMap &map);
hipError_t launch_attn_splitk_f16_die(const AttnParams &p, const AttnBatch &b, const DieMap &map,
                                      uint32_t total_partials, hipStream_t stream,
                                      const FoldedParams *folded = nullptr);
// The latency-shaped form of the same path for decode steps (attn_decode_f16.hip): every item
// one new row, at most one block per wavefront, splits merged inside the launch. `takes` is
// asked after the batch has been planned and AttnParams::exchange set.
bool attn_decode_f16_takes(const AttnParams &p, const AttnBatch &b);
// Workgroups of that kernel the device holds at once (the smallest figure over its
// instantiations, asked of the runtime once).
uint32_t attn_decode_f16_resident_groups();
hipError_t launch_attn_decode_f16(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                  hipStream_t stream, bool q_two_halves = false);
// f32 MFMA split-K path: f32 pools (row-major planes), head_dim 128, rows*group <= 16, implied
// query positions. Partials are in log2 domain (combine with base2 = 1).
bool attn_splitk_f32_supports(const PoolGeom &g, uint32_t group, uint32_t max_rows);
// True when such a launch also appends the step's rows (k_new / v_new in its parameters).
bool attn_splitk_f32_appends(const PoolGeom &g, uint32_t group, uint32_t max_rows);
uint32_t attn_splitk_f32_plan(const PoolGeom &g, AttnBatch &b, uint32_t q_heads);
hipError_t launch_attn_splitk_f32(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                  hipStream_t stream);
// MFMA block path (speculative blocks and prefill chunks): same pools, any number of rows,
// group dividing 16; K/V staged through LDS, split over the context when the launch would
// otherwise not fill the device. Partials are in log2 domain (combine with base2 = 1).
bool attn_prefill_f16_supports(const PoolGeom &g, uint32_t group);
uint32_t attn_prefill_f16_plan(const PoolGeom &g, AttnBatch &b, uint32_t group, uint32_t q_heads,
                               uint32_t window, bool appends = false);
// True when a launch of the block kernel over items of at most `most_rows` rows and
// `most_blocks` key blocks appends the items' rows itself (k_new / v_new in its parameters).
bool attn_prefill_f16_appends(const PoolGeom &g, uint32_t group, uint32_t most_rows,
                              uint32_t most_blocks);
hipError_t launch_attn_prefill_f16(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                   hipStream_t stream);
// The same at head dims 64, 96 and 256 (instantiated in a file of their own); `one` = the
// one-tile form, as launch_attn_prefill_f16 decides it.
// The two-halves form (head_dim 128, two tiles, no rows brought along).
hipError_t launch_attn_prefill_f16_qlo(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                       hipStream_t stream);
hipError_t launch_attn_prefill_f16_dims(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                        bool one, hipStream_t stream);
// Merge of split partials; total_rows = query rows of the batch. With `gate` the merged rows
// are multiplied by sigmoid(gate) as they are written (items with one split are not touched:
// their writer was the attention kernel).
hipError_t launch_attn_combine(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                               uint32_t total_rows, int base2, hipStream_t stream,
                               const float *gate = nullptr);

}  // namespace itak
