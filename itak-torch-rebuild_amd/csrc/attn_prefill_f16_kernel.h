// The block kernel and its launch templates, included by the files that instantiate it
// (attn_prefill_f16.hip: head_dim 128 and the planner; attn_prefill_f16_dims.hip: the other head
// dims), so that the two sets of instantiations compile side by side.
//
// Chunked causal prefill attention for gfx950, f16 KV, head_dim 64, 96, 128 or 256 (a template
// argument; the figures in these comments are those of head_dim 128): QK^T and PV on
// v_mfma_f32_16x16x32_f16, everything else (scale, softcap, mask, online softmax) in f32.
//
// One workgroup of four wavefronts owns (item, kv head, tile of 128 query vectors), where a
// query vector is one query row of one Q head of the KV group: with a group of 8 that is
// 16 consecutive rows x 8 heads, all reading the same K and V. Each wavefront keeps 32 of
// the vectors (2 MFMA column tiles): Q^T as f16 B-operands in registers for the whole
// kernel, O^T as f32 accumulators; at most 256 registers, so two workgroups share a compute
// unit and one wavefront's softmax runs under another's MFMAs. The workgroup walks the
// context in 32-key blocks. Per block and column tile:
//   S^T = K . Q^T (8 MFMA), softcap / causal mask, softmax in the lane's own column,
//   O^T += V^T . P^T (8 MFMA).
//
// K/V blocks travel HBM -> LDS without passing through registers (global_load_lds_dwordx4:
// lane i of the instruction writes 16 bytes at M0 + 16*i) into a ring of four stages, so
// the loads of three blocks are in flight while one is multiplied; the latency of a miss is
// about a microsecond, more than two block times. The planes are stored as the MFMA
// consumes them, so the key block is a straight 8 KiB copy; the 16-byte pieces of the value
// block are permuted on the way in (the source address of such a load is free per lane, the
// destination is lane-linear) so that every operand read of a wavefront is one KiB of
// consecutive LDS: no bank conflicts.
//
// The softmax keeps a *reference* maximum per column instead of the exact running maximum:
//   * the reference enters the score MFMA as its initial accumulator (-ref), so the product
//     comes out as s - ref and the exponent needs no subtraction;
//   * the reference moves only when some score of the block exceeds it by more than
//     kRefSlack (P is bounded by 2^kRefSlack, far inside f16 and f32 range), which after
//     the first blocks is rare: the cross-lane maximum, the rescale of the accumulators and
//     the branch around them leave the common path. The result is the same softmax: every
//     term of numerator and denominator carries the same factor 2^-ref.
// A column with nothing visible yet has ref = 0 and threshold -inf, so its first finite
// score sets the reference exactly.
//
// The chunk's own K/V rows are appended before this kernel runs; row r of the chunk sits at
// position pos0 + r and sees keys <= its position (attention.rs:77-85 with no window).
// Blocks of up to kFuseRows rows in the one-tile form bring their rows along instead
// (AttnParams::k_new / v_new): every workgroup whose run of key blocks reaches the new
// positions converts them in its prologue, keeps them in registers (16 pieces of 4 channels a
// thread) and writes them over what the ring's loads brought into LDS for those blocks, and
// one workgroup per KV head stores them to the planes. That is one launch and its gap less per
// layer for the blocks where a launch is a sixth of the layer.
#pragma once

#include "internal.h"
#include "mfma_common.h"
#include "timeline.h"

#include <algorithm>

namespace itak {

namespace {

constexpr int kWaves = 4;
constexpr int kMaxTiles = 2;  // MFMA column tiles (16 query vectors) per wavefront: 1 or 2
// Halves in one plane block (8 KiB at head_dim 128) and bytes in one stage of the LDS ring (one
// key block + one value block).
constexpr int block_elems(int d) { return kBlockKeys * d; }
constexpr int stage_bytes(int d) { return 2 * block_elems(d) * 2; }
constexpr float kRefSlack = 8.0f;
// The smallest divisor of 16 that holds a GQA group of up to 16 heads.
__host__ __device__ inline uint32_t padded_group(uint32_t group) {
    return group <= 1 ? 1 : group <= 2 ? 2 : group <= 4 ? 4 : group <= 8 ? 8 : 16;
}
// New rows a launch that appends its own rows carries at most: sixteen 16-byte pieces a thread.
constexpr int fuse_rows(int d) { return d <= 128 ? 64 : 16; }
constexpr uint32_t kOneTileBlocks = 520;  // key blocks up to which blocks of <= 512 vectors take one tile

__device__ __forceinline__ float column_max4(float v) {
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const auto c = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(c[0]), __uint_as_float(c[1]));
}
// The largest of three, none of them a signalling NaN (scores and -inf): one instruction, no
// quieting of the inputs.
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// The direct-to-LDS load is issued from inline assembly: the compiler then neither tracks it
// (it would make every LDS read wait for all of them) nor needs to, because the only consumer
// is ordered by the explicit s_waitcnt vmcnt + s_barrier at the top of each iteration.
constexpr int kStages = 4;      // blocks of the LDS ring: three in flight while one is read
constexpr int kDeepStages = 8;  // for short runs of blocks, one workgroup per compute unit

__device__ __forceinline__ void lds_dma16(const void *src, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(src), "s"(lds_addr)
                 : "memory");
}
// s_waitcnt vmcnt(n), other counters untouched.
template <int n>
__device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt(0x0f70 | (n & 15) | ((n >> 4) << 14));
}

// RING = the layer is windowed (blocks start at the window, live in a ring, the mask has a
// lower edge); global layers run the instantiation without any of it.
// D = head_dim. At 256 a stage of the ring is 32 KiB and a wavefront's accumulators alone are 64
// to 128 registers: one workgroup per compute unit, up to 512 registers a lane.
// QLO (ITAK_POOL_Q_TWO_HALVES; head_dim 128, two tiles): the scaled queries are held as two
// halves, q = hi + lo with hi = f16(q) and lo = f16(q - hi), and every score is K.hi + K.lo: the
// queries' rounding to f16, which is relative to each channel and so grows with the scores,
// leaves the scores. Half as many score products again on a kernel the matrix pipe bounds.
template <int N, bool SOFTCAP, int kTiles, bool RING, int STAGES, int D, bool QLO = false>
__global__ __launch_bounds__(kWaves * 64, D <= 128 ? 2 : 1) void attn_prefill_f16_kernel(
    AttnParams p, AttnBatchT<N> b, uint32_t total_partials) {
    constexpr int kD = D;
    constexpr int kSteps = D / 32;  // MFMAs of one score tile (32 channels each)
    constexpr int kOut = D / 16;    // output tiles of 16 channels
    constexpr int kBlockElems = block_elems(D);
    constexpr int kStageBytes = stage_bytes(D);
    constexpr int kPieces = (D + 63) / 64;  // KiB pieces of a key (or value) block each wavefront moves
    constexpr int kLoads = 2 * kPieces;  // ring loads a thread issues per block
    constexpr int kChunks = D / 4;       // 16-byte pieces of one side of a new f32 row
    constexpr int kRowsPerPass = kWaves * 64 / (2 * kChunks);  // new rows the workgroup loads at once
    constexpr int kFuseRows = fuse_rows(D);
    constexpr int kFusePieces = (kFuseRows + kRowsPerPass - 1) / kRowsPerPass;  // per thread
    constexpr int kVecPerWave = kTiles * 16;
    // The row-by-row product for values that are not finite is compiled into every form (the
    // switch is kept for measurements of what it costs: 0 to 2 %, head_dim 96 5 % on chunks).
    constexpr bool kByRow = true;
    constexpr int kVecPerGroup = kWaves * kVecPerWave;  // query vectors per workgroup
    extern __shared__ __attribute__((aligned(16))) uint16_t lds_ring[];  // [kStages][K block | V block]

    const uint32_t tid = threadIdx.x;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const uint32_t g = lane >> 4, jl = lane & 15;
    ITAK_MARK_BEGIN
    ITAK_MARK(0)

    const AttnItem item = b.item[b.find_by_block(blockIdx.x)];
    // A query row's heads of one KV group fill `gp` consecutive columns: the group size padded
    // to the next divisor of 16 (a group of 5 takes 8 columns, three of them zero queries whose
    // results are dropped), so that a row never straddles two MFMA tiles.
    const uint32_t group = p.group, gp = padded_group(group);
    const uint32_t rows_per_group = kVecPerGroup / gp;
    const uint32_t rows_per_wave = kVecPerWave / gp;
    // Workgroup -> (row tile, kv head, split of the context).
    const uint32_t local = blockIdx.x - item.block0;
    uint32_t unit = local / item.splits;
    const uint32_t split = local - unit * item.splits;
    const uint32_t tiles = (item.rows + rows_per_group - 1) / rows_per_group;
    // Units are handed out longest row tile first. All of an unsplit causal launch's first two
    // runs (one workgroup per compute unit each) are resident from the start, the second run
    // beside the first: taken in the same order, the longest tiles would share their compute
    // units with the longest of the second half. Every second run is taken in reverse.
    // The row tiles are reversed, not the KV heads: workgroup i of a launch runs on compute die
    // i mod 8, so with unit mod kv_heads as the head every die keeps reading the K/V of one head
    // (two dies per head with 4 KV heads) and the head's blocks are fetched into two L2s, not four.
    if (p.fold_units) {
        const uint32_t run = unit / p.fold_units, idx = unit - run * p.fold_units;
        const uint32_t span = min(p.fold_units, tiles * p.g.kv_heads - run * p.fold_units);
        if (run & 1) {
            const uint32_t t = idx / p.g.kv_heads, h = idx - t * p.g.kv_heads;
            unit = run * p.fold_units + (span / p.g.kv_heads - 1 - t) * p.g.kv_heads + h;
        }
        unit = __builtin_amdgcn_readfirstlane(unit);  // (the divisions run on the vector unit)
    }
    const uint32_t kv_head = unit % p.g.kv_heads;
    const uint32_t tile = tiles - 1 - unit / p.g.kv_heads;  // longest first
    const uint32_t row_begin = tile * rows_per_group + wave * rows_per_wave;
    const uint32_t wg_row_end = min(item.rows, (tile + 1) * rows_per_group);

    const uint16_t *kplane = static_cast<const uint16_t *>(p.layer_base) +
                             item.slot * p.g.slot_stride + kv_head * p.g.head_stride;
    const uint16_t *vplane = kplane + p.g.side_stride;

    // Blocks of this workgroup: its split's run of the blocks its rows can see (on a windowed
    // layer those start at the window of the workgroup's first row, not at the item's).
    const uint32_t blocks_per_split = item.keys_per_split / kBlockKeys;
    const uint32_t window = RING ? p.window : 0, kv_lo = RING ? item.kv_lo : 0;
    const uint32_t wg_lo =
        lowest_visible(item.pos0 + min(tile * rows_per_group, item.rows - 1), window, kv_lo);
    const uint32_t kb_begin = wg_lo / kBlockKeys + split * blocks_per_split;
    // (Rows that stand ahead of the stored length see all of it and nothing more.)
    const uint32_t nblocks =
        min((min(item.pos0 + wg_row_end, item.kv_len) + kBlockKeys - 1) / kBlockKeys,
            kb_begin + blocks_per_split);
    const uint32_t wave_row_end = min(item.rows, row_begin + rows_per_wave);
    [[maybe_unused]] const uint32_t wave_rows = wave_row_end - min(wave_row_end, row_begin);
    [[maybe_unused]] const uint32_t gp_shift = __builtin_amdgcn_readfirstlane(__builtin_ctz(gp));
    const uint32_t wave_blocks =
        row_begin < item.rows
            ? (min(item.pos0 + wave_row_end, item.kv_len) + kBlockKeys - 1) / kBlockKeys
            : 0;
    const uint32_t first_masked = (min(item.pos0 + row_begin, item.kv_len - 1) + 1) / kBlockKeys;
    // Lower edge: blocks before wave_first hold nothing this wavefront's rows see; blocks
    // before low_masked_end hold positions too old for some of them.
    // [wave_lo, wave_hi): the positions some row of this wavefront sees. Outside it the value
    // operand is cleared (stale ring rows, rows past the stored length, and rows that only other
    // wavefronts' rows see: a masked key's zero weight times a value that is not finite would
    // be NaN); a wavefront with one row needs nothing else to be exact.
    const uint32_t wave_lo = lowest_visible(item.pos0 + min(row_begin, item.rows - 1), window, kv_lo);
    const uint32_t wave_hi = min(item.pos0 + max(wave_row_end, 1u), item.kv_len);
    const uint32_t wave_first = wave_lo / kBlockKeys;
    const uint32_t low_masked_end =
        (lowest_visible(item.pos0 + wave_row_end - 1, window, kv_lo) + kBlockKeys - 1) / kBlockKeys;

    // Each wavefront moves kPieces 1 KiB pieces of the key block and as many of the value block
    // (piece w + 4i for wavefront w). When the block is not a multiple of 4 KiB (head_dim 96: six
    // pieces), the wavefronts whose last piece would lie past it fetch their previous piece twice:
    // every wavefront then has the same number of loads in flight, which is what the waits count.
    static_assert(D % 32 == 0 && (D % 64 == 0 || kPieces >= 2), "piece plan");
    const uint32_t last_piece = wave + 4u * (kPieces - 1) < uint32_t(D / 16) ? kPieces - 1 : kPieces - 2;
    const uint4 *kg = reinterpret_cast<const uint4 *>(kplane) + tid;
    // Value pieces are permuted on the way in: LDS position dt*64 + g*16 + jl holds the
    // 16 bytes (channel dt*16 + jl, keys g*8 .. g*8+7), so that the operand read of a
    // wavefront is linear in the lane number like the key read (the plane's own order,
    // channel-major, would make 16 consecutive lanes read at a 64-byte stride: bank
    // conflicts). The pieces of one load still come from one contiguous KiB.
    const uint4 *vg = reinterpret_cast<const uint4 *>(vplane) + (wave * 16 + jl) * 4 + g;
    constexpr uint32_t kBlockVec = kBlockElems / 8;
    const uint32_t ring_base =
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)(lds_ring);  // LDS byte address
    const uint32_t dma_base = ring_base + wave * 1024;
    // Storage block of the next block to fetch: position blocks are consecutive, so it climbs
    // by one and wraps at the end of a windowed layer's ring.
    const uint32_t ring_blocks = RING ? p.ring_blocks : 1;
    uint32_t next_sb = RING ? kb_begin % ring_blocks : 0;
    auto issue_block = [&](uint32_t kb) {
        // Past the end the last block is fetched again into a stage nobody reads: the
        // number of loads in flight stays the same in every iteration.
        const uint64_t off = uint64_t(RING ? next_sb : min(kb, max(nblocks, 1u) - 1)) * kBlockVec;
        if (RING && kb + 1 < nblocks) next_sb = next_sb + 1 == ring_blocks ? 0 : next_sb + 1;
        const uint32_t dst = dma_base + (kb % STAGES) * kStageBytes;
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const uint32_t ii = i == kPieces - 1 ? last_piece : uint32_t(i);
            lds_dma16(kg + off + 256 * ii, dst + 4096 * ii);
        }
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const uint32_t ii = i == kPieces - 1 ? last_piece : uint32_t(i);
            lds_dma16(vg + off + 256 * ii, dst + 2 * kBlockElems + 4096 * ii);
        }
    };
    const bool any_block = kb_begin < nblocks;  // a split past the rows' horizon has none
    ITAK_MARK(1)

    // With a softcap the score MFMA yields the argument of tanh's exponential directly
    // (2 * log2(e) * s / cap): one multiply less on every score.
    const float softcap = p.softcap;
    const float cap2 = SOFTCAP ? softcap * kLog2e : 0.0f;
    const float qscale = SOFTCAP ? p.scale * (2.0f * kLog2e / softcap) : p.scale * kLog2e;
    // Q^T of the wavefront's vectors. The Q loads go out first, the ring is filled behind them,
    // and Q is converted as soon as it is in: loads return in order, so Q is not held up by
    // three to seven blocks of keys and values, which a short run of blocks could not hide.
    // The compiler cannot count the ring's loads (they are issued from assembly), so it would
    // wait for everything before the first use of Q: the Q loads are issued from assembly too
    // and waited for by count. Between such a load and the wait that names its registers the
    // code is a straight line: across a branch the compiler may copy a register it believes
    // loaded, and would copy what was there before. So the ring is always filled (a workgroup
    // without blocks fetches block 0 into stages nobody reads), rows past the block's end
    // re-read its last row and are scaled to zero columns, and the variant that also brings new
    // rows is a second straight line, not a branch inside this one.
    //
    // New rows (one-tile form only): piece u of this thread is row nrow + kRowsPerPass * u, side
    // nside, channels nc4 .. nc4 + 3 (at head_dim 128: row (tid >> 6) + 4u, side (tid >> 5) & 1,
    // channels (tid & 31) * 4), requested ahead of Q and waited for with it.
    // At head_dim 96 a row is 48 pieces: five rows a pass, the last sixteen threads idle.
    constexpr bool kCanFuse = kTiles == 1;
    const bool fused = kCanFuse && p.k_new != nullptr;
    const uint32_t nrow = tid / (2 * kChunks);
    const bool nlane = nrow < uint32_t(kRowsPerPass);  // false only where a row is not a divisor of 256 lanes
    const uint32_t nside = (tid / kChunks) & 1u, nc4 = (tid % kChunks) * 4;
    // Does this workgroup's run of blocks reach the new positions? Is it the one that stores them?
    const bool patches = fused && any_block && nblocks * kBlockKeys > item.pos0;
    const bool stores_new = fused && unit < p.g.kv_heads && split == item.splits - 1;
    const bool with_new = patches || stores_new;
    // (See the stores below. The new rows touch up to three consecutive position blocks; on a ring
    // of fewer storage blocks two of them are the same storage block, and the stage of the later
    // one, fetched before the earlier one was stored, would put the old rows back over the new.)
    const bool by_stage = stores_new && patches && item.rows >= 8 && (!RING || ring_blocks >= 3);
    [[maybe_unused]] uint2 npk[kCanFuse ? kFusePieces : 1];
    half8 qb[kTiles][kSteps];
    static_assert(!QLO || (kTiles == 2 && D == 128), "the two-halves form exists for two tiles at head_dim 128");
    [[maybe_unused]] half8 qb_lo[QLO ? kTiles : 1][kSteps];
    uint32_t colpos[kTiles], collo[kTiles];
    const float *qp[kTiles];
    float qsc[kTiles];
#pragma unroll
    for (int qt = 0; qt < kTiles; ++qt) {
        const uint32_t j = qt * 16 + jl;
        const uint32_t row = row_begin + j / gp, hq = j % gp;
        colpos[qt] = min(item.pos0 + row, item.kv_len - 1);
        collo[qt] = lowest_visible(item.pos0 + row, window, kv_lo);
        const uint32_t head = kv_head * group + min(hq, group - 1);
        qp[qt] = p.q + (uint64_t(item.q_row0 + min(row, item.rows - 1)) * p.q_heads + head) * kD + g * 8;
        qsc[qt] = row < item.rows && hq < group ? qscale : 0.0f;
    }
#define ITAK_Q_LOADS(qraw)                                                                      \
    _Pragma("unroll") for (int qt = 0; qt < kTiles; ++qt)                                       \
        _Pragma("unroll") for (int s = 0; s < 2 * kSteps; ++s)                                  \
            asm volatile("global_load_dwordx4 %0, %1, off"                                      \
                         : "=v"(qraw[qt][s])                                                    \
                         : "v"(qp[qt] + (s >> 1) * 32 + (s & 1) * 4)                            \
                         : "memory");
#define ITAK_RING_FILL                                                                          \
    _Pragma("unroll") for (int ahead = 0; ahead < STAGES - 1; ++ahead) issue_block(kb_begin + ahead);
// Everything older than the ring's loads has landed. The registers named after the wait pass
// through an (empty) statement behind it, so that nothing that reads them is scheduled ahead.
#define ITAK_WAIT_BEHIND_RING asm volatile("s_waitcnt vmcnt(%0)" : : "n"(kLoads * (STAGES - 1)) : "memory");
#define ITAK_Q_ARRIVED(qraw)                                                                    \
    _Pragma("unroll") for (int qt = 0; qt < kTiles; ++qt)                                       \
        _Pragma("unroll") for (int s = 0; s < 2 * kSteps; ++s) asm volatile("" : "+v"(qraw[qt][s]));
#define ITAK_Q_CONVERT(qraw)                                                                    \
    _Pragma("unroll") for (int qt = 0; qt < kTiles; ++qt)                                       \
        _Pragma("unroll") for (int s = 0; s < kSteps; ++s) {                                    \
            const floatx4 a = qraw[qt][2 * s], c = qraw[qt][2 * s + 1];                         \
            const float sc = qsc[qt];                                                           \
            qb[qt][s] = half8{static_cast<_Float16>(a[0] * sc), static_cast<_Float16>(a[1] * sc), \
                              static_cast<_Float16>(a[2] * sc), static_cast<_Float16>(a[3] * sc), \
                              static_cast<_Float16>(c[0] * sc), static_cast<_Float16>(c[1] * sc), \
                              static_cast<_Float16>(c[2] * sc), static_cast<_Float16>(c[3] * sc)}; \
            if constexpr (QLO) {                                                                \
                _Pragma("unroll") for (int e = 0; e < 8; ++e) {                                 \
                    const float full = (e < 4 ? a[e & 3] : c[e & 3]) * sc;                      \
                    qb_lo[qt][s][e] = static_cast<_Float16>(full - float(qb[qt][s][e]));        \
                }                                                                               \
            }                                                                                   \
        }
    bool took_new = false;
    if constexpr (kCanFuse) {
        if (with_new) {
            took_new = true;
            floatx4 nraw[kFusePieces], qraw[kTiles][2 * kSteps];
            const uint32_t row_width = p.g.kv_heads * kD;
            const float *src = (nside ? p.v_new : p.k_new) + uint64_t(item.q_row0) * row_width +
                               kv_head * kD + nc4;
#pragma unroll
            for (int u = 0; u < kFusePieces; ++u) {
                const uint32_t r = min(nrow + uint32_t(kRowsPerPass) * u, item.rows - 1);
                asm volatile("global_load_dwordx4 %0, %1, off"
                             : "=v"(nraw[u])
                             : "v"(src + uint64_t(r) * row_width)
                             : "memory");
            }
            ITAK_Q_LOADS(qraw)
            ITAK_RING_FILL
            ITAK_MARK(2)
            ITAK_WAIT_BEHIND_RING
            ITAK_Q_ARRIVED(qraw)
#pragma unroll
            for (int u = 0; u < kFusePieces; ++u) asm volatile("" : "+v"(nraw[u]));
            ITAK_Q_CONVERT(qraw)
            // The conversion rule (f32_to_f16_bits) is the hardware's rounding plus a fixed
            // pattern for NaNs: a sum that is not a NaN proves its four terms are not, so the
            // wavefront converts in pairs and takes the element-wise rule only when some lane
            // met a NaN (or an infinity that cancelled). Pieces past the block's rows repeat
            // its last row and are never written anywhere: skipped.
            bool nan_seen = false;
#pragma unroll
            for (int u = 0; u < kFusePieces; ++u) {
                const float sum = (nraw[u][0] + nraw[u][1]) + (nraw[u][2] + nraw[u][3]);
                nan_seen = nan_seen || sum != sum;
            }
            const bool by_element = __builtin_amdgcn_ballot_w64(nan_seen) != 0;
#pragma unroll
            for (int u = 0; u < kFusePieces; ++u) {
                // (Uniform over the wavefront when a row is 64 lanes.)
                if (!nlane || (2 * kChunks == 64 ? wave : nrow) + uint32_t(kRowsPerPass) * u >= item.rows) continue;
                if (by_element) {
                    const uint32_t h0 = f32_to_f16_bits(nraw[u][0]), h1 = f32_to_f16_bits(nraw[u][1]);
                    const uint32_t h2 = f32_to_f16_bits(nraw[u][2]), h3 = f32_to_f16_bits(nraw[u][3]);
                    npk[u] = uint2{h0 | (h1 << 16), h2 | (h3 << 16)};
                } else {
                    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
                    const half2_t lo{static_cast<_Float16>(nraw[u][0]), static_cast<_Float16>(nraw[u][1])};
                    const half2_t hi{static_cast<_Float16>(nraw[u][2]), static_cast<_Float16>(nraw[u][3])};
                    npk[u] = uint2{__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi)};
                }
            }
        }
    }
    if (!took_new) {
        floatx4 qraw[kTiles][2 * kSteps];
        ITAK_Q_LOADS(qraw)
        ITAK_RING_FILL
        ITAK_MARK(2)
        ITAK_WAIT_BEHIND_RING  // that is Q
        ITAK_Q_ARRIVED(qraw)
        ITAK_Q_CONVERT(qraw)
    }
#undef ITAK_Q_CONVERT
#undef ITAK_Q_ARRIVED
#undef ITAK_WAIT_BEHIND_RING
#undef ITAK_RING_FILL
#undef ITAK_Q_LOADS
    if constexpr (kCanFuse) {
        // As the append kernel lays them out (k_offset / v_offset). From registers, a value row
        // leaves as one two-byte store per channel (sixty-four such stores a thread for a 64-row
        // block, each touching as many cache lines as it has lanes: 6 us in the one workgroup per
        // KV head that stores, the last to finish). Blocks of eight rows or more are therefore
        // stored block by block from the LDS stage once the rows have been written over it (below),
        // sixteen bytes a thread and store; what remains here are short blocks and rows of key
        // blocks that lie before this workgroup's run.
        if (stores_new) {
            uint16_t *kp = const_cast<uint16_t *>(kplane), *vp = const_cast<uint16_t *>(vplane);
#pragma unroll
            for (int u = 0; u < kFusePieces; ++u) {
                const uint32_t r = nrow + uint32_t(kRowsPerPass) * u;
                if (!nlane || r >= item.rows) continue;
                const uint32_t key = item.pos0 + r, kin = key % kBlockKeys;
                if (by_stage && key / kBlockKeys >= kb_begin) continue;
                const uint32_t sb = RING ? (key / kBlockKeys) % ring_blocks : key / kBlockKeys;
                const uint64_t blk = uint64_t(sb) * kBlockElems;
                if (nside == 0) {
                    const uint32_t kt = (kin >> 2) & 1, ki = (kin >> 3) * 4 + (kin & 3);
                    *reinterpret_cast<uint2 *>(kp + blk + ((kt * (kD / 8) + (nc4 >> 3)) * 16 + ki) * 8 +
                                               (nc4 & 7)) = npk[u];
                } else {
                    uint16_t *vd = vp + blk + nc4 * kBlockKeys + kin;
                    vd[0] = uint16_t(npk[u].x);
                    vd[kBlockKeys] = uint16_t(npk[u].x >> 16);
                    vd[2 * kBlockKeys] = uint16_t(npk[u].y);
                    vd[3 * kBlockKeys] = uint16_t(npk[u].y >> 16);
                }
            }
        }
    }
    ITAK_MARK(3)
    // The denominator goes through the matrix pipe: one more MFMA per tile and block with an
    // all-ones A operand leaves the block's sum of P (as rounded for P.V, over all 32 keys) in
    // every row of a 16x16 accumulator. That replaces eight additions per tile and block, and
    // ordinary vector instructions are what this loop runs out of (they do not overlap with a
    // SIMD's MFMAs; the extra MFMA costs a quarter of the additions' issue time).
    float ref[kTiles], thr[kTiles];
    floatx4 l[kTiles];
    floatx4 negref[kTiles];
    const half8 ones = {_Float16(1.0f), _Float16(1.0f), _Float16(1.0f), _Float16(1.0f),
                        _Float16(1.0f), _Float16(1.0f), _Float16(1.0f), _Float16(1.0f)};
    floatx4 o[kTiles][kOut];
#pragma unroll
    for (int qt = 0; qt < kTiles; ++qt) {
        ref[qt] = 0.0f;
        thr[qt] = -INFINITY;
        l[qt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        negref[qt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int dt = 0; dt < kOut; ++dt) o[qt][dt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    }

    for (uint32_t kb = kb_begin; kb < nblocks; ++kb) {
        // This thread's pieces of block kb have landed (the loads of the next STAGES - 2 blocks
        // may still fly); after the barrier everybody's have, and everybody is done with
        // block kb - 1, whose stage the loads for block kb + 3 may now overwrite.
        wait_vmcnt<kLoads * (STAGES - 2)>();
        if (kb == kb_begin) { ITAK_MARK(7) }
        __builtin_amdgcn_s_barrier();
        if (kb == kb_begin) { ITAK_MARK(8) }
        issue_block(kb + STAGES - 1);
        const uint16_t *lds_k = lds_ring + (kb % STAGES) * (kStageBytes / 2);
        const uint16_t *lds_v = lds_k + kBlockElems;
        if constexpr (kCanFuse) {
            if (patches && (kb + 1) * kBlockKeys > item.pos0) {
                // The block holds new positions: what the loads brought for them is whatever
                // the planes held (the storing workgroup may or may not have got there yet);
                // the rows themselves go over it, in the stage's layouts.
                uint16_t *sk = lds_ring + (kb % STAGES) * (kStageBytes / 2), *sv = sk + kBlockElems;
#pragma unroll
                for (int u = 0; u < kFusePieces; ++u) {
                    const uint32_t r = nrow + uint32_t(kRowsPerPass) * u;
                    const uint32_t key = item.pos0 + r, kin = key % kBlockKeys;
                    if (!nlane || r >= item.rows || key / kBlockKeys != kb) continue;
                    if (nside == 0) {
                        const uint32_t kt = (kin >> 2) & 1, ki = (kin >> 3) * 4 + (kin & 3);
                        *reinterpret_cast<uint2 *>(sk + ((kt * (kD / 8) + (nc4 >> 3)) * 16 + ki) * 8 +
                                                   (nc4 & 7)) = npk[u];
                    } else {
                        // piece (channel c, keys g*8..g*8+7) sits at (c/16)*64 + g*16 + c%16
                        uint16_t *vd = sv + (((nc4 >> 4) * 64 + (kin >> 3) * 16 + (nc4 & 15)) * 8) + (kin & 7);
                        vd[0] = uint16_t(npk[u].x);
                        vd[8] = uint16_t(npk[u].x >> 16);
                        vd[16] = uint16_t(npk[u].y);
                        vd[24] = uint16_t(npk[u].y >> 16);
                    }
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
                if (by_stage) {
                    // The stage now is what the planes' block should hold (rows past the new ones
                    // are what the loads brought from there): back it goes, the key block as it
                    // lies, the value pieces to where their load took them from.
                    const uint32_t sb = RING ? kb % ring_blocks : kb;
                    uint4 *kdst = reinterpret_cast<uint4 *>(const_cast<uint16_t *>(kplane)) + uint64_t(sb) * kBlockVec;
                    uint4 *vdst = reinterpret_cast<uint4 *>(const_cast<uint16_t *>(vplane)) + uint64_t(sb) * kBlockVec;
                    const uint4 *ks = reinterpret_cast<const uint4 *>(sk), *vs = reinterpret_cast<const uint4 *>(sv);
#pragma unroll
                    for (uint32_t i = tid; i < kBlockVec; i += kWaves * 64) {
                        kdst[i] = ks[i];
                        const uint32_t dt = i >> 6, gg = (i >> 4) & 3, jj = i & 15;
                        vdst[(dt * 16 + jj) * 4 + gg] = vs[i];
                    }
                }
                if (kb == kb_begin) { ITAK_MARK(9) }
            }
        }

        if (kb < wave_blocks && (!RING || kb >= wave_first)) {
            const uint32_t key_base = kb * kBlockKeys + g * 8;
            floatx4 x[kTiles][2];
            __builtin_amdgcn_s_setprio(0);  // raised again below, for the block's second half
            {
                half8 ka[2][kSteps];
                const uint16_t *kl = lds_k + (g * 16 + jl) * 8;
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int s = 0; s < kSteps; ++s)
                        ka[t][s] =
                            *reinterpret_cast<const half8 *>(kl + ((t * (kD / 8) + s * 4) * 16) * 8);
#pragma unroll
                for (int qt = 0; qt < kTiles; ++qt)
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        floatx4 s = negref[qt];
#pragma unroll
                        for (int k = 0; k < kSteps; ++k)
                            s = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[t][k], qb[qt][k], s, 0, 0, 0);
                        if constexpr (QLO) {
#pragma unroll
                            for (int k = 0; k < kSteps; ++k)
                                s = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[t][k], qb_lo[qt][k], s, 0, 0, 0);
                        }
                        x[qt][t] = s;
                    }
            }
            half8 va[kOut];
            const uint16_t *vl = lds_v + lane * 8;
#pragma unroll
            for (int dt = 0; dt < kOut; ++dt)
                va[dt] = *reinterpret_cast<const half8 *>(vl + dt * 64 * 8);

            if constexpr (SOFTCAP) {  // negref stays zero: x is the raw scaled score here
#pragma unroll
                for (int qt = 0; qt < kTiles; ++qt)
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        x[qt][e >> 2][e & 3] = softcap_of_exp2_arg(x[qt][e >> 2][e & 3], cap2, ref[qt]);
            }
            // A block at an edge of the mask whose values are not all finite: the wavefront's rows
            // share the value operand, and a masked key's zero weight times such a value is NaN,
            // where gqa_attention never reads the value row of a key a query does not see
            // (crates/attention/src/attention.rs:160-173). P.V is then taken row by row (below).
            [[maybe_unused]] bool by_row = false;
            if (RING && kb < low_masked_end) {
#pragma unroll
                for (int qt = 0; qt < kTiles; ++qt)
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (key_base + e < collo[qt]) x[qt][e >> 2][e & 3] = -INFINITY;
                if (kb * kBlockKeys < wave_lo) {
                    // Ring rows older than anything the wavefront's queries see may be stale.
                    const uint32_t stale = min(wave_lo - min(wave_lo, key_base), 8u);
                    const u32x4 keep = ~first_halves(stale);
#pragma unroll
                    for (int dt = 0; dt < kOut; ++dt)
                        va[dt] = keep_halves(va[dt], keep);
                }
                if constexpr (kByRow) by_row = true;
            }
            if (kb >= first_masked) {
#pragma unroll
                for (int qt = 0; qt < kTiles; ++qt)
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (key_base + e > colpos[qt]) x[qt][e >> 2][e & 3] = -INFINITY;
                if ((kb + 1) * kBlockKeys > wave_hi) {
                    // Rows past the stored length may hold stale data, rows past the wavefront's
                    // last row values that are not finite: keep them out of P.V.
                    const uint32_t stored = min(wave_hi - min(wave_hi, key_base), 8u);
                    const u32x4 keep = first_halves(stored);
#pragma unroll
                    for (int dt = 0; dt < kOut; ++dt)
                        va[dt] = keep_halves(va[dt], keep);
                }
                if constexpr (kByRow) by_row = true;
            }
            if constexpr (kByRow) {
                if (by_row && wave_rows > 1) {
                    // Is any value of the block not finite? Asked of the matrix pipe: the values
                    // times a zero operand sum to zero unless one of them is an infinity or a NaN
                    // (eight MFMAs and a comparison, where looking at the 32 registers' exponent
                    // fields takes a hundred vector instructions).
                    // At head_dim 96 the values are read from the stage again, here and in the
                    // row-by-row loop below: given the operand registers in a second kind of
                    // product and a cleared copy of them further down, the compiler keeps the
                    // operand as separate halves there and puts it together again in every
                    // block (24 permutes, a 512-row chunk 65 -> 71 us per layer; with the second
                    // read 68). The stage's copy has not had the stale and unstored rows cleared:
                    // at worst the row-by-row path is taken for a block that did not need it,
                    // and its own masks, one row's at a time, leave those rows out as well.
                    floatx4 t = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
                    const half8 zero = half8{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                    for (int dt = 0; dt < kOut; ++dt) {
                        half8 v;
                        if constexpr (D == 96)
                            v = *reinterpret_cast<const half8 *>(vl + dt * 64 * 8);
                        else
                            v = va[dt];
                        t = __builtin_amdgcn_mfma_f32_16x16x32_f16(v, zero, t, 0, 0, 0);
                    }
                    const float any = (t[0] + t[1]) + (t[2] + t[3]);
                    by_row = __builtin_amdgcn_ballot_w64(any != any) != 0;
                } else {
                    by_row = false;
                }
            }
            float lmax[kTiles];
            bool over = false;
#pragma unroll
            for (int qt = 0; qt < kTiles; ++qt) {
                float mx = max3(x[qt][0][0], x[qt][0][1], x[qt][0][2]);
                mx = max3(mx, x[qt][0][3], x[qt][1][0]);
                mx = max3(mx, x[qt][1][1], x[qt][1][2]);
                lmax[qt] = max3(mx, x[qt][1][3], x[qt][1][3]);
                over = over || lmax[qt] > thr[qt];
            }
            if (__builtin_amdgcn_ballot_w64(over) != 0) {
                // Some column's scores ran past its reference (or it saw its first key).
#pragma unroll
                for (int qt = 0; qt < kTiles; ++qt) {
                    const float cm = column_max4(lmax[qt]);
                    const bool live = thr[qt] != -INFINITY;
                    float delta = live ? fmaxf(cm, 0.0f) : cm;
                    if (cm == -INFINITY) delta = 0.0f;
                    const float alpha = live ? fast_exp2(-delta) : 1.0f;
                    ref[qt] += delta;
                    if (cm != -INFINITY) thr[qt] = kRefSlack;
                    l[qt] *= alpha;
#pragma unroll
                    for (int dt = 0; dt < kOut; ++dt) o[qt][dt] *= alpha;
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int r = 0; r < 4; ++r) x[qt][t][r] -= delta;
                    if constexpr (!SOFTCAP) {
                        const float nr = -ref[qt];
                        negref[qt] = floatx4{nr, nr, nr, nr};
                    }
                }
            }
            // From here to the block's last MFMA this wavefront goes first when the SIMD picks
            // an instruction: the exponentials and P.V of the wavefront that is ahead then do
            // not wait behind the score MFMAs of the one that shares its SIMD, which keeps the
            // two half a block apart (one in the matrix pipe, one in vector work) instead of
            // drifting into step (measured on the 2048-row chunk: +4.5 %; the other placements
            // of the raised stretch tried, scores only or masks and maxima only, gave +3 %).
            __builtin_amdgcn_s_setprio(1);
            half8 pb[kTiles];
#pragma unroll
            for (int qt = 0; qt < kTiles; ++qt) {
                float pe[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) pe[e] = fast_exp2(x[qt][e >> 2][e & 3]);
#pragma unroll
                for (int e = 0; e < 8; ++e) pb[qt][e] = static_cast<_Float16>(pe[e]);
            }
            if constexpr (kByRow) {
                if (__builtin_expect(by_row, false)) {
                    // Once per row of the wavefront's tile, with the columns of the keys that row
                    // does not see cleared; a lane keeps the sum of its own column's row. The
                    // accumulators are written in place, and the value operand is cleared
                    // afterwards, so that the products below, which every block runs, add zeros:
                    // one definition of the accumulators reaches the loop's end, not two that the
                    // compiler would have to copy into one another every block.
#pragma unroll
                    for (int qt = 0; qt < kTiles; ++qt) {
                        __builtin_amdgcn_sched_barrier(0);  // one tile after the other: registers
                        // (gp is a power of two; the shift is made here and not taken from the
                        // prologue's division, whose result would otherwise be held through
                        // every block for this path's sake.)
                        uint32_t jl_here = jl;
                        asm volatile("" : "+v"(jl_here));  // (nor moved out of the loop by the compiler)
                        const uint32_t my_row = row_begin + ((uint32_t(qt) * 16 + jl_here) >> gp_shift);
#pragma unroll 1
                        for (uint32_t r = row_begin; r < wave_row_end; ++r) {
                            const uint32_t pos = min(item.pos0 + r, item.kv_len - 1);
                            const uint32_t lo = RING ? lowest_visible(item.pos0 + r, window, kv_lo) : 0u;
                            const uint32_t end = min(pos + 1 - min(pos + 1, key_base), 8u);
                            const uint32_t first = RING ? min(lo - min(lo, key_base), 8u) : 0u;
                            const bool mine = my_row == r;
#pragma unroll
                            for (int dt = 0; dt < kOut; ++dt) {
                                // (The mask is made per product from the two counts: four registers
                                // fewer to hold across the products, in a path no speed is asked of.)
                                u32x4 keep = first_halves(end);
                                if constexpr (RING) keep &= ~first_halves(first);
                                asm volatile("" : "+v"(keep));
                                // (The one-tile form, which holds all 256 registers, reads the
                                // values from the stage again: the stage keeps them until the next
                                // block's barrier, and the operand registers are then free for
                                // this loop. The two-tile form has the registers, and with the
                                // second read in it a windowed chunk ran 5 % slower; head_dim 96
                                // reads again in both forms, see the detection above.)
                                half8 v;
                                if constexpr (kTiles == 1 || D == 96)
                                    v = *reinterpret_cast<const half8 *>(vl + dt * 64 * 8);
                                else
                                    v = va[dt];
                                const floatx4 sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                    keep_halves(v, keep), pb[qt], o[qt][dt], 0, 0, 0);
                                if (mine) o[qt][dt] = sum;
                                __builtin_amdgcn_sched_barrier(0);
                            }
                        }
                    }
#pragma unroll
                    for (int dt = 0; dt < kOut; ++dt) va[dt] = half8{0, 0, 0, 0, 0, 0, 0, 0};
                }
            }
#pragma unroll
            for (int qt = 0; qt < kTiles; ++qt) {
                l[qt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, pb[qt], l[qt], 0, 0, 0);
#pragma unroll
                for (int dt = 0; dt < kOut; ++dt)
                    o[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va[dt], pb[qt], o[qt][dt], 0, 0, 0);
            }
        }
        if (kb == kb_begin) { ITAK_MARK(4) }
    }
    ITAK_MARK(5)
    wait_vmcnt<0>();  // the surplus loads of the last iterations (or of the prologue alone)

    // One split: the normalised output. Several: the partial (m, l, acc[128]) of this split
    // in the log2 domain, merged by the combine launch; a column that saw nothing writes
    // m = -inf and zeros.
    const bool final_out = item.splits == 1;
    float *const ws_acc = p.ws;
    float *const ws_ml = p.ws + uint64_t(total_partials) * kD;
    // (The column's row and head are worked out again here, from a lane number the compiler
    // cannot tie to the prologue's: kept from there they would hold registers across the loop.)
    uint32_t jl_again = jl;
    asm volatile("" : "+v"(jl_again));
#pragma unroll
    for (int qt = 0; qt < kTiles; ++qt) {
        const float lt = l[qt][0];
        const uint32_t j = qt * 16 + jl_again;
        const uint32_t row = row_begin + j / gp, hq = j % gp, head = kv_head * group + hq;
        if (row >= item.rows || hq >= group) continue;
        if (final_out) {
            const float inv = 1.0f / lt;
            float *dst = p.out + (uint64_t(item.q_row0 + row) * p.q_heads + head) * kD + g * 4;
#pragma unroll
            for (int dt = 0; dt < kOut; ++dt)
                *reinterpret_cast<floatx4 *>(dst + dt * 16) = o[qt][dt] * inv;
        } else {
            const uint64_t ps = item.ws0 + (uint64_t(row) * p.q_heads + head) * item.splits + split;
            float *dst = ws_acc + ps * kD + g * 4;
#pragma unroll
            for (int dt = 0; dt < kOut; ++dt) *reinterpret_cast<floatx4 *>(dst + dt * 16) = o[qt][dt];
            if (g == 0)
                *reinterpret_cast<float2 *>(ws_ml + ps * 2) =
                    make_float2(thr[qt] == -INFINITY ? -INFINITY : ref[qt], lt);
        }
    }
    ITAK_MARK(6)
    ITAK_MARK_END
}

template <int N, bool SOFTCAP, int TILES, bool RING, int STAGES, int D, bool QLO = false>
hipError_t launch_prefill_ring(const AttnParams &p, const AttnBatch &b,
                                      uint32_t total_partials, hipStream_t stream) {
    constexpr size_t lds = size_t(STAGES) * stage_bytes(D);
    static const hipError_t granted = hipFuncSetAttribute(
        reinterpret_cast<const void *>(&attn_prefill_f16_kernel<N, SOFTCAP, TILES, RING, STAGES, D, QLO>),
        hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
    if (granted != hipSuccess) return granted;
    attn_prefill_f16_kernel<N, SOFTCAP, TILES, RING, STAGES, D, QLO>
        <<<b.total_blocks, kWaves * 64, lds, stream>>>(p, AttnBatchT<N>(b), total_partials);
    return hipGetLastError();
}

template <int N, bool SOFTCAP, int TILES, bool RING, int D, bool QLO = false>
hipError_t launch_prefill(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                 hipStream_t stream) {
    if constexpr (D <= 128) {
        if (b.deep_ring)
            return launch_prefill_ring<N, SOFTCAP, TILES, RING, kDeepStages, D, QLO>(p, b, total_partials, stream);
    } else if (b.deep_ring) {
        return hipErrorInvalidValue;
    }
    return launch_prefill_ring<N, SOFTCAP, TILES, RING, kStages, D, QLO>(p, b, total_partials, stream);
}

// Softcap, ring and tile count chosen for one head_dim. BY_CLASS: an instantiation per batch
// size class (the batch table is a kernel argument, and a large argument block costs a launch
// about a microsecond), which head_dim 128 has; the other head dims have two, one item and any
// number.
template <int D, bool BY_CLASS>
hipError_t launch_prefill_head_dim(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                   bool one, hipStream_t stream) {
    hipError_t e = hipSuccess;
#define ITAK_LAUNCH_N(SC, TILES, RING)                                                          \
    do {                                                                                        \
        if constexpr (BY_CLASS)                                                                 \
            ITAK_DISPATCH_BATCH(b.n, (e = launch_prefill<N, SC, TILES, RING, D>(p, b, total_partials, stream))); \
        else if (b.n <= 1)                                                                      \
            e = launch_prefill<1, SC, TILES, RING, D>(p, b, total_partials, stream);            \
        else                                                                                    \
            e = launch_prefill<kMaxBatchItems, SC, TILES, RING, D>(p, b, total_partials, stream); \
    } while (0)
#define ITAK_LAUNCH_TILES(SC, RING)      \
    do {                                 \
        if (one)                         \
            ITAK_LAUNCH_N(SC, 1, RING);  \
        else                             \
            ITAK_LAUNCH_N(SC, 2, RING);  \
    } while (0)
#define ITAK_LAUNCH_RING(SC)              \
    do {                                  \
        if (p.ring_blocks)                \
            ITAK_LAUNCH_TILES(SC, true);  \
        else                              \
            ITAK_LAUNCH_TILES(SC, false); \
    } while (0)
    if (p.softcap > 0.0f)
        ITAK_LAUNCH_RING(true);
    else
        ITAK_LAUNCH_RING(false);
#undef ITAK_LAUNCH_RING
#undef ITAK_LAUNCH_TILES
#undef ITAK_LAUNCH_N
    return e;
}

}  // namespace

}  // namespace itak
