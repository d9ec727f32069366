// GQA flash-decode for gfx950, f16 KV, head_dim 128: split over the context, K and V
// consumed straight from their planes as MFMA operands.
//
// One workgroup owns (item, kv head, split = a run of 32-key blocks). Each wavefront walks
// its own blocks with a private online softmax and never synchronises inside the loop;
// the wavefronts merge once through LDS at the end. Per 32-key block and per tile of 16
// query vectors (a query vector = one query row of one Q head of the group):
//
//   S^T = K . Q^T   v_mfma_f32_16x16x32_f16, A = 16 key rows x 32 channels from the key
//                   plane (16 bytes per lane), B = Q^T converted to f16 once per kernel.
//   softmax         the lane that holds query vector j holds 8 consecutive keys of it, so
//                   max/sum need two cross-lane steps; m, l and the rescale factor live in
//                   the lane's own column.
//   O^T += V^T . P^T  A = 16 channels x 32 keys from the blocked value plane (16 contiguous
//                   bytes per lane, 1 KiB contiguous per wavefront load), B = P in the
//                   registers the scores were produced in.
//
// All query heads of the KV group (and all rows of a speculative block) are columns of the
// same MFMA, so K and V are read from HBM once per group. Scores, softmax state and
// accumulators are f32; P and Q enter the MFMA as f16.
//
// Semantics: gqa_attention in crates/attention/src/attention.rs:104-215 (key kp visible to a
// query at position p iff kp <= p and, on a windowed layer, kp > p - window), with the
// optional softcap
// cap*tanh(s/cap) of crates/torch-math/src/logits.rs:26-37 applied to the scaled scores.
#include "attn_splitk_f16_kernel.h"

#include <math.h>

#include <algorithm>

// Timeline marks (timeline.h). Split-K kernel: 0 first instruction, 1 addresses known, 2 loads
// issued, 3 bookkeeping done, 4 Q staged, 5 past the barrier, 6 blocks done, 7 O^T in LDS, 8 past
// the barrier, 9 partials issued, 11 all done. Merge kernel (records in the buffer's second
// half): 0 first instruction, 1 addresses known, 2 loads issued, 7 sums done, 8 past the
// barrier, 9 output issued, 11 all done.
ITAK_TIMELINE_READER(itak_timeline_read_splitk)

namespace itak {

bool attn_splitk_f16_supports(const PoolGeom &g, uint32_t group, uint32_t max_rows) {
    return g.v_block == kVBlock && g.head_dim == kD && group >= 1 && max_rows >= 1 &&
           max_rows <= uint32_t(kMaxNewRows) && max_rows * group <= 64;
}

// ---- variants and planning ---------------------------------------------------------------
// The kernel is built for 16, 32 and 64 query vectors per KV head (NQ = 1, 2, 4 tiles) and,
// for 16 vectors, with four or eight wavefronts per workgroup: eight-wave workgroups halve
// the partials and win on large batches, four-wave ones are faster at a few hundred blocks
// (context 4096, batch 1); two-wave workgroups lose everywhere, because the partials they
// double are paid for at the kernel boundary and in the merge launch.
struct Variant {
    int nq, waves, index;
};
static Variant pick_variant(const PoolGeom &g, const AttnBatch &b, uint32_t group) {
    uint32_t nvec = 0, rows = 0;
    uint64_t blocks = 0;
    for (uint32_t i = 0; i < b.n; ++i) {
        nvec = std::max(nvec, b.item[i].rows * group);
        rows = std::max(rows, b.item[i].rows);
        blocks += uint64_t(g.kv_heads) * item_block_count(b.item[i]);
    }
    if (nvec > 32) return {4, 4, 3};
    if (nvec > 16) return {2, 4, 2};
    // (Eight wavefronts for one-row steps only: that variant leaves out the exact treatment of
    // non-finite values that a step of several rows may need.)
    return blocks >= 4096 && rows == 1 ? Variant{1, 8, 1} : Variant{1, 4, 0};
}
// The variant a planned batch takes: 0 = 16 vectors on four wavefronts, 1 = on eight, 2 = 32
// vectors, 3 = 64 vectors.
int attn_splitk_f16_variant(const PoolGeom &g, const AttnBatch &b, uint32_t group) {
    return pick_variant(g, b, group).index;
}
template <int NQ, int W, bool PREP = false>
static hipError_t grant_lds(size_t lds) {
    static size_t granted = 64 * 1024;
    if (lds <= granted) return hipSuccess;
    // The attribute is per kernel function: set it on each batch-size instantiation.
    const void *plain[] = {
        reinterpret_cast<const void *>(&attn_splitk_f16_kernel<NQ, W, 1, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_kernel<NQ, W, 8, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_kernel<NQ, W, 64, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_kernel<NQ, W, 1, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_kernel<NQ, W, 8, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_kernel<NQ, W, 64, true>)};
    const void *prepping[] = {
        reinterpret_cast<const void *>(&attn_splitk_f16_prep_kernel<NQ, W, 1, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_prep_kernel<NQ, W, 8, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_prep_kernel<NQ, W, 64, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_prep_kernel<NQ, W, 1, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_prep_kernel<NQ, W, 8, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_prep_kernel<NQ, W, 64, true>)};
    const void *const *kernels = PREP ? prepping : plain;
    hipError_t e = hipSuccess;
    for (int k = 0; k < 6; ++k)
        if (e == hipSuccess)
            e = hipFuncSetAttribute(kernels[k], hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
    if (e == hipSuccess) granted = lds;
    return e;
}
// Workgroups of a variant the device holds at once (registers and LDS decide), asked of the
// runtime once per variant: the smallest figure over every instantiation a launch of the
// variant may be (batch sizes, ring and preparing forms differ in registers). A launch of at
// most this many workgroups runs in one wave of dispatch, so its duration is that of its
// largest workgroup, and every one of its workgroups is running or done when another waits
// for it (the in-launch exchange relies on that).
template <int NQ, int W>
static uint32_t resident_groups() {
    static uint32_t cached = 0;
    if (cached) return cached;
    const size_t lds = variant_lds(NQ, W);
    int cus = 0, dev = 0;
    if (grant_lds<NQ, W>(lds) != hipSuccess || grant_lds<NQ, W, true>(lds) != hipSuccess ||
        hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) {
        (void)hipGetLastError();
        return 256;
    }
    const void *kernels[] = {
        reinterpret_cast<const void *>(&attn_splitk_f16_kernel<NQ, W, 1, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_kernel<NQ, W, 8, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_kernel<NQ, W, 64, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_kernel<NQ, W, 1, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_kernel<NQ, W, 8, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_kernel<NQ, W, 64, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_prep_kernel<NQ, W, 1, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_prep_kernel<NQ, W, 8, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_prep_kernel<NQ, W, 64, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_prep_kernel<NQ, W, 1, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_prep_kernel<NQ, W, 8, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_prep_kernel<NQ, W, 64, true>)};
    int least = 1 << 30;
    for (const void *k : kernels) {
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, k, W * 64, lds) != hipSuccess || per_cu < 1) {
            (void)hipGetLastError();
            return 256;
        }
        least = std::min(least, per_cu);
    }
    cached = uint32_t(least) * uint32_t(cus);
    return cached;
}
static uint32_t variant_capacity(const Variant &v) {
    switch (v.index) {
        case 0: return resident_groups<1, 4>();
        case 1: return resident_groups<1, 8>();
        case 2: return resident_groups<2, 4>();
        default: return resident_groups<4, 4>();
    }
}

// Fills splits / keys_per_split / block0 / ws0 for a batch (the caller has set slot, rows,
// pos0, q_row0, kv_len) and returns the number of partials the launch will write.
// Every (item, KV head) is cut into equal runs of at most T blocks, T the smallest run for
// which the whole batch fits the device in one wave of dispatch; a run is never shorter
// than one block per wavefront.
uint32_t attn_splitk_f16_plan(const PoolGeom &g, AttnBatch &b, uint32_t q_heads) {
    const Variant v = pick_variant(g, b, q_heads / g.kv_heads);
    const uint64_t capacity = variant_capacity(v);
    uint64_t blocks = 0;
    for (uint32_t i = 0; i < b.n; ++i) blocks += uint64_t(g.kv_heads) * item_block_count(b.item[i]);
    uint64_t T = std::max<uint64_t>((blocks + capacity - 1) / capacity, uint64_t(v.waves));
    for (;; ++T) {
        uint64_t groups = 0;
        for (uint32_t i = 0; i < b.n; ++i) {
            const uint64_t nb = item_block_count(b.item[i]);
            groups += uint64_t(g.kv_heads) * std::max<uint64_t>((nb + T - 1) / T, 1);
        }
        if (groups <= capacity || T >= blocks) break;
    }
    uint32_t block0 = 0, ws0 = 0;
    for (uint32_t i = 0; i < b.n; ++i) {
        AttnItem &it = b.item[i];
        const uint32_t nblocks = item_block_count(it);
        it.splits = std::max<uint32_t>(uint32_t((nblocks + T - 1) / T), 1);
        const uint32_t bps = std::max<uint32_t>((nblocks + it.splits - 1) / it.splits, 1);
        it.splits = std::max<uint32_t>((nblocks + bps - 1) / bps, 1);
        it.keys_per_split = bps * kBlockKeys;
        it.splits_magic =
            it.splits > 1 ? uint32_t(((uint64_t(1) << 32) + it.splits - 1) / it.splits) : 0;
        it.block0 = block0;
        it.ws0 = ws0;
        block0 += g.kv_heads * it.splits;
        if (it.splits > 1) ws0 += it.rows * q_heads * it.splits;
    }
    b.total_blocks = block0;
    b.rows_per_block = 0;
    return ws0;
}

// Decides whether a planned batch can merge its splits inside the split-K launch, and if so
// re-bases every item's ws0 on the exchange buffer (in records of kExchangeWords words, after
// the header). Returns the 64-bit words the buffer must hold, 0 when the batch keeps its merge
// launch: nothing is split, or some workgroup would have more words to gather than its
// threads and its merge area take.
uint64_t attn_splitk_f16_plan_exchange(const PoolGeom &g, AttnBatch &b, uint32_t q_heads) {
    const uint32_t group = q_heads / g.kv_heads;
    const Variant v = pick_variant(g, b, group);
    const uint64_t threads = uint64_t(v.waves) * 64;
    bool any = false;
    for (uint32_t i = 0; i < b.n; ++i) {
        const AttnItem &it = b.item[i];
        if (it.splits <= 1) continue;
        any = true;
        const uint64_t slices = uint64_t(it.rows) * group * 4;
        const uint64_t max_local = (slices + it.splits - 1) / it.splits;
        if (max_local * it.splits * kExchangeWords > threads * kExchangePerThread) return 0;
        if (slices + it.splits >= 65536) return 0;  // the kernel divides by multiplication
    }
    if (!any) return 0;
    // A workgroup of the exchange polls for its group's others: all of the launch must be on the
    // device together. The launch may be the single-row decode kernel (its own registers and
    // LDS), so that kernel's figure bounds 16-vector launches too.
    uint64_t held = variant_capacity(v);
    if (v.index == 0) held = std::min<uint64_t>(held, attn_decode_f16_resident_groups());
    if (b.total_blocks > held) return 0;
    uint64_t records = 0;
    for (uint32_t i = 0; i < b.n; ++i) {
        AttnItem &it = b.item[i];
        if (it.splits <= 1) continue;
        const uint64_t slices = uint64_t(it.rows) * group * 4;
        const uint64_t max_local = (slices + it.splits - 1) / it.splits;
        if (records > 0xffffffffull) return 0;
        it.ws0 = uint32_t(records);
        records += uint64_t(g.kv_heads) * it.splits * max_local * it.splits;
    }
    return kExchangeHeaderWords + records * kExchangeWords;
}

hipError_t launch_attn_splitk_f16(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                  uint32_t max_rows, hipStream_t stream,
                                  const FoldedParams *folded, bool q_two_halves) {
    (void)max_rows;
    if (b.total_blocks == 0) return hipSuccess;
    const Variant v = pick_variant(p.g, b, p.group);
    const bool prep = folded && folded->prep_on;
    if (!prep && v.index == 0 && attn_decode_f16_takes(p, b))
        return launch_attn_decode_f16(p, b, total_partials, stream, q_two_halves);
    if (q_two_halves) return launch_attn_splitk_f16_qlo(p, b, total_partials, stream, folded);
#define ITAK_LAUNCH(NQ, W)                                                                \
    do {                                                                                  \
        const size_t lds = variant_lds(NQ, W);                                            \
        hipError_t e = grant_lds<NQ, W>(lds);                                             \
        if (e != hipSuccess) return e;                                                    \
        if (p.ring_blocks)                                                                \
            attn_splitk_f16_kernel<NQ, W, N, true><<<b.total_blocks, W * 64, lds, stream>>>(  \
                p, AttnBatchT<N>(b), total_partials);                                     \
        else                                                                              \
            attn_splitk_f16_kernel<NQ, W, N, false><<<b.total_blocks, W * 64, lds, stream>>>( \
                p, AttnBatchT<N>(b), total_partials);                                     \
    } while (0)
#define ITAK_LAUNCH_PREP(NQ, W)                                                           \
    do {                                                                                  \
        const size_t lds = variant_lds(NQ, W);                                            \
        hipError_t e = grant_lds<NQ, W, true>(lds);                                       \
        if (e != hipSuccess) return e;                                                    \
        if (p.ring_blocks)                                                                \
            attn_splitk_f16_prep_kernel<NQ, W, N, true>                                   \
                <<<b.total_blocks, W * 64, lds, stream>>>(p, AttnBatchT<N>(b), total_partials, \
                                                          *folded);                       \
        else                                                                              \
            attn_splitk_f16_prep_kernel<NQ, W, N, false>                                  \
                <<<b.total_blocks, W * 64, lds, stream>>>(p, AttnBatchT<N>(b), total_partials, \
                                                          *folded);                       \
    } while (0)
#define ITAK_LAUNCH_NQ()                                  \
    do {                                                  \
        switch (v.index + (prep ? 4 : 0)) {               \
            case 0: ITAK_LAUNCH(1, 4); break;             \
            case 1: ITAK_LAUNCH(1, 8); break;             \
            case 2: ITAK_LAUNCH(2, 4); break;             \
            case 3: ITAK_LAUNCH(4, 4); break;             \
            case 4: ITAK_LAUNCH_PREP(1, 4); break;        \
            case 5: ITAK_LAUNCH_PREP(1, 8); break;        \
            case 6: ITAK_LAUNCH_PREP(2, 4); break;        \
            default: ITAK_LAUNCH_PREP(4, 4); break;       \
        }                                                 \
    } while (0)
    ITAK_DISPATCH_BATCH(b.n, ITAK_LAUNCH_NQ());
#undef ITAK_LAUNCH_NQ
#undef ITAK_LAUNCH_PREP
#undef ITAK_LAUNCH
    return hipGetLastError();
}

// ------------------------------------------------------------------------------ combine
// Merges the split partials of one (query row, Q head): weights w_s = exp(m_s - M), output
// sum_s w_s * acc_s / sum_s w_s * l_s. One 256-thread workgroup per (row, head): thread =
// (4 channels, one of 8 split lanes). Every thread issues all its accumulator loads before
// the weights are known, so the merge costs one memory round trip, not one per split.
// grid = all (row, head) pairs of the batch; items whose splits == 1 exit at once.
constexpr int kCombineThreads = 256;
constexpr int kCombineMaxLoads = 8;  // accumulator loads in flight per thread and pass

template <int N>
__global__ __launch_bounds__(kCombineThreads) void attn_combine_kernel(AttnParams p,
                                                                       AttnBatchT<N> b,
                                                                       uint32_t total_partials,
                                                                       int base2,
                                                                       const float *gate) {
    __shared__ float w_s[1024];
    __shared__ float red[8];
    __shared__ float4 part[kCombineThreads];
    const uint32_t tid = threadIdx.x;
    const uint32_t D = p.g.head_dim;
    const uint32_t pair = blockIdx.x;
    const uint32_t grow = pair / p.q_heads, head = pair % p.q_heads;
    const AttnItem item = b.item[b.find_by_row(grow)];
    if (item.splits == 1) return;
    const uint32_t row = grow - (item.q_row0 - b.base_row);
    const uint64_t ps0 = item.ws0 + (uint64_t(row) * p.q_heads + head) * item.splits;
    const float *ws_acc = p.ws + ps0 * D;
    const float *ws_ml = p.ws + uint64_t(total_partials) * D + ps0 * 2;
    const uint32_t S = item.splits;

    // Thread layout for the accumulators: chunk c of 4 channels, split lane sl.
    const uint32_t chunks = (D + 3) / 4;                       // 32 for head_dim 128
    const uint32_t lanes = kCombineThreads / chunks ? kCombineThreads / chunks : 1;
    const uint32_t c = tid % chunks, sl = tid / chunks;
    const bool vec_ok = (D % 4 == 0) && sl < lanes;

    // First pass of accumulator loads goes out before anything waits on m/l.
    float4 x[kCombineMaxLoads];
    if (vec_ok) {
#pragma unroll
        for (int u = 0; u < kCombineMaxLoads; ++u) {
            const uint32_t s = sl + u * lanes;
            x[u] = s < S ? *reinterpret_cast<const float4 *>(ws_acc + uint64_t(s) * D + c * 4)
                         : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    float mx = -INFINITY;
    for (uint32_t s = tid; s < S; s += kCombineThreads) mx = fmaxf(mx, ws_ml[s * 2]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if ((tid & 63) == 0) red[tid >> 6] = mx;
    __syncthreads();
    const float M = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float lsum = 0.0f;
    for (uint32_t s = tid; s < S; s += kCombineThreads) {
        const float ms = ws_ml[s * 2];
        const float w = (ms == -INFINITY) ? 0.0f : (base2 ? exp2f(ms - M) : expf(ms - M));
        w_s[s] = w;
        lsum += w * ws_ml[s * 2 + 1];
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) lsum += __shfl_xor(lsum, o);
    if ((tid & 63) == 0) red[4 + (tid >> 6)] = lsum;
    __syncthreads();
    const float inv = 1.0f / (red[4] + red[5] + red[6] + red[7]);
    float *dst = p.out + (uint64_t(item.q_row0 + row) * p.q_heads + head) * D;

    if (D % 4 != 0) {  // scalar path for odd head dims
        for (uint32_t d = tid; d < D; d += kCombineThreads) {
            float acc = 0.0f;
            for (uint32_t s = 0; s < S; ++s) acc = fmaf(ws_acc[uint64_t(s) * D + d], w_s[s], acc);
            dst[d] = acc * inv * (gate ? sigmoid_fast(gate[(dst - p.out) + d]) : 1.0f);
        }
        return;
    }
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (vec_ok) {
#pragma unroll
        for (int u = 0; u < kCombineMaxLoads; ++u) {
            const uint32_t s = sl + u * lanes;
            const float w = s < S ? w_s[s] : 0.0f;
            acc.x = fmaf(x[u].x, w, acc.x);
            acc.y = fmaf(x[u].y, w, acc.y);
            acc.z = fmaf(x[u].z, w, acc.z);
            acc.w = fmaf(x[u].w, w, acc.w);
        }
        for (uint32_t s0 = kCombineMaxLoads * lanes; s0 < S; s0 += kCombineMaxLoads * lanes) {
#pragma unroll
            for (int u = 0; u < kCombineMaxLoads; ++u) {
                const uint32_t s = s0 + sl + u * lanes;
                x[u] = s < S ? *reinterpret_cast<const float4 *>(ws_acc + uint64_t(s) * D + c * 4)
                             : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int u = 0; u < kCombineMaxLoads; ++u) {
                const uint32_t s = s0 + sl + u * lanes;
                const float w = s < S ? w_s[s] : 0.0f;
                acc.x = fmaf(x[u].x, w, acc.x);
                acc.y = fmaf(x[u].y, w, acc.y);
                acc.z = fmaf(x[u].z, w, acc.z);
                acc.w = fmaf(x[u].w, w, acc.w);
            }
        }
    }
    part[tid] = acc;
    __syncthreads();
    if (tid < chunks) {
        float4 sum = part[tid];
        for (uint32_t l = 1; l < lanes; ++l) {
            const float4 y = part[tid + l * chunks];
            sum.x += y.x;
            sum.y += y.y;
            sum.z += y.z;
            sum.w += y.w;
        }
        float4 o = make_float4(sum.x * inv, sum.y * inv, sum.z * inv, sum.w * inv);
        if (gate) {
            const float4 gt = *reinterpret_cast<const float4 *>(gate + (dst - p.out) + tid * 4);
            o = make_float4(o.x * sigmoid_fast(gt.x), o.y * sigmoid_fast(gt.y),
                            o.z * sigmoid_fast(gt.z), o.w * sigmoid_fast(gt.w));
        }
        *reinterpret_cast<float4 *>(dst + tid * 4) = o;
    }
}

// The same merge for head_dim 128, shaped for latency (it runs for under two microseconds per
// decode layer): grid = (Q head, query row); wavefront w owns channels 32w .. 32w+31, lane =
// (4 channels c of its 8 chunks, split lane sl of 8). A lane issues every load of its first 8
// splits, accumulators and (m, l) pairs alike, before it waits for anything, folds them with its
// own running maximum, and the eight split lanes meet through lane permutes: one memory round
// trip, no LDS and no barrier, and no stretch that a single wavefront runs while three wait (the
// form with a barrier and 32 threads finishing cost 0.4 us more per launch).
// SL = split lanes of a chunk: lanes that differ in the bits above log2(64 / SL).
template <int SL>
__device__ __forceinline__ float split_lanes_max(float v) {
    if constexpr (SL >= 16) v = fmaxf(v, dpp_lane<0x124>(v));  // row_ror:4
    if constexpr (SL >= 8) v = fmaxf(v, dpp_lane<0x128>(v));   // row_ror:8
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const auto c = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(c[0]), __uint_as_float(c[1]));
}
template <int SL>
__device__ __forceinline__ float split_lanes_sum(float v) {
    if constexpr (SL >= 16) v += dpp_lane<0x124>(v);
    if constexpr (SL >= 8) v += dpp_lane<0x128>(v);
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const auto c = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(c[0]) + __uint_as_float(c[1]);
}
// D = head_dim (64, 96, 128 or 256): a wavefront owns D/4 channels, i.e. D/16 chunks, in the next
// power of two of lanes (at 96 two of eight sit idle), and the other lane bits are split lanes.
template <int N, bool BASE2, bool GATE, int D = 128>
__device__ __forceinline__ void attn_combine128_body(const AttnParams &p, const AttnBatchT<N> &b,
                                                     uint32_t total_partials,
                                                     [[maybe_unused]] const float *gate) {
    constexpr uint32_t kChunks = D / 16;                                   // per wavefront
    constexpr uint32_t kChunkLanes = kChunks <= 4 ? 4 : kChunks <= 8 ? 8 : 16;
    constexpr int SL = 64 / kChunkLanes;                                   // split lanes
    const uint32_t tid = threadIdx.x;
    ITAK_MARK_BEGIN
    ITAK_MARK(0)
    const uint32_t head = blockIdx.x, grow = blockIdx.y;
    if (N == 1)  // fetch every kernel argument in one batch of scalar loads
        asm volatile("" ::"s"(p.out), "s"(p.ws), "s"(p.q_heads), "s"(total_partials),
                     "s"(b.base_row), "s"(b.item[0].q_row0), "s"(b.item[0].splits),
                     "s"(b.item[0].ws0));
    if (N == 1 && GATE) asm volatile("" ::"s"(gate));
    const AttnItem item = b.item[b.find_by_row(grow)];
    const uint32_t S = item.splits;
    if (S == 1) return;
    const uint32_t row = grow - (item.q_row0 - b.base_row);
    const uint64_t ps0 = item.ws0 + (uint64_t(row) * p.q_heads + head) * S;
    const uint32_t wave = tid >> 6, lane = tid & 63;
    const uint32_t cl = lane % kChunkLanes, sl = lane / kChunkLanes;  // chunk of the wavefront, split lane
    const bool holds = cl < kChunks;                                   // (false only at head_dim 96)
    const uint32_t c = wave * kChunks + min(cl, kChunks - 1);          // chunk of 4 channels
    const float *ws_acc = p.ws + ps0 * D + c * 4;
    const float2 *ws_ml = reinterpret_cast<const float2 *>(p.ws + uint64_t(total_partials) * D) + ps0;
    const uint64_t at = (uint64_t(item.q_row0 + row) * p.q_heads + head) * D + c * 4;
    // The gate of the lanes that write the output, fetched with the partials.
    [[maybe_unused]] float4 gt = make_float4(0.f, 0.f, 0.f, 0.f);
    if (GATE && sl == 0 && holds) gt = *reinterpret_cast<const float4 *>(gate + at);
    ITAK_MARK(1)

    float m_run = -INFINITY, l_run = 0.0f;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (uint32_t s0 = 0; s0 < S; s0 += 8 * SL) {
        float4 x[8];
        float2 ml[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {  // clamped, so the loads need no branch
            const uint32_t s = min(s0 + sl + u * SL, S - 1);
            x[u] = *reinterpret_cast<const float4 *>(ws_acc + uint64_t(s) * D);
            ml[u] = ws_ml[s];
        }
        // Nothing below may move above this line and no load below it: left to itself the
        // scheduler issues half of the accumulator loads after the first weights are computed.
        __builtin_amdgcn_sched_barrier(0);
        if (s0 == 0) { ITAK_MARK(2) }
        float mx = m_run;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            // A lane past the last split holds a second copy of that split's partial: its
            // weight is zero, and so must the copy be, or a value in it that is not finite
            // (which the rows that see the key are due) would make the product NaN.
            if (s0 + sl + u * SL >= S) {
                ml[u].x = -INFINITY;
                x[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            }
            mx = fmaxf(mx, ml[u].x);
        }
        // Nothing visible in these splits (nor before): every weight below is exp(-inf) = 0
        // against a finite stand-in. No branch around the arithmetic: behind one the compiler
        // fetches the maxima first and the accumulators after it has looked at them, two memory
        // round trips instead of one.
        const float ref = mx == -INFINITY ? 0.0f : mx;
        const float alpha = BASE2 ? fast_exp2(m_run - ref) : __expf(m_run - ref);  // 0 at first
        acc.x *= alpha, acc.y *= alpha, acc.z *= alpha, acc.w *= alpha;
        l_run *= alpha;
        m_run = mx;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float w = BASE2 ? fast_exp2(ml[u].x - ref) : __expf(ml[u].x - ref);  // exp(-inf) = 0
            l_run = fmaf(ml[u].y, w, l_run);
            acc.x = fmaf(x[u].x, w, acc.x);
            acc.y = fmaf(x[u].y, w, acc.y);
            acc.z = fmaf(x[u].z, w, acc.z);
            acc.w = fmaf(x[u].w, w, acc.w);
        }
    }
    ITAK_MARK(7)
    // The eight split lanes of a chunk: a common maximum, then the weighted sums.
    const float M = split_lanes_max<SL>(m_run);
    const float w = m_run == -INFINITY ? 0.0f : (BASE2 ? fast_exp2(m_run - M) : __expf(m_run - M));
    const float L = split_lanes_sum<SL>(l_run * w);
    float4 sum = make_float4(split_lanes_sum<SL>(acc.x * w), split_lanes_sum<SL>(acc.y * w),
                             split_lanes_sum<SL>(acc.z * w), split_lanes_sum<SL>(acc.w * w));
    ITAK_MARK(8)
    if (sl == 0 && holds) {
        const float inv = __builtin_amdgcn_rcpf(L);  // within an ulp: far inside either pool's bar
        float4 o = make_float4(sum.x * inv, sum.y * inv, sum.z * inv, sum.w * inv);
        if (GATE)
            o = make_float4(o.x * sigmoid_fast(gt.x), o.y * sigmoid_fast(gt.y),
                            o.z * sigmoid_fast(gt.z), o.w * sigmoid_fast(gt.w));
        *reinterpret_cast<float4 *>(p.out + at) = o;
    }
    ITAK_MARK(9)
    ITAK_MARK_END_AT(ITAK_TIMELINE_WAVES / 2)
}
template <int N, bool BASE2>
__global__ __launch_bounds__(256) void attn_combine128_kernel(AttnParams p, AttnBatchT<N> b,
                                                              uint32_t total_partials) {
    attn_combine128_body<N, BASE2, false>(p, b, total_partials, nullptr);
}
// The same merge whose writers multiply by sigmoid(gate) (cpu.rs:657-673).
template <int N, bool BASE2>
__global__ __launch_bounds__(256) void attn_combine128_gate_kernel(AttnParams p, AttnBatchT<N> b,
                                                                   uint32_t total_partials,
                                                                   const float *gate) {
    attn_combine128_body<N, BASE2, true>(p, b, total_partials, gate);
}

// The same merge at head dims 64, 96 and 256 (the partials of the block kernel and, at 64, of the
// f32 kernel).
template <int N, bool BASE2, bool GATE, int D>
__global__ __launch_bounds__(256) void attn_combine_lanes_kernel(AttnParams p, AttnBatchT<N> b,
                                                                 uint32_t total_partials,
                                                                 const float *gate) {
    attn_combine128_body<N, BASE2, GATE, D>(p, b, total_partials, gate);
}

// The same merge for items of at most 16 splits, one wavefront per (row, Q head): lane =
// (4 channels c, split lane sl of 2), every load of the wavefront's 16 splits issued at once,
// the two split lanes joined by a half-wave swap. A workgroup is four such wavefronts (four
// heads of one row) that never meet: no LDS, no barrier, and a quarter of the wavefronts of the
// form above, whose launch of a few microseconds is mostly wavefront dispatch once a block of
// several rows has hundreds of (row, head) pairs to merge.
__device__ __forceinline__ float half_max(float v) {
    const auto c = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(c[0]), __uint_as_float(c[1]));
}
__device__ __forceinline__ float half_sum(float v) {
    const auto c = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(c[0]) + __uint_as_float(c[1]);
}
// A load with the streaming hint: split partials are read once, by the merge, and what they
// would otherwise displace from L2 on their way through is the next layer's use (measured with
// the hint on the wave kernel's loads: the verify block 23.85 -> 23.23 us per layer, the 64-row
// chunk 20.16 -> 19.56; the decode merge, a twentieth of the bytes, does not change).
__device__ __forceinline__ float4 load_once4(const float *p) {
    typedef float f4v __attribute__((ext_vector_type(4)));
    const f4v v = __builtin_nontemporal_load(reinterpret_cast<const f4v *>(p));
    return make_float4(v[0], v[1], v[2], v[3]);
}
template <int N, bool BASE2, bool GATE>
__global__ __launch_bounds__(256) void attn_combine128_wave_kernel(AttnParams p, AttnBatchT<N> b,
                                                                   uint32_t total_partials,
                                                                   const float *gate) {
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const uint32_t head = blockIdx.x * 4 + wave, grow = blockIdx.y;
    if (head >= p.q_heads) return;
    const AttnItem item = b.item[b.find_by_row(grow)];
    const uint32_t S = item.splits;
    if (S == 1) return;
    const uint32_t row = grow - (item.q_row0 - b.base_row);
    const uint64_t ps0 = item.ws0 + (uint64_t(row) * p.q_heads + head) * S;
    const uint32_t c = lane & 31, sl = lane >> 5;
    const float *ws_acc = p.ws + ps0 * 128 + c * 4;
    const float2 *ws_ml = reinterpret_cast<const float2 *>(p.ws + uint64_t(total_partials) * 128) + ps0;
    const uint64_t at = (uint64_t(item.q_row0 + row) * p.q_heads + head) * 128 + c * 4;
    [[maybe_unused]] float4 gt = make_float4(0.f, 0.f, 0.f, 0.f);
    if (GATE && sl == 0) gt = *reinterpret_cast<const float4 *>(gate + at);
    float4 x[8];
    float2 ml[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {  // clamped, so the loads need no branch
        const uint32_t s = min(sl + u * 2, S - 1);
        x[u] = load_once4(ws_acc + uint64_t(s) * 128);
        ml[u] = ws_ml[s];
    }
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        if (sl + u * 2 >= S) {  // a second copy of the last split: weight zero, and cleared
            ml[u].x = -INFINITY;
            x[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        mx = fmaxf(mx, ml[u].x);
    }
    const float M = half_max(mx);
    float l = 0.0f;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const float w = ml[u].x == -INFINITY ? 0.0f : (BASE2 ? fast_exp2(ml[u].x - M) : __expf(ml[u].x - M));
        l = fmaf(ml[u].y, w, l);
        acc.x = fmaf(x[u].x, w, acc.x);
        acc.y = fmaf(x[u].y, w, acc.y);
        acc.z = fmaf(x[u].z, w, acc.z);
        acc.w = fmaf(x[u].w, w, acc.w);
    }
    const float inv = 1.0f / half_sum(l);
    float4 o = make_float4(half_sum(acc.x) * inv, half_sum(acc.y) * inv, half_sum(acc.z) * inv,
                           half_sum(acc.w) * inv);
    if (sl == 0) {
        if (GATE)
            o = make_float4(o.x * sigmoid_fast(gt.x), o.y * sigmoid_fast(gt.y),
                            o.z * sigmoid_fast(gt.z), o.w * sigmoid_fast(gt.w));
        *reinterpret_cast<float4 *>(p.out + at) = o;
    }
}

hipError_t launch_attn_combine(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                               uint32_t total_rows, int base2, hipStream_t stream, const float *gate) {
    bool any = false;
    for (uint32_t i = 0; i < b.n; ++i) any = any || b.item[i].splits > 1;
    if (!any || total_rows == 0) return hipSuccess;
    uint32_t most_splits = 0;
    for (uint32_t i = 0; i < b.n; ++i) most_splits = std::max(most_splits, b.item[i].splits);
    if (p.g.head_dim == 128 && most_splits <= 16 && uint64_t(total_rows) * p.q_heads >= 128) {
        const dim3 grid((p.q_heads + 3) / 4, total_rows);
        if (gate && base2)
            ITAK_DISPATCH_BATCH(b.n, (attn_combine128_wave_kernel<N, true, true><<<grid, 256, 0, stream>>>(
                                         p, AttnBatchT<N>(b), total_partials, gate)));
        else if (gate)
            ITAK_DISPATCH_BATCH(b.n, (attn_combine128_wave_kernel<N, false, true><<<grid, 256, 0, stream>>>(
                                         p, AttnBatchT<N>(b), total_partials, gate)));
        else if (base2)
            ITAK_DISPATCH_BATCH(b.n, (attn_combine128_wave_kernel<N, true, false><<<grid, 256, 0, stream>>>(
                                         p, AttnBatchT<N>(b), total_partials, nullptr)));
        else
            ITAK_DISPATCH_BATCH(b.n, (attn_combine128_wave_kernel<N, false, false><<<grid, 256, 0, stream>>>(
                                         p, AttnBatchT<N>(b), total_partials, nullptr)));
        return hipGetLastError();
    }
    if (p.g.head_dim == 128) {
        const dim3 grid(p.q_heads, total_rows);
        if (gate && base2)
            ITAK_DISPATCH_BATCH(b.n, (attn_combine128_gate_kernel<N, true><<<grid, 256, 0, stream>>>(
                                         p, AttnBatchT<N>(b), total_partials, gate)));
        else if (gate)
            ITAK_DISPATCH_BATCH(b.n, (attn_combine128_gate_kernel<N, false><<<grid, 256, 0, stream>>>(
                                         p, AttnBatchT<N>(b), total_partials, gate)));
        else if (base2)
            ITAK_DISPATCH_BATCH(b.n, (attn_combine128_kernel<N, true><<<grid, 256, 0, stream>>>(
                                         p, AttnBatchT<N>(b), total_partials)));
        else
            ITAK_DISPATCH_BATCH(b.n, (attn_combine128_kernel<N, false><<<grid, 256, 0, stream>>>(
                                         p, AttnBatchT<N>(b), total_partials)));
        return hipGetLastError();
    }
    // (A workgroup per output pays where the merge is a matter of latency; with thousands of
    // outputs, a 512-row chunk, the general kernel below is the faster one by a tenth of the step.)
    if ((p.g.head_dim == 64 || p.g.head_dim == 96 || p.g.head_dim == 256) &&
        uint64_t(total_rows) * p.q_heads <= 4096) {
        const dim3 grid(p.q_heads, total_rows);
#define ITAK_LANES(B2, G, D)                                                                  \
    ITAK_DISPATCH_BATCH(b.n, (attn_combine_lanes_kernel<N, B2, G, D><<<grid, 256, 0, stream>>>( \
                                 p, AttnBatchT<N>(b), total_partials, gate)))
#define ITAK_LANES_D(D)                                \
    do {                                               \
        if (gate && base2) ITAK_LANES(true, true, D);  \
        else if (gate) ITAK_LANES(false, true, D);     \
        else if (base2) ITAK_LANES(true, false, D);    \
        else ITAK_LANES(false, false, D);              \
    } while (0)
        if (p.g.head_dim == 64) ITAK_LANES_D(64);
        else if (p.g.head_dim == 96) ITAK_LANES_D(96);
        else ITAK_LANES_D(256);
#undef ITAK_LANES_D
#undef ITAK_LANES
        return hipGetLastError();
    }
    ITAK_DISPATCH_BATCH(b.n, (attn_combine_kernel<N><<<total_rows * p.q_heads, kCombineThreads, 0,
                                                      stream>>>(p, AttnBatchT<N>(b), total_partials,
                                                                base2, gate)));
    return hipGetLastError();
}

}  // namespace itak
