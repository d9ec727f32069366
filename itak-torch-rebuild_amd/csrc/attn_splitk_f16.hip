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
#include "internal.h"
#include "mfma_common.h"
#include "split_exchange.h"
#include "timeline.h"

#include <math.h>

#include <algorithm>

// Timeline marks (timeline.h). Split-K kernel: 0 first instruction, 1 addresses known, 2 loads
// issued, 3 bookkeeping done, 4 Q staged, 5 past the barrier, 6 blocks done, 7 O^T in LDS, 8 past
// the barrier, 9 partials issued, 11 all done. Merge kernel (records in the buffer's second
// half): 0 first instruction, 1 addresses known, 2 loads issued, 7 sums done, 8 past the
// barrier, 9 output issued, 11 all done.
ITAK_TIMELINE_READER(itak_timeline_read_splitk)

namespace itak {

namespace {

template <int NQ>
struct WaveState {
    float m[NQ];         // running max of this lane's query-vector column (log2 domain)
    float l[NQ];         // this lane's share of the running denominator
    floatx4 o[NQ][8];    // O^T accumulators: channel dt*16 + g*4 + r, query vector column
};

// K/V are read once per launch: streaming (non-temporal) loads keep them from displacing the
// kernel's code, arguments and split partials in L2 (measured: 6 % off a decode layer at
// context 4096, 10 % more bandwidth on 16 slots x 16384).
#define ITAK_KV_LOAD(p) __builtin_nontemporal_load(p)

struct BlockOperands {
    half8 k[2][4];  // [key half t][channel step s]
    half8 v[8];     // [channel tile dt]
};

// Position block kb lives in storage block kb % ring_blocks on a windowed layer.
__device__ __forceinline__ uint32_t storage_block(uint32_t kb, uint32_t ring_blocks) {
    return ring_blocks ? kb % ring_blocks : kb;
}

__device__ __forceinline__ void load_block(BlockOperands &b, const uint16_t *kplane,
                                           const uint16_t *vplane, uint32_t kb, uint32_t g,
                                           uint32_t i) {
    // Key rows of MFMA tile t are interleaved so that the lane group g ends up holding
    // scores of the 8 consecutive keys g*8 .. g*8+7: row i of tile t is key
    // (i/4)*8 + t*4 + i%4 of the block. The blocked key plane stores the 16-byte piece
    // (tile t, channel chunk c, row i) at ((t*16 + c)*16 + i)*8, so the 64 lanes of the load
    // for (t, s) (chunks s*4 .. s*4+3, rows 0..15) read 1 KiB of contiguous memory.
    const uint16_t *kb_base = kplane + uint64_t(kb) * (kBlockKeys * kD) + (g * 16 + i) * 8;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int s = 0; s < 4; ++s)
            b.k[t][s] = ITAK_KV_LOAD(reinterpret_cast<const half8 *>(kb_base + ((t * 16 + s * 4) * 16) * 8));
    const uint16_t *vb = vplane + uint64_t(kb) * (kBlockKeys * kD) + i * kBlockKeys + g * 8;
#pragma unroll
    for (int dt = 0; dt < 8; ++dt)
        b.v[dt] = ITAK_KV_LOAD(reinterpret_cast<const half8 *>(vb + dt * 16 * kBlockKeys));
}

// Fused append. The workgroup that owns the blocks holding the new positions
// [pos0, kv_len) converts the new K/V rows once (all threads, coalesced), keeps them in LDS
// and stores them into the planes; the wavefront that multiplies such a block replaces the
// operand elements of the new keys from LDS. No other workgroup reads these positions, so
// nothing depends on the stores within the launch.
constexpr int kNewStride = kD + 8;  // LDS row stride of the staged new rows (halves)

__device__ __forceinline__ void patch_new_rows(BlockOperands &b, const _Float16 *sm_newk,
                                               const _Float16 *sm_newv, uint32_t kb, uint32_t g,
                                               uint32_t i, uint32_t pos0, uint32_t kv_len) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const uint32_t key = kb * kBlockKeys + (i >> 2) * 8 + t * 4 + (i & 3);
        if (key >= pos0 && key < kv_len) {
            const _Float16 *src = sm_newk + (key - pos0) * kNewStride + g * 8;
#pragma unroll
            for (int s = 0; s < 4; ++s) b.k[t][s] = *reinterpret_cast<const half8 *>(src + s * 32);
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t key = kb * kBlockKeys + g * 8 + e;
        if (key >= pos0 && key < kv_len) {
            const _Float16 *src = sm_newv + (key - pos0) * kNewStride + i;
#pragma unroll
            for (int dt = 0; dt < 8; ++dt) b.v[dt][e] = src[dt * 16];
        }
    }
}

// Reductions over the four lanes that share a query-vector column (lanes l, l^16, l^32,
// l^48) with the gfx950 row and half swaps: they run at VALU speed, not through the LDS
// crossbar. permlane16_swap exchanges the odd rows of its first operand with the even rows
// of its second, permlane32_swap the upper half of the first with the lower half of the
// second; with both operands equal, combining the two results folds l with l^16 (l^32).
__device__ __forceinline__ float column_max(float v) {
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const auto c = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(c[0]), __uint_as_float(c[1]));
}
__device__ __forceinline__ float column_sum(float v) {
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const auto c = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(c[0]) + __uint_as_float(c[1]);
}

// One 32-key block against all NQ tiles of query vectors. FIRST = the wavefront's first
// block: the running state is written, not rescaled (most decode wavefronts see one block).
// Up to 32 vectors the Q^T operand lives in registers (qreg), beyond that it is re-read
// from LDS per block: lane (g, jl) holds channels k*32 + g*8 .. +8 of vector jl.
template <int NQ, bool FIRST, bool RING>
__device__ __forceinline__ void process_block(WaveState<NQ> &st, BlockOperands &b,
                                              const half8 *qreg, const _Float16 *sm_q,
                                              uint32_t kb, uint32_t g, uint32_t jl,
                                              const uint32_t *colpos, const uint32_t *collo,
                                              uint32_t pos0, uint32_t kv_len, uint32_t lo_min,
                                              uint32_t lo_max, float softcap, float inv_cap) {
    const uint32_t key_base = kb * kBlockKeys + g * 8;  // first of this lane's 8 keys
    const bool tail = (kb + 1) * kBlockKeys > kv_len || (RING && kb * kBlockKeys < lo_min);
    auto zero_tail = [&] {
        // Rows past the stored length, and ring rows older than anything the block's queries
        // see, may hold stale data: keep them out of P.V even as 0*x.
        const uint32_t end = min(kv_len - min(kv_len, key_base), 8u);
        const uint32_t first = RING ? min(lo_min - min(lo_min, key_base), 8u) : 0u;
        const u32x4 keep = first_halves(end) & ~first_halves(first);
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) b.v[dt] = keep_halves(b.v[dt], keep);
    };
    if (NQ <= 2 && tail) zero_tail();
    [[maybe_unused]] half8 pbs[NQ > 2 ? NQ : 1];
    [[maybe_unused]] float alphas[NQ > 2 ? NQ : 1];
    const bool need_mask =
        (kb + 1) * kBlockKeys > pos0 + 1 || (RING && kb * kBlockKeys < lo_max);
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt) {
        half8 qb[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            if constexpr (NQ <= 2)
                qb[k] = qreg[qt * 4 + k];
            else
                qb[k] = *reinterpret_cast<const half8 *>(sm_q + (qt * 16 + jl) * kQStride +
                                                         k * 32 + g * 8);
        }
        floatx4 s[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            s[t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int k = 0; k < 4; ++k)
                s[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b.k[t][k], qb[k], s[t], 0, 0, 0);
        }
        float sc[8];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) sc[t * 4 + r] = s[t][r];
        if (softcap > 0.0f) {
#pragma unroll
            for (int e = 0; e < 8; ++e) sc[e] = softcap_log2(sc[e], softcap, inv_cap);
        }
        if (need_mask) {
            const uint32_t pos = colpos[qt];  // this column's query position
            const uint32_t lo = RING ? collo[qt] : 0;  // and the oldest position it sees
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (key_base + e > pos || (RING && key_base + e < lo)) sc[e] = -INFINITY;
        }
        float mx = sc[0];
#pragma unroll
        for (int e = 1; e < 8; ++e) mx = fmaxf(mx, sc[e]);
        mx = column_max(mx);
        // 64 vectors: the column's reference follows the block maximum only when that runs
        // more than kSlack ahead of it (P stays below 2^kSlack, far inside f16 and f32 range;
        // every term of numerator and denominator carries the same factor, so the softmax is
        // the same). Rescaling the 32 accumulators of a tile, which live in accumulation
        // registers there and cost three instructions an element, then leaves the common path.
        constexpr float kSlack = NQ > 2 ? 8.0f : 0.0f;
        const float m_new = FIRST ? mx : (mx > st.m[qt] + kSlack ? mx : st.m[qt]);
        const bool dead = m_new == -INFINITY;  // nothing visible to this column so far
        float p[8];
        float sum = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            p[e] = dead ? 0.0f : fast_exp2(sc[e] - m_new);
            sum += p[e];
        }
        half8 pb;
#pragma unroll
        for (int e = 0; e < 8; ++e) pb[e] = static_cast<_Float16>(p[e]);
        const float alpha = (FIRST || dead) ? 1.0f : fast_exp2(st.m[qt] - m_new);
        st.l[qt] = FIRST ? sum : st.l[qt] * alpha + sum;
        st.m[qt] = m_new;
        if constexpr (NQ > 2) {
            // 64 vectors: P.V of all tiles after the scores of all tiles, so that the value
            // operands (fetched after the keys, with no block of lead) are not needed before
            // four tiles of score MFMAs and softmax have run.
            pbs[qt] = pb;
            alphas[qt] = alpha;
        } else if constexpr (FIRST) {
#pragma unroll
            for (int dt = 0; dt < 8; ++dt)
                st.o[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                    b.v[dt], pb, floatx4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
        } else {
#pragma unroll
            for (int dt = 0; dt < 8; ++dt) {
                st.o[qt][dt] *= alpha;
                st.o[qt][dt] =
                    __builtin_amdgcn_mfma_f32_16x16x32_f16(b.v[dt], pb, st.o[qt][dt], 0, 0, 0);
            }
        }
    }
    if constexpr (NQ > 2) {
        if (tail) zero_tail();
        if constexpr (!FIRST) {
#pragma unroll
            for (int qt = 0; qt < NQ; ++qt)
                if (__builtin_amdgcn_ballot_w64(alphas[qt] != 1.0f) != 0) {  // some reference moved
#pragma unroll
                    for (int dt = 0; dt < 8; ++dt) st.o[qt][dt] *= alphas[qt];
                }
        }
#pragma unroll
        for (int qt = 0; qt < NQ; ++qt)
#pragma unroll
            for (int dt = 0; dt < 8; ++dt) {
                if constexpr (FIRST) {
                    st.o[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        b.v[dt], pbs[qt], floatx4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
                } else {
                    st.o[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b.v[dt], pbs[qt],
                                                                          st.o[qt][dt], 0, 0, 0);
                }
            }
    }
}

// This kernel runs for a few microseconds at decode shapes, so its shape follows latency,
// not throughput: every global load is issued before anything waits (new rows, then the
// query vectors, then the wavefront's first K/V block, all unconditional so that the
// in-order load counter lets the queries be staged while K/V are still in flight),
// integer divisions are replaced by multiplications with host-made reciprocals, and the
// bookkeeping the epilogue needs is computed in the shadow of the loads.
// RING = the layer is windowed: blocks start at the window, live in a ring, and the mask has a
// lower edge. Global layers run the instantiation without any of it.
// ---- preparation folded into the step (PREP instantiations) -----------------------------
// The reference's model norms and rotates Q and K between their projections and attention
// (per-head RMSNorm, crates/torch-math/src/norm.rs:40-51; RoPE, rope_interleaved.rs:103-114 /
// rope.rs:99-114; order of calls crates/muse-glimmer/src/model.rs:445-451). A decode step is a
// few thousand elements, so as a launch of its own that work costs a launch; here every
// workgroup prepares the 16 query vectors it stages anyway, and the workgroup that appends
// the new K rows prepares those. A 128-channel head row lies across 32 consecutive lanes, four
// channels each (c4 = 4 * (lane % 32)), which is how Q and the new rows are loaded.
//
// Arithmetic: the angle position * base^(-2i/rot) is formed and reduced to [-pi, pi] in f64
// (an f32 angle is off by 8e-3 rad at position 100,000); norm, sine, cosine and rotation are
// f32. The results feed f16 storage and f16 MFMA operands, so they differ from the
// reference's f64 chain by parts in 1e7 before that rounding: at most one f16 step after it.
struct PrepTrig {
    float c[4], s[4];  // per pair held by this lane: 2 (interleaved) or 4 (half split)
};

__device__ __forceinline__ void prep_trig(PrepTrig &t, double position, const double (&freq)[4],
                                          int pairs) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (i >= pairs) break;
        // The angle in turns, reduced to [-1/2, 1/2] exactly in f64; the sine and cosine
        // instructions take turns. Their error (about 1e-6 absolute) is a five-hundredth of
        // the f16 step the results are rounded to.
        const double turns = position * freq[i] * 0.15915494309189535;
        const float frac = float(turns - rint(turns));
        t.s[i] = __builtin_amdgcn_sinf(frac);
        t.c[i] = __builtin_amdgcn_cosf(frac);
    }
}

// Sum over the 32 lanes that share a head row: four DPP steps inside each row of 16 lanes
// (neighbour, other pair, mirrored half, mirrored row), then the row 16 lanes away.
__device__ __forceinline__ float row_sum32(float v) {
    v += dpp_lane<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_lane<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_lane<0x141>(v);  // row_half_mirror
    v += dpp_lane<0x140>(v);  // row_mirror
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(a[0]) + __uint_as_float(a[1]);
}

// x = channels c4 .. c4+3 of a head row, w = the norm weight's same channels.
__device__ __forceinline__ float4 prep_chunk(float4 x, bool norm, float4 w, float eps, uint32_t c4,
                                             uint32_t lane, uint32_t rot, bool interleaved,
                                             const PrepTrig &t) {
    if (norm) {
        const float ss = row_sum32(x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w);
        const float inv = __builtin_amdgcn_rsqf(ss * (1.0f / kD) + eps);
        x = make_float4(x.x * inv * w.x, x.y * inv * w.y, x.z * inv * w.z, x.w * inv * w.w);
    }
    if (rot == 0) return x;
    if (interleaved) {  // pairs (c4, c4+1) and (c4+2, c4+3)
        float4 y = x;
        if (c4 < rot) {
            y.x = x.x * t.c[0] - x.y * t.s[0];
            y.y = x.x * t.s[0] + x.y * t.c[0];
        }
        if (c4 + 2 < rot) {
            y.z = x.z * t.c[1] - x.w * t.s[1];
            y.w = x.z * t.s[1] + x.w * t.c[1];
        }
        return y;
    }
    // Half split: channel c < rot/2 turns with channel c + rot/2, four lanes-of-four apart.
    const uint32_t half = rot >> 1;
    const bool low = c4 < half, turn = c4 < rot;
    const uint32_t partner = (lane & 32u) | (((lane & 31u) + (low ? half / 4 : 32u - half / 4)) & 31u);
    const float4 o = make_float4(__shfl(x.x, partner), __shfl(x.y, partner), __shfl(x.z, partner),
                                 __shfl(x.w, partner));
    if (!turn) return x;
    if (low)
        return make_float4(x.x * t.c[0] - o.x * t.s[0], x.y * t.c[1] - o.y * t.s[1],
                           x.z * t.c[2] - o.z * t.s[2], x.w * t.c[3] - o.w * t.s[3]);
    return make_float4(o.x * t.s[0] + x.x * t.c[0], o.y * t.s[1] + x.y * t.c[1],
                       o.z * t.s[2] + x.z * t.c[2], o.w * t.s[3] + x.w * t.c[3]);
}


template <int NQ, int WAVES, int N, bool RING, bool PREP>
__device__ __forceinline__ void attn_splitk_f16_body(const AttnParams &p, const AttnBatchT<N> &b,
                                                     uint32_t total_partials,
                                                     [[maybe_unused]] const FoldedParams &fold) {
    extern __shared__ float lds[];
    float *sm_m = lds;                          // [WAVES][NQ*16]
    float *sm_l = sm_m + WAVES * NQ * 16;       // [WAVES][NQ*16]
    float *sm_o = sm_l + WAVES * NQ * 16;       // [WAVES][NQ][8][64][4]
    _Float16 *sm_q = reinterpret_cast<_Float16 *>(sm_o + WAVES * NQ * 8 * 64 * 4);  // [NQ*16][kQStride]
    _Float16 *sm_newk = sm_q + NQ * 16 * kQStride;  // [kMaxNewRows][kNewStride]
    _Float16 *sm_newv = sm_newk + kMaxNewRows * kNewStride;

    const uint32_t tid = threadIdx.x;
    const uint32_t wave = tid >> 6, lane = tid & 63;
    const uint32_t g = lane >> 4, jl = lane & 15;
    ITAK_MARK_BEGIN
    ITAK_MARK(0)

    // Kernel arguments arrive through scalar loads that the compiler would issue one
    // dependent batch at a time, each a round trip; naming them all in one place makes it
    // fetch them together.
    if (N == 1)
        asm volatile("" ::"s"(p.layer_base), "s"(p.q), "s"(p.out), "s"(p.ws), "s"(p.k_new),
                     "s"(p.v_new), "s"(p.g.slot_stride), "s"(p.g.head_stride),
                     "s"(p.g.side_stride), "s"(p.g.kv_heads), "s"(p.q_heads), "s"(p.group),
                     "s"(p.group_magic), "s"(p.scale), "s"(p.softcap), "s"(total_partials),
                     "s"(b.item[0].slot), "s"(b.item[0].rows), "s"(b.item[0].pos0),
                     "s"(b.item[0].q_row0), "s"(b.item[0].kv_len), "s"(b.item[0].splits),
                     "s"(b.item[0].keys_per_split), "s"(b.item[0].block0), "s"(b.item[0].ws0),
                     "s"(b.item[0].splits_magic), "s"(b.item[0].kv_lo), "s"(p.window),
                     "s"(p.ring_blocks));
    if (N == 1 && PREP)
        asm volatile("" ::"s"(fold.prep_q_weight), "s"(fold.prep_k_weight), "s"(fold.prep_eps),
                     "s"(fold.prep_rot), "s"(fold.prep_interleaved), "s"(fold.prep_freq_step), "s"(fold.gate));
    const AttnItem item = b.item[b.find_by_block(blockIdx.x)];
    const uint32_t local = blockIdx.x - item.block0;
    const uint32_t kv_head = item.splits > 1 ? __umulhi(local, item.splits_magic) : local;
    const uint32_t split = local - kv_head * item.splits;
    const uint32_t group = p.group, magic = p.group_magic;
    const uint32_t nvec = item.rows * group;

    uint16_t *kplane = static_cast<uint16_t *>(const_cast<void *>(p.layer_base)) +
                       item.slot * p.g.slot_stride + kv_head * p.g.head_stride;
    uint16_t *vplane = kplane + p.g.side_stride;
    const uint32_t row_width = p.g.kv_heads * kD;

    const uint32_t nblocks = (item.kv_len + kBlockKeys - 1) / kBlockKeys;
    const uint32_t blocks_per_split = item.keys_per_split / kBlockKeys;
    const uint32_t kb_begin = (RING ? item_first_block(item) : 0) + split * blocks_per_split;
    const uint32_t kb_end = min(nblocks, kb_begin + blocks_per_split);
    const uint32_t ring_blocks = RING ? p.ring_blocks : 0;
    const uint32_t window = RING ? p.window : 0, kv_lo = RING ? item.kv_lo : 0;
    const bool fused = p.k_new != nullptr;
    const bool owns_new = fused && kb_end * kBlockKeys > item.pos0;
    float *const ws_acc = p.ws;
    float *const ws_ml = p.ws + uint64_t(total_partials) * kD;
    ITAK_MARK(1)

    // ---- 1. new K/V rows into registers: rows x {K, V} x 32 chunks of 4 channels, read by
    // the one workgroup per KV head whose blocks hold the new positions.
    constexpr int NL = (kMaxNewRows * 2 * (kD / 4) + WAVES * 64 - 1) / (WAVES * 64);
    float4 nreg[NL];
    if (owns_new) {
        const float *k_new = p.k_new + uint64_t(item.q_row0) * row_width + kv_head * kD;
        const float *v_new = p.v_new + uint64_t(item.q_row0) * row_width + kv_head * kD;
#pragma unroll
        for (int u = 0; u < NL; ++u) {
            const uint32_t f = tid + u * WAVES * 64;
            const uint32_t r = f >> 6, side = (f >> 5) & 1, c4 = (f & 31) * 4;
            nreg[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (r < item.rows)
                nreg[u] = *reinterpret_cast<const float4 *>((side ? v_new : k_new) +
                                                            uint64_t(r) * row_width + c4);
        }
    }

    // ---- 2. query vectors into registers (vector j = query row j / group, Q head
    // kv_head*group + j % group); padding vectors re-read the last real one and are zeroed
    // when staged, so the loads need no branch.
    constexpr int QL = (NQ * 16 * (kD / 4)) / (WAVES * 64);
    static_assert(QL >= 1, "too many wavefronts for the query tile");
    float4 qld[QL];
#pragma unroll
    for (int u = 0; u < QL; ++u) {
        const uint32_t f = tid + u * WAVES * 64;
        const uint32_t j = min(f >> 5, nvec - 1), c4 = (f & 31) * 4;
        const uint32_t row = (j * magic) >> 16, head = kv_head * group + (j - row * group);
        qld[u] = *reinterpret_cast<const float4 *>(
            p.q + (uint64_t(item.q_row0 + row) * p.q_heads + head) * kD + c4);
    }

    // PREP: the norm weights of this lane's four channels (Q's and K's), issued with Q.
    const uint32_t pc4 = (tid & 31u) * 4;
    [[maybe_unused]] float4 wq = make_float4(1.f, 1.f, 1.f, 1.f), wk = wq;
    if constexpr (PREP) {
        if (fold.prep_q_weight) wq = *reinterpret_cast<const float4 *>(fold.prep_q_weight + pc4);
        if (fold.prep_k_weight) wk = *reinterpret_cast<const float4 *>(fold.prep_k_weight + pc4);
    }

    // ---- 3. the wavefront's first block (a wavefront without one loads the split's first
    // block and ignores it).
    BlockOperands buf_a;
    [[maybe_unused]] BlockOperands buf_b;
    uint32_t kb = kb_begin + wave;
    const bool has_block = kb < kb_end;
    load_block(buf_a, kplane, vplane, storage_block(has_block ? kb : kb_begin, ring_blocks), g, jl);
    ITAK_MARK(2)

    // ---- 4. in the shadow of the loads: what the mask and the epilogue need per column.
    uint32_t colpos[NQ], collo[NQ], colout[NQ], colps[NQ];
    const uint32_t lo_min = lowest_visible(item.pos0, window, kv_lo);
    const uint32_t lo_max = lowest_visible(item.pos0 + item.rows - 1, window, kv_lo);
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt) {
        const uint32_t j = qt * 16 + jl;
        const uint32_t row = (j * magic) >> 16, head = kv_head * group + (j - row * group);
        // A query ahead of the stored rows sees them all: for the mask its position is the
        // last stored one (its window still follows from where it really stands).
        colpos[qt] = min(item.pos0 + row, item.kv_len - 1);
        collo[qt] = lowest_visible(item.pos0 + row, window, kv_lo);
        colout[qt] = (item.q_row0 + row) * p.q_heads + head;
        colps[qt] = item.ws0 + (row * p.q_heads + head) * item.splits + split;
    }
    const float softcap = p.softcap;
    const float inv_cap = softcap > 0.0f ? 1.0f / softcap : 0.0f;
    const float qscale = softcap > 0.0f ? p.scale : p.scale * kLog2e;
    // PREP: this lane's pairs and their rotation at the step's first position, still in the
    // shadow of the loads (nothing here depends on what they bring).
    [[maybe_unused]] PrepTrig trig0;
    [[maybe_unused]] double freq[4] = {0.0, 0.0, 0.0, 0.0};
    [[maybe_unused]] int trig_pairs = 0;
    const uint32_t prot = PREP ? fold.prep_rot : 0;
    const bool pinter = PREP && fold.prep_interleaved != 0;
    if constexpr (PREP) {
        if (prot) {
            const uint32_t half = prot >> 1;
            // First pair index of this lane: interleaved pairs are (2i, 2i+1); half-split pair i
            // joins channels i and i + rot/2.
            const uint32_t pair0 = pinter ? pc4 >> 1 : (pc4 < half ? pc4 : pc4 - half);
            trig_pairs = pinter ? 2 : 4;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (i < trig_pairs) freq[i] = exp2(double(pair0 + i) * fold.prep_freq_step);
            prep_trig(trig0, double(item.pos0), freq, trig_pairs);
        }
    }
    ITAK_MARK(3)

    // ---- 5. stage Q^T (scaled, f16) and the new rows (f16, also stored to the planes).
#pragma unroll
    for (int u = 0; u < QL; ++u) {
        const uint32_t f = tid + u * WAVES * 64;
        const uint32_t j = f >> 5, c4 = (f & 31) * 4;
        float4 a = qld[u];
        if constexpr (PREP) {
            const uint32_t jr = min(j, nvec - 1), row = (jr * magic) >> 16;
            PrepTrig t = trig0;
            if (prot && row != 0) prep_trig(t, double(item.pos0 + row), freq, trig_pairs);
            a = prep_chunk(a, fold.prep_q_weight != nullptr, wq, fold.prep_eps, c4, lane, prot, pinter, t);
        }
        half4 h{static_cast<_Float16>(a.x * qscale), static_cast<_Float16>(a.y * qscale),
                static_cast<_Float16>(a.z * qscale), static_cast<_Float16>(a.w * qscale)};
        if (j >= nvec) h = half4{0, 0, 0, 0};
        *reinterpret_cast<half4 *>(sm_q + j * kQStride + c4) = h;
    }
    if (owns_new) {
#pragma unroll
        for (int u = 0; u < NL; ++u) {
            const uint32_t f = tid + u * WAVES * 64;
            const uint32_t r = f >> 6, side = (f >> 5) & 1, c4 = (f & 31) * 4;
            float4 a = nreg[u];
            if constexpr (PREP) {  // lanes 0..31 of a wavefront hold a K row, 32..63 its V row
                PrepTrig t = trig0;
                if (prot && r != 0 && r < item.rows) prep_trig(t, double(item.pos0 + r), freq, trig_pairs);
                const float4 k = prep_chunk(a, fold.prep_k_weight != nullptr, wk, fold.prep_eps, c4, lane, prot,
                                            pinter, t);
                if (side == 0) a = k;
            }
            if (r >= item.rows) continue;
            const uint16_t h0 = f32_to_f16_bits(a.x), h1 = f32_to_f16_bits(a.y);
            const uint16_t h2 = f32_to_f16_bits(a.z), h3 = f32_to_f16_bits(a.w);
            uint2 packed{uint32_t(h0) | (uint32_t(h1) << 16), uint32_t(h2) | (uint32_t(h3) << 16)};
            *reinterpret_cast<uint2 *>((side ? sm_newv : sm_newk) + r * kNewStride + c4) = packed;
            const uint32_t key = item.pos0 + r, kin = key % kBlockKeys;
            const uint64_t blk =
                uint64_t(storage_block(key / kBlockKeys, ring_blocks)) * (kBlockKeys * kD);
            if (side == 0) {
                const uint32_t kt = (kin >> 2) & 1, ki = (kin >> 3) * 4 + (kin & 3);
                *reinterpret_cast<uint2 *>(kplane + blk + ((kt * 16 + (c4 >> 3)) * 16 + ki) * 8 +
                                           (c4 & 7)) = packed;
            } else {
                uint16_t *vd = vplane + blk + c4 * kBlockKeys + kin;
                vd[0] = h0;
                vd[kBlockKeys] = h1;
                vd[2 * kBlockKeys] = h2;
                vd[3 * kBlockKeys] = h3;
            }
        }
    }
    ITAK_MARK(4)
    __syncthreads();
    half8 qreg[NQ <= 2 ? NQ * 4 : 1];
    if constexpr (NQ <= 2) {
#pragma unroll
        for (int qt = 0; qt < NQ; ++qt)
#pragma unroll
            for (int k = 0; k < 4; ++k)
                qreg[qt * 4 + k] = *reinterpret_cast<const half8 *>(
                    sm_q + (qt * 16 + jl) * kQStride + k * 32 + g * 8);
    }
    ITAK_MARK(5)

    // ---- this wavefront's blocks. Up to 32 query vectors there are registers for two
    // operand sets, so the next block's loads fly while the current one is multiplied; with
    // 64 vectors the accumulators take that room and the other wavefronts hide the latency.
    WaveState<NQ> st;
#define ITAK_BLOCK(FIRST, BUF, KB)                                                               \
    do {                                                                                         \
        if (fused && ((KB) + 1) * kBlockKeys > item.pos0)                                        \
            patch_new_rows(BUF, sm_newk, sm_newv, KB, g, jl, item.pos0, item.kv_len);            \
        process_block<NQ, FIRST, RING>(st, BUF, qreg, sm_q, KB, g, jl, colpos, collo,                  \
                                 min(item.pos0, item.kv_len - 1), item.kv_len, lo_min, lo_max,   \
                                 softcap, inv_cap);                                              \
    } while (0)
    if (has_block) {
        if constexpr (NQ <= 2) {
            uint32_t kb2 = kb + WAVES;
            bool more = kb2 < kb_end;
            if (more) load_block(buf_b, kplane, vplane, storage_block(kb2, ring_blocks), g, jl);
            ITAK_BLOCK(true, buf_a, kb);
            while (more) {
                const uint32_t kb3 = kb2 + WAVES;
                const bool more3 = kb3 < kb_end;
                if (more3) load_block(buf_a, kplane, vplane, storage_block(kb3, ring_blocks), g, jl);
                ITAK_BLOCK(false, buf_b, kb2);
                if (!more3) break;
                kb2 = kb3 + WAVES;
                more = kb2 < kb_end;
                if (more) load_block(buf_b, kplane, vplane, storage_block(kb2, ring_blocks), g, jl);
                ITAK_BLOCK(false, buf_a, kb3);
            }
        } else {
            ITAK_BLOCK(true, buf_a, kb);
            for (kb += WAVES; kb < kb_end; kb += WAVES) {
                load_block(buf_a, kplane, vplane, storage_block(kb, ring_blocks), g, jl);
                ITAK_BLOCK(false, buf_a, kb);
            }
        }
    } else {
#pragma unroll
        for (int qt = 0; qt < NQ; ++qt) {
            st.m[qt] = -INFINITY;
            st.l[qt] = 0.0f;
#pragma unroll
            for (int dt = 0; dt < 8; ++dt) st.o[qt][dt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
#undef ITAK_BLOCK

    // ---- merge the wavefronts through LDS ------------------------------------------------
    ITAK_MARK(6)
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt) {
        const float l = column_sum(st.l[qt]);
        if (g == 0) {
            sm_m[wave * NQ * 16 + qt * 16 + jl] = st.m[qt];
            sm_l[wave * NQ * 16 + qt * 16 + jl] = l;
        }
#pragma unroll
        for (int dt = 0; dt < 8; ++dt)
            *reinterpret_cast<floatx4 *>(sm_o + (((wave * NQ + qt) * 8 + dt) * 64 + lane) * 4) =
                st.o[qt][dt];
    }
    ITAK_MARK(7)
    __syncthreads();
    ITAK_MARK(8)

    // Every LDS read of the merge is issued before the first one is used.
    constexpr int kDtPerWave = 8 / WAVES;  // channel tiles each wavefront finishes
    const bool final_out = item.splits == 1;
    // The merge inside the launch: this group's run of the exchange buffer (p.ws).
    const bool exchanges = p.exchange != 0 && !final_out;
    ExchangeGroup xg;
    if (exchanges) xg.init(p.ws, item, kv_head, split, nvec);
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt) {
        const uint32_t j = qt * 16 + jl;
        floatx4 ow[kDtPerWave][WAVES];
        float mw[WAVES], lw[WAVES];
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            mw[w] = sm_m[w * NQ * 16 + qt * 16 + jl];
            lw[w] = sm_l[w * NQ * 16 + qt * 16 + jl];
        }
#pragma unroll
        for (int x = 0; x < kDtPerWave; ++x)
#pragma unroll
            for (int w = 0; w < WAVES; ++w)
                ow[x][w] = *reinterpret_cast<const floatx4 *>(
                    sm_o + (((w * NQ + qt) * 8 + wave * kDtPerWave + x) * 64 + lane) * 4);
        float M = mw[0];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) M = fmaxf(M, mw[w]);
        float L = 0.0f, wgt[WAVES];
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            wgt[w] = (mw[w] == -INFINITY) ? 0.0f : fast_exp2(mw[w] - M);
            L = fmaf(lw[w], wgt[w], L);
        }
        if (j >= nvec) continue;
        if (exchanges) {
            // Publish this wavefront's channel tiles of vector j to the slices' owners.
#pragma unroll
            for (int x = 0; x < kDtPerWave; ++x) {
                floatx4 acc = ow[x][0] * wgt[0];
#pragma unroll
                for (int w = 1; w < WAVES; ++w) acc += ow[x][w] * wgt[w];
                xg.publish(j, wave * kDtPerWave + x, g, acc, M, L);
            }
            continue;
        }
        float *dst = final_out ? p.out + uint64_t(colout[qt]) * kD
                               : ws_acc + uint64_t(colps[qt]) * kD;
        const float post = final_out ? __builtin_amdgcn_rcpf(L) : 1.0f;
#pragma unroll
        for (int x = 0; x < kDtPerWave; ++x) {
            floatx4 acc = ow[x][0] * wgt[0];
#pragma unroll
            for (int w = 1; w < WAVES; ++w) acc += ow[x][w] * wgt[w];
            acc *= post;
            if (PREP && final_out && fold.gate) {
                const float4 gt = *reinterpret_cast<const float4 *>(
                    fold.gate + uint64_t(colout[qt]) * kD + (wave * kDtPerWave + x) * 16 + g * 4);
                acc = floatx4{acc[0] * sigmoid_fast(gt.x), acc[1] * sigmoid_fast(gt.y),
                              acc[2] * sigmoid_fast(gt.z), acc[3] * sigmoid_fast(gt.w)};
            }
            *reinterpret_cast<floatx4 *>(dst + (wave * kDtPerWave + x) * 16 + g * 4) = acc;
        }
        if (!final_out && wave == 0 && g == 0)
            *reinterpret_cast<float2 *>(ws_ml + uint64_t(colps[qt]) * 2) = make_float2(M, L);
    }
    ITAK_MARK(9)
    if (exchanges) {
        const float *gate = nullptr;
        if constexpr (PREP) gate = fold.gate;
        xg.template finish<WAVES * 64, kExchangePerThread, 1>(reinterpret_cast<unsigned long long *>(sm_o), p, item, kv_head,
                                       group, magic, gate);
    }
    ITAK_MARK_END
}

template <int NQ, int WAVES, int N, bool RING>
__global__ __launch_bounds__(WAVES * 64) void attn_splitk_f16_kernel(AttnParams p, AttnBatchT<N> b,
                                                                     uint32_t total_partials) {
    attn_splitk_f16_body<NQ, WAVES, N, RING, false>(p, b, total_partials, FoldedParams{});
}
// The same variants with the preparation and the gate folded in.
template <int NQ, int WAVES, int N, bool RING>
__global__ __launch_bounds__(WAVES * 64) void attn_splitk_f16_prep_kernel(AttnParams p,
                                                                          AttnBatchT<N> b,
                                                                          uint32_t total_partials,
                                                                          FoldedParams f) {
    attn_splitk_f16_body<NQ, WAVES, N, RING, true>(p, b, total_partials, f);
}

}  // namespace

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
    uint32_t nvec = 0;
    uint64_t blocks = 0;
    for (uint32_t i = 0; i < b.n; ++i) {
        nvec = std::max(nvec, b.item[i].rows * group);
        blocks += uint64_t(g.kv_heads) * item_block_count(b.item[i]);
    }
    if (nvec > 32) return {4, 4, 3};
    if (nvec > 16) return {2, 4, 2};
    return blocks >= 4096 ? Variant{1, 8, 1} : Variant{1, 4, 0};
}
static size_t variant_lds(int nq, int waves) {
    return (size_t(2) * waves * nq * 16 + size_t(waves) * nq * 8 * 64 * 4) * 4 +
           size_t(nq) * 16 * kQStride * 2 + size_t(2) * kMaxNewRows * kNewStride * 2;
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
// runtime once per variant. A launch of at most this many workgroups runs in one wave of
// dispatch, so its duration is that of its largest workgroup.
template <int NQ, int W>
static uint32_t resident_groups() {
    static uint32_t cached = 0;
    if (cached) return cached;
    const size_t lds = variant_lds(NQ, W);
    int per_cu = 0, cus = 0, dev = 0;
    if (grant_lds<NQ, W>(lds) != hipSuccess || hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(
            &per_cu, reinterpret_cast<const void *>(&attn_splitk_f16_kernel<NQ, W, 1, false>), W * 64,
            lds) != hipSuccess ||
        per_cu < 1 || cus < 1) {
        (void)hipGetLastError();
        return 256;
    }
    cached = uint32_t(per_cu) * uint32_t(cus);
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
                                  const FoldedParams *folded) {
    (void)max_rows;
    if (b.total_blocks == 0) return hipSuccess;
    const Variant v = pick_variant(p.g, b, p.group);
    const bool prep = folded && folded->prep_on;
    if (!prep && v.index == 0 && attn_decode_f16_takes(p, b)) return launch_attn_decode_f16(p, b, total_partials, stream);
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
            if (s0 + sl + u * SL >= S) ml[u].x = -INFINITY;
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
        if (sl + u * 2 >= S) ml[u].x = -INFINITY;
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
