// The split-K attention kernel of f16 pools at head_dim 128 (see attn_splitk_f16.hip for what it
// computes): the kernel body, included by the files that instantiate it. DIE = false is the form
// whose splits a second launch merges (or the exchange of split_exchange.h); DIE = true places
// every split of a (sequence, KV head) unit on one compute die and lets the last workgroup of
// the unit to finish merge the unit's partials out of that die's L2 (attn_splitk_f16_die.hip).
#pragma once

#include "internal.h"
#include "mfma_common.h"
#include "split_exchange.h"
#include "timeline.h"

#include <math.h>

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

// What the exact treatment of non-finite value rows needs to know of the item's query rows.
struct RowSpan {
    uint32_t pos0;    // position of the item's first query row (not clamped)
    uint32_t rows;
    uint32_t window;  // 0 on a global layer
    uint32_t kv_lo;
    uint32_t magic;   // j / group == (j * magic) >> 16
    // The step appends its own rows (they are then the only keys at the causal edge that some
    // rows see and others do not), and whether one of their values is not finite.
    bool appends, new_not_finite;
};

// O^T += V^T . P^T of one tile of query vectors, row of the step by row, for a block in which
// the rows do not all see the same keys and some value is not finite. The rows of a step share
// the block's value operand, a key that only some of them see is one column of it, and a
// masked key's zero weight times a value that is not finite is NaN in every row of the
// product, where gqa_attention never reads the value row of a key a query does not see
// (crates/attention/src/attention.rs:160-173). So the product is taken once per query row,
// with the value columns of the keys that row does not see cleared, and each lane keeps the
// result of the row its own column belongs to.
template <bool RING>
__device__ __forceinline__ void accumulate_by_row(floatx4 (&o)[8], const BlockOperands &b, half8 pb,
                                                  uint32_t qt, uint32_t key_base, uint32_t jl,
                                                  uint32_t kv_len, const RowSpan &span) {
    const uint32_t my_row = ((qt * 16 + jl) * span.magic) >> 16;
#pragma unroll 1
    for (uint32_t r = 0; r < span.rows; ++r) {
        const uint32_t pos = min(span.pos0 + r, kv_len - 1);
        const uint32_t lo = RING ? lowest_visible(span.pos0 + r, span.window, span.kv_lo) : 0u;
        const uint32_t end = min(pos + 1 - min(pos + 1, key_base), 8u);   // this lane's keys up to pos
        const uint32_t first = min(lo - min(lo, key_base), 8u);             // and from lo on
        const u32x4 keep = first_halves(end) & ~first_halves(first);
        const bool mine = my_row == r;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) {
            const floatx4 part = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                keep_halves(b.v[dt], keep), pb, floatx4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
            if (mine) o[dt] += part;
            // One channel tile at a time: left to itself the scheduler starts all eight products
            // before it adds the first, and their 32 registers do not fit beside the loop's.
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// One 32-key block against all NQ tiles of query vectors. FIRST = the wavefront's first
// block: the running state is written, not rescaled (most decode wavefronts see one block).
// Up to 32 vectors the Q^T operand lives in registers (qreg), beyond that it is re-read
// from LDS per block: lane (g, jl) holds channels k*32 + g*8 .. +8 of vector jl.
// BYROW = false compiles the exact treatment of non-finite values out: for the eight-wavefront
// variant, which the planners give to steps of one row per item only (its registers are all
// taken, and one row alone never needs it).
// QLO: the scaled queries are held as two halves, q = hi + lo with hi = f16(q) and lo = f16(q -
// hi), and every score is K.hi + K.lo: the queries' rounding to f16, which is relative to each
// channel and so grows with the scores, leaves the scores (the keys are exact, they are stored
// as f16). The low halves are read from LDS (sm_q_lo) block by block.
template <int NQ, bool FIRST, bool RING, bool BYROW, bool QLO>
__device__ __forceinline__ void process_block(WaveState<NQ> &st, BlockOperands &b,
                                              const half8 *qreg, const _Float16 *sm_q,
                                              [[maybe_unused]] const _Float16 *sm_q_lo,
                                              uint32_t kb, uint32_t g, uint32_t jl,
                                              const uint32_t *colpos, const uint32_t *collo,
                                              uint32_t pos0, uint32_t kv_len, uint32_t lo_min,
                                              uint32_t lo_max, float softcap, float inv_cap,
                                              const RowSpan &span) {
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
    // A block of several rows that do not all see the same keys: values that are not finite go
    // the exact way (accumulate_by_row). One row alone sees what zero_tail left.
    // (Where the step appends its own rows the answer for the causal edge was settled when they
    // were converted; looking through the operand registers is a hundred instructions that the
    // workgroup at the end of every item would otherwise run, cold.)
    auto suspect = [&]() -> bool {
        const bool low_edge = RING && kb * kBlockKeys < lo_max;
        if (!low_edge && span.appends) return span.new_not_finite;
        return any_not_finite(b.v);
    };
    const bool by_row = BYROW && span.rows > 1 && need_mask && (NQ <= 2 || !tail) && suspect();
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
        if constexpr (QLO) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const half8 ql = *reinterpret_cast<const half8 *>(sm_q_lo + (qt * 16 + jl) * kQStride +
                                                                  k * 32 + g * 8);
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    s[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b.k[t][k], ql, s[t], 0, 0, 0);
            }
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
        // Nothing finite visible to this column so far: its scores are -inf (weight zero, taken
        // against a reference of zero, since -inf - -inf is NaN) or NaN (a key that is not
        // finite: the maximum passes over it, as the reference's comparison does
        // (attention.rs:160-173), and its weight and with it the whole row must come out NaN).
        const bool dead = m_new == -INFINITY;
        const float m_ref = dead ? 0.0f : m_new;
        float p[8];
        float sum = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            p[e] = fast_exp2(sc[e] - m_ref);
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
        } else if (__builtin_expect(by_row, false)) {
#pragma unroll
            for (int dt = 0; dt < 8; ++dt)
                st.o[qt][dt] = FIRST ? floatx4{0.0f, 0.0f, 0.0f, 0.0f} : st.o[qt][dt] * alpha;
            accumulate_by_row<RING>(st.o[qt], b, pb, qt, key_base, jl, kv_len, span);
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
        // (The values are looked at after the tail is cleared: what lies past the stored rows
        // is nobody's to see.)
        const bool by_row_late = by_row || (BYROW && span.rows > 1 && need_mask && tail && suspect());
        if constexpr (!FIRST) {
#pragma unroll
            for (int qt = 0; qt < NQ; ++qt)
                if (__builtin_amdgcn_ballot_w64(alphas[qt] != 1.0f) != 0) {  // some reference moved
#pragma unroll
                    for (int dt = 0; dt < 8; ++dt) st.o[qt][dt] *= alphas[qt];
                }
        }
        if (__builtin_expect(by_row_late, false)) {
#pragma unroll
            for (int qt = 0; qt < NQ; ++qt) {
                if constexpr (FIRST) {
#pragma unroll
                    for (int dt = 0; dt < 8; ++dt) st.o[qt][dt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
                }
                accumulate_by_row<RING>(st.o[qt], b, pbs[qt], qt, key_base, jl, kv_len, span);
            }
            if constexpr (FIRST) return;
            // Later blocks fall through to the products every block runs, with the value operand
            // cleared (they add zeros): the accumulators then have one definition at the end of
            // the block, not two that the compiler must copy into one another.
#pragma unroll
            for (int dt = 0; dt < 8; ++dt) b.v[dt] = half8{0, 0, 0, 0, 0, 0, 0, 0};
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


// Dynamic LDS of a variant: the wavefronts' (m, l) and O^T for their merge, Q^T, the new rows.
inline size_t variant_lds(int nq, int waves, bool q_two_halves = false) {
    return (size_t(2) * waves * nq * 16 + size_t(waves) * nq * 8 * 64 * 4) * 4 +
           size_t(nq) * 16 * kQStride * 2 * (q_two_halves && nq <= 2 ? 2 : 1) +
           size_t(2) * kMaxNewRows * kNewStride * 2;
}

// ---- the merge of a unit's splits on the unit's own compute die (DIE instantiations) -------
// The device is eight compute dies, each with its own L2; workgroup i of a launch runs on die
// i % 8 (a probe at pool creation holds the device to that, and every workgroup of a DIE launch
// looks at the hardware's die number and counts itself in DieMap::faults when it differs). With
// every split of a unit on one die, the partials can stay in that die's L2: a workgroup stores
// its partial with ordinary stores, waits until the L2 has acknowledged them, and draws a
// ticket from the unit's counter (an atomic the L2 executes). Whoever draws the last ticket
// knows that every partial of the unit is in the L2 it reads from, puts the counter back to
// zero and merges. Nobody waits for anybody: no spin, no bound, nothing that can hang. The
// merging workgroup's vector cache cannot hold an older copy of what it reads: it is emptied
// when a kernel starts, and units do not share cache lines (they begin on multiples of 16
// partials).
__device__ __forceinline__ uint32_t compute_die() {
    uint32_t v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    return v & 0xfu;
}
// Merges the first S splits of the unit's first `count` query vectors (partials unit_ps0 +
// s * nvec + j) and, with `write`, stores the output rows. A thread takes (vector, 4 channels)
// after (vector, 4 channels) and walks the splits eight at a time, the loads of a trip in flight
// together; no lane needs another's values. The order of the sums depends on the split
// numbers only, never on which workgroup came last.
//
// The code is kept short on purpose. Only one workgroup per unit merges, and what few
// workgroups run they fetch cold, at some nanoseconds an instruction. For the same reason the
// workgroups that are not last run it once over their own partial without writing (the caller
// passes S = 1, a handful of vectors and write = false): they have finished, and the first of
// them on a die brings the code into that die's L2 ahead of the workgroups that need it.
template <int WAVES>
__device__ __forceinline__ void die_merge(const AttnParams &p, const AttnItem &item,
                                          uint32_t kv_head, uint32_t nvec, uint32_t count,
                                          uint32_t unit_ps0, uint32_t S,
                                          uint32_t total_partials, const float *gate, bool write) {
    const float2 *ws_ml = reinterpret_cast<const float2 *>(p.ws + uint64_t(total_partials) * kD);
#pragma unroll 1
    for (uint32_t task = threadIdx.x; task < count * 32; task += WAVES * 64) {
        const uint32_t jv = task >> 5, c = task & 31;
        float m_run = -INFINITY, l_run = 0.0f;
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 1
        for (uint32_t s0 = 0; s0 < S; s0 += 8) {
            float4 x[8];
            float2 ml[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {  // clamped, so the loads need no branch
                const uint64_t at = uint64_t(unit_ps0) + min(s0 + u, S - 1) * nvec + jv;
                x[u] = *reinterpret_cast<const float4 *>(p.ws + at * kD + c * 4);
                ml[u] = ws_ml[at];
            }
            float mx = m_run;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (s0 + u >= S) {  // a second copy of the last split: weight zero, and cleared
                    ml[u].x = -INFINITY;
                    x[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                }
                mx = fmaxf(mx, ml[u].x);
            }
            const float ref = mx == -INFINITY ? 0.0f : mx;  // exp2(-inf - finite) = 0
            const float alpha = fast_exp2(m_run - ref);
            acc.x *= alpha, acc.y *= alpha, acc.z *= alpha, acc.w *= alpha;
            l_run *= alpha;
            m_run = mx;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const float w = fast_exp2(ml[u].x - ref);
                l_run = fmaf(ml[u].y, w, l_run);
                acc.x = fmaf(x[u].x, w, acc.x);
                acc.y = fmaf(x[u].y, w, acc.y);
                acc.z = fmaf(x[u].z, w, acc.z);
                acc.w = fmaf(x[u].w, w, acc.w);
            }
        }
        const float inv = 1.0f / l_run;
        float4 o = make_float4(acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv);
        const uint32_t j = jv;
        const uint32_t row = (j * p.group_magic) >> 16;
        const uint32_t head = kv_head * p.group + (j - row * p.group);
        const uint64_t at = (uint64_t(item.q_row0 + row) * p.q_heads + head) * kD + c * 4;
        if (gate) {
            const float4 gt = *reinterpret_cast<const float4 *>(gate + at);
            o = make_float4(o.x * sigmoid_fast(gt.x), o.y * sigmoid_fast(gt.y),
                            o.z * sigmoid_fast(gt.z), o.w * sigmoid_fast(gt.w));
        }
        if (write) *reinterpret_cast<float4 *>(p.out + at) = o;
    }
}

template <int NQ, int WAVES, int N, bool RING, bool PREP, bool DIE, bool QLO = false>
__device__ __forceinline__ void attn_splitk_f16_body(const AttnParams &p, const AttnBatchT<N> &b,
                                                     uint32_t total_partials,
                                                     [[maybe_unused]] const FoldedParams &fold,
                                                     [[maybe_unused]] const DieMap &dm) {
    extern __shared__ float lds[];
    float *sm_m = lds;                          // [WAVES][NQ*16]
    float *sm_l = sm_m + WAVES * NQ * 16;       // [WAVES][NQ*16]
    float *sm_o = sm_l + WAVES * NQ * 16;       // [WAVES][NQ][8][64][4]
    _Float16 *sm_q = reinterpret_cast<_Float16 *>(sm_o + WAVES * NQ * 8 * 64 * 4);  // [NQ*16][kQStride]
    _Float16 *sm_newk = sm_q + NQ * 16 * kQStride;  // [kMaxNewRows][kNewStride]
    _Float16 *sm_newv = sm_newk + kMaxNewRows * kNewStride;
    // QLO: the queries' low halves, [NQ*16][kQStride]. With 64 vectors there is no LDS left for
    // them: they lie in the area the wavefronts' merge takes over when the blocks are done
    // (a barrier stands between the last read and the merge's first write).
    [[maybe_unused]] _Float16 *sm_q_lo =
        NQ > 2 ? reinterpret_cast<_Float16 *>(sm_o) : sm_newv + kMaxNewRows * kNewStride;

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
    const uint32_t group = p.group, magic = p.group_magic;
    // Which (item, KV head, split) this workgroup is. DIE: workgroup i runs on compute die
    // i % 8, and die d serves KV head d % heads of the items of bin d / heads, one after the
    // other along the die's own index i / 8.
    uint32_t item_at = 0, kv_head = 0, split = 0;
    if constexpr (DIE) {
        const uint32_t die = blockIdx.x & (kDieCount - 1), idx = blockIdx.x >> 3;
        const uint32_t bin = die >> dm.shift;
        // The bin's entries picked by comparisons: every word of the map is then fetched at a
        // fixed offset, in one batch of scalar loads, instead of one dependent load per lookup.
        uint32_t count = 0, item_end = 0;
#pragma unroll
        for (uint32_t k = 0; k < kDieCount; ++k)
            if (bin == k) {
                count = dm.bin_count[k];
                item_at = dm.bin_first[k];
                item_end = dm.bin_first[k + 1];
            }
        if (idx >= count) return;
        kv_head = die & ((1u << dm.shift) - 1u);
#pragma unroll 1
        while (item_at + 1 < item_end && idx >= b.block0[item_at + 1]) ++item_at;
        if (tid == 0 && (compute_die() & (kDieCount - 1)) != die)
            __hip_atomic_fetch_add(dm.faults, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
        item_at = b.find_by_block(blockIdx.x);
    }
    const AttnItem item = b.item[item_at];
    const uint32_t nvec = item.rows * group;
    if constexpr (DIE) {
        split = blockIdx.x / kDieCount - item.block0;
    } else {
        const uint32_t local = blockIdx.x - item.block0;
        kv_head = item.splits > 1 ? __umulhi(local, item.splits_magic) : local;
        split = local - kv_head * item.splits;
    }
    // DIE: first partial of this (item, KV head) unit, partial (split, vector j) at
    // unit_ps0 + split * nvec + j; units start on multiples of 16 partials, so that no cache
    // line of the (m, l) pairs is shared between units.
    const uint32_t unit_ps0 = item.ws0 + kv_head * ((item.splits * nvec + 15u) & ~15u);

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
        colps[qt] = DIE ? unit_ps0 + split * nvec + j
                        : item.ws0 + (row * p.q_heads + head) * item.splits + split;
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
        const float4 as = make_float4(a.x * qscale, a.y * qscale, a.z * qscale, a.w * qscale);
        half4 h{static_cast<_Float16>(as.x), static_cast<_Float16>(as.y),
                static_cast<_Float16>(as.z), static_cast<_Float16>(as.w)};
        if (j >= nvec) h = half4{0, 0, 0, 0};
        *reinterpret_cast<half4 *>(sm_q + j * kQStride + c4) = h;
        if constexpr (QLO) {  // what the rounding to f16 dropped, as a second f16
            half4 l{static_cast<_Float16>(as.x - float(h[0])), static_cast<_Float16>(as.y - float(h[1])),
                    static_cast<_Float16>(as.z - float(h[2])), static_cast<_Float16>(as.w - float(h[3]))};
            if (j >= nvec) l = half4{0, 0, 0, 0};
            *reinterpret_cast<half4 *>(sm_q_lo + j * kQStride + c4) = l;
        }
    }
    __shared__ uint32_t sm_new_not_finite[WAVES];
    if (owns_new) {
        uint32_t not_finite = 0;  // exponent field all ones in some half of a new value row
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
            if (side)
                not_finite |= ((packed.x & 0x7c007c00u) + 0x04000400u) | ((packed.y & 0x7c007c00u) + 0x04000400u);
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
        const bool wave_saw = __builtin_amdgcn_ballot_w64((not_finite & 0x80008000u) != 0) != 0;
        if (lane == 0) sm_new_not_finite[wave] = wave_saw ? 1u : 0u;
    }
    ITAK_MARK(4)
    __syncthreads();
    bool new_not_finite = false;
    if (owns_new) {
#pragma unroll
        for (int w = 0; w < WAVES; ++w) new_not_finite = new_not_finite || sm_new_not_finite[w] != 0;
    }
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
    const RowSpan span{item.pos0, item.rows, window, kv_lo, magic, fused, new_not_finite};
#define ITAK_BLOCK(FIRST, BUF, KB)                                                               \
    do {                                                                                         \
        if (fused && ((KB) + 1) * kBlockKeys > item.pos0)                                        \
            patch_new_rows(BUF, sm_newk, sm_newv, KB, g, jl, item.pos0, item.kv_len);            \
        /* Two copies of the block's arithmetic: the one with the exact treatment of values   \
           that are not finite only for blocks in which the step's rows do not all see the    \
           same keys, so that every other block runs code that knows nothing of it. */        \
        if constexpr (NQ > 2) { /* (no room for two copies beside 128 accumulators; the one copy  \
           costs the 7-row verify block 3 %: 23.7 -> 24.5 us per layer, same box) */             \
            process_block<NQ, FIRST, RING, true, QLO>(st, BUF, qreg, sm_q, sm_q_lo, KB, g, jl, colpos, \
                                 collo, min(item.pos0, item.kv_len - 1), item.kv_len, lo_min,    \
                                 lo_max, softcap, inv_cap, span);                                \
        } else if (WAVES != 8 && item.rows > 1 &&                                                \
            (((KB) + 1) * kBlockKeys > min(item.pos0, item.kv_len - 1) + 1 ||                    \
             (RING && (KB) * kBlockKeys < lo_max)))                                              \
            process_block<NQ, FIRST, RING, WAVES != 8, QLO>(st, BUF, qreg, sm_q, sm_q_lo, KB, g, jl, colpos, \
                                 collo, min(item.pos0, item.kv_len - 1), item.kv_len, lo_min,    \
                                 lo_max, softcap, inv_cap, span);                                \
        else                                                                                     \
            process_block<NQ, FIRST, RING, false, QLO>(st, BUF, qreg, sm_q, sm_q_lo, KB, g, jl, colpos, collo, \
                                 min(item.pos0, item.kv_len - 1), item.kv_len, lo_min, lo_max,   \
                                 softcap, inv_cap, span);                                        \
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
    if constexpr (QLO && NQ > 2) __syncthreads();  // everybody is done with the low halves in sm_o
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
    const bool exchanges = !DIE && p.exchange != 0 && !final_out;
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
    if constexpr (DIE) {
        __shared__ uint32_t sm_last;
        if (item.splits > 1) {
            // The unit's ticket is drawn once every partial store of this workgroup has been
            // acknowledged by the die's L2.
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            if (tid == 0) {
                uint32_t *ticket = dm.tickets + uint64_t(item.splits_magic + kv_head) * kDieTicketStride;
                const uint32_t t = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED,
                                                          __HIP_MEMORY_SCOPE_WORKGROUP);
                const uint32_t last = t + 1 == item.splits ? 1u : 0u;
                if (last) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                sm_last = last;
            }
            __syncthreads();
            ITAK_MARK(10)
            // (Not last: one pass over this workgroup's own partial, nothing written.)
            const bool last = sm_last != 0;
            die_merge<WAVES>(p, item, kv_head, nvec, last ? nvec : min(nvec, uint32_t(WAVES * 2)),
                             last ? unit_ps0 : unit_ps0 + split * nvec, last ? item.splits : 1u,
                             total_partials, dm.gate, last);
        }
    }
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
    attn_splitk_f16_body<NQ, WAVES, N, RING, false, false>(p, b, total_partials, FoldedParams{}, DieMap{});
}
// The same variants with the preparation and the gate folded in.
template <int NQ, int WAVES, int N, bool RING>
__global__ __launch_bounds__(WAVES * 64) void attn_splitk_f16_prep_kernel(AttnParams p,
                                                                          AttnBatchT<N> b,
                                                                          uint32_t total_partials,
                                                                          FoldedParams f) {
    attn_splitk_f16_body<NQ, WAVES, N, RING, true, false>(p, b, total_partials, f, DieMap{});
}
// The same with the queries as two halves (ITAK_POOL_Q_TWO_HALVES).
template <int NQ, int WAVES, int N, bool RING>
__global__ __launch_bounds__(WAVES * 64) void attn_splitk_f16_qlo_kernel(AttnParams p, AttnBatchT<N> b,
                                                                         uint32_t total_partials) {
    attn_splitk_f16_body<NQ, WAVES, N, RING, false, false, true>(p, b, total_partials, FoldedParams{}, DieMap{});
}
template <int NQ, int WAVES, int N, bool RING>
__global__ __launch_bounds__(WAVES * 64) void attn_splitk_f16_qlo_prep_kernel(AttnParams p,
                                                                              AttnBatchT<N> b,
                                                                              uint32_t total_partials,
                                                                              FoldedParams f) {
    attn_splitk_f16_body<NQ, WAVES, N, RING, true, false, true>(p, b, total_partials, f, DieMap{});
}
// The variants that merge each unit's splits on the unit's compute die.
template <int NQ, int WAVES, int N, bool RING>
__global__ __launch_bounds__(WAVES * 64) void attn_splitk_f16_die_kernel(AttnParams p, DieMap dm,
                                                                         AttnBatchT<N> b,
                                                                         uint32_t total_partials) {
    attn_splitk_f16_body<NQ, WAVES, N, RING, false, true>(p, b, total_partials, FoldedParams{}, dm);
}
template <int NQ, int WAVES, int N, bool RING>
__global__ __launch_bounds__(WAVES * 64) void attn_splitk_f16_die_prep_kernel(AttnParams p, DieMap dm,
                                                                              AttnBatchT<N> b,
                                                                              uint32_t total_partials,
                                                                              FoldedParams f) {
    attn_splitk_f16_body<NQ, WAVES, N, RING, true, true>(p, b, total_partials, f, dm);
}

}  // namespace

}  // namespace itak
