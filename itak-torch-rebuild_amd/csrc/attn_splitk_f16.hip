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
// Semantics: gqa_attention in crates/attention/src/attention.rs:104-215 on a global layer
// (key kp visible to a query at position p iff kp <= p), with the optional softcap
// cap*tanh(s/cap) of crates/torch-math/src/logits.rs:26-37 applied to the scaled scores.
#include "internal.h"
#include "mfma_common.h"

#include <math.h>

namespace itak {

namespace {

template <int NQ>
struct WaveState {
    float m[NQ];         // running max of this lane's query-vector column (log2 domain)
    float l[NQ];         // this lane's share of the running denominator
    floatx4 o[NQ][8];    // O^T accumulators: channel dt*16 + g*4 + r, query vector column
};

struct BlockOperands {
    half8 k[2][4];  // [key half t][channel step s]
    half8 v[8];     // [channel tile dt]
};

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
            b.k[t][s] = *reinterpret_cast<const half8 *>(kb_base + ((t * 16 + s * 4) * 16) * 8);
    const uint16_t *vb = vplane + uint64_t(kb) * (kBlockKeys * kD) + i * kBlockKeys + g * 8;
#pragma unroll
    for (int dt = 0; dt < 8; ++dt)
        b.v[dt] = *reinterpret_cast<const half8 *>(vb + dt * 16 * kBlockKeys);
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

template <int NQ>
__device__ __forceinline__ void process_block(WaveState<NQ> &st, BlockOperands &b,
                                              const _Float16 *sm_q, uint32_t kb, uint32_t g,
                                              uint32_t jl, uint32_t pos0, uint32_t group,
                                              uint32_t kv_len, float softcap, float inv_cap) {
    const uint32_t key_base = kb * kBlockKeys + g * 8;  // first of this lane's 8 keys
    const bool tail = (kb + 1) * kBlockKeys > kv_len;
    if (tail) {
        // Rows past the stored length may hold stale data: keep them out of P.V even as 0*x.
#pragma unroll
        for (int dt = 0; dt < 8; ++dt)
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (key_base + e >= kv_len) b.v[dt][e] = _Float16(0.0f);
    }
    const bool need_mask = (kb + 1) * kBlockKeys > pos0 + 1;
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt) {
        // Q^T operand of this tile: lane (g, jl) holds channels k*32 + g*8 .. +8 of vector jl.
        half8 qb[4];
#pragma unroll
        for (int k = 0; k < 4; ++k)
            qb[k] = *reinterpret_cast<const half8 *>(sm_q + (qt * 16 + jl) * kQStride + k * 32 +
                                                     g * 8);
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
            const uint32_t pos = pos0 + (qt * 16 + jl) / group;  // this column's query position
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (key_base + e > pos) sc[e] = -INFINITY;
        }
        float mx = sc[0];
#pragma unroll
        for (int e = 1; e < 8; ++e) mx = fmaxf(mx, sc[e]);
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(st.m[qt], mx);
        const bool dead = m_new == -INFINITY;  // nothing visible to this column so far
        const float alpha = dead ? 1.0f : fast_exp2(st.m[qt] - m_new);
        float p[8];
        float sum = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            p[e] = dead ? 0.0f : fast_exp2(sc[e] - m_new);
            sum += p[e];
        }
        st.m[qt] = m_new;
        st.l[qt] = st.l[qt] * alpha + sum;
        half8 pb;
#pragma unroll
        for (int e = 0; e < 8; ++e) pb[e] = static_cast<_Float16>(p[e]);
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) {
            st.o[qt][dt] *= alpha;
            st.o[qt][dt] =
                __builtin_amdgcn_mfma_f32_16x16x32_f16(b.v[dt], pb, st.o[qt][dt], 0, 0, 0);
        }
    }
}

template <int NQ, int WAVES, int N>
__global__ __launch_bounds__(WAVES * 64) void attn_splitk_f16_kernel(AttnParams p, AttnBatchT<N> b,
                                                                     uint32_t total_partials) {
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

    const AttnItem item = b.item[b.find_by_block(blockIdx.x)];
    const uint32_t local = blockIdx.x - item.block0;
    const uint32_t split = local % item.splits;
    const uint32_t kv_head = local / item.splits;
    const uint32_t group = p.group;
    const uint32_t nvec = item.rows * group;

    uint16_t *kplane = static_cast<uint16_t *>(const_cast<void *>(p.layer_base)) +
                       item.slot * p.g.slot_stride + kv_head * p.g.head_stride;
    uint16_t *vplane = kplane + p.g.side_stride;
    const uint32_t row_width = p.g.kv_heads * kD;
    const bool fused = p.k_new != nullptr;
    const float *k_new = fused ? p.k_new + uint64_t(item.q_row0) * row_width + kv_head * kD : nullptr;
    const float *v_new = fused ? p.v_new + uint64_t(item.q_row0) * row_width + kv_head * kD : nullptr;

    const uint32_t nblocks = (item.kv_len + kBlockKeys - 1) / kBlockKeys;
    const uint32_t blocks_per_split = item.keys_per_split / kBlockKeys;
    const uint32_t kb_begin = split * blocks_per_split;
    const uint32_t kb_end = min(nblocks, kb_begin + blocks_per_split);

    // Start the first block's loads before anything else: this kernel is latency bound.
    BlockOperands buf_a;
    [[maybe_unused]] BlockOperands buf_b;
    uint32_t kb = kb_begin + wave;
    if (kb < kb_end) load_block(buf_a, kplane, vplane, kb, g, jl);

    // ---- Q^T as the B operand: lane (g, jl) holds channels s*32 + g*8 .. +8 of vector jl.
    // The workgroup reads its query vectors once, coalesced, scales and converts them to
    // f16 into LDS; each wavefront reads its operand registers from there per block.
    const float softcap = p.softcap;
    const float inv_cap = softcap > 0.0f ? 1.0f / softcap : 0.0f;
    const float qscale = softcap > 0.0f ? p.scale : p.scale * kLog2e;
    for (uint32_t f = tid; f < NQ * 16 * (kD / 4); f += WAVES * 64) {
        const uint32_t j = f / (kD / 4), c4 = (f % (kD / 4)) * 4;
        half4 h{0, 0, 0, 0};
        if (j < nvec) {
            const uint32_t row = j / group, head = kv_head * group + j % group;
            const float4 a = *reinterpret_cast<const float4 *>(
                p.q + (uint64_t(item.q_row0 + row) * p.q_heads + head) * kD + c4);
            h = half4{static_cast<_Float16>(a.x * qscale), static_cast<_Float16>(a.y * qscale),
                      static_cast<_Float16>(a.z * qscale), static_cast<_Float16>(a.w * qscale)};
        }
        *reinterpret_cast<half4 *>(sm_q + j * kQStride + c4) = h;
    }
    const bool owns_new = fused && kb_end * kBlockKeys > item.pos0;
    if (owns_new) {
        // rows x {K, V} x 32 chunks of 4 channels: convert, keep in LDS, store to the planes.
        for (uint32_t f = tid; f < item.rows * 2 * (kD / 4); f += WAVES * 64) {
            const uint32_t r = f / (2 * (kD / 4)), side = (f / (kD / 4)) & 1, c4 = (f % (kD / 4)) * 4;
            const float4 a = *reinterpret_cast<const float4 *>((side ? v_new : k_new) +
                                                               uint64_t(r) * row_width + c4);
            const uint16_t h0 = f32_to_f16_bits(a.x), h1 = f32_to_f16_bits(a.y);
            const uint16_t h2 = f32_to_f16_bits(a.z), h3 = f32_to_f16_bits(a.w);
            uint2 packed{uint32_t(h0) | (uint32_t(h1) << 16), uint32_t(h2) | (uint32_t(h3) << 16)};
            *reinterpret_cast<uint2 *>((side ? sm_newv : sm_newk) + r * kNewStride + c4) = packed;
            const uint32_t key = item.pos0 + r, kin = key % kBlockKeys;
            const uint64_t blk = uint64_t(key / kBlockKeys) * (kBlockKeys * kD);
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
    __syncthreads();

    WaveState<NQ> st;
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt) {
        st.m[qt] = -INFINITY;
        st.l[qt] = 0.0f;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) st.o[qt][dt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    }

    // ---- this wavefront's blocks. Up to 32 query vectors there are registers for two
    // operand sets, so the next block's loads fly while the current one is multiplied; with
    // 64 vectors the accumulators take that room and the other wavefronts hide the latency.
    if constexpr (NQ <= 2) {
        if (kb < kb_end) {
            for (;;) {
                const uint32_t kb2 = kb + WAVES;
                const bool has2 = kb2 < kb_end;
                if (has2) load_block(buf_b, kplane, vplane, kb2, g, jl);
                if (fused && (kb + 1) * kBlockKeys > item.pos0)
                    patch_new_rows(buf_a, sm_newk, sm_newv, kb, g, jl, item.pos0, item.kv_len);
                process_block<NQ>(st, buf_a, sm_q, kb, g, jl, item.pos0, group, item.kv_len,
                                  softcap, inv_cap);
                if (!has2) break;
                const uint32_t kb3 = kb2 + WAVES;
                const bool has3 = kb3 < kb_end;
                if (has3) load_block(buf_a, kplane, vplane, kb3, g, jl);
                if (fused && (kb2 + 1) * kBlockKeys > item.pos0)
                    patch_new_rows(buf_b, sm_newk, sm_newv, kb2, g, jl, item.pos0, item.kv_len);
                process_block<NQ>(st, buf_b, sm_q, kb2, g, jl, item.pos0, group, item.kv_len,
                                  softcap, inv_cap);
                if (!has3) break;
                kb = kb3;
            }
        }
    } else {
        while (kb < kb_end) {
            if (fused && (kb + 1) * kBlockKeys > item.pos0)
                patch_new_rows(buf_a, sm_newk, sm_newv, kb, g, jl, item.pos0, item.kv_len);
            process_block<NQ>(st, buf_a, sm_q, kb, g, jl, item.pos0, group, item.kv_len, softcap,
                              inv_cap);
            kb += WAVES;
            if (kb < kb_end) load_block(buf_a, kplane, vplane, kb, g, jl);
        }
    }

    // ---- merge the wavefronts through LDS ------------------------------------------------
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt) {
        float l = st.l[qt];
        l += __shfl_xor(l, 16);
        l += __shfl_xor(l, 32);
        if (g == 0) {
            sm_m[wave * NQ * 16 + qt * 16 + jl] = st.m[qt];
            sm_l[wave * NQ * 16 + qt * 16 + jl] = l;
        }
#pragma unroll
        for (int dt = 0; dt < 8; ++dt)
            *reinterpret_cast<floatx4 *>(sm_o + (((wave * NQ + qt) * 8 + dt) * 64 + lane) * 4) =
                st.o[qt][dt];
    }
    __syncthreads();

    float *ws_acc = p.ws;
    float *ws_ml = p.ws + uint64_t(total_partials) * kD;
    constexpr int kDtPerWave = 8 / WAVES;  // channel tiles each wavefront finishes
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt) {
        const uint32_t j = qt * 16 + jl;
        float mw[WAVES], M = -INFINITY;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            mw[w] = sm_m[w * NQ * 16 + qt * 16 + jl];
            M = fmaxf(M, mw[w]);
        }
        float L = 0.0f, wgt[WAVES];
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            wgt[w] = (mw[w] == -INFINITY) ? 0.0f : fast_exp2(mw[w] - M);
            L += sm_l[w * NQ * 16 + qt * 16 + jl] * wgt[w];
        }
        if (j >= nvec) continue;
        const uint32_t row = j / group, head = kv_head * group + j % group;
        const uint64_t ps = item.ws0 + (uint64_t(row) * p.q_heads + head) * item.splits + split;
#pragma unroll
        for (int x = 0; x < kDtPerWave; ++x) {
            const int dt = wave * kDtPerWave + x;
            floatx4 acc{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int w = 0; w < WAVES; ++w)
                acc += *reinterpret_cast<const floatx4 *>(
                           sm_o + (((w * NQ + qt) * 8 + dt) * 64 + lane) * 4) *
                       wgt[w];
            const uint32_t d = dt * 16 + g * 4;
            if (item.splits == 1) {
                const float inv = 1.0f / L;
                acc *= inv;
                *reinterpret_cast<floatx4 *>(
                    p.out + (uint64_t(item.q_row0 + row) * p.q_heads + head) * kD + d) = acc;
            } else {
                *reinterpret_cast<floatx4 *>(ws_acc + ps * kD + d) = acc;
            }
        }
        if (item.splits > 1 && wave == 0 && g == 0) {
            ws_ml[ps * 2] = M;
            ws_ml[ps * 2 + 1] = L;
        }
    }
}

}  // namespace

bool attn_splitk_f16_supports(const PoolGeom &g, uint32_t group, uint32_t max_rows) {
    return g.v_block == kVBlock && g.head_dim == kD && group >= 1 && max_rows >= 1 &&
           max_rows <= uint32_t(kMaxNewRows) && max_rows * group <= 64;
}

// Fills splits / keys_per_split / block0 / ws0 for a batch (the caller has set slot, rows,
// pos0, q_row0, kv_len) and returns the number of partials the launch will write.
// Wavefronts per workgroup. The 16-vector (decode) kernel is built with four and with
// eight: eight-wave workgroups halve the partials and measured about 4 % faster on large
// ragged batches, four-wave ones are faster at a few hundred blocks (context 4096, batch 1);
// two-wave workgroups were slower everywhere (the merge launch pays for the doubled partials).
constexpr uint32_t kSplitWaves = 4;
static uint32_t splitk_waves(const PoolGeom &g, const AttnBatch &b, uint32_t group) {
    uint64_t blocks = 0;
    for (uint32_t i = 0; i < b.n; ++i) {
        if (b.item[i].rows * group > 16) return kSplitWaves;
        blocks += uint64_t(g.kv_heads) * ((b.item[i].kv_len + kBlockKeys - 1) / kBlockKeys);
    }
    return blocks >= 4096 ? 8 : kSplitWaves;
}

uint32_t attn_splitk_f16_plan(const PoolGeom &g, AttnBatch &b, uint32_t q_heads) {
    uint64_t blocks = 0;
    for (uint32_t i = 0; i < b.n; ++i)
        blocks += uint64_t(g.kv_heads) * ((b.item[i].kv_len + kBlockKeys - 1) / kBlockKeys);
    const uint32_t waves = splitk_waves(g, b, q_heads / g.kv_heads);
    // About four workgroups per CU keeps every SIMD fed; short contexts get one block per
    // wavefront, the least work a workgroup can usefully have.
    constexpr uint64_t kTargetGroups = 1024;
    uint64_t bps = (blocks + kTargetGroups - 1) / kTargetGroups;
    bps = (bps + waves - 1) / waves * waves;
    if (bps < waves) bps = waves;
    uint32_t block0 = 0, ws0 = 0;
    for (uint32_t i = 0; i < b.n; ++i) {
        AttnItem &it = b.item[i];
        const uint32_t nblocks = (it.kv_len + kBlockKeys - 1) / kBlockKeys;
        it.keys_per_split = uint32_t(bps) * kBlockKeys;
        it.splits = uint32_t((nblocks + bps - 1) / bps);
        if (it.splits == 0) it.splits = 1;
        it.block0 = block0;
        it.ws0 = ws0;
        block0 += g.kv_heads * it.splits;
        if (it.splits > 1) ws0 += it.rows * q_heads * it.splits;
    }
    b.total_blocks = block0;
    b.rows_per_block = 0;
    return ws0;
}

hipError_t launch_attn_splitk_f16(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                  uint32_t max_rows, hipStream_t stream) {
    if (b.total_blocks == 0) return hipSuccess;
    const uint32_t nvec = max_rows * p.group;
    const uint32_t waves = splitk_waves(p.g, b, p.group);
#define ITAK_LAUNCH(NQ, W)                                                                       \
    do {                                                                                         \
        const size_t lds = (size_t(2) * W * NQ * 16 + size_t(W) * NQ * 8 * 64 * 4) * 4 +          \
                           size_t(NQ) * 16 * kQStride * 2 + size_t(2) * kMaxNewRows * (kD + 8) * 2; \
        static size_t granted = 64 * 1024;                                                       \
        if (lds > granted) {                                                                     \
            hipError_t e = hipFuncSetAttribute(                                                  \
                reinterpret_cast<const void *>(&attn_splitk_f16_kernel<NQ, W, N>),               \
                hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));                           \
            if (e != hipSuccess) return e;                                                       \
            granted = lds;                                                                       \
        }                                                                                        \
        attn_splitk_f16_kernel<NQ, W, N><<<b.total_blocks, W * 64, lds, stream>>>(               \
            p, AttnBatchT<N>(b), total_partials);                                                \
    } while (0)
#define ITAK_LAUNCH_NQ()                \
    do {                                \
        if (nvec <= 16) {               \
            if (waves == 8)             \
                ITAK_LAUNCH(1, 8);      \
            else                        \
                ITAK_LAUNCH(1, 4);      \
        } else if (nvec <= 32) {        \
            ITAK_LAUNCH(2, 4);          \
        } else {                        \
            ITAK_LAUNCH(4, 4);          \
        }                               \
    } while (0)
    ITAK_DISPATCH_BATCH(b.n, ITAK_LAUNCH_NQ());
#undef ITAK_LAUNCH_NQ
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
                                                                       int base2) {
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
            dst[d] = acc * inv;
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
        *reinterpret_cast<float4 *>(dst + tid * 4) =
            make_float4(sum.x * inv, sum.y * inv, sum.z * inv, sum.w * inv);
    }
}

hipError_t launch_attn_combine(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                               uint32_t total_rows, int base2, hipStream_t stream) {
    bool any = false;
    for (uint32_t i = 0; i < b.n; ++i) any = any || b.item[i].splits > 1;
    if (!any || total_rows == 0) return hipSuccess;
    ITAK_DISPATCH_BATCH(b.n, (attn_combine_kernel<N><<<total_rows * p.q_heads, kCombineThreads, 0,
                                                      stream>>>(p, AttnBatchT<N>(b), total_partials,
                                                                base2)));
    return hipGetLastError();
}

}  // namespace itak
