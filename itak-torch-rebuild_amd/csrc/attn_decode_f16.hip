// GQA flash-decode for gfx950 shaped for latency: one new position per sequence, f16 KV,
// head_dim 128, at most one 32-key block per wavefront, the split merge inside the launch.
//
// At a few thousand positions a decode layer moves a few MiB: about a microsecond of HBM time
// inside a launch that costs more than that to start. What the layer then costs is the longest
// chain of dependent round trips in its one launch, and how much code each wavefront has to
// fetch on the way (the instruction cache starts cold), so this kernel is the general
// split-K kernel (attn_splitk_f16.hip) with everything taken out that a decode step does not
// need:
//   - every wavefront owns one block and issues all of its loads at once: its share of the
//     group's query vectors (staged through LDS as f16 while the block is in flight: loading
//     them per lane in operand order costs the address unit as much as the block itself),
//     the new row's pieces where it owns them, then 8 x 16 bytes of keys and 8 x 16 of values;
//   - S^T = K . Q^T and O^T = V^T . P^T are 8 + 8 v_mfma_f32_16x16x32_f16 with the scores'
//     registers feeding P (the layouts are those of attn_splitk_f16.hip);
//   - the workgroup that owns the block of the new position converts the new K/V row once
//     (64 lanes, four channels each), stores it to the planes and hands it through LDS to the
//     wavefront that multiplies the block, which patches its operands in registers;
//   - the four wavefronts meet once in LDS; the workgroups of a KV head then merge among
//     themselves through the exchange buffer (split_exchange.h) and write the output.
//
// Semantics: gqa_attention, crates/attention/src/attention.rs:104-215, for one query per
// sequence at the sequence's newest position, after KvCache::append of that position
// (crates/attention/src/cache.rs:423-474) with the f32 -> f16 rule of
// crates/wgpu-compute/src/kernels/k1_q4k_gemv.rs:285-329; softcap as in attn_splitk_f16.hip.
#include "internal.h"
#include "mfma_common.h"
#include "split_exchange.h"
#include "timeline.h"

#include <math.h>

#include <algorithm>


// Timeline marks of attn_decode_f16_kernel: 0 first instruction, 1 addresses known (the kernel
// arguments have arrived), 2 every load issued, 3 scores done (keys and queries have arrived),
// 4 O^T written to LDS (values have arrived), 5 past the barrier, 6 partials or exchange words
// issued, 7 every exchange word gathered (in-launch merge only), 11 everything in flight done.
ITAK_TIMELINE_READER(itak_timeline_read_decode)

namespace itak {

namespace {

constexpr int kWaves = 4;
constexpr int kDecodeWords = 4;  // exchange words one thread gathers at most
constexpr int kDecodeLooks = 4;  // looks at the exchange buffer kept in flight

__device__ __forceinline__ float column_max4(float v) {
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const auto c = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(c[0]), __uint_as_float(c[1]));
}
__device__ __forceinline__ float column_sum4(float v) {
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const auto c = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(c[0]) + __uint_as_float(c[1]);
}

__device__ __forceinline__ half8 to_half8_rne(float4 a, float4 b) {
    half8 h;
    h[0] = __builtin_bit_cast(_Float16, f32_to_f16_bits(a.x));
    h[1] = __builtin_bit_cast(_Float16, f32_to_f16_bits(a.y));
    h[2] = __builtin_bit_cast(_Float16, f32_to_f16_bits(a.z));
    h[3] = __builtin_bit_cast(_Float16, f32_to_f16_bits(a.w));
    h[4] = __builtin_bit_cast(_Float16, f32_to_f16_bits(b.x));
    h[5] = __builtin_bit_cast(_Float16, f32_to_f16_bits(b.y));
    h[6] = __builtin_bit_cast(_Float16, f32_to_f16_bits(b.z));
    h[7] = __builtin_bit_cast(_Float16, f32_to_f16_bits(b.w));
    return h;
}

// QLO: the queries as two f16 halves, q = hi + lo, scores K.hi + K.lo (attn_splitk_f16_qlo.hip
// says why).
template <int N, bool RING, bool QLO = false>
__global__ __launch_bounds__(kWaves * 64) void attn_decode_f16_kernel(AttnParams p, AttnBatchT<N> b,
                                                                       uint32_t total_partials) {
    __shared__ float sm_m[kWaves * 16];
    __shared__ float sm_l[kWaves * 16];
    __shared__ __attribute__((aligned(16))) float sm_o[kWaves * 8 * 64 * 4];
    __shared__ __attribute__((aligned(16))) _Float16 sm_q[16 * kQStride];
    [[maybe_unused]] __shared__ __attribute__((aligned(16))) _Float16 sm_q_lo[QLO ? 16 * kQStride : 8];
    __shared__ __attribute__((aligned(16))) _Float16 sm_new[2 * kD];  // the new K row, then the new V row

    const uint32_t tid = threadIdx.x;
    const uint32_t wave = tid >> 6, lane = tid & 63;
    const uint32_t g = lane >> 4, jl = lane & 15;
    ITAK_MARK_BEGIN
    ITAK_MARK(0)
    // Kernel arguments arrive through scalar loads; naming them in one place makes the
    // compiler fetch them in one batch instead of one dependent round trip after another.
    if (N == 1)
        asm volatile("" ::"s"(p.layer_base), "s"(p.q), "s"(p.out), "s"(p.ws), "s"(p.k_new),
                     "s"(p.v_new), "s"(p.g.slot_stride), "s"(p.g.head_stride),
                     "s"(p.g.side_stride), "s"(p.g.kv_heads), "s"(p.q_heads), "s"(p.group),
                     "s"(p.group_magic), "s"(p.scale), "s"(p.softcap), "s"(p.spin_limit),
                     "s"(b.item[0].slot), "s"(b.item[0].pos0), "s"(b.item[0].q_row0),
                     "s"(b.item[0].kv_len), "s"(b.item[0].splits), "s"(b.item[0].keys_per_split),
                     "s"(b.item[0].block0), "s"(b.item[0].ws0), "s"(b.item[0].splits_magic),
                     "s"(b.item[0].kv_lo), "s"(p.window), "s"(p.ring_blocks));
    const AttnItem item = b.item[b.find_by_block(blockIdx.x)];
    const uint32_t local = blockIdx.x - item.block0;
    // Workgroups reach the device in the order of their index and the launch ends with its
    // slowest: the last split of every KV head, which holds the new position and has the most to
    // do, takes the first indices (split-major order, last split first).
    const uint32_t heads = p.g.kv_heads;
    uint32_t kv_head = local, split = 0;
    if (item.splits > 1) {
        uint32_t behind;  // splits after this one
        if ((heads & (heads - 1)) == 0) {
            behind = local >> __builtin_ctz(heads);
            kv_head = local & (heads - 1);
        } else {
            behind = local / heads;
            kv_head = local - behind * heads;
        }
        split = item.splits - 1 - behind;
    }
    const uint32_t group = p.group;

    uint16_t *kplane = static_cast<uint16_t *>(const_cast<void *>(p.layer_base)) +
                       item.slot * p.g.slot_stride + kv_head * p.g.head_stride;
    uint16_t *vplane = kplane + p.g.side_stride;

    const uint32_t pos = item.kv_len - 1;  // the query's position: the newest row
    const uint32_t nblocks = (item.kv_len + kBlockKeys - 1) / kBlockKeys;
    const uint32_t blocks_per_split = item.keys_per_split / kBlockKeys;  // at most kWaves
    const uint32_t kb_begin = (RING ? item_first_block(item) : 0) + split * blocks_per_split;
    const uint32_t kb_end = min(nblocks, kb_begin + blocks_per_split);
    const uint32_t kb = kb_begin + wave;
    const bool has_block = kb < kb_end;
    const uint32_t ring_blocks = RING ? p.ring_blocks : 0;
    uint32_t sb = has_block ? kb : kb_begin;  // a wavefront without a block loads one and ignores it
    if (RING) sb %= ring_blocks;
    ITAK_MARK(1)

    // ---- every load of the wavefront. Queries first (they and the keys gate the first MFMA and
    // loads return in order): thread f holds channels 4*(f%32) .. +3 of vector f/32.
    // Vectors beyond the group re-read the last real one and are zeroed when staged, so the
    // loads need no branch (a branch would make the compiler wait for them inside it).
    float4 qraw[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const uint32_t f = tid + u * kWaves * 64, j = min(f >> 5, group - 1), c4 = (f & 31) * 4;
        qraw[u] = *reinterpret_cast<const float4 *>(
            p.q + (uint64_t(item.q_row0) * p.q_heads + kv_head * group + j) * kD + c4);
    }
    // The new position's row is not in the planes yet. In the workgroup whose blocks hold it,
    // wavefront 0 reads the f32 row (lanes 0..31 the keys, 32..63 the values, four channels
    // each), converts it as append does, stores it to the planes and leaves it in LDS; the
    // wavefront that multiplies the block takes its operand pieces from there.
    const uint32_t new_kb = pos / kBlockKeys, kk = pos % kBlockKeys;
    const bool owns_new = p.k_new != nullptr && new_kb >= kb_begin && new_kb < kb_end;
    float4 nraw = make_float4(0.f, 0.f, 0.f, 0.f);
    if (owns_new && wave == 0) {
        const uint32_t row_width = p.g.kv_heads * kD;
        const float *src = (lane < 32 ? p.k_new : p.v_new) + uint64_t(item.q_row0) * row_width + kv_head * kD;
        nraw = *reinterpret_cast<const float4 *>(src + (lane & 31) * 4);
    }
    // Key rows of MFMA tile t are interleaved so that lane group g ends up holding the scores of
    // the 8 consecutive keys g*8 .. g*8+7 (the layout of internal.h).
    half8 bk[2][4], bv[8];
    {
        const uint16_t *kb_base = kplane + uint64_t(sb) * (kBlockKeys * kD) + (g * 16 + jl) * 8;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int s = 0; s < 4; ++s)
                bk[t][s] = __builtin_nontemporal_load(
                    reinterpret_cast<const half8 *>(kb_base + ((t * 16 + s * 4) * 16) * 8));
        const uint16_t *vb = vplane + uint64_t(sb) * (kBlockKeys * kD) + jl * kBlockKeys + g * 8;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt)
            bv[dt] = __builtin_nontemporal_load(reinterpret_cast<const half8 *>(vb + dt * 16 * kBlockKeys));
    }
    ITAK_MARK(2)

    // ---- Q^T as f16 through LDS while the block is in flight.
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const uint32_t f = tid + u * kWaves * 64, j = f >> 5, c4 = (f & 31) * 4;
        half4 h{static_cast<_Float16>(qraw[u].x), static_cast<_Float16>(qraw[u].y),
                static_cast<_Float16>(qraw[u].z), static_cast<_Float16>(qraw[u].w)};
        if (j >= group) h = half4{0, 0, 0, 0};
        *reinterpret_cast<half4 *>(sm_q + j * kQStride + c4) = h;
        if constexpr (QLO) {
            half4 l{static_cast<_Float16>(qraw[u].x - float(h[0])), static_cast<_Float16>(qraw[u].y - float(h[1])),
                    static_cast<_Float16>(qraw[u].z - float(h[2])), static_cast<_Float16>(qraw[u].w - float(h[3]))};
            if (j >= group) l = half4{0, 0, 0, 0};
            *reinterpret_cast<half4 *>(sm_q_lo + j * kQStride + c4) = l;
        }
    }
    uint2 packed{0u, 0u};
    if (owns_new && wave == 0) {
        const uint32_t c4 = (lane & 31) * 4;
        const uint32_t h0 = f32_to_f16_bits(nraw.x), h1 = f32_to_f16_bits(nraw.y);
        const uint32_t h2 = f32_to_f16_bits(nraw.z), h3 = f32_to_f16_bits(nraw.w);
        packed = uint2{h0 | (h1 << 16), h2 | (h3 << 16)};
        *reinterpret_cast<uint2 *>(sm_new + (lane >> 5) * kD + c4) = packed;
    }
    lds_barrier();
    half8 qb[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
        qb[k] = *reinterpret_cast<const half8 *>(sm_q + jl * kQStride + k * 32 + g * 8);

    if (owns_new && kb == new_kb) {
        // Keys: lane (g, i) holds row i of tile t; the new key is row i_new of tile t_new.
        const uint32_t t_new = (kk >> 2) & 1, i_new = (kk >> 3) * 4 + (kk & 3);
        if (jl == i_new) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const half8 h = *reinterpret_cast<const half8 *>(sm_new + s * 32 + g * 8);
                if (t_new == 0) bk[0][s] = h; else bk[1][s] = h;
            }
        }
    }

    // ---- S^T = K . Q^T
    const float softcap = p.softcap;
    const float qscale = softcap > 0.0f ? p.scale : p.scale * kLog2e;
    floatx4 s[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        s[t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int k = 0; k < 4; ++k)
            s[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bk[t][k], qb[k], s[t], 0, 0, 0);
    }
    if constexpr (QLO) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const half8 ql = *reinterpret_cast<const half8 *>(sm_q_lo + jl * kQStride + k * 32 + g * 8);
#pragma unroll
            for (int t = 0; t < 2; ++t)
                s[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bk[t][k], ql, s[t], 0, 0, 0);
        }
    }
    ITAK_MARK(3)
    float sc[8];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) sc[t * 4 + r] = s[t][r] * qscale;
    if (softcap > 0.0f) {
        const float inv_cap = 1.0f / softcap;
#pragma unroll
        for (int e = 0; e < 8; ++e) sc[e] = softcap_log2(sc[e], softcap, inv_cap);
    }
    // Keys the query does not see: beyond its position (rows past the stored length included)
    // or, on a windowed layer, before its window. Their values leave the product too, whatever
    // they hold: the reference never reads them (attention.rs:160-173).
    const uint32_t key_base = kb * kBlockKeys + g * 8;
    const uint32_t lo = RING ? lowest_visible(pos, p.window, item.kv_lo) : 0;
    if ((kb + 1) * kBlockKeys > pos + 1 || (RING && kb * kBlockKeys < lo)) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (key_base + e > pos || (RING && key_base + e < lo)) sc[e] = -INFINITY;
    }
    float mx = sc[0];
#pragma unroll
    for (int e = 1; e < 8; ++e) mx = fmaxf(mx, sc[e]);
    mx = column_max4(mx);
    const bool dead = mx == -INFINITY || !has_block;
    // (A block with nothing finite in sight: -inf weighs zero against a reference of zero, and a
    // NaN score, which the maximum passes over as the reference's comparison does, stays NaN.)
    const float m_ref = mx == -INFINITY ? 0.0f : mx;
    float sum = 0.0f;
    half8 pb;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float pe = has_block ? fast_exp2(sc[e] - m_ref) : 0.0f;
        sum += pe;
        pb[e] = static_cast<_Float16>(pe);
    }
    // ---- O^T = V^T . P^T, then the wavefronts meet in LDS.
    // What touches the value registers comes here, after the scores: the keys arrive first and
    // the softmax runs while the values are still on their way.
    if (owns_new && kb == new_kb) {
        // Values: lane (g, jl) holds keys g*8 .. g*8+7 of channel dt*16 + jl.
        if (g == (kk >> 3)) {
            // Half kk % 8 of each register group is replaced through a mask: no jump into one
            // of eight copies of the insertion, on a path one workgroup per KV head runs, cold.
            const u32x4 at = first_halves((kk & 7u) + 1) & ~first_halves(kk & 7u);
#pragma unroll
            for (int dt = 0; dt < 8; ++dt) {
                const uint32_t h = reinterpret_cast<const uint16_t *>(sm_new)[kD + dt * 16 + jl];
                const uint32_t both = h | (h << 16);
                const u32x4 old = __builtin_bit_cast(u32x4, bv[dt]);
                bv[dt] = __builtin_bit_cast(half8, (old & ~at) | (u32x4{both, both, both, both} & at));
            }
        }
    }
    if ((kb + 1) * kBlockKeys > pos + 1 || (RING && kb * kBlockKeys < lo)) {
        // This lane's keys [first, end) stay.
        const uint32_t end = min(pos + 1 - min(pos + 1, key_base), 8u);
        const uint32_t first = RING ? min(lo - min(lo, key_base), 8u) : 0u;
        const u32x4 keep = first_halves(end) & ~first_halves(first);
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) bv[dt] = keep_halves(bv[dt], keep);
    }
    const float l_wave = column_sum4(sum);
    if (g == 0) {
        sm_m[wave * 16 + jl] = dead ? -INFINITY : mx;
        sm_l[wave * 16 + jl] = l_wave;
    }
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) {
        floatx4 o = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        if (has_block) o = __builtin_amdgcn_mfma_f32_16x16x32_f16(bv[dt], pb, o, 0, 0, 0);
        *reinterpret_cast<floatx4 *>(sm_o + ((wave * 8 + dt) * 64 + lane) * 4) = o;
    }
    ITAK_MARK(4)
    lds_barrier();
    ITAK_MARK(5)
    // Wavefront w finishes channel tiles 2w and 2w+1 of every column.
    float mw[kWaves], lw[kWaves];
    floatx4 ow[2][kWaves];
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        mw[w] = sm_m[w * 16 + jl];
        lw[w] = sm_l[w * 16 + jl];
    }
#pragma unroll
    for (int x = 0; x < 2; ++x)
#pragma unroll
        for (int w = 0; w < kWaves; ++w)
            ow[x][w] = *reinterpret_cast<const floatx4 *>(sm_o + ((w * 8 + wave * 2 + x) * 64 + lane) * 4);
    float M = mw[0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) M = fmaxf(M, mw[w]);
    float L = 0.0f;
    floatx4 acc[2] = {floatx4{0.0f, 0.0f, 0.0f, 0.0f}, floatx4{0.0f, 0.0f, 0.0f, 0.0f}};
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        const float wgt = mw[w] == -INFINITY ? 0.0f : fast_exp2(mw[w] - M);
        L = fmaf(lw[w], wgt, L);
        acc[0] += ow[0][w] * wgt;
        acc[1] += ow[1][w] * wgt;
    }
    // The new row goes to the planes as append lays it out (k_offset / v_offset). Nothing in this
    // launch reads it from there, so the stores are the last thing their wavefront issues: the
    // others of its workgroup never wait behind them.
    auto store_new_row = [&] {
    if (owns_new && wave == 0) {
            const uint32_t c4 = (lane & 31) * 4;
            uint32_t nsb = new_kb;
            if (RING) nsb %= ring_blocks;
            const uint64_t blk = uint64_t(nsb) * (kBlockKeys * kD);
            if (lane < 32) {
                const uint32_t kt = (kk >> 2) & 1, ki = (kk >> 3) * 4 + (kk & 3);
                *reinterpret_cast<uint2 *>(kplane + blk + ((kt * 16 + (c4 >> 3)) * 16 + ki) * 8 + (c4 & 7)) = packed;
            } else {
                uint16_t *vd = vplane + blk + c4 * kBlockKeys + kk;
                vd[0] = uint16_t(packed.x);
                vd[kBlockKeys] = uint16_t(packed.x >> 16);
                vd[2 * kBlockKeys] = uint16_t(packed.y);
                vd[3 * kBlockKeys] = uint16_t(packed.y >> 16);
            }
        }
    };
    if (item.splits == 1) {
        if (jl < group) {
            float *dst = p.out + (uint64_t(item.q_row0) * p.q_heads + kv_head * group + jl) * kD;
            const float inv = __builtin_amdgcn_rcpf(L);
#pragma unroll
            for (int x = 0; x < 2; ++x)
                *reinterpret_cast<floatx4 *>(dst + (wave * 2 + x) * 16 + g * 4) = acc[x] * inv;
        }
        store_new_row();
        ITAK_MARK_END
        return;
    }
    if (!p.exchange) {
        // Partials for the merge launch: accumulators first, then (m, l) pairs (internal.h).
        if (jl < group) {
            const uint32_t ps = item.ws0 + (kv_head * group + jl) * item.splits + split;
            float *dst = p.ws + uint64_t(ps) * kD;
#pragma unroll
            for (int x = 0; x < 2; ++x)
                *reinterpret_cast<floatx4 *>(dst + (wave * 2 + x) * 16 + g * 4) = acc[x];
            if (wave == 0 && g == 0)
                *reinterpret_cast<float2 *>(p.ws + uint64_t(total_partials) * kD + uint64_t(ps) * 2) =
                    make_float2(M, L);
        }
        ITAK_MARK(6)
        store_new_row();
        ITAK_MARK_END
        return;
    }
    ExchangeGroup xg;
    xg.init(p.ws, item, kv_head, split, group);
    if (jl < group) {
        xg.publish(jl, wave * 2, g, acc[0], M, L);
        xg.publish(jl, wave * 2 + 1, g, acc[1], M, L);
    }
    ITAK_MARK(6)
    store_new_row();
    unsigned long long gathered_at = 0;
    xg.template finish<kWaves * 64, kDecodeWords, kDecodeLooks>(reinterpret_cast<unsigned long long *>(sm_o), p, item, kv_head, group,
                                    p.group_magic, nullptr, &gathered_at);
#ifdef ITAK_TIMELINE
    tm_[7] = gathered_at;
#endif
    ITAK_MARK_END
}

}  // namespace

// Takes a planned split-K batch when every item is one new row and no wavefront would own more
// than one block (and, where the splits merge inside the launch, no thread more words than
// the kernel gathers).
bool attn_decode_f16_takes(const AttnParams &p, const AttnBatch &b) {
    if (p.g.v_block != kVBlock || p.g.head_dim != kD || p.group < 1 || p.group > 16) return false;
    for (uint32_t i = 0; i < b.n; ++i) {
        const AttnItem &it = b.item[i];
        if (it.rows != 1 || it.pos0 + 1 != it.kv_len) return false;
        if (it.keys_per_split > uint32_t(kWaves * kBlockKeys)) return false;
        if (it.splits > 1 && p.exchange) {
            const uint32_t slices = p.group * 4, max_local = (slices + it.splits - 1) / it.splits;
            if (max_local * it.splits * kExchangeWords > uint32_t(kDecodeWords * kWaves * 64)) return false;
        }
    }
    return true;
}

uint32_t attn_decode_f16_resident_groups() {
    static uint32_t cached = 0;
    if (cached) return cached;
    int cus = 0, dev = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) {
        (void)hipGetLastError();
        return 256;
    }
    const void *kernels[] = {reinterpret_cast<const void *>(&attn_decode_f16_kernel<1, false>),
                             reinterpret_cast<const void *>(&attn_decode_f16_kernel<8, false>),
                             reinterpret_cast<const void *>(&attn_decode_f16_kernel<64, false>),
                             reinterpret_cast<const void *>(&attn_decode_f16_kernel<1, true>),
                             reinterpret_cast<const void *>(&attn_decode_f16_kernel<8, true>),
                             reinterpret_cast<const void *>(&attn_decode_f16_kernel<64, true>)};
    int least = 1 << 30;
    for (const void *k : kernels) {
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, k, kWaves * 64, 0) != hipSuccess || per_cu < 1) {
            (void)hipGetLastError();
            return 256;
        }
        least = std::min(least, per_cu);
    }
    cached = uint32_t(least) * uint32_t(cus);
    return cached;
}

hipError_t launch_attn_decode_f16(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                  hipStream_t stream, bool q_two_halves) {
    if (b.total_blocks == 0) return hipSuccess;
    if (q_two_halves) {
#define ITAK_LAUNCH_DECODE_QLO()                                                                   \
    do {                                                                                           \
        if (p.ring_blocks)                                                                         \
            attn_decode_f16_kernel<N, true, true><<<b.total_blocks, kWaves * 64, 0, stream>>>(p, AttnBatchT<N>(b), total_partials); \
        else                                                                                       \
            attn_decode_f16_kernel<N, false, true><<<b.total_blocks, kWaves * 64, 0, stream>>>(p, AttnBatchT<N>(b), total_partials); \
    } while (0)
        ITAK_DISPATCH_BATCH(b.n, ITAK_LAUNCH_DECODE_QLO());
#undef ITAK_LAUNCH_DECODE_QLO
        return hipGetLastError();
    }
#define ITAK_LAUNCH_DECODE()                                                                       \
    do {                                                                                           \
        if (p.ring_blocks)                                                                         \
            attn_decode_f16_kernel<N, true><<<b.total_blocks, kWaves * 64, 0, stream>>>(p, AttnBatchT<N>(b), total_partials); \
        else                                                                                       \
            attn_decode_f16_kernel<N, false><<<b.total_blocks, kWaves * 64, 0, stream>>>(p, AttnBatchT<N>(b), total_partials); \
    } while (0)
    ITAK_DISPATCH_BATCH(b.n, ITAK_LAUNCH_DECODE());
#undef ITAK_LAUNCH_DECODE
    return hipGetLastError();
}

}  // namespace itak
