// GQA attention for gfx950 over f32 KV (the reference's own storage type), head_dim 128:
// decode steps, verify blocks and prefill chunks, split over the context like the f16 kernels,
// products on v_mfma_f32_16x16x4_f32 (f32 in, f32 out: the 1e-5 bar of f32 pools holds), K and V
// read straight from their row-major planes with 16-byte loads, no LDS in the loop; a short
// step's new rows are appended by the same launch. Other head dims and explicit query
// positions stay on the generic kernel.
//
// One workgroup of four wavefronts owns (item, kv head, tile of 16 query vectors, split = a run
// of 32-key blocks), a query vector being one row of one Q head of the group; a block of more
// than 16 vectors is several tiles, each walking the keys its own rows see (tiles of later rows
// first: they have the longest runs). Each wavefront walks its own blocks with a private online
// softmax, the four merge once through LDS. The MFMA takes one float per lane and operand: A[i][k] from lane i + 16k, B[k][j] from
// lane j + 16k, and returns rows 4g .. 4g+3 of column j to lane j + 16g. A dot product does
// not care in which order its terms are taken, so the channels (for K.Q^T) and the keys (for
// V^T.P^T) are assigned to the MFMA's k index in whatever order lets every lane fetch 16
// contiguous bytes:
//
//   S^T = K . Q^T   per 16-key tile t, 32 steps (s, e): lane (i, g) supplies K[key 16t + i]
//                   [channel 16s + 4g + e], i.e. the float4 at channels 16s + 4g of its key
//                   row covers the four e of a step group; Q^T is held the same way.
//                   Lane (j, g) receives the scores of keys 16t + 4g + r, r = 0..3.
//   O^T += V^T . P^T  per tile t and r = 0..3 the k index g stands for key 16t + 4g + r, whose
//                   probability is exactly what lane (j, g) holds in score register r: P needs
//                   no shuffle. Output tile (h, e) row i is channel 64h + 4i + e, so lane
//                   (i, g) fetches the float4 at channels 64h + 4i of value row 16t + 4g + r.
//
// Semantics: gqa_attention in crates/attention/src/attention.rs:104-215, softcap as
// crates/torch-math/src/logits.rs:26-37. Partials are in the log2 domain.
#include "internal.h"
#include "mfma_common.h"

#include <math.h>

#include <algorithm>

namespace itak {

namespace {

constexpr int kWavesF32 = 4;

__device__ __forceinline__ float lanes4_max(float v) {  // over lanes l, l^16, l^32, l^48
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const auto c = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(c[0]), __uint_as_float(c[1]));
}
__device__ __forceinline__ float lanes4_sum(float v) {
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const auto c = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(c[0]) + __uint_as_float(c[1]);
}

// D = head_dim: 64 or 128 (a multiple of 64: a value row is read as D / 64 float4 per lane).
// K/V rows that one workgroup alone reads (a step of one tile of vectors per KV head: decode rows,
// short blocks) are read with the streaming hint, so that they do not displace the kernel's
// code, arguments and split partials in L2 (decode at context 4096 13.6 -> 12.65 us per layer, the
// ragged batch 86.1 -> 81.5). Rows that several tiles' workgroups read keep the plain load: with
// the hint a 2048-row chunk took 4.4 ms instead of 3.3.
template <bool STREAM>
__device__ __forceinline__ float4 kv_load(const float *p) {
    if constexpr (STREAM) {
        typedef float f4v __attribute__((ext_vector_type(4)));
        const f4v v = __builtin_nontemporal_load(reinterpret_cast<const f4v *>(p));
        return make_float4(v[0], v[1], v[2], v[3]);
    } else {
        return *reinterpret_cast<const float4 *>(p);
    }
}

// BYROW: the launch holds an item of several rows (the exact treatment of values that are not
// finite is compiled in; launches of one row per item run the kernel without it).
template <int N, bool RING, int D, bool STREAM, bool BYROW>
__global__ __launch_bounds__(kWavesF32 * 64) void attn_splitk_f32_kernel(AttnParams p,
                                                                         AttnBatchT<N> b,
                                                                         uint32_t total_partials) {
    constexpr int kD = D;          // shadows the f16 kernels' constant inside this kernel
    constexpr int kSteps = D / 16;  // float4 steps of a key row per lane group
    constexpr int kH = D / 64;      // float4 pieces of a value row per lane
    __shared__ float sm_m[kWavesF32][16], sm_l[kWavesF32][16];
    __shared__ float sm_o[kWavesF32][kH * 4][64][4];  // [wave][tile (h, e)][lane][row of the lane]

    const uint32_t tid = threadIdx.x;
    const uint32_t wave = tid >> 6, lane = tid & 63;
    const uint32_t g = lane >> 4, jl = lane & 15;

    const AttnItem item = b.item[b.find_by_block(blockIdx.x)];
    const uint32_t local = blockIdx.x - item.block0;
    const uint32_t unit = local / item.splits, split = local % item.splits;
    const uint32_t group = p.group, nvec = item.rows * group;
    const uint32_t vtiles = (nvec + 15) / 16;
    const uint32_t kv_head = unit % p.g.kv_heads, vtile = vtiles - 1 - unit / p.g.kv_heads;
    // The rows this tile's vectors belong to bound the keys it walks.
    const uint32_t row_first = (vtile * 16) / group;
    const uint32_t row_last = min(item.rows - 1, (vtile * 16 + 15) / group);

    const float *kplane = static_cast<const float *>(p.layer_base) + item.slot * p.g.slot_stride +
                          kv_head * p.g.head_stride;
    const float *vplane = kplane + p.g.side_stride;

    const uint32_t ring = RING ? p.ring_blocks * kBlockKeys : 0;
    const uint32_t window = RING ? p.window : 0, kv_lo = RING ? item.kv_lo : 0;
    const uint32_t nblocks =
        (min(item.pos0 + row_last + 1, item.kv_len) + kBlockKeys - 1) / kBlockKeys;
    const uint32_t blocks_per_split = item.keys_per_split / kBlockKeys;
    const uint32_t kb_begin =
        (RING ? lowest_visible(item.pos0 + row_first, window, kv_lo) / kBlockKeys : 0) +
        split * blocks_per_split;
    const uint32_t kb_end = min(nblocks, kb_begin + blocks_per_split);

    // Fused append (p.k_new set): the last `rows` positions are not in the planes yet. The
    // workgroups whose blocks reach them copy the new rows in (f32 to f32, all threads, 16 bytes
    // each) and meet at a barrier before anybody reads a block; where two splits both reach
    // them both write the same bytes. No other workgroup reads these positions.
    if (p.k_new != nullptr && kb_end * kBlockKeys > item.pos0) {
        const uint32_t row_width = p.g.kv_heads * kD;
        constexpr uint32_t kChunks = kD / 4;  // float4 pieces of one side of a row
        for (uint32_t f = tid; f < item.rows * 2 * kChunks; f += kWavesF32 * 64) {
            const uint32_t r = f / (2 * kChunks), side = (f / kChunks) & 1, c4 = (f % kChunks) * 4;
            const float *src = (side ? p.v_new : p.k_new) + uint64_t(item.q_row0 + r) * row_width +
                               kv_head * kD + c4;
            const uint32_t pos = item.pos0 + r;
            float *dst = const_cast<float *>(side ? vplane : kplane) +
                         uint64_t(RING ? pos % ring : pos) * kD + c4;
            *reinterpret_cast<float4 *>(dst) = *reinterpret_cast<const float4 *>(src);
        }
        __syncthreads();
    }

    // This lane's query vector (column jl of the tile) and what its mask and its output need.
    const uint32_t jv = vtile * 16 + jl;
    const uint32_t j = min(jv, nvec - 1);
    const uint32_t row = j / group, head = kv_head * group + j % group;
    const uint32_t colpos = min(item.pos0 + row, item.kv_len - 1);
    const uint32_t collo = lowest_visible(item.pos0 + row, window, kv_lo);
    // [tile_lo, tile_hi): the positions some row of this tile sees.
    const uint32_t tile_lo = lowest_visible(item.pos0 + row_first, window, kv_lo);
    const uint32_t tile_hi = min(item.pos0 + row_last + 1, item.kv_len);
    const float softcap = p.softcap;
    const float inv_cap = softcap > 0.0f ? 1.0f / softcap : 0.0f;
    const float qscale = softcap > 0.0f ? p.scale : p.scale * kLog2e;

    // Q^T as B operands: step (s, e) takes channel 16s + 4g + e of vector jl.
    float4 qreg[kSteps];
    {
        const float *qp = p.q + (uint64_t(item.q_row0 + row) * p.q_heads + head) * kD + 4 * g;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            float4 a = *reinterpret_cast<const float4 *>(qp + 16 * s);
            if (jv >= nvec) a = make_float4(0.f, 0.f, 0.f, 0.f);
            qreg[s] = make_float4(a.x * qscale, a.y * qscale, a.z * qscale, a.w * qscale);
        }
    }

    float m_run = -INFINITY, l_run = 0.0f;
    floatx4 o[kH][4];
#pragma unroll
    for (int h = 0; h < kH; ++h)
#pragma unroll
        for (int e = 0; e < 4; ++e) o[h][e] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

    for (uint32_t kb = kb_begin + wave; kb < kb_end; kb += kWavesF32) {
        const uint32_t key0 = kb * kBlockKeys;
        // Rows past the stored length are fetched from the last stored row instead (the
        // plane may end there) and masked; a position's storage row on a ring is pos % ring.
        auto storage_row = [&](uint32_t pos) {
            const uint32_t q = min(pos, item.kv_len - 1);
            return RING ? q % ring : q;
        };
        float4 kreg[2][kSteps], vreg[2][4][kH];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const float *kr = kplane + uint64_t(storage_row(key0 + 16 * t + jl)) * kD + 4 * g;
#pragma unroll
            for (int s = 0; s < kSteps; ++s) kreg[t][s] = kv_load<STREAM>(kr + 16 * s);
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float *vr = vplane + uint64_t(storage_row(key0 + 16 * t + 4 * g + r)) * kD + 4 * jl;
#pragma unroll
                for (int h = 0; h < kH; ++h)
                    vreg[t][r][h] = kv_load<STREAM>(vr + 64 * h);
            }

        // Scores of keys key0 + 16t + 4g + r for this lane's vector.
        float sc[2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            floatx4 acc = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int s = 0; s < kSteps; ++s) {
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(kreg[t][s].x, qreg[s].x, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(kreg[t][s].y, qreg[s].y, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(kreg[t][s].z, qreg[s].z, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(kreg[t][s].w, qreg[s].w, acc, 0, 0, 0);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) sc[t][r] = acc[r];
        }
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t kp = key0 + 16 * t + 4 * g + r;
                float v = sc[t][r];
                if (softcap > 0.0f) v = softcap_log2(v, softcap, inv_cap);
                if (kp > colpos || (RING && kp < collo)) v = -INFINITY;
                sc[t][r] = v;
                mx = fmaxf(mx, v);
                // A row no query of the tile sees (past the stored length or the tile's last
                // row, or older than its oldest window on a ring) may hold anything, stale data
                // or a value that is not finite: keep it out of P.V even as 0*x. A tile of one
                // row needs nothing else to be exact.
                if (kp >= tile_hi || (RING && kp < tile_lo)) {
#pragma unroll
                    for (int h = 0; h < kH; ++h) vreg[t][r][h] = make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
        mx = lanes4_max(mx);
        const float m_new = fmaxf(m_run, mx);
        const bool dead = m_new == -INFINITY;
        const float alpha = (dead || m_run == -INFINITY) ? (dead ? 1.0f : 0.0f) : fast_exp2(m_run - m_new);
        float sum = 0.0f;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                // (Nothing finite in sight so far: -inf weighs zero against a reference of zero,
                // and a NaN score, which the maximum passes over as the reference's comparison
                // does, stays NaN and takes the row with it.)
                const float pe = fast_exp2(sc[t][r] - (dead ? 0.0f : m_new));
                sc[t][r] = pe;
                sum += pe;
            }
        l_run = l_run * alpha + sum;
        m_run = m_new;
#pragma unroll
        for (int h = 0; h < kH; ++h)
#pragma unroll
            for (int e = 0; e < 4; ++e) o[h][e] *= alpha;
        // A block in which the tile's rows do not all see the same keys, holding a value that is
        // not finite: gqa_attention never reads the value row of a key a query does not see
        // (crates/attention/src/attention.rs:160-173), but the rows share the value operand here
        // and a masked key's zero weight times such a value is NaN. The product is then taken
        // once per query row of the tile, the values of the keys that row does not see
        // cleared, and each lane keeps the result of the row its own column belongs to.
        if (BYROW && row_last > row_first &&
            (key0 + kBlockKeys > min(item.pos0 + row_first, item.kv_len - 1) + 1 ||
             (RING && key0 < lowest_visible(item.pos0 + row_last, window, kv_lo)))) {
            uint32_t seen = 0;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r)
#pragma unroll
                    for (int h = 0; h < kH; ++h) {
                        const float4 a = vreg[t][r][h];  // exponent all ones: 0x7f800000 + 0x00800000 = 0x80000000
                        seen |= ((__float_as_uint(a.x) & 0x7f800000u) + 0x00800000u) |
                                ((__float_as_uint(a.y) & 0x7f800000u) + 0x00800000u) |
                                ((__float_as_uint(a.z) & 0x7f800000u) + 0x00800000u) |
                                ((__float_as_uint(a.w) & 0x7f800000u) + 0x00800000u);
                    }
            if (__builtin_amdgcn_ballot_w64((seen & 0x80000000u) != 0) != 0) {
#pragma unroll 1
                for (uint32_t rr = row_first; rr <= row_last; ++rr) {
                    const uint32_t pos = min(item.pos0 + rr, item.kv_len - 1);
                    const uint32_t lo = RING ? lowest_visible(item.pos0 + rr, window, kv_lo) : 0u;
                    const bool mine = row == rr;
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const uint32_t kp = key0 + 16 * t + 4 * g + r;
                            const bool seen_by_row = kp <= pos && kp >= lo;
#pragma unroll
                            for (int h = 0; h < kH; ++h) {
                                const float4 v = vreg[t][r][h];
                                const float4 a = seen_by_row ? v : make_float4(0.f, 0.f, 0.f, 0.f);
                                const floatx4 zero = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
                                const floatx4 p0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, sc[t][r], zero, 0, 0, 0);
                                const floatx4 p1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, sc[t][r], zero, 0, 0, 0);
                                const floatx4 p2 = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, sc[t][r], zero, 0, 0, 0);
                                const floatx4 p3 = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, sc[t][r], zero, 0, 0, 0);
                                if (mine) {
                                    o[h][0] += p0;
                                    o[h][1] += p1;
                                    o[h][2] += p2;
                                    o[h][3] += p3;
                                }
                                __builtin_amdgcn_sched_barrier(0);
                            }
                        }
                }
                continue;
            }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int h = 0; h < kH; ++h) {
                    const float4 a = vreg[t][r][h];
                    o[h][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, sc[t][r], o[h][0], 0, 0, 0);
                    o[h][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, sc[t][r], o[h][1], 0, 0, 0);
                    o[h][2] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, sc[t][r], o[h][2], 0, 0, 0);
                    o[h][3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, sc[t][r], o[h][3], 0, 0, 0);
                }
    }

    // ---- merge the wavefronts through LDS: wavefront w finishes tiles 2w and 2w + 1.
    const float l_col = lanes4_sum(l_run);
    if (g == 0) {
        sm_m[wave][jl] = m_run;
        sm_l[wave][jl] = l_col;
    }
#pragma unroll
    for (int h = 0; h < kH; ++h)
#pragma unroll
        for (int e = 0; e < 4; ++e)
            *reinterpret_cast<floatx4 *>(&sm_o[wave][h * 4 + e][lane][0]) = o[h][e];
    __syncthreads();

    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < kWavesF32; ++w) M = fmaxf(M, sm_m[w][jl]);
    float L = 0.0f, wgt[kWavesF32];
#pragma unroll
    for (int w = 0; w < kWavesF32; ++w) {
        const float mw = sm_m[w][jl];
        wgt[w] = mw == -INFINITY ? 0.0f : fast_exp2(mw - M);
        L = fmaf(sm_l[w][jl], wgt[w], L);
    }
    if (jv >= nvec) return;
    const bool final_out = item.splits == 1;
    const uint64_t ps = item.ws0 + (uint64_t(row) * p.q_heads + head) * item.splits + split;
    float *dst = final_out ? p.out + (uint64_t(item.q_row0 + row) * p.q_heads + head) * kD
                           : p.ws + ps * kD;
    const float post = final_out ? 1.0f / L : 1.0f;
    // Tile (h, e), lane (jl, g), register rr holds channel 64h + 16g + 4rr + e. The kH * 4 tiles
    // are shared out among the four wavefronts: two consecutive e of one h each at head_dim 128
    // (8 contiguous bytes per register), one tile each at head_dim 64.
    constexpr int kTilesPerWave = kH * 4 / kWavesF32;
    floatx4 fin[kTilesPerWave];
#pragma unroll
    for (int x = 0; x < kTilesPerWave; ++x) {
        fin[x] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int w = 0; w < kWavesF32; ++w)
            fin[x] += *reinterpret_cast<const floatx4 *>(&sm_o[w][wave * kTilesPerWave + x][lane][0]) * wgt[w];
        fin[x] *= post;
    }
    if constexpr (kTilesPerWave == 2) {
        const uint32_t h = wave >> 1, e0 = (wave & 1) * 2;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr)
            *reinterpret_cast<float2 *>(dst + 64 * h + 16 * g + 4 * rr + e0) =
                make_float2(fin[0][rr], fin[1][rr]);
    } else {
#pragma unroll
        for (int x = 0; x < kTilesPerWave; ++x) {
            const uint32_t tile = wave * kTilesPerWave + x, h = tile >> 2, e = tile & 3;
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) dst[64 * h + 16 * g + 4 * rr + e] = fin[x][rr];
        }
    }
    if (!final_out && wave == 0 && g == 0)
        *reinterpret_cast<float2 *>(p.ws + uint64_t(total_partials) * kD + ps * 2) = make_float2(M, L);
}

}  // namespace

bool attn_splitk_f32_supports(const PoolGeom &g, uint32_t group, uint32_t max_rows) {
    return g.v_block == 0 && (g.head_dim == 128 || g.head_dim == 64) && group >= 1 && max_rows >= 1;
}
// Steps of up to 16 query vectors per KV head bring their rows along: every workgroup that
// reaches the new positions copies all of them in, which is nothing for a row or two and would
// be the whole chunk for a prefill.
bool attn_splitk_f32_appends(const PoolGeom &g, uint32_t group, uint32_t max_rows) {
    return attn_splitk_f32_supports(g, group, max_rows) && max_rows * group <= 16;
}

// Fills splits / keys_per_split / block0 / ws0 (slot, rows, pos0, q_row0, kv_len, kv_lo are
// set) and returns the number of partials. Every (item, KV head) is cut into equal runs of at
// most T blocks, T the smallest run for which the batch is at most two workgroups per
// compute unit, and never shorter than one block per wavefront.
uint32_t attn_splitk_f32_plan(const PoolGeom &g, AttnBatch &b, uint32_t q_heads) {
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        (void)hipGetLastError();
    const uint64_t capacity = uint64_t(2) * uint64_t(cus > 0 ? cus : 256);
    const uint32_t group = q_heads / g.kv_heads;
    auto units_of = [&](const AttnItem &it) {
        return uint64_t(g.kv_heads) * ((uint64_t(it.rows) * group + 15) / 16);
    };
    uint64_t blocks = 0;
    for (uint32_t i = 0; i < b.n; ++i) blocks += units_of(b.item[i]) * item_block_count(b.item[i]);
    uint64_t T = std::max<uint64_t>((blocks + capacity - 1) / capacity, uint64_t(kWavesF32));
    for (;; ++T) {
        uint64_t groups = 0;
        for (uint32_t i = 0; i < b.n; ++i) {
            const uint64_t nb = item_block_count(b.item[i]);
            groups += units_of(b.item[i]) * std::max<uint64_t>((nb + T - 1) / T, 1);
        }
        // (Units that alone outnumber the device are left whole: nothing is gained by splitting.)
        if (groups <= capacity || T >= blocks || T >= 4096) break;
    }
    uint32_t block0 = 0, ws0 = 0;
    for (uint32_t i = 0; i < b.n; ++i) {
        AttnItem &it = b.item[i];
        const uint32_t nblocks = item_block_count(it);
        it.splits = std::max<uint32_t>(uint32_t((nblocks + T - 1) / T), 1);
        const uint32_t bps = std::max<uint32_t>((nblocks + it.splits - 1) / it.splits, 1);
        it.splits = std::max<uint32_t>((nblocks + bps - 1) / bps, 1);
        it.keys_per_split = bps * kBlockKeys;
        it.splits_magic = 0;
        it.block0 = block0;
        it.ws0 = ws0;
        block0 += uint32_t(units_of(it)) * it.splits;
        if (it.splits > 1) ws0 += it.rows * q_heads * it.splits;
    }
    b.total_blocks = block0;
    b.rows_per_block = 0;
    return ws0;
}

hipError_t launch_attn_splitk_f32(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                  hipStream_t stream) {
    if (b.total_blocks == 0) return hipSuccess;
    // One tile of vectors per KV head in every item: each K/V row is read by one workgroup.
    // (And only where the keys and values would not stay in the last-level cache anyway: a pool
    // small enough to live there reads faster without the hint, 33.9 against 37.2 us for 4 slots
    // of 8192 rows on two layers.)
    bool single = p.kv_streams != 0;
    for (uint32_t i = 0; i < b.n; ++i) single = single && b.item[i].rows * p.group <= 16;
    bool several = false;
    for (uint32_t i = 0; i < b.n; ++i) several = several || b.item[i].rows > 1;
#define ITAK_LAUNCH_F32_B(RING, D, STREAM, BYROW)                                                 \
    ITAK_DISPATCH_BATCH(b.n, (attn_splitk_f32_kernel<N, RING, D, STREAM, BYROW>                     \
                              <<<b.total_blocks, kWavesF32 * 64, 0, stream>>>(p, AttnBatchT<N>(b), total_partials)))
#define ITAK_LAUNCH_F32_S(RING, D, STREAM)              \
    do {                                                \
        if (several)                                    \
            ITAK_LAUNCH_F32_B(RING, D, STREAM, true);   \
        else                                            \
            ITAK_LAUNCH_F32_B(RING, D, STREAM, false);  \
    } while (0)
#define ITAK_LAUNCH_F32(RING, D)                 \
    do {                                         \
        if (single)                              \
            ITAK_LAUNCH_F32_S(RING, D, true);    \
        else                                     \
            ITAK_LAUNCH_F32_S(RING, D, false);   \
    } while (0)
    if (p.g.head_dim == 64) {
        if (p.ring_blocks) ITAK_LAUNCH_F32(true, 64); else ITAK_LAUNCH_F32(false, 64);
    } else {
        if (p.ring_blocks) ITAK_LAUNCH_F32(true, 128); else ITAK_LAUNCH_F32(false, 128);
    }
#undef ITAK_LAUNCH_F32_S
#undef ITAK_LAUNCH_F32_B
#undef ITAK_LAUNCH_F32
    return hipGetLastError();
}

}  // namespace itak
