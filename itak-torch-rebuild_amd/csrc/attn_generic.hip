// Generic GQA attention for gfx950: f32 or f16 KV storage, any head_dim <= 256, any
// GQA group that fits the block, explicit or implied query positions, optional logit
// softcap, split over the key range (partials are merged by attn_combine_kernel).
// It is the path every shape can take (and the only f32-storage path); the tuned f16
// kernels elsewhere in this directory cover the shapes the engine actually serves.
//
// Semantics follow gqa_attention in crates/attention/src/attention.rs:104-215: a key at
// position kp is visible to a query at position p iff kp <= p and, on a windowed layer,
// kp > p - window (attention.rs:77-85), query head
// h reads KV head h / group, scores are dot(q, k) * scale, softmax over the visible keys,
// output = sum of weights * values. The reference's two-pass softmax becomes an online
// softmax over key tiles; sums are f32.
#include "internal.h"

#include <math.h>

namespace itak {

namespace {

constexpr int kThreads = 256;
constexpr int kMaxR = 64;   // query vectors (rows x group heads) per workgroup
constexpr int kMaxI = 16;   // accumulator slots per thread

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(uint16_t bits) {
    return static_cast<float>(__builtin_bit_cast(_Float16, bits));
}

struct Shape {
    uint32_t d;        // head_dim
    uint32_t tile;     // keys per tile (64 or 32)
    uint32_t kstride;  // LDS row stride of the key tile (floats)
    uint32_t ncol;     // d / VEC
    uint32_t rgroups;  // kThreads / ncol
};

template <int VEC>
__device__ __forceinline__ Shape make_shape(uint32_t d) {
    Shape s;
    s.d = d;
    s.tile = d <= 128 ? 64 : 32;
    s.kstride = d + VEC;
    s.ncol = d / VEC;
    s.rgroups = kThreads / s.ncol;
    return s;
}

template <typename T, int VEC, int N>
__global__ __launch_bounds__(kThreads) void attn_generic_kernel(AttnParams p, AttnBatchT<N> b,
                                                                uint32_t total_partials) {
    extern __shared__ float lds[];
    const Shape sh = make_shape<VEC>(p.g.head_dim);
    const uint32_t D = sh.d, TILE = sh.tile;
    float *Qs = lds;                      // [kMaxR][D]
    float *Ks = Qs + kMaxR * D;           // [TILE][kstride]
    float *Vs = Ks + TILE * sh.kstride;   // [TILE][D]
    float *Ss = Vs + TILE * D;            // [kMaxR][TILE]
    float *m_s = Ss + kMaxR * TILE;       // [kMaxR]
    float *l_s = m_s + kMaxR;
    float *a_s = l_s + kMaxR;

    const uint32_t tid = threadIdx.x;

    // ---- which work item is this workgroup? -------------------------------------
    const AttnItem item = b.item[b.find_by_block(blockIdx.x)];
    const uint32_t local = blockIdx.x - item.block0;
    const uint32_t split = local % item.splits;
    const uint32_t rest = local / item.splits;
    const uint32_t kv_head = rest % p.g.kv_heads;
    const uint32_t qblock = rest / p.g.kv_heads;

    const uint32_t row_begin = qblock * b.rows_per_block;
    const uint32_t row_end = min(item.rows, row_begin + b.rows_per_block);
    const uint32_t nrows = row_end - row_begin;
    const uint32_t R = nrows * p.group;

    // Keys this workgroup may touch: the split's range, clipped to what the block's
    // last row can see.
    uint32_t kend = item.kv_len;
    if (p.q_pos == nullptr) kend = min(kend, item.pos0 + row_end);
    const uint32_t k_begin = min(kend, item.kv_lo + split * item.keys_per_split);
    const uint32_t k_end = min(kend, k_begin + item.keys_per_split);
    const uint32_t ring = p.ring_blocks * 32;

    const T *kplane = static_cast<const T *>(p.layer_base) + item.slot * p.g.slot_stride +
                      kv_head * p.g.head_stride;
    const T *vplane = kplane + p.g.side_stride;

    // ---- stage the queries -----------------------------------------------------------
    for (uint32_t i = tid; i < R * D; i += kThreads) {
        const uint32_t r = i / D, d = i % D;
        const uint32_t row = row_begin + r / p.group;
        const uint32_t head = kv_head * p.group + r % p.group;
        Qs[r * D + d] = p.q[(uint64_t(item.q_row0 + row) * p.q_heads + head) * D + d];
    }
    if (tid < kMaxR) {
        m_s[tid] = -INFINITY;
        l_s[tid] = 0.0f;
        a_s[tid] = 0.0f;
    }

    // PV accumulators: thread owns column chunk dc and rows rbase + rgroups*i.
    const uint32_t dc = tid % sh.ncol;
    const uint32_t rbase = tid / sh.ncol;
    const bool pv_active = rbase < sh.rgroups;
    float acc[kMaxI][VEC];
#pragma unroll
    for (int i = 0; i < kMaxI; ++i)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[i][e] = 0.0f;

    // Score mapping: thread owns key column j and rows sgroup + sgroups*i.
    const uint32_t j = tid % TILE;
    const uint32_t sgroup = tid / TILE;
    const uint32_t sgroups = kThreads / TILE;

    __syncthreads();

    for (uint32_t t0 = k_begin; t0 < k_end; t0 += TILE) {
        const uint32_t tn = min(TILE, k_end - t0);
        // ---- load K and V tile (converted to f32) -----------------------------------
        for (uint32_t i = tid; i < TILE * sh.ncol; i += kThreads) {
            const uint32_t kj = i / sh.ncol, c = (i % sh.ncol) * VEC;
            float kv[VEC], vv[VEC];
            if (kj < tn) {
                const uint32_t srow = ring ? (t0 + kj) % ring : t0 + kj;
                const uint64_t koff = k_offset(p.g, srow, c);  // VEC channels share a piece
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    kv[e] = to_f32(kplane[koff + e]);
                    vv[e] = to_f32(vplane[v_offset(p.g, srow, c + e)]);
                }
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) kv[e] = vv[e] = 0.0f;
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                Ks[kj * sh.kstride + c + e] = kv[e];
                Vs[kj * D + c + e] = vv[e];
            }
        }
        __syncthreads();

        // ---- scores -----------------------------------------------------------------
        for (uint32_t i0 = 0; sgroup + sgroups * i0 < R; i0 += 8) {
            float s[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) s[i] = 0.0f;
            for (uint32_t d = 0; d < D; d += VEC) {
                float kk[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e) kk[e] = Ks[j * sh.kstride + d + e];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint32_t r = sgroup + sgroups * (i0 + i);
                    if (r < R) {
#pragma unroll
                        for (int e = 0; e < VEC; ++e) s[i] = fmaf(Qs[r * D + d + e], kk[e], s[i]);
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t r = sgroup + sgroups * (i0 + i);
                if (r < R) {
                    const uint32_t row = row_begin + r / p.group;
                    const uint32_t pos =
                        p.q_pos ? p.q_pos[item.q_row0 + row] : item.pos0 + row;
                    float v = s[i] * p.scale;
                    if (p.softcap > 0.0f) v = p.softcap * tanhf(v / p.softcap);
                    const uint32_t kp = t0 + j;
                    if (j >= tn || kp > pos || kp < lowest_visible(pos, p.window, item.kv_lo))
                        v = -INFINITY;
                    Ss[r * TILE + j] = v;
                }
            }
        }
        __syncthreads();

        // ---- online softmax, one wave per query vector at a time --------------------------
        {
            const uint32_t wave = tid >> 6, lane = tid & 63;
            for (uint32_t r = wave; r < R; r += kThreads / 64) {
                float v = lane < TILE ? Ss[r * TILE + lane] : -INFINITY;
                float mx = v;
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
                const float m_old = m_s[r];
                const float m_new = fmaxf(m_old, mx);
                const float pexp = (v == -INFINITY) ? 0.0f : expf(v - m_new);
                float sum = pexp;
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
                if (lane < TILE) Ss[r * TILE + lane] = pexp;
                if (lane == 0) {
                    const float alpha = (m_old == -INFINITY) ? 0.0f : expf(m_old - m_new);
                    a_s[r] = alpha;
                    l_s[r] = l_s[r] * alpha + sum;
                    m_s[r] = m_new;
                }
            }
        }
        __syncthreads();

        // ---- PV ---------------------------------------------------------------------
        if (pv_active) {
#pragma unroll
            for (int i = 0; i < kMaxI; ++i) {
                const uint32_t r = rbase + sh.rgroups * i;
                if (r < R) {
                    const float alpha = a_s[r];
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc[i][e] *= alpha;
                }
            }
            for (uint32_t kj = 0; kj < tn; ++kj) {
                float vv[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e) vv[e] = Vs[kj * D + dc * VEC + e];
#pragma unroll
                for (int i = 0; i < kMaxI; ++i) {
                    const uint32_t r = rbase + sh.rgroups * i;
                    if (r < R) {
                        const float w = Ss[r * TILE + kj];
#pragma unroll
                        for (int e = 0; e < VEC; ++e) acc[i][e] = fmaf(w, vv[e], acc[i][e]);
                    }
                }
            }
        }
        __syncthreads();
    }

    // ---- epilogue ----------------------------------------------------------------------
    if (item.splits == 1) {
        if (pv_active) {
#pragma unroll
            for (int i = 0; i < kMaxI; ++i) {
                const uint32_t r = rbase + sh.rgroups * i;
                if (r < R) {
                    const uint32_t row = row_begin + r / p.group;
                    const uint32_t head = kv_head * p.group + r % p.group;
                    const float inv = 1.0f / l_s[r];
                    float *o = p.out + (uint64_t(item.q_row0 + row) * p.q_heads + head) * D +
                               dc * VEC;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) o[e] = acc[i][e] * inv;
                }
            }
        }
        return;
    }

    // Partials: acc in ws[0 .. total_partials*D), then (m, l) pairs.
    float *ws_acc = p.ws;
    float *ws_ml = p.ws + uint64_t(total_partials) * D;
    if (pv_active) {
#pragma unroll
        for (int i = 0; i < kMaxI; ++i) {
            const uint32_t r = rbase + sh.rgroups * i;
            if (r < R) {
                const uint32_t row = row_begin + r / p.group;
                const uint32_t head = kv_head * p.group + r % p.group;
                const uint64_t ps =
                    item.ws0 + (uint64_t(row) * p.q_heads + head) * item.splits + split;
                float *o = ws_acc + ps * D + dc * VEC;
#pragma unroll
                for (int e = 0; e < VEC; ++e) o[e] = acc[i][e];
                if (dc == 0) {
                    ws_ml[ps * 2] = m_s[r];
                    ws_ml[ps * 2 + 1] = l_s[r];
                }
            }
        }
    }
}

size_t lds_bytes(uint32_t d, int vec) {
    const uint32_t tile = d <= 128 ? 64 : 32;
    const size_t floats = size_t(kMaxR) * d + size_t(tile) * (d + vec) + size_t(tile) * d +
                          size_t(kMaxR) * tile + 3 * kMaxR;
    return floats * sizeof(float);
}

}  // namespace

// Query vectors one workgroup can carry for a head_dim: bounded by the accumulator slots
// of the PV mapping (kMaxI rows per thread column group).
static uint32_t max_vectors(uint32_t d) {
    const int vec = d % 4 == 0 ? 4 : 1;
    const uint32_t ncol = d / vec;
    const uint32_t rgroups = kThreads / ncol;
    uint32_t r = kMaxI * rgroups;
    return r > kMaxR ? kMaxR : r;
}

uint32_t attn_generic_rows_per_block(uint32_t group, uint32_t head_dim) {
    if (group == 0 || head_dim == 0 || head_dim > 256) return 0;
    return max_vectors(head_dim) / group;
}

uint32_t attn_generic_tile(uint32_t head_dim) { return head_dim <= 128 ? 64 : 32; }

hipError_t launch_attn_generic(int elem_f16, const AttnParams &p, const AttnBatch &b,
                               uint32_t total_partials, hipStream_t stream) {
    if (b.total_blocks == 0) return hipSuccess;
    const uint32_t d = p.g.head_dim;
    const int vec = d % 4 == 0 ? 4 : 1;
    const size_t lds = lds_bytes(d, vec);
// Dynamic LDS above 64 KiB has to be granted per kernel before the first launch that
// needs it; the grant is raised whenever a launch needs more than any earlier one.
#define ITAK_LAUNCH(T, V)                                                                        \
    do {                                                                                         \
        static size_t granted = 64 * 1024;                                                       \
        if (lds > granted) {                                                                     \
            hipError_t e = hipFuncSetAttribute(                                                  \
                reinterpret_cast<const void *>(&attn_generic_kernel<T, V, N>),                   \
                hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));                           \
            if (e != hipSuccess) return e;                                                       \
            granted = lds;                                                                       \
        }                                                                                        \
        attn_generic_kernel<T, V, N><<<b.total_blocks, kThreads, lds, stream>>>(                 \
            p, AttnBatchT<N>(b), total_partials);                                                \
    } while (0)
#define ITAK_LAUNCH_TV()                 \
    do {                                 \
        if (elem_f16) {                  \
            if (vec == 4)                \
                ITAK_LAUNCH(uint16_t, 4);\
            else                         \
                ITAK_LAUNCH(uint16_t, 1);\
        } else {                         \
            if (vec == 4)                \
                ITAK_LAUNCH(float, 4);   \
            else                         \
                ITAK_LAUNCH(float, 1);   \
        }                                \
    } while (0)
    ITAK_DISPATCH_BATCH(b.n, ITAK_LAUNCH_TV());
#undef ITAK_LAUNCH_TV
#undef ITAK_LAUNCH
    return hipGetLastError();
}

}  // namespace itak
