// KV row movement kernels for gfx950: append (f32 -> f16 RNE or f32 copy), zero fill of
// dropped rows, snapshot gather-restore and row readback. All of them are pure byte
// movement bound by HBM (or, for a pinned-host source, by the host link). Sources and
// the reference's own cache use [row][kv_head][d]; the pool stores one plane per KV head,
// and value planes of f16 pools in 32-row transposed blocks (see PoolGeom).
#include "internal.h"

namespace itak {

__device__ __forceinline__ void store4(float *dst, const float4 &v) {
    *reinterpret_cast<float4 *>(dst) = v;
}
__device__ __forceinline__ void store4(uint16_t *dst, const float4 &v) {
    uint2 packed;
    packed.x = uint32_t(f32_to_f16_bits(v.x)) | (uint32_t(f32_to_f16_bits(v.y)) << 16);
    packed.y = uint32_t(f32_to_f16_bits(v.z)) | (uint32_t(f32_to_f16_bits(v.w)) << 16);
    *reinterpret_cast<uint2 *>(dst) = packed;
}
__device__ __forceinline__ void store1(float *dst, float v) { *dst = v; }
__device__ __forceinline__ void store1(uint16_t *dst, float v) { *dst = f32_to_f16_bits(v); }
__device__ __forceinline__ void store1(uint16_t *dst, uint16_t v) { *dst = v; }

// ---------------------------------------------------------------------------- append
// Thread = one (row, side, kv head, VEC-element chunk) of the new rows. Key planes
// (row-major or blocked) and row-major value planes take one vector store; blocked value
// planes take VEC 2-byte stores 64 bytes apart (an append moves a few KiB, so their width
// does not matter).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void kv_append_kernel(T *__restrict__ layer_base, PoolGeom g,
                                                        AppendBatch b,
                                                        const float *__restrict__ k_src,
                                                        const float *__restrict__ v_src) {
    const uint32_t chunks = g.head_dim / VEC;
    const uint64_t per_row = 2ull * g.kv_heads * chunks;
    const uint64_t idx = blockIdx.x * 256ull + threadIdx.x;
    if (idx >= per_row * b.total_rows) return;
    uint32_t row = uint32_t(idx / per_row);  // among the rows this launch moves, then in the source
    if (b.gap_rows && row >= b.gap_at) row += b.gap_rows;
    uint32_t rem = uint32_t(idx % per_row);
    const uint32_t side = rem / (g.kv_heads * chunks);
    rem -= side * g.kv_heads * chunks;
    const uint32_t head = rem / chunks;
    const uint32_t d = (rem % chunks) * VEC;
    uint32_t it = 0;
    while (it + 1 < b.n && row >= b.item[it + 1].src_row0) ++it;
    const AppendItem item = b.item[it];
    uint32_t dst_row = item.pos0 + (row - item.src_row0);
    if (b.ring) dst_row %= b.ring;  // cache.rs:168-173 with the device ring in place of the window
    const float *src = (side ? v_src : k_src) + (uint64_t(row) * g.kv_heads + head) * g.head_dim + d;
    T *plane = layer_base + item.slot * g.slot_stride + side * g.side_stride + head * g.head_stride;
    if constexpr (VEC == 4) {
        const float4 v = *reinterpret_cast<const float4 *>(src);
        if (side == 0 || g.v_block == 0) {
            // Four channels never straddle an 8-channel piece of the blocked key layout.
            store4(plane + k_offset(g, dst_row, d), v);
        } else {
            T *dst = plane + v_offset(g, dst_row, d);
            store1(dst, v.x);
            store1(dst + kVBlock, v.y);
            store1(dst + 2 * kVBlock, v.z);
            store1(dst + 3 * kVBlock, v.w);
        }
    } else {
        store1(plane + kv_offset(g, side, dst_row, d), *src);
    }
}

hipError_t launch_append(void *layer_base, int elem_f16, const PoolGeom &g, const AppendBatch &b,
                         const float *k_src, const float *v_src, hipStream_t stream) {
    if (b.total_rows == 0) return hipSuccess;
    const bool vec = (g.head_dim % 4 == 0) && (reinterpret_cast<uintptr_t>(k_src) % 16 == 0) &&
                     (reinterpret_cast<uintptr_t>(v_src) % 16 == 0);
    const uint64_t per_row = 2ull * g.kv_heads * (vec ? g.head_dim / 4 : g.head_dim);
    const uint64_t threads = per_row * b.total_rows;
    const uint32_t blocks = uint32_t((threads + 255) / 256);
    if (elem_f16) {
        auto *base = static_cast<uint16_t *>(layer_base);
        if (vec)
            kv_append_kernel<uint16_t, 4><<<blocks, 256, 0, stream>>>(base, g, b, k_src, v_src);
        else
            kv_append_kernel<uint16_t, 1><<<blocks, 256, 0, stream>>>(base, g, b, k_src, v_src);
    } else {
        auto *base = static_cast<float *>(layer_base);
        if (vec)
            kv_append_kernel<float, 4><<<blocks, 256, 0, stream>>>(base, g, b, k_src, v_src);
        else
            kv_append_kernel<float, 1><<<blocks, 256, 0, stream>>>(base, g, b, k_src, v_src);
    }
    return hipGetLastError();
}

// ------------------------------------------------------------------------- zero rows
// grid = (blocks over the widest item's elements, item, layer * 2 * kv_heads planes).
template <typename T>
__global__ __launch_bounds__(256) void kv_zero_rows(T *__restrict__ pool_base, PoolGeom g,
                                                    uint32_t layer_from, ZeroBatch b) {
    const ZeroItem item = b.item[blockIdx.y];
    if (item.row_to <= item.row_from) return;
    const uint32_t planes_per_layer = 2 * g.kv_heads;
    const uint32_t layer = layer_from + blockIdx.z / planes_per_layer;
    const uint32_t plane_id = blockIdx.z % planes_per_layer;  // side * kv_heads + head
    const uint32_t side = plane_id / g.kv_heads;
    T *plane = pool_base + layer * g.layer_stride + item.slot * g.slot_stride +
               plane_id * g.head_stride;
    const uint64_t total = uint64_t(item.row_to - item.row_from) * g.head_dim;
    const bool blocked = g.v_block != 0;
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < total; i += gridDim.x * 256ull) {
        if (blocked) {
            const uint32_t rows = item.row_to - item.row_from;
            const uint32_t d = uint32_t(i / rows);
            const uint32_t row = item.row_from + uint32_t(i % rows);
            plane[kv_offset(g, side, row, d)] = T(0);
        } else {
            plane[uint64_t(item.row_from) * g.head_dim + i] = T(0);
        }
    }
}

hipError_t launch_zero_rows(void *pool_base, int elem_f16, const PoolGeom &g, uint32_t layer_from,
                            uint32_t layer_to, const ZeroBatch &b, hipStream_t stream) {
    if (b.n == 0 || b.max_rows == 0 || layer_to <= layer_from) return hipSuccess;
    const uint64_t elems = uint64_t(b.max_rows) * g.head_dim;
    uint32_t bx = uint32_t((elems + 255) / 256);
    if (bx > 1024) bx = 1024;
    const uint32_t planes_per_layer = 2 * g.kv_heads;
    // gridDim.z is limited to 65535: walk the layers in slices that fit.
    const uint32_t layers_per_launch = 65535 / planes_per_layer ? 65535 / planes_per_layer : 1;
    for (uint32_t l = layer_from; l < layer_to; l += layers_per_launch) {
        const uint32_t n = (layer_to - l < layers_per_launch) ? layer_to - l : layers_per_launch;
        dim3 grid(bx, b.n, n * planes_per_layer);
        if (elem_f16)
            kv_zero_rows<uint16_t><<<grid, 256, 0, stream>>>(static_cast<uint16_t *>(pool_base), g,
                                                             l, b);
        else
            kv_zero_rows<float><<<grid, 256, 0, stream>>>(static_cast<float *>(pool_base), g, l, b);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// ---------------------------------------------------------------------------- restore
// Gather from [row][kv_head][d] sources (possibly pinned host memory, read in place) into
// the planes. Row-major planes: thread = one 16-byte source vector, a wave covers 1 KiB
// of contiguous source. grid = (blocks, side, layer entry).
template <typename S, typename D>
__global__ __launch_bounds__(256) void kv_restore_rows(D *__restrict__ pool_base, PoolGeom g,
                                                       RestoreBatch b, uint32_t sides_from) {
    constexpr int VEC = 16 / sizeof(S);
    const RestoreLayer L = b.layer[blockIdx.z];
    const uint32_t side = sides_from + blockIdx.y;
    const uint32_t chunks = g.head_dim / VEC;
    const uint64_t total = uint64_t(L.rows) * g.kv_heads * chunks;
    const S *src = static_cast<const S *>(side ? L.values : L.keys);
    D *dst_side = pool_base + L.layer * g.layer_stride + b.slot * g.slot_stride +
                  side * g.side_stride;
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < total; i += gridDim.x * 256ull) {
        const uint32_t row = uint32_t(i / (g.kv_heads * chunks));
        const uint32_t rem = uint32_t(i % (g.kv_heads * chunks));
        const uint32_t head = rem / chunks;
        const uint32_t d = (rem % chunks) * VEC;
        // side 1 only gets here with row-major planes; VEC (4 or 8) channels stay inside one
        // 8-channel piece of the blocked key layout.
        D *dst = dst_side + head * g.head_stride +
                 (side ? uint64_t(L.first_row + row) * g.head_dim + d
                       : k_offset(g, L.first_row + row, d));
        if constexpr (sizeof(S) == 4) {
            store4(dst, *reinterpret_cast<const float4 *>(src + i * VEC));
        } else {
            *reinterpret_cast<uint4 *>(dst) = *reinterpret_cast<const uint4 *>(src + i * VEC);
        }
    }
}

// Blocked planes, both sides in one launch: a workgroup moves one (32-row block, kv head) of
// keys and of values. The 32 source rows of each side are read coalesced into LDS (converted):
// whole 256- or 512-byte runs, which is what a source in pinned host memory needs to keep the
// host link at its rate (a variant whose threads fetch their key piece directly, 64-byte
// runs, gains 4 % from HBM and loses 12 % over the link). The key block then leaves as the
// 8 KiB of 16-byte pieces the MFMA kernels read (piece (tile t, channel chunk c, row i) at
// ((t*(D/8) + c)*16 + i)*8, k_offset above) and the value block transposed, every thread
// storing 16 contiguous bytes. Requires first_row % 32 == 0; rows of the last block past the source are written as
// zeros, which is what a fresh layer holds there. grid = (row blocks, kv_heads, layer entry).
// HD = the head_dim the index arithmetic is compiled for (shifts instead of divisions: at
// 128 bytes moved per thread the divisions by a run-time head_dim cost more than the copy);
// 0 = any head_dim, read from the geometry.
template <typename S, int HD>
__global__ __launch_bounds__(256) void kv_restore_blocked(uint16_t *__restrict__ pool_base,
                                                          PoolGeom g, RestoreBatch b) {
    // Every byte is read once and written once: loads and stores carry the streaming hint
    // (3.83 -> 4.03 TB/s on the 48-layer snapshot).
    typedef float f4v __attribute__((ext_vector_type(4)));
    typedef uint32_t u4v __attribute__((ext_vector_type(4)));
    extern __shared__ uint16_t tile[];  // [2][32][head_dim + 8]: keys, values
    const RestoreLayer L = b.layer[blockIdx.z];
    const uint32_t head = blockIdx.y;
    const uint32_t D = HD ? uint32_t(HD) : g.head_dim;
    const uint32_t stride = D + 8;
    uint16_t *ktile = tile, *vtile = tile + kVBlock * stride;
    uint16_t *kplane = pool_base + L.layer * g.layer_stride + b.slot * g.slot_stride +
                       head * g.head_stride;
    uint16_t *vplane = kplane + g.side_stride;
    const uint32_t nblocks = (L.rows + kVBlock - 1) / kVBlock;
    constexpr int VEC = 16 / sizeof(S);
    const uint32_t chunks = D / VEC;
    for (uint32_t blk = blockIdx.x; blk < nblocks; blk += gridDim.x) {
        const uint32_t row0 = blk * kVBlock;
        for (uint32_t i = threadIdx.x; i < 2 * kVBlock * chunks; i += 256) {
            const uint32_t side = i / (kVBlock * chunks), j = i % (kVBlock * chunks);
            const uint32_t r = j / chunks, c = (j % chunks) * VEC;
            uint16_t *t = (side ? vtile : ktile) + r * stride + c;
            if (row0 + r < L.rows) {
                const S *s = static_cast<const S *>(side ? L.values : L.keys) +
                             (uint64_t(row0 + r) * g.kv_heads + head) * D + c;
                if constexpr (sizeof(S) == 4) {
                    const f4v q = __builtin_nontemporal_load(reinterpret_cast<const f4v *>(s));
                    store4(t, make_float4(q[0], q[1], q[2], q[3]));
                } else {
                    *reinterpret_cast<u4v *>(t) = __builtin_nontemporal_load(reinterpret_cast<const u4v *>(s));
                }
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) t[e] = 0;
            }
        }
        __syncthreads();
        const uint64_t block_at = uint64_t(L.first_row / kVBlock + blk) * (kVBlock * D);
        for (uint32_t piece = threadIdx.x; piece < kVBlock * (D / 8); piece += 256) {
            const uint32_t i = piece % 16, tc = piece / 16, c = tc % (D / 8), t = tc / (D / 8);
            const uint32_t key = (i >> 2) * 8 + t * 4 + (i & 3);
            __builtin_nontemporal_store(*reinterpret_cast<const u4v *>(ktile + key * stride + c * 8),
                                        reinterpret_cast<u4v *>(kplane + block_at + uint64_t(piece) * 8));
        }
        for (uint32_t i = threadIdx.x; i < D * (kVBlock / 8); i += 256) {
            const uint32_t d = i / (kVBlock / 8), r8 = (i % (kVBlock / 8)) * 8;
            uint16_t v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = vtile[(r8 + e) * stride + d];
            uint4 packed;
            packed.x = v[0] | (uint32_t(v[1]) << 16);
            packed.y = v[2] | (uint32_t(v[3]) << 16);
            packed.z = v[4] | (uint32_t(v[5]) << 16);
            packed.w = v[6] | (uint32_t(v[7]) << 16);
            __builtin_nontemporal_store(u4v{packed.x, packed.y, packed.z, packed.w},
                                        reinterpret_cast<u4v *>(vplane + block_at + d * kVBlock + r8));
        }
        __syncthreads();
    }
}

// Element-wise fallback for head dims or alignments the vector paths cannot take.
template <typename S, typename D>
__global__ __launch_bounds__(256) void kv_restore_scalar(D *__restrict__ pool_base, PoolGeom g,
                                                         RestoreBatch b) {
    const RestoreLayer L = b.layer[blockIdx.z];
    const uint32_t side = blockIdx.y;
    const uint64_t total = uint64_t(L.rows) * g.kv_heads * g.head_dim;
    const S *src = static_cast<const S *>(side ? L.values : L.keys);
    D *dst_side = pool_base + L.layer * g.layer_stride + b.slot * g.slot_stride +
                  side * g.side_stride;
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < total; i += gridDim.x * 256ull) {
        const uint32_t row = uint32_t(i / (g.kv_heads * g.head_dim));
        const uint32_t rem = uint32_t(i % (g.kv_heads * g.head_dim));
        const uint32_t head = rem / g.head_dim;
        const uint32_t d = rem % g.head_dim;
        store1(dst_side + head * g.head_stride + kv_offset(g, side, L.first_row + row, d), src[i]);
    }
}

hipError_t launch_restore(void *pool_base, int dst_f16, int src_f16, const PoolGeom &g,
                          const RestoreBatch &b, hipStream_t stream) {
    if (b.n == 0 || b.max_rows == 0) return hipSuccess;
    bool aligned = true, block_aligned = true;
    for (uint32_t i = 0; i < b.n; ++i) {
        aligned = aligned && (reinterpret_cast<uintptr_t>(b.layer[i].keys) % 16 == 0) &&
                  (reinterpret_cast<uintptr_t>(b.layer[i].values) % 16 == 0);
        block_aligned = block_aligned && (b.layer[i].first_row % kVBlock == 0);
    }
    const uint32_t vec = src_f16 ? 8 : 4;
    const bool use_vec = aligned && (g.head_dim % vec == 0);
    if (!use_vec || (g.v_block != 0 && !block_aligned)) {
        const uint64_t per_layer = uint64_t(b.max_rows) * g.kv_heads * g.head_dim;
        uint32_t bx = uint32_t((per_layer + 255) / 256);
        if (bx > 2048) bx = 2048;
        dim3 grid(bx, 2, b.n);
        if (src_f16)
            kv_restore_scalar<uint16_t, uint16_t><<<grid, 256, 0, stream>>>(
                static_cast<uint16_t *>(pool_base), g, b);
        else if (dst_f16)
            kv_restore_scalar<float, uint16_t><<<grid, 256, 0, stream>>>(
                static_cast<uint16_t *>(pool_base), g, b);
        else
            kv_restore_scalar<float, float><<<grid, 256, 0, stream>>>(
                static_cast<float *>(pool_base), g, b);
        return hipGetLastError();
    }
    if (g.v_block != 0) {  // blocked planes: keys and values of a block in one workgroup
        uint32_t nblocks = (b.max_rows + kVBlock - 1) / kVBlock;
        if (nblocks > 2048) nblocks = 2048;
        dim3 grid(nblocks, g.kv_heads, b.n);
        const size_t lds = size_t(2) * kVBlock * (g.head_dim + 8) * sizeof(uint16_t);
        uint16_t *base = static_cast<uint16_t *>(pool_base);
        if (g.head_dim == 128 && src_f16)
            kv_restore_blocked<uint16_t, 128><<<grid, 256, lds, stream>>>(base, g, b);
        else if (g.head_dim == 128)
            kv_restore_blocked<float, 128><<<grid, 256, lds, stream>>>(base, g, b);
        else if (src_f16)
            kv_restore_blocked<uint16_t, 0><<<grid, 256, lds, stream>>>(base, g, b);
        else
            kv_restore_blocked<float, 0><<<grid, 256, lds, stream>>>(base, g, b);
        return hipGetLastError();
    }
    const uint64_t per_layer = uint64_t(b.max_rows) * g.kv_heads * (g.head_dim / vec);
    uint32_t bx = uint32_t((per_layer + 255) / 256);
    if (bx > 2048) bx = 2048;
    dim3 grid(bx, 2, b.n);
    if (src_f16)
        kv_restore_rows<uint16_t, uint16_t><<<grid, 256, 0, stream>>>(
            static_cast<uint16_t *>(pool_base), g, b, 0);
    else if (dst_f16)
        kv_restore_rows<float, uint16_t><<<grid, 256, 0, stream>>>(
            static_cast<uint16_t *>(pool_base), g, b, 0);
    else
        kv_restore_rows<float, float><<<grid, 256, 0, stream>>>(static_cast<float *>(pool_base), g,
                                                               b, 0);
    return hipGetLastError();
}

// --------------------------------------------------------------------------- readback
// planes -> [row][kv_head][d], one element per thread (readback is a test and capture
// path, not a token-loop path).
template <typename T>
__global__ __launch_bounds__(256) void kv_read_rows(const T *__restrict__ layer_base, PoolGeom g,
                                                    uint32_t slot, uint32_t first_row,
                                                    uint32_t rows, uint32_t ring,
                                                    T *__restrict__ keys_out,
                                                    T *__restrict__ values_out) {
    const uint32_t side = blockIdx.y;
    T *out = side ? values_out : keys_out;
    if (out == nullptr) return;
    const uint64_t total = uint64_t(rows) * g.kv_heads * g.head_dim;
    const T *src_side = layer_base + slot * g.slot_stride + side * g.side_stride;
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < total; i += gridDim.x * 256ull) {
        const uint32_t row = uint32_t(i / (g.kv_heads * g.head_dim));
        const uint32_t rem = uint32_t(i % (g.kv_heads * g.head_dim));
        const uint32_t head = rem / g.head_dim;
        const uint32_t d = rem % g.head_dim;
        const uint32_t srow = ring ? (first_row + row) % ring : first_row + row;
        out[i] = src_side[head * g.head_stride + kv_offset(g, side, srow, d)];
    }
}

// ------------------------------------------------------- ring rows aside and back
// One element per thread and step: a checkpoint deeper than the headroom is taken once per
// speculative round at most and moves a few MB.
template <typename T, bool TO_RING>
__global__ __launch_bounds__(256) void kv_ring_rows_kernel(T *__restrict__ pool_base_w, PoolGeom g,
                                                           RingRowsBatch b, T *__restrict__ saved) {
    const RingRowsLayer L = b.layer[blockIdx.z];
    const uint32_t side = blockIdx.y;
    const uint32_t row_elems = g.kv_heads * g.head_dim;
    const uint64_t total = uint64_t(L.rows) * row_elems;
    T *plane_side = pool_base_w + L.layer * g.layer_stride + b.slot * g.slot_stride +
                    side * g.side_stride;
    T *buf = saved + L.saved_off + (uint64_t(side) * L.saved_rows + L.saved_row0) * row_elems;
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < total; i += gridDim.x * 256ull) {
        const uint32_t row = uint32_t(i / row_elems), rem = uint32_t(i % row_elems);
        const uint32_t head = rem / g.head_dim, d = rem % g.head_dim;
        const uint32_t srow = (L.pos0 + row) % L.ring;
        T *at = plane_side + head * g.head_stride + kv_offset(g, side, srow, d);
        if (TO_RING)
            *at = buf[i];
        else
            buf[i] = *at;
    }
}

hipError_t launch_ring_rows(void *pool_base_w, int elem_f16, const PoolGeom &gw,
                            const RingRowsBatch &b, void *saved, bool to_ring, hipStream_t stream) {
    if (b.n == 0 || b.max_rows == 0) return hipSuccess;
    const uint64_t total = uint64_t(b.max_rows) * gw.kv_heads * gw.head_dim;
    uint32_t bx = uint32_t((total + 255) / 256);
    if (bx > 1024) bx = 1024;
    dim3 grid(bx, 2, b.n);
#define ITAK_RING_ROWS(T, TO)                                                                  \
    kv_ring_rows_kernel<T, TO><<<grid, 256, 0, stream>>>(static_cast<T *>(pool_base_w), gw, b, \
                                                         static_cast<T *>(saved))
    if (elem_f16) {
        if (to_ring) ITAK_RING_ROWS(uint16_t, true); else ITAK_RING_ROWS(uint16_t, false);
    } else {
        if (to_ring) ITAK_RING_ROWS(float, true); else ITAK_RING_ROWS(float, false);
    }
#undef ITAK_RING_ROWS
    return hipGetLastError();
}

hipError_t launch_read_rows(const void *layer_base, int elem_f16, const PoolGeom &g, uint32_t slot,
                            uint32_t first_row, uint32_t rows, uint32_t ring, void *keys_out,
                            void *values_out, hipStream_t stream) {
    if (rows == 0) return hipSuccess;
    const uint64_t total = uint64_t(rows) * g.kv_heads * g.head_dim;
    uint32_t bx = uint32_t((total + 255) / 256);
    if (bx > 4096) bx = 4096;
    dim3 grid(bx, 2, 1);
    if (elem_f16) {
        kv_read_rows<uint16_t><<<grid, 256, 0, stream>>>(
            static_cast<const uint16_t *>(layer_base), g, slot, first_row, rows, ring,
            static_cast<uint16_t *>(keys_out), static_cast<uint16_t *>(values_out));
    } else {
        kv_read_rows<float><<<grid, 256, 0, stream>>>(
            static_cast<const float *>(layer_base), g, slot, first_row, rows, ring,
            static_cast<float *>(keys_out), static_cast<float *>(values_out));
    }
    return hipGetLastError();
}

// ------------------------------------------------------------------- bare conversion
__global__ __launch_bounds__(256) void convert_f32_to_f16(const float *__restrict__ src,
                                                          uint16_t *__restrict__ dst,
                                                          uint64_t count) {
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < count; i += gridDim.x * 256ull)
        dst[i] = f32_to_f16_bits(src[i]);
}

hipError_t launch_convert_f16(const float *src, uint16_t *dst, uint64_t count, hipStream_t stream) {
    if (count == 0) return hipSuccess;
    uint64_t blocks = (count + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    convert_f32_to_f16<<<uint32_t(blocks), 256, 0, stream>>>(src, dst, count);
    return hipGetLastError();
}

// f16 -> f32 is exact for every half (crates/gguf/src/dequant.rs:12-34 is the host rule).
__global__ __launch_bounds__(256) void widen_f16_to_f32(const uint16_t *__restrict__ src,
                                                        float *__restrict__ dst, uint64_t count) {
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < count; i += gridDim.x * 256ull)
        dst[i] = static_cast<float>(__builtin_bit_cast(_Float16, src[i]));
}

hipError_t launch_widen_f16(const uint16_t *src, float *dst, uint64_t count, hipStream_t stream) {
    if (count == 0) return hipSuccess;
    uint64_t blocks = (count + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    widen_f16_to_f32<<<uint32_t(blocks), 256, 0, stream>>>(src, dst, count);
    return hipGetLastError();
}

// ------------------------------------------------- host-pointer call: in and done
// The small inputs of a host-pointer call lie packed in pinned host memory. One launch reads
// them over the host link into device memory (a copy engine's command costs more than this
// launch at 20 KB), and a one-thread launch at the end of the call's work writes the call's
// number into pinned memory, where the host is watching for it: finding out from the runtime
// that a stream has drained costs several microseconds more than seeing a word change.
__global__ __launch_bounds__(256) void stage_in_kernel(const uint4 *__restrict__ pinned,
                                                       uint4 *__restrict__ dst, uint32_t n) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i < n) dst[i] = pinned[i];
}
__global__ void signal_done_kernel(uint32_t *pinned_word, uint32_t value) {
    if (threadIdx.x == 0) {
        __hip_atomic_store(pinned_word, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}
hipError_t launch_stage_in(const void *pinned, void *dst, uint64_t bytes, hipStream_t stream) {
    const uint32_t n = uint32_t((bytes + 15) / 16);
    if (n == 0) return hipSuccess;
    stage_in_kernel<<<(n + 255) / 256, 256, 0, stream>>>(static_cast<const uint4 *>(pinned),
                                                         static_cast<uint4 *>(dst), n);
    return hipGetLastError();
}
hipError_t launch_signal_done(uint32_t *pinned_word, uint32_t value, hipStream_t stream) {
    signal_done_kernel<<<1, 64, 0, stream>>>(pinned_word, value);
    return hipGetLastError();
}

// ------------------------------------------------------------- word fill
// Sets 64-bit words to one value: the empty pattern of the split-K exchange buffer. A kernel,
// not a memset, so that a stream under capture can carry it.
__global__ __launch_bounds__(256) void fill_words_kernel(unsigned long long *dst, uint64_t n,
                                                         unsigned long long value) {
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < n; i += gridDim.x * 256ull)
        dst[i] = value;
}
hipError_t launch_fill_words(unsigned long long *dst, uint64_t count, unsigned long long value,
                             hipStream_t stream) {
    if (count == 0) return hipSuccess;
    uint64_t blocks = (count + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    fill_words_kernel<<<uint32_t(blocks), 256, 0, stream>>>(dst, count, value);
    return hipGetLastError();
}

// ------------------------------------------------------------- measurement aids
// A plain streaming copy of known size (the yardstick the FETCH_SIZE / WRITE_SIZE counters
// are scaled by) and an empty kernel (the per-launch floor of a stream of dependent
// launches).
__global__ __launch_bounds__(256) void probe_copy_kernel(const uint4 *__restrict__ src,
                                                         uint4 *__restrict__ dst, uint64_t n) {
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < n; i += gridDim.x * 256ull)
        dst[i] = src[i];
}

// A plain streaming read of known size: every 16 bytes fetched once, four loads in flight per
// thread, nothing written (the read half of what the attention kernels of a decode step do).
typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void probe_read_kernel(const probe_u32x4 *__restrict__ src, uint64_t n,
                                                         uint32_t *sink) {
    const uint64_t stride = gridDim.x * 256ull;
    probe_u32x4 acc = {0, 0, 0, 0};
    uint64_t i = blockIdx.x * 256ull + threadIdx.x;
    for (; i + 3 * stride < n; i += 4 * stride) {
        const probe_u32x4 a = __builtin_nontemporal_load(src + i), b = __builtin_nontemporal_load(src + i + stride);
        const probe_u32x4 c = __builtin_nontemporal_load(src + i + 2 * stride),
                          d = __builtin_nontemporal_load(src + i + 3 * stride);
        acc ^= a ^ b ^ c ^ d;
    }
    for (; i < n; i += stride) acc ^= __builtin_nontemporal_load(src + i);
    // (Never true for the buffers the probe is given; it keeps the loads alive.)
    if (sink != nullptr && (acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) *sink = acc[0];
}

__global__ void probe_empty_kernel(uint32_t *sink) {
    if (sink == nullptr) return;
    if (threadIdx.x == 0xffffffffu) *sink = 0;
}

hipError_t launch_probe_copy(const void *src, void *dst, uint64_t bytes, hipStream_t stream) {
    const uint64_t n = bytes / 16;
    if (n == 0) return hipSuccess;
    uint64_t blocks = (n + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    probe_copy_kernel<<<uint32_t(blocks), 256, 0, stream>>>(static_cast<const uint4 *>(src),
                                                            static_cast<uint4 *>(dst), n);
    return hipGetLastError();
}

hipError_t launch_probe_read(const void *src, uint64_t bytes, hipStream_t stream) {
    const uint64_t n = bytes / 16;
    if (n == 0) return hipSuccess;
    uint64_t blocks = (n + 1023) / 1024;
    if (blocks > 8192) blocks = 8192;
    probe_read_kernel<<<uint32_t(blocks), 256, 0, stream>>>(static_cast<const probe_u32x4 *>(src), n, nullptr);
    return hipGetLastError();
}

hipError_t launch_probe_empty(hipStream_t stream) {
    probe_empty_kernel<<<1, 64, 0, stream>>>(nullptr);
    return hipGetLastError();
}

// What the matrix pipe sustains by itself: `iters` trips of 32 v_mfma_f32_16x16x32_f16 into 16
// accumulators (two in a row per accumulator, the pattern of the block kernel's P.V), operands
// held in registers, two wavefronts a SIMD on every compute unit. RANDOM fills the operands
// with pseudo-random halves in (-1, 1), else with one constant: the clock the chip holds under
// the instruction depends on how many operand bits change from one product to the next, and so
// does what "the peak" is for data like a model's. clocks[0..1] receive the shader clock's and
// the 100 MHz constant clock's ticks over the loop of workgroup 0 (their ratio is the clock).
typedef _Float16 probe_half8 __attribute__((ext_vector_type(8)));
typedef float probe_floatx4 __attribute__((ext_vector_type(4)));
template <bool RANDOM>
__global__ __launch_bounds__(256, 2) void probe_mfma_kernel(uint32_t iters, unsigned long long *clocks,
                                                            float *sink) {
    const uint32_t tid = threadIdx.x;
    probe_half8 a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t h = (tid * 131u + blockIdx.x * 977u + i * 17u + e) * 2654435761u;
            a[i][e] = RANDOM ? (_Float16)(float((h >> 16) & 1023) / 512.0f - 1.0f) : (_Float16)0.0625f;
            b[i][e] = RANDOM ? (_Float16)(0.2f * (float((h >> 6) & 1023) / 512.0f - 1.0f)) : (_Float16)0.0625f;
        }
    probe_floatx4 c[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) c[i] = probe_floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    const unsigned long long c0 = clock64(), w0 = wall_clock64();
    for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            c[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i & 7], b[(i + 1) & 7], c[i], 0, 0, 0);
            c[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[(i + 3) & 7], b[i & 7], c[i], 0, 0, 0);
        }
        if ((it & 1023u) == 1023u) {  // the sums stay in range however long the loop
#pragma unroll
            for (int i = 0; i < 16; ++i) c[i] *= 0.001f;
        }
    }
    if (clocks != nullptr && blockIdx.x == 0 && tid == 0) {
        clocks[0] = clock64() - c0;
        clocks[1] = wall_clock64() - w0;
    }
    probe_floatx4 acc = probe_floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < 16; ++i) acc += c[i];
    // (Never true; it keeps the products alive.)
    if (sink != nullptr && acc[0] == 12345.678f) sink[blockIdx.x * 256 + tid] = acc[1] + acc[2] + acc[3];
}

hipError_t launch_probe_mfma(bool random_operands, uint32_t iters, unsigned long long *clocks,
                             uint32_t *workgroups, hipStream_t stream) {
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        (void)hipGetLastError();
    const uint32_t grid = 2u * uint32_t(cus > 0 ? cus : 256);
    if (workgroups) *workgroups = grid;
    if (random_operands)
        probe_mfma_kernel<true><<<grid, 256, 0, stream>>>(iters, clocks, nullptr);
    else
        probe_mfma_kernel<false><<<grid, 256, 0, stream>>>(iters, clocks, nullptr);
    return hipGetLastError();
}

}  // namespace itak
