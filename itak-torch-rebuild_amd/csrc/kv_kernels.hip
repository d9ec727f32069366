// KV row movement kernels for gfx950: append (f32 -> f16 RNE or f32 copy), zero fill of
// dropped rows, snapshot gather-restore and row readback. All of them are pure byte
// movement bound by HBM (or, for a pinned-host source, by the host link): every thread
// moves one 16-byte source vector and the grid covers the rows exactly.
#include "internal.h"

#include <hip/hip_fp16.h>

namespace itak {

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

__device__ __forceinline__ void store4(float *dst, const float4 &v) {
    *reinterpret_cast<float4 *>(dst) = v;
}
__device__ __forceinline__ void store4(uint16_t *dst, const float4 &v) {
    uint2 packed;
    packed.x = uint32_t(f32_to_f16_bits(v.x)) | (uint32_t(f32_to_f16_bits(v.y)) << 16);
    packed.y = uint32_t(f32_to_f16_bits(v.z)) | (uint32_t(f32_to_f16_bits(v.w)) << 16);
    *reinterpret_cast<uint2 *>(dst) = packed;
}

// ---------------------------------------------------------------------------- append
// Thread = one (row, side, kv head, 4-element chunk). head_dim % 4 == 0 takes the vector
// path; other head dims go through the scalar kernel below.
template <typename T>
__global__ __launch_bounds__(256) void kv_append_vec4(T *__restrict__ layer_base, PoolGeom g,
                                                      AppendBatch b,
                                                      const float *__restrict__ k_src,
                                                      const float *__restrict__ v_src) {
    const uint32_t chunks = g.head_dim >> 2;
    const uint64_t per_row = 2ull * g.kv_heads * chunks;
    const uint64_t idx = blockIdx.x * 256ull + threadIdx.x;
    if (idx >= per_row * b.total_rows) return;
    uint32_t row = uint32_t(idx / per_row);
    uint32_t rem = uint32_t(idx % per_row);
    const uint32_t side = rem / (g.kv_heads * chunks);
    rem -= side * g.kv_heads * chunks;
    const uint32_t head = rem / chunks;
    const uint32_t d = (rem % chunks) << 2;
    uint32_t it = 0;
    while (it + 1 < b.n && row >= b.item[it + 1].src_row0) ++it;
    const AppendItem item = b.item[it];
    const uint32_t local = row - item.src_row0;
    const float *src = (side ? v_src : k_src) + (uint64_t(row) * g.kv_heads + head) * g.head_dim + d;
    const float4 v = *reinterpret_cast<const float4 *>(src);
    T *dst = layer_base + item.slot * g.slot_stride + side * g.side_stride +
             head * g.head_stride + uint64_t(item.pos0 + local) * g.head_dim + d;
    store4(dst, v);
}

__device__ __forceinline__ void store1(float *dst, float v) { *dst = v; }
__device__ __forceinline__ void store1(uint16_t *dst, float v) { *dst = f32_to_f16_bits(v); }

template <typename T>
__global__ __launch_bounds__(256) void kv_append_scalar(T *__restrict__ layer_base, PoolGeom g,
                                                        AppendBatch b,
                                                        const float *__restrict__ k_src,
                                                        const float *__restrict__ v_src) {
    const uint64_t per_row = 2ull * g.kv_heads * g.head_dim;
    const uint64_t idx = blockIdx.x * 256ull + threadIdx.x;
    if (idx >= per_row * b.total_rows) return;
    uint32_t row = uint32_t(idx / per_row);
    uint32_t rem = uint32_t(idx % per_row);
    const uint32_t side = rem / (g.kv_heads * g.head_dim);
    rem -= side * g.kv_heads * g.head_dim;
    const uint32_t head = rem / g.head_dim;
    const uint32_t d = rem % g.head_dim;
    uint32_t it = 0;
    while (it + 1 < b.n && row >= b.item[it + 1].src_row0) ++it;
    const AppendItem item = b.item[it];
    const uint32_t local = row - item.src_row0;
    const float *src = (side ? v_src : k_src) + (uint64_t(row) * g.kv_heads + head) * g.head_dim + d;
    T *dst = layer_base + item.slot * g.slot_stride + side * g.side_stride +
             head * g.head_stride + uint64_t(item.pos0 + local) * g.head_dim + d;
    store1(dst, *src);
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
            kv_append_vec4<uint16_t><<<blocks, 256, 0, stream>>>(base, g, b, k_src, v_src);
        else
            kv_append_scalar<uint16_t><<<blocks, 256, 0, stream>>>(base, g, b, k_src, v_src);
    } else {
        auto *base = static_cast<float *>(layer_base);
        if (vec)
            kv_append_vec4<float><<<blocks, 256, 0, stream>>>(base, g, b, k_src, v_src);
        else
            kv_append_scalar<float><<<blocks, 256, 0, stream>>>(base, g, b, k_src, v_src);
    }
    return hipGetLastError();
}

// ------------------------------------------------------------------------- zero rows
// grid = (blocks over the widest item's bytes, item, layer*2*kv_heads planes).
__global__ __launch_bounds__(256) void kv_zero_rows(unsigned char *__restrict__ pool_base,
                                                    uint32_t elem_bytes, PoolGeom g,
                                                    uint32_t layer_from, ZeroBatch b) {
    const ZeroItem item = b.item[blockIdx.y];
    if (item.row_to <= item.row_from) return;
    const uint32_t planes_per_layer = 2 * g.kv_heads;
    const uint32_t layer = layer_from + blockIdx.z / planes_per_layer;
    const uint32_t plane = blockIdx.z % planes_per_layer;  // side*kv_heads + head
    const uint64_t row_bytes = uint64_t(g.head_dim) * elem_bytes;
    const uint64_t bytes = uint64_t(item.row_to - item.row_from) * row_bytes;
    unsigned char *dst = pool_base +
                         (layer * g.layer_stride + item.slot * g.slot_stride +
                          plane * g.head_stride + uint64_t(item.row_from) * g.head_dim) *
                             elem_bytes;
    // Row starts are multiples of head_dim*elem_bytes; use 4-byte words when that allows.
    if ((row_bytes & 3) == 0) {
        const uint64_t words = bytes >> 2;
        for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < words; i += gridDim.x * 256ull)
            reinterpret_cast<uint32_t *>(dst)[i] = 0u;
    } else {
        for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < bytes; i += gridDim.x * 256ull)
            dst[i] = 0;
    }
}

hipError_t launch_zero_rows(void *pool_base, int elem_f16, const PoolGeom &g, uint32_t layer_from,
                            uint32_t layer_to, const ZeroBatch &b, hipStream_t stream) {
    if (b.n == 0 || b.max_rows == 0 || layer_to <= layer_from) return hipSuccess;
    const uint32_t elem_bytes = elem_f16 ? 2 : 4;
    const uint64_t words = (uint64_t(b.max_rows) * g.head_dim * elem_bytes + 3) / 4;
    uint32_t bx = uint32_t((words + 255) / 256);
    if (bx > 1024) bx = 1024;
    if (bx == 0) bx = 1;
    const uint32_t planes_per_layer = 2 * g.kv_heads;
    // gridDim.z is limited to 65535: walk the layers in slices that fit.
    const uint32_t layers_per_launch = 65535 / planes_per_layer ? 65535 / planes_per_layer : 1;
    for (uint32_t l = layer_from; l < layer_to; l += layers_per_launch) {
        const uint32_t n = (layer_to - l < layers_per_launch) ? layer_to - l : layers_per_launch;
        dim3 grid(bx, b.n, n * planes_per_layer);
        kv_zero_rows<<<grid, 256, 0, stream>>>(static_cast<unsigned char *>(pool_base), elem_bytes,
                                               g, l, b);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// ---------------------------------------------------------------------------- restore
// Gather: source rows are [row][kv_head][d] (the snapshot's and the reference cache's
// layout), destination planes are per KV head. grid = (blocks over rows*kv_heads*chunks,
// side, layer entry). Sources may live in pinned host memory: each thread issues one
// 16-byte read, so a wave covers 1 KiB of contiguous source per instruction.
template <typename D>
__global__ __launch_bounds__(256) void kv_restore_from_f32(D *__restrict__ pool_base, PoolGeom g,
                                                           RestoreBatch b) {
    const RestoreLayer L = b.layer[blockIdx.z];
    const uint32_t side = blockIdx.y;
    const uint32_t chunks = g.head_dim >> 2;
    const uint64_t total = uint64_t(L.rows) * g.kv_heads * chunks;
    const float *src = static_cast<const float *>(side ? L.values : L.keys);
    D *dst_layer = pool_base + L.layer * g.layer_stride + b.slot * g.slot_stride +
                   side * g.side_stride;
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < total; i += gridDim.x * 256ull) {
        const uint32_t row = uint32_t(i / (g.kv_heads * chunks));
        const uint32_t rem = uint32_t(i % (g.kv_heads * chunks));
        const uint32_t head = rem / chunks;
        const uint32_t d = (rem % chunks) << 2;
        const float4 v = *reinterpret_cast<const float4 *>(src + i * 4);
        store4(dst_layer + head * g.head_stride + uint64_t(L.first_row + row) * g.head_dim + d, v);
    }
}

// f16 source into an f16 pool: raw 16-byte copies (8 halves), bit-exact by construction.
__global__ __launch_bounds__(256) void kv_restore_from_f16(uint16_t *__restrict__ pool_base,
                                                           PoolGeom g, RestoreBatch b) {
    const RestoreLayer L = b.layer[blockIdx.z];
    const uint32_t side = blockIdx.y;
    const uint32_t chunks = g.head_dim >> 3;
    const uint64_t total = uint64_t(L.rows) * g.kv_heads * chunks;
    const uint16_t *src = static_cast<const uint16_t *>(side ? L.values : L.keys);
    uint16_t *dst_layer = pool_base + L.layer * g.layer_stride + b.slot * g.slot_stride +
                          side * g.side_stride;
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < total; i += gridDim.x * 256ull) {
        const uint32_t row = uint32_t(i / (g.kv_heads * chunks));
        const uint32_t rem = uint32_t(i % (g.kv_heads * chunks));
        const uint32_t head = rem / chunks;
        const uint32_t d = (rem % chunks) << 3;
        const uint4 v = *reinterpret_cast<const uint4 *>(src + i * 8);
        *reinterpret_cast<uint4 *>(dst_layer + head * g.head_stride +
                                   uint64_t(L.first_row + row) * g.head_dim + d) = v;
    }
}

// Scalar fallback for head dims the vector paths cannot take.
template <typename S, typename D>
__global__ __launch_bounds__(256) void kv_restore_scalar(D *__restrict__ pool_base, PoolGeom g,
                                                         RestoreBatch b) {
    const RestoreLayer L = b.layer[blockIdx.z];
    const uint32_t side = blockIdx.y;
    const uint64_t total = uint64_t(L.rows) * g.kv_heads * g.head_dim;
    const S *src = static_cast<const S *>(side ? L.values : L.keys);
    D *dst_layer = pool_base + L.layer * g.layer_stride + b.slot * g.slot_stride +
                   side * g.side_stride;
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < total; i += gridDim.x * 256ull) {
        const uint32_t row = uint32_t(i / (g.kv_heads * g.head_dim));
        const uint32_t rem = uint32_t(i % (g.kv_heads * g.head_dim));
        const uint32_t head = rem / g.head_dim;
        const uint32_t d = rem % g.head_dim;
        D *dst = dst_layer + head * g.head_stride + uint64_t(L.first_row + row) * g.head_dim + d;
        if constexpr (sizeof(S) == sizeof(D)) {
            *dst = src[i];
        } else {
            store1(dst, src[i]);
        }
    }
}

hipError_t launch_restore(void *pool_base, int dst_f16, int src_f16, const PoolGeom &g,
                          const RestoreBatch &b, hipStream_t stream) {
    if (b.n == 0 || b.max_rows == 0) return hipSuccess;
    bool aligned = true;
    for (uint32_t i = 0; i < b.n; ++i) {
        aligned = aligned && (reinterpret_cast<uintptr_t>(b.layer[i].keys) % 16 == 0) &&
                  (reinterpret_cast<uintptr_t>(b.layer[i].values) % 16 == 0);
    }
    const uint32_t vec = src_f16 ? 8 : 4;
    const bool use_vec = aligned && (g.head_dim % vec == 0);
    const uint64_t per_layer =
        uint64_t(b.max_rows) * g.kv_heads * (use_vec ? g.head_dim / vec : g.head_dim);
    uint32_t bx = uint32_t((per_layer + 255) / 256);
    if (bx > 2048) bx = 2048;
    dim3 grid(bx, 2, b.n);
    if (src_f16) {
        auto *base = static_cast<uint16_t *>(pool_base);
        if (use_vec)
            kv_restore_from_f16<<<grid, 256, 0, stream>>>(base, g, b);
        else
            kv_restore_scalar<uint16_t, uint16_t><<<grid, 256, 0, stream>>>(base, g, b);
    } else if (dst_f16) {
        auto *base = static_cast<uint16_t *>(pool_base);
        if (use_vec)
            kv_restore_from_f32<uint16_t><<<grid, 256, 0, stream>>>(base, g, b);
        else
            kv_restore_scalar<float, uint16_t><<<grid, 256, 0, stream>>>(base, g, b);
    } else {
        auto *base = static_cast<float *>(pool_base);
        if (use_vec)
            kv_restore_from_f32<float><<<grid, 256, 0, stream>>>(base, g, b);
        else
            kv_restore_scalar<float, float><<<grid, 256, 0, stream>>>(base, g, b);
    }
    return hipGetLastError();
}

// --------------------------------------------------------------------------- readback
// planes -> [row][kv_head][d], one element per thread (readback is a test and capture
// path, not a token-loop path).
template <typename T>
__global__ __launch_bounds__(256) void kv_read_rows(const T *__restrict__ layer_base, PoolGeom g,
                                                    uint32_t slot, uint32_t first_row,
                                                    uint32_t rows, T *__restrict__ keys_out,
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
        out[i] = src_side[head * g.head_stride + uint64_t(first_row + row) * g.head_dim + d];
    }
}

hipError_t launch_read_rows(const void *layer_base, int elem_f16, const PoolGeom &g, uint32_t slot,
                            uint32_t first_row, uint32_t rows, void *keys_out, void *values_out,
                            hipStream_t stream) {
    if (rows == 0) return hipSuccess;
    const uint64_t total = uint64_t(rows) * g.kv_heads * g.head_dim;
    uint32_t bx = uint32_t((total + 255) / 256);
    if (bx > 4096) bx = 4096;
    dim3 grid(bx, 2, 1);
    if (elem_f16) {
        kv_read_rows<uint16_t><<<grid, 256, 0, stream>>>(
            static_cast<const uint16_t *>(layer_base), g, slot, first_row, rows,
            static_cast<uint16_t *>(keys_out), static_cast<uint16_t *>(values_out));
    } else {
        kv_read_rows<float><<<grid, 256, 0, stream>>>(
            static_cast<const float *>(layer_base), g, slot, first_row, rows,
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

}  // namespace itak
