// Shared declarations between the host logic (pool.hip) and the kernel files.
// Nothing here is part of the public ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace itak {

// Device layout of the KV pool, in elements of the storage type. One "plane" is the
// rows of one (layer, slot, side, kv_head): capacity x head_dim elements, contiguous,
// so a workgroup that streams one KV head reads one unbroken run of memory.
//   plane(layer, slot, side, head) =
//     layer*layer_stride + slot*slot_stride + side*side_stride + head*head_stride
// side 0 = keys, 1 = values. Key planes are row-major: row*head_dim + d. Value planes are
// row-major too unless v_block != 0: then they are stored in blocks of v_block (= 32) rows,
// each block transposed, element (row, d) at
//     (row / 32) * 32 * head_dim + d * 32 + row % 32
// so that the 8 consecutive rows an MFMA lane needs for one channel are 16 contiguous
// bytes and a wavefront's operand load covers 1 KiB of contiguous memory.
struct PoolGeom {
    uint32_t kv_heads;
    uint32_t head_dim;
    uint32_t capacity;  // rows per plane (a multiple of 32 when v_block != 0)
    uint32_t max_slots;
    uint32_t v_block;   // 0 or 32
    uint32_t pad;
    uint64_t head_stride;   // capacity * head_dim
    uint64_t side_stride;   // kv_heads * head_stride
    uint64_t slot_stride;   // 2 * side_stride
    uint64_t layer_stride;  // max_slots * slot_stride
};

constexpr uint32_t kVBlock = 32;

// Element offset of (row, d) inside a value plane.
__host__ __device__ inline uint64_t v_offset(const PoolGeom &g, uint32_t row, uint32_t d) {
    if (g.v_block == 0) return uint64_t(row) * g.head_dim + d;
    return uint64_t(row / kVBlock) * (kVBlock * g.head_dim) + uint64_t(d) * kVBlock + row % kVBlock;
}

constexpr int kMaxBatchItems = 64;

// ---- append ---------------------------------------------------------------------
struct AppendItem {
    uint32_t slot;
    uint32_t rows;
    uint32_t pos0;      // storage row of the item's first new row
    uint32_t src_row0;  // row offset of the item inside k_src / v_src
};
struct AppendBatch {
    uint32_t n;
    uint32_t total_rows;
    AppendItem item[kMaxBatchItems];
};
hipError_t launch_append(void *layer_base, int elem_f16, const PoolGeom &g, const AppendBatch &b,
                         const float *k_src, const float *v_src, hipStream_t stream);

// ---- zero fill of dropped rows (truncate scrub, slot reset) ------------------------
struct ZeroItem {
    uint32_t slot;
    uint32_t row_from;
    uint32_t row_to;  // exclusive
    uint32_t pad;
};
struct ZeroBatch {
    uint32_t n;
    uint32_t max_rows;
    ZeroItem item[kMaxBatchItems];
};
hipError_t launch_zero_rows(void *pool_base, int elem_f16, const PoolGeom &g, uint32_t layer_from,
                            uint32_t layer_to, const ZeroBatch &b, hipStream_t stream);

// ---- snapshot restore (gather from [row][kv_head][d] sources into the planes) --------
constexpr int kMaxRestoreLayers = 64;
struct RestoreLayer {
    const void *keys;
    const void *values;
    uint32_t layer;
    uint32_t rows;
    uint32_t first_row;  // destination storage row of source row 0
    uint32_t pad;
};
struct RestoreBatch {
    uint32_t n;
    uint32_t max_rows;
    uint32_t slot;
    uint32_t pad;
    RestoreLayer layer[kMaxRestoreLayers];
};
hipError_t launch_restore(void *pool_base, int dst_f16, int src_f16, const PoolGeom &g,
                          const RestoreBatch &b, hipStream_t stream);

// ---- row readback: planes -> [row][kv_head][d] ---------------------------------------
hipError_t launch_read_rows(const void *layer_base, int elem_f16, const PoolGeom &g, uint32_t slot,
                            uint32_t first_row, uint32_t rows, void *keys_out, void *values_out,
                            hipStream_t stream);

hipError_t launch_convert_f16(const float *src, uint16_t *dst, uint64_t count, hipStream_t stream);

// ---- attention ----------------------------------------------------------------------
// One item = one slot's query rows against that slot's rows of one layer. Query row r
// sits at position pos0 + r unless q_pos is given. A workgroup owns (item, row block,
// kv head, split of the key range) and writes either the final output (splits == 1) or
// a partial (m, l, acc[head_dim]) per query vector; a second, small launch merges the
// partials of each (row, Q head). Partials live in `ws`: first total_partials*head_dim
// accumulators, then total_partials (m, l) pairs; the partial of (row, head, split) of
// an item is ws0 + (row*q_heads + head)*splits + split.
struct AttnItem {
    uint32_t slot;
    uint32_t rows;
    uint32_t pos0;
    uint32_t q_row0;        // first row of the item in q / out
    uint32_t kv_len;        // stored rows visible to the item's last query row (exclusive end)
    uint32_t splits;
    uint32_t keys_per_split;
    uint32_t block0;        // first workgroup index of the item
    uint32_t ws0;           // first partial index of the item
    uint32_t pad;
};
struct AttnBatch {
    uint32_t n;
    uint32_t total_blocks;
    uint32_t rows_per_block;
    uint32_t pad;
    AttnItem item[kMaxBatchItems];
};
struct AttnParams {
    const void *layer_base;
    PoolGeom g;
    const float *q;
    float *out;
    const uint32_t *q_pos;  // optional explicit positions, [sum rows]
    float *ws;              // partials: (head_dim + 2) floats each
    uint32_t q_heads;
    uint32_t group;         // q_heads / kv_heads
    float scale;
    float softcap;
};

// Generic VALU path: f32 or f16 storage, any head_dim <= 256, group <= 64. Partials are in
// natural-log domain (combine with base2 = 0).
hipError_t launch_attn_generic(int elem_f16, const AttnParams &p, const AttnBatch &b,
                               uint32_t total_partials, hipStream_t stream);
// Query rows one workgroup of the generic kernel carries (0 = shape not supported).
uint32_t attn_generic_rows_per_block(uint32_t group, uint32_t head_dim);
// Keys per tile of the generic kernel for a head_dim.
uint32_t attn_generic_tile(uint32_t head_dim);

// MFMA split-K path: f16 pools with blocked value planes, head_dim 128, rows*group <= 64.
// Partials are in log2 domain (combine with base2 = 1).
bool attn_splitk_f16_supports(const PoolGeom &g, uint32_t group, uint32_t max_rows);
uint32_t attn_splitk_f16_plan(const PoolGeom &g, AttnBatch &b, uint32_t q_heads);
hipError_t launch_attn_splitk_f16(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                  uint32_t max_rows, hipStream_t stream);
// Merge of split partials; total_rows = query rows of the batch.
hipError_t launch_attn_combine(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                               uint32_t total_rows, int base2, hipStream_t stream);

}  // namespace itak
