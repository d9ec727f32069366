// The block kernel's host side: which launches it takes, their plan, and the head_dim 128
// instantiations (attn_prefill_f16_kernel.h has the kernel).
#include "attn_prefill_f16_kernel.h"

// Timeline marks of attn_prefill_f16_kernel: 0 first instruction, 1 addresses known, 2 first
// blocks and Q requested, 3 Q converted (it has arrived), 4 first block multiplied, 5 last block
// multiplied, 6 output or partials issued, 11 all done; of the first block: 7 its loads have
// landed, 8 past the barrier, 9 new rows written over it.
ITAK_TIMELINE_READER(itak_timeline_read_prefill)

namespace itak {

// A launch may bring its items' new rows along (AttnParams::k_new / v_new) when it takes the
// one-tile form and no item has more than kFuseRows rows.
bool attn_prefill_f16_appends(const PoolGeom &g, uint32_t group, uint32_t most_rows,
                              uint32_t most_blocks) {
    return attn_prefill_f16_supports(g, group) && most_rows <= uint32_t(fuse_rows(int(g.head_dim))) &&
           most_rows * padded_group(group) <= 512 && most_blocks <= kOneTileBlocks;
}

bool attn_prefill_f16_supports(const PoolGeom &g, uint32_t group) {
    return g.v_block == kVBlock &&
           (g.head_dim == 64 || g.head_dim == 96 || g.head_dim == 128 || g.head_dim == 256) &&
           group >= 1 && group <= 16;
}

// Up to 64 query vectors per KV head (speculative blocks) take one 16-vector tile per
// wavefront, so that all four wavefronts of the workgroup have columns; more take two.
// So do blocks of up to 512 vectors over at most kOneTileBlocks key blocks (a draft tree of 16
// to 32 tokens, or a 64-row chunk, at a context up to 16384): the launch has to split the
// context anyway, with twice the row tiles it needs half the splits, half the partials to
// write and merge, and the one-tile form appends the block's rows itself (measured per layer,
// one tile and its own append against two tiles behind an append launch: context 8192, 9 / 16 /
// 32 / 64 rows 19.7 / 22.6 / 25.9 / 30.3 -> 16.6 / 19.2 / 20.9 / 30.2 us; context 16384, 23.1 /
// 25.6 / 30.2 / 37.6 -> 20.3 / 21.1 / 26.2 / 36.5; at context 30720 the second pass over the
// keys costs more than it saves: 26.7 -> 29.0 and 38.4 -> 45.2 us for 9 and 32 rows).
static int tiles_for(const AttnBatch &b, uint32_t group) {
    uint32_t nvec = 0, nblocks = 0;
    for (uint32_t i = 0; i < b.n; ++i) {
        nvec = std::max(nvec, b.item[i].rows * padded_group(group));
        nblocks = std::max(nblocks, item_block_count(b.item[i]));
    }
    if (b.two_halves) return kMaxTiles;  // the form with the registers for the second halves
    if (nvec <= uint32_t(kWaves * 16)) return 1;
    return nvec <= 512 && nblocks <= kOneTileBlocks ? 1 : kMaxTiles;
}

// Fills splits / keys_per_split / block0 / ws0 for a batch (slot, rows, pos0, q_row0, kv_len
// already set) and returns the number of partials the launch will write. A unit is one
// (row tile, KV head) of an item; the context of every unit is cut into equal runs of at
// most T blocks, T the smallest run length for which the launch has at least two
// workgroups per compute unit's worth of work units, and never shorter than 8 blocks
// (a workgroup needs that many to amortise filling its load pipeline).
// Key blocks one (row tile, KV head) unit of an item walks at most: everything up to the
// item's end on a global layer, the window of its first row plus its own rows on a windowed
// one (the kernel starts each workgroup at its own first visible block).
static uint32_t unit_block_count(const AttnItem &it, uint32_t rows_per_group, uint32_t window) {
    const uint32_t all = item_block_count(it);
    if (window == 0) return all;
    const uint32_t span = window + std::min(rows_per_group, it.rows) + 2 * kBlockKeys - 2;
    return std::min(all, span / kBlockKeys);
}

uint32_t attn_prefill_f16_plan(const PoolGeom &g, AttnBatch &b, uint32_t group, uint32_t q_heads,
                               uint32_t window, bool appends) {
    const uint32_t rows_per_group = uint32_t(tiles_for(b, group) * kWaves * 16) / padded_group(group);
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        (void)hipGetLastError();
    const uint64_t per_cu = uint64_t(cus > 0 ? cus : 256);
    uint64_t unit_blocks = 0;
    for (uint32_t i = 0; i < b.n; ++i) {
        const uint64_t units = uint64_t(g.kv_heads) * ((b.item[i].rows + rows_per_group - 1) / rows_per_group);
        unit_blocks += units * unit_block_count(b.item[i], rows_per_group, window);
    }
    // Two workgroups per compute unit hide each other's waits when their runs are long. When
    // the whole launch is 8 to 40 blocks per compute unit, a run is over before that pays:
    // then one workgroup per compute unit with twice the blocks in flight (the deep ring), so
    // that its handful of blocks arrive behind one another after a single memory latency
    // (measured: 64 rows at context 4096 30.8 -> 27.1 us, 256 rows 52.6 -> 48.4 us, 16 rows at
    // context 30720 36.3 -> 31.6 us; above the range it loses, below it nothing changes).
    // (Eight stages of head_dim 256 do not fit the LDS.)
    const bool deep = unit_blocks >= 8 * per_cu && unit_blocks <= 40 * per_cu && g.head_dim <= 128;
    b.deep_ring = deep ? 1 : 0;
    b.fold_units = 0;
    const uint64_t target = deep ? per_cu : 2 * per_cu;
    uint64_t T = std::max<uint64_t>((unit_blocks + target - 1) / target, 8);
    // Rounding the splits up per unit can leave a few workgroups more than the device takes at
    // once, and those few run alone in a second round (96 rows at context 4096: 264 workgroups
    // on 256 compute units, 38.5 us where 128 rows take 34.4): lengthen the runs until the
    // launch fits, when the first estimate says it nearly does (96 / 160 / 192 / 384 rows at
    // context 4096: 38.5 / 48.1 / 51.9 / 63.0 -> 29.2 / 36.6 / 38.0 / 52.0 us).
    // (Never by more than half: when the units alone outnumber the target, no run length fits,
    // and a search to the end would leave every item unsplit, the decode rows of a mixed batch
    // walking their whole context in one workgroup.)
    const uint64_t T0 = T;
    for (; T < unit_blocks; ++T) {
        uint64_t groups = 0;
        for (uint32_t i = 0; i < b.n; ++i) {
            const uint64_t nb = unit_block_count(b.item[i], rows_per_group, window);
            const uint64_t units = uint64_t(g.kv_heads) * ((b.item[i].rows + rows_per_group - 1) / rows_per_group);
            groups += units * std::max<uint64_t>((nb + T - 1) / T, 1);
        }
        if (groups <= target || groups > target + target / 4) break;
        if (T >= T0 + T0 / 2) {
            T = T0;
            break;
        }
    }
    uint32_t block0 = 0, ws0 = 0;
    for (uint32_t i = 0; i < b.n; ++i) {
        AttnItem &it = b.item[i];
        const uint32_t nblocks = unit_block_count(it, rows_per_group, window);
        const uint32_t units = g.kv_heads * ((it.rows + rows_per_group - 1) / rows_per_group);
        uint32_t splits = std::max<uint32_t>(uint32_t((nblocks + T - 1) / T), 1);
        // A short context is not worth splitting once the row tiles alone keep a good part of
        // the device busy: the partials and the merge launch cost more than the blocks saved
        // (no prefix, 384 / 512 / 768 rows: 31.0 / 35.4 / 49.1 -> 20.7 / 25.4 / 31.6 us per
        // layer; 192 / 256 / 512 rows over a 512-row prefix: 29.2 / 31.7 / 40.4 -> 25.4 / 26.6 /
        // 35.0; with 32 units, a 64-row chunk, the splits are what fills the device and stay).
        if (nblocks < 40 && units >= 48) splits = 1;
        // Nor is any context, once the units give most compute units their two workgroups
        // (384 units, 1536 rows: no prefix 83.6 -> 49.3 us, over 2048 rows 138 -> 100, over
        // 8192 290 -> 262, over 30720 829 -> 792), or each its one on a context under 128
        // blocks (256 units over 2048 rows: 83.8 -> 77.4; from 160 blocks on the split form,
        // two workgroups of half the run on every compute unit, is the faster one).
        if (uint64_t(units) * 2 >= 3 * per_cu || (units >= per_cu && nblocks < 128)) splits = 1;
        uint32_t bps = std::max<uint32_t>((nblocks + splits - 1) / splits, 1);
        // A launch that appends its own rows: the workgroups of a unit's last split convert
        // the new rows and write them over their last blocks, about a block's time for every
        // eight rows, and the launch ends with them; their run is made that much shorter and
        // the other splits share the difference.
        if (appends && splits > 1) {
            const uint32_t extra = std::min<uint32_t>(it.rows / 8 + 1, bps / 2);
            const uint32_t longer = (nblocks + extra + splits - 1) / splits;
            if (uint64_t(splits - 1) * longer < nblocks) bps = longer;
        }
        splits = std::max<uint32_t>((nblocks + bps - 1) / bps, 1);
        it.splits = splits;
        it.keys_per_split = bps * kBlockKeys;
        it.splits_magic = 0;
        it.block0 = block0;
        it.ws0 = ws0;
        block0 += units * splits;
        if (splits > 1) ws0 += it.rows * q_heads * splits;
    }
    b.total_blocks = block0;
    b.rows_per_block = rows_per_group;
    // One unsplit item whose row tiles see different numbers of blocks (no window) and whose
    // workgroups are all resident from the start, two to a compute unit: fold the second run
    // (see the kernel; 2048 rows without a prefix 64.9 -> 61.6 us per layer). With more runs
    // the later workgroups go wherever one ends, which balances better unfolded (4096 and 8192
    // rows measured 1 to 3 % slower folded).
    if (b.n == 1 && b.item[0].splits == 1 && window == 0 && !deep && block0 > per_cu &&
        block0 <= 2 * per_cu && per_cu % g.kv_heads == 0)
        b.fold_units = uint32_t(per_cu);
    return ws0;
}

hipError_t launch_attn_prefill_f16(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                   hipStream_t stream) {
    if (b.total_blocks == 0) return hipSuccess;
    const bool one = tiles_for(b, p.group) == 1;
    if (p.k_new && !one) return hipErrorInvalidValue;  // only the one-tile form appends
    if (b.two_halves) return launch_attn_prefill_f16_qlo(p, b, total_partials, stream);
    if (p.g.head_dim == 128) return launch_prefill_head_dim<128, true>(p, b, total_partials, one, stream);
    return launch_attn_prefill_f16_dims(p, b, total_partials, one, stream);
}

}  // namespace itak
