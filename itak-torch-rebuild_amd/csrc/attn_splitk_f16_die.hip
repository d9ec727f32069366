// The split-K attention kernel of f16 pools at head_dim 128 (attn_splitk_f16_kernel.h) in the
// form that merges a unit's splits on the unit's own compute die: the placement plan, the
// probe that holds the device to the dealing order the plan relies on, and the launches.
//
// What the plan replaces: the merge launch behind every split-K launch (its dispatch gap, its
// own start and end, a round trip of the partials through HBM). What it gives up: a unit's
// splits run on the 32 compute units of one die instead of anywhere, so the batch must deal
// out evenly over the eight dies; batches that do not keep the ordinary plan.
//
// Semantics: gqa_attention in crates/attention/src/attention.rs:104-215 (see
// attn_splitk_f16.hip).
#include "attn_splitk_f16_kernel.h"

#include <algorithm>
#include <mutex>
#include <vector>

ITAK_TIMELINE_READER(itak_timeline_read_splitk_die)

namespace itak {

namespace {

__global__ void die_probe_kernel(uint32_t *ids) {
    if (threadIdx.x == 0) ids[blockIdx.x] = compute_die();
}

struct DeviceDies {
    int state = 0;  // 0 not probed, 1 dealt round-robin over eight dies, -1 anything else
    uint32_t cus_per_die = 0;
};
DeviceDies g_dies[64];
std::mutex g_dies_mutex;

struct DieVariant {
    int nq, waves, index;
};
// 16-vector steps with four or eight wavefronts, as the ordinary plan picks them, or 32 vectors.
DieVariant pick_die_variant(const PoolGeom &g, const AttnBatch &b, uint32_t group) {
    uint32_t nvec = 0, rows = 0;
    uint64_t blocks = 0;
    for (uint32_t i = 0; i < b.n; ++i) {
        nvec = std::max(nvec, b.item[i].rows * group);
        rows = std::max(rows, b.item[i].rows);
        blocks += uint64_t(g.kv_heads) * item_block_count(b.item[i]);
    }
    if (nvec > 16) return {2, 4, 2};
    return blocks >= 4096 && rows == 1 ? DieVariant{1, 8, 1} : DieVariant{1, 4, 0};
}

template <int NQ, int W>
hipError_t grant_die_lds(size_t lds) {
    static size_t granted = 64 * 1024;
    if (lds <= granted) return hipSuccess;
    const void *kernels[] = {
        reinterpret_cast<const void *>(&attn_splitk_f16_die_kernel<NQ, W, 1, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_die_kernel<NQ, W, 8, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_die_kernel<NQ, W, 64, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_die_kernel<NQ, W, 1, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_die_kernel<NQ, W, 8, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_die_kernel<NQ, W, 64, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_die_prep_kernel<NQ, W, 1, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_die_prep_kernel<NQ, W, 8, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_die_prep_kernel<NQ, W, 64, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_die_prep_kernel<NQ, W, 1, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_die_prep_kernel<NQ, W, 8, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_die_prep_kernel<NQ, W, 64, true>)};
    hipError_t e = hipSuccess;
    for (const void *k : kernels)
        if (e == hipSuccess)
            e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
    if (e == hipSuccess) granted = lds;
    return e;
}

// Workgroups of a variant one compute unit holds at once: the smallest figure over the
// instantiations a launch of the variant may be (the ring and preparing forms use more
// registers), asked of the runtime once.
template <int NQ, int W>
uint32_t die_groups_per_cu() {
    static uint32_t cached = 0;
    if (cached) return cached;
    const size_t lds = variant_lds(NQ, W);
    if (grant_die_lds<NQ, W>(lds) != hipSuccess) {
        (void)hipGetLastError();
        return 1;
    }
    const void *kernels[] = {
        reinterpret_cast<const void *>(&attn_splitk_f16_die_kernel<NQ, W, 64, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_die_kernel<NQ, W, 64, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_die_prep_kernel<NQ, W, 64, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_die_prep_kernel<NQ, W, 64, true>)};
    int least = 1 << 30;
    for (const void *k : kernels) {
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, k, W * 64, lds) != hipSuccess ||
            per_cu < 1) {
            (void)hipGetLastError();
            return 1;
        }
        least = std::min(least, per_cu);
    }
    cached = uint32_t(least);
    return cached;
}
uint32_t variant_groups_per_cu(const DieVariant &v) {
    switch (v.index) {
        case 0: return die_groups_per_cu<1, 4>();
        case 1: return die_groups_per_cu<1, 8>();
        default: return die_groups_per_cu<2, 4>();
    }
}

}  // namespace

bool die_layout_ok(int device) {
    if (device < 0 || device >= 64) return false;
    std::lock_guard<std::mutex> lock(g_dies_mutex);
    DeviceDies &d = g_dies[device];
    if (d.state != 0) return d.state > 0;
    d.state = -1;
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess ||
        cus < int(kDieCount) || cus % int(kDieCount) != 0) {
        (void)hipGetLastError();
        return false;
    }
    // Grids below, at and far above what the device holds at once.
    constexpr uint32_t kMost = 4096;
    uint32_t *ids = nullptr;
    if (hipMalloc(reinterpret_cast<void **>(&ids), kMost * sizeof(uint32_t)) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    bool ok = true;
    std::vector<uint32_t> host(kMost);
    for (uint32_t grid : {8u, 136u, uint32_t(cus), 1000u, kMost}) {
        die_probe_kernel<<<grid, 64, 0, nullptr>>>(ids);
        if (hipStreamSynchronize(nullptr) != hipSuccess ||
            hipMemcpy(host.data(), ids, grid * sizeof(uint32_t), hipMemcpyDeviceToHost) != hipSuccess) {
            (void)hipGetLastError();
            ok = false;
            break;
        }
        for (uint32_t i = 0; i < grid; ++i) ok = ok && host[i] == i % kDieCount;
    }
    (void)hipFree(ids);
    if (ok) {
        d.state = 1;
        d.cus_per_die = uint32_t(cus) / kDieCount;
    }
    return ok;
}

uint32_t attn_splitk_f16_plan_die(const PoolGeom &g, const AttnBatch &b, uint32_t q_heads,
                                  AttnBatch &out, DieMap &map) {
    const uint32_t heads = g.kv_heads;
    if (heads != 1 && heads != 2 && heads != 4 && heads != 8) return 0;
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 0;
    uint32_t cus_per_die = 0;
    {
        std::lock_guard<std::mutex> lock(g_dies_mutex);
        if (g_dies[device].state <= 0) return 0;
        cus_per_die = g_dies[device].cus_per_die;
    }
    const uint32_t group = q_heads / heads;
    const uint32_t bins = kDieCount / heads;
    if (b.n < bins || uint64_t(b.n) * heads > kDieMaxUnits) return 0;
    // Steps of more than 32 query vectors per KV head keep the merge launch: one compute unit
    // merging the 458 KB of a 7-row block's partials takes as long as the merge launch does, and
    // such an item cut into two units of 32 vectors on one die (both reading the KV head's
    // blocks) ran 28.8 us per layer against the merge launch's 23.4.
    uint32_t most_vec = 0;
    for (uint32_t i = 0; i < b.n; ++i) most_vec = std::max(most_vec, b.item[i].rows * group);
    if (most_vec > 32) return 0;
    const DieVariant v = pick_die_variant(g, b, group);
    uint32_t nb[kMaxBatchItems], order[kMaxBatchItems], bin_of[kMaxBatchItems];
    bool splits_any = false;
    uint64_t total = 0;
    uint32_t longest = 1;
    for (uint32_t i = 0; i < b.n; ++i) {
        nb[i] = std::max<uint32_t>(item_block_count(b.item[i]), 1);
        splits_any = splits_any || nb[i] > uint32_t(v.waves);
        total += nb[i];
        longest = std::max(longest, nb[i]);
    }
    if (!splits_any) return 0;
    // The shortest run of blocks per split, T, with which every die takes its workgroups at
    // once. For each T the items go over the bins longest first, each into the lightest bin (by
    // blocks) that still has room for its workgroups at that T; the first T at which every item
    // finds room is taken, if the bins' blocks are then even enough.
    const uint64_t cap = uint64_t(variant_groups_per_cu(v)) * cus_per_die;
    for (uint32_t i = 0; i < b.n; ++i) order[i] = i;
    std::stable_sort(order, order + b.n, [&](uint32_t x, uint32_t y) { return nb[x] > nb[y]; });
    uint64_t T = std::max<uint64_t>((total + cap * bins - 1) / (cap * bins), uint64_t(v.waves));
    uint64_t heaviest = 0;
    for (;; ++T) {
        uint64_t count[kDieCount] = {0}, load[kDieCount] = {0};
        bool fits = true;
        for (uint32_t k = 0; k < b.n; ++k) {
            const uint32_t i = order[k];
            const uint64_t mine = (nb[i] + T - 1) / T;
            uint32_t best = bins;
            for (uint32_t bin = 0; bin < bins; ++bin)
                if (count[bin] + mine <= cap && (best == bins || load[bin] < load[best])) best = bin;
            if (best == bins) {  // no room anywhere: the lightest bin, and a longer T next
                fits = false;
                best = uint32_t(std::min_element(load, load + bins) - load);
            }
            bin_of[i] = best;
            count[best] += mine;
            load[best] += nb[i];
        }
        heaviest = *std::max_element(load, load + bins);
        if (fits || T >= longest) break;
    }
    // A die that carries a tenth more than its share would cost more than the merge launch.
    if (heaviest * bins * 10 > total * 11) return 0;

    out = AttnBatch{};
    out.n = b.n;
    map.shift = heads == 1 ? 0 : heads == 2 ? 1 : heads == 4 ? 2 : 3;
    uint32_t at = 0, ws0 = 0, unit0 = 0, most = 0;
    bool merges = false;
    for (uint32_t bin = 0; bin < kDieCount; ++bin) {
        map.bin_first[bin] = at;
        uint32_t idx = 0;
        for (uint32_t k = 0; bin < bins && k < b.n; ++k) {
            const uint32_t i = order[k];
            if (bin_of[i] != bin) continue;
            AttnItem it = b.item[i];
            it.splits = uint32_t((nb[i] + T - 1) / T);
            const uint32_t bps = (nb[i] + it.splits - 1) / it.splits;
            it.splits = (nb[i] + bps - 1) / bps;
            it.keys_per_split = bps * kBlockKeys;
            it.block0 = idx;
            it.ws0 = ws0;
            it.splits_magic = unit0;  // the item's first ticket (one per KV head)
            idx += it.splits;
            unit0 += heads;
            if (it.splits > 1) {
                ws0 += heads * ((it.splits * it.rows * group + 15u) & ~15u);
                merges = true;
            }
            out.item[at++] = it;
        }
        map.bin_count[bin] = idx;
        most = std::max(most, idx);
    }
    map.bin_first[kDieCount] = at;
    out.total_blocks = most * kDieCount;
    out.rows_per_block = uint32_t(v.index);  // host side: the variant the launch takes
    return merges ? ws0 : 0;
}

hipError_t launch_attn_splitk_f16_die(const AttnParams &p, const AttnBatch &b, const DieMap &map,
                                      uint32_t total_partials, hipStream_t stream,
                                      const FoldedParams *folded) {
    if (b.total_blocks == 0) return hipSuccess;
    const bool prep = folded && folded->prep_on;
#define ITAK_LAUNCH(NQ, W)                                                                        \
    do {                                                                                          \
        const size_t lds = variant_lds(NQ, W);                                                    \
        hipError_t e = grant_die_lds<NQ, W>(lds);                                                 \
        if (e != hipSuccess) return e;                                                            \
        if (prep && p.ring_blocks)                                                                \
            attn_splitk_f16_die_prep_kernel<NQ, W, N, true><<<b.total_blocks, W * 64, lds, stream>>>( \
                p, map, AttnBatchT<N>(b), total_partials, *folded);                               \
        else if (prep)                                                                            \
            attn_splitk_f16_die_prep_kernel<NQ, W, N, false><<<b.total_blocks, W * 64, lds, stream>>>( \
                p, map, AttnBatchT<N>(b), total_partials, *folded);                               \
        else if (p.ring_blocks)                                                                   \
            attn_splitk_f16_die_kernel<NQ, W, N, true><<<b.total_blocks, W * 64, lds, stream>>>(  \
                p, map, AttnBatchT<N>(b), total_partials);                                        \
        else                                                                                      \
            attn_splitk_f16_die_kernel<NQ, W, N, false><<<b.total_blocks, W * 64, lds, stream>>>( \
                p, map, AttnBatchT<N>(b), total_partials);                                        \
    } while (0)
#define ITAK_LAUNCH_NQ()                      \
    do {                                      \
        switch (b.rows_per_block) {           \
            case 0: ITAK_LAUNCH(1, 4); break; \
            case 1: ITAK_LAUNCH(1, 8); break; \
            default: ITAK_LAUNCH(2, 4); break; \
        }                                     \
    } while (0)
    ITAK_DISPATCH_BATCH(b.n, ITAK_LAUNCH_NQ());
#undef ITAK_LAUNCH_NQ
#undef ITAK_LAUNCH
    return hipGetLastError();
}

}  // namespace itak
