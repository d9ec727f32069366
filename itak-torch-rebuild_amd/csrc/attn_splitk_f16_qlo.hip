// The split-K attention kernel of f16 pools at head_dim 128 (attn_splitk_f16_kernel.h) with the
// queries as two f16 halves: the instantiations and their launches, in a file of their own so
// that they compile beside the ordinary ones.
//
// Q enters the score products as f16. Its rounding is relative to each channel, so the error
// of a score grows with the score: at scaled scores of standard deviation 4 and more the
// outputs leave the 2e-3 bar of f16 pools. With q = hi + lo (hi = f16(q), lo = f16(q - hi))
// and scores K.hi + K.lo the queries are good to 2^-22 and what remains is the rounding of the
// softmax weights. The kernels these launches replace wait for memory, not for the matrix pipe:
// the second product per score tile is free.
//
// Semantics: gqa_attention in crates/attention/src/attention.rs:104-215 (see
// attn_splitk_f16.hip).
#include "attn_splitk_f16_kernel.h"

namespace itak {

namespace {

template <int NQ, int W>
hipError_t grant_qlo_lds(size_t lds) {
    static size_t granted = 64 * 1024;
    if (lds <= granted) return hipSuccess;
    const void *kernels[] = {
        reinterpret_cast<const void *>(&attn_splitk_f16_qlo_kernel<NQ, W, 1, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_qlo_kernel<NQ, W, 8, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_qlo_kernel<NQ, W, 64, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_qlo_kernel<NQ, W, 1, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_qlo_kernel<NQ, W, 8, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_qlo_kernel<NQ, W, 64, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_qlo_prep_kernel<NQ, W, 1, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_qlo_prep_kernel<NQ, W, 8, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_qlo_prep_kernel<NQ, W, 64, false>),
        reinterpret_cast<const void *>(&attn_splitk_f16_qlo_prep_kernel<NQ, W, 1, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_qlo_prep_kernel<NQ, W, 8, true>),
        reinterpret_cast<const void *>(&attn_splitk_f16_qlo_prep_kernel<NQ, W, 64, true>)};
    hipError_t e = hipSuccess;
    for (const void *k : kernels)
        if (e == hipSuccess)
            e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
    if (e == hipSuccess) granted = lds;
    return e;
}

}  // namespace

hipError_t launch_attn_splitk_f16_qlo(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                      hipStream_t stream, const FoldedParams *folded) {
    if (b.total_blocks == 0) return hipSuccess;
    const bool prep = folded && folded->prep_on;
    const int variant = attn_splitk_f16_variant(p.g, b, p.group);
#define ITAK_LAUNCH(NQ, W)                                                                         \
    do {                                                                                           \
        const size_t lds = variant_lds(NQ, W, true);                                               \
        hipError_t e = grant_qlo_lds<NQ, W>(lds);                                                  \
        if (e != hipSuccess) return e;                                                             \
        if (prep && p.ring_blocks)                                                                 \
            attn_splitk_f16_qlo_prep_kernel<NQ, W, N, true><<<b.total_blocks, W * 64, lds, stream>>>(  \
                p, AttnBatchT<N>(b), total_partials, *folded);                                     \
        else if (prep)                                                                             \
            attn_splitk_f16_qlo_prep_kernel<NQ, W, N, false><<<b.total_blocks, W * 64, lds, stream>>>( \
                p, AttnBatchT<N>(b), total_partials, *folded);                                     \
        else if (p.ring_blocks)                                                                    \
            attn_splitk_f16_qlo_kernel<NQ, W, N, true><<<b.total_blocks, W * 64, lds, stream>>>(   \
                p, AttnBatchT<N>(b), total_partials);                                              \
        else                                                                                       \
            attn_splitk_f16_qlo_kernel<NQ, W, N, false><<<b.total_blocks, W * 64, lds, stream>>>(  \
                p, AttnBatchT<N>(b), total_partials);                                              \
    } while (0)
#define ITAK_LAUNCH_NQ()                      \
    do {                                      \
        switch (variant) {                    \
            case 0: ITAK_LAUNCH(1, 4); break; \
            case 1: ITAK_LAUNCH(1, 8); break; \
            case 2: ITAK_LAUNCH(2, 4); break; \
            default: ITAK_LAUNCH(4, 4); break; \
        }                                     \
    } while (0)
    ITAK_DISPATCH_BATCH(b.n, ITAK_LAUNCH_NQ());
#undef ITAK_LAUNCH_NQ
#undef ITAK_LAUNCH
    return hipGetLastError();
}

}  // namespace itak
