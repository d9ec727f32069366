// The block kernel with the queries as two f16 halves (ITAK_POOL_Q_TWO_HALVES): head_dim 128, the
// two-tile form (attn_prefill_f16_kernel.h has the kernel, attn_prefill_f16.hip the planner and
// the entry point that calls this).
#include "attn_prefill_f16_kernel.h"

namespace itak {

hipError_t launch_attn_prefill_f16_qlo(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                       hipStream_t stream) {
    if (p.g.head_dim != 128 || p.k_new) return hipErrorInvalidValue;
    hipError_t e = hipSuccess;
    // Two argument sizes, one item and any number: the form is opt-in and its launches are long.
#define ITAK_LAUNCH_QLO(SC, RING)                                                                       \
    do {                                                                                                \
        if (b.n <= 1)                                                                                   \
            e = launch_prefill<1, SC, 2, RING, 128, true>(p, b, total_partials, stream);                \
        else                                                                                            \
            e = launch_prefill<kMaxBatchItems, SC, 2, RING, 128, true>(p, b, total_partials, stream);   \
    } while (0)
    if (p.softcap > 0.0f) {
        if (p.ring_blocks)
            ITAK_LAUNCH_QLO(true, true);
        else
            ITAK_LAUNCH_QLO(true, false);
    } else {
        if (p.ring_blocks)
            ITAK_LAUNCH_QLO(false, true);
        else
            ITAK_LAUNCH_QLO(false, false);
    }
#undef ITAK_LAUNCH_QLO
    return e;
}

}  // namespace itak
