// The block kernel at the head dims other than 128 (attn_prefill_f16_kernel.h has the kernel,
// attn_prefill_f16.hip the planner and the entry point that calls this).
#include "attn_prefill_f16_kernel.h"

// The marks of attn_prefill_f16_kernel's instantiations in this file.
ITAK_TIMELINE_READER(itak_timeline_read_prefill_dims)

namespace itak {

hipError_t launch_attn_prefill_f16_dims(const AttnParams &p, const AttnBatch &b, uint32_t total_partials,
                                        bool one, hipStream_t stream) {
    switch (p.g.head_dim) {
        case 64: return launch_prefill_head_dim<64, false>(p, b, total_partials, one, stream);
        case 96: return launch_prefill_head_dim<96, false>(p, b, total_partials, one, stream);
        case 256: return launch_prefill_head_dim<256, false>(p, b, total_partials, one, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace itak
