// The split merge done inside the attention launch (split-K kernels of f16 pools).
//
// A decode layer at a few thousand positions is a few microseconds of work, and a second
// launch that merges the split partials costs as much again. With AttnParams::exchange set
// the workgroups of one (item, KV head) merge among themselves instead. The S workgroups
// (splits) of the group each own the slices s with s % S == split, a slice being 32 channels
// of one query vector together with the vector's (m, l). Every workgroup publishes its share
// of every slice into the owner's run of the exchange buffer, then gathers its own slices from
// all S producers and writes that part of the final output. The record of (owner c, local
// slice n, producer p) is 17 words of 64 bits at ((c * max_local + n) * S + p) * 17 from the
// group's base: words 0..15 hold channel pairs, word 16 holds (m, l).
//
// Nothing is fenced. Every word is written and read with relaxed agent-scope atomics of 64
// bits and proves itself: the buffer holds kExchangeEmpty wherever nothing has been published,
// published words never carry that pattern (a NaN with all bits set is rewritten to the default
// NaN first), and a consumer polls the words that are still empty. Having read a word it puts
// the pattern back, so the buffer is clean again when the launch ends; coherence of a single
// location orders that store after the producer's. Consumers wait only for workgroups of their
// own launch, and the planner never makes a launch larger than the device holds at once, so
// every producer is running or done; the wait is bounded all the same (AttnParams::spin_limit
// polls, about a microsecond each), after which the consumer gives up, writes NaN and counts
// itself in the buffer's first word.
#pragma once

#include "internal.h"
#include "mfma_common.h"

namespace itak {

constexpr unsigned long long kExchangeEmpty = kExchangeEmptyWord;
constexpr int kExchangeWords = 17;        // 64-bit words per record
constexpr int kExchangePerThread = 16;    // words one thread gathers at most
constexpr int kExchangeHeaderWords = 32;  // words before the first record (word 0, low half: give-ups)

__device__ __forceinline__ unsigned long long exchange_pack(float a, float b) {
    uint32_t lo = __float_as_uint(a), hi = __float_as_uint(b);
    lo = lo == 0xffffffffu ? 0x7fc00000u : lo;
    hi = hi == 0xffffffffu ? 0x7fc00000u : hi;
    return uint64_t(lo) | (uint64_t(hi) << 32);
}
__device__ __forceinline__ void exchange_store(unsigned long long *dst, unsigned long long v) {
    __hip_atomic_store(dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long exchange_load(const unsigned long long *src) {
    return __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// A barrier for code that has global stores in flight: only LDS traffic is waited for.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}
// Reductions over the 16 lanes of a DPP row, result in every lane.
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_lane<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_lane<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_lane<0x141>(v);  // row_half_mirror
    v += dpp_lane<0x140>(v);  // row_mirror
    return v;
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_lane<0xB1>(v));
    v = fmaxf(v, dpp_lane<0x4E>(v));
    v = fmaxf(v, dpp_lane<0x141>(v));
    v = fmaxf(v, dpp_lane<0x140>(v));
    return v;
}

// One workgroup's view of its group's run of the exchange buffer.
struct ExchangeGroup {
    unsigned long long *base;  // the group's first record
    uint32_t splits, magic;    // S and ceil(2^32 / S)
    uint32_t split;            // this workgroup's place in the group
    uint32_t slices;           // 4 per query vector
    uint32_t max_local;        // slices an owner holds at most

    __device__ __forceinline__ void init(float *ws, const AttnItem &item, uint32_t kv_head,
                                         uint32_t split_, uint32_t nvec) {
        splits = item.splits;
        magic = item.splits_magic;
        split = split_;
        slices = nvec * 4;
        max_local = __umulhi(slices + splits - 1, magic);
        base = reinterpret_cast<unsigned long long *>(ws) + kExchangeHeaderWords +
               (uint64_t(item.ws0) + uint64_t(kv_head) * splits * max_local * splits) * kExchangeWords;
    }

    // Channels dt*16 + g*4 .. +3 of query vector j, weighted sums not yet divided by l; the
    // lane with g == 0 of an even tile also carries the vector's (m, l).
    __device__ __forceinline__ void publish(uint32_t j, uint32_t dt, uint32_t g, floatx4 acc, float m,
                                            float l) const {
        const uint32_t slice = j * 4 + (dt >> 1);
        const uint32_t local_slice = __umulhi(slice, magic);
        const uint32_t owner = slice - local_slice * splits;
        unsigned long long *rec =
            base + (uint64_t(owner * max_local + local_slice) * splits + split) * kExchangeWords;
        exchange_store(rec + (dt & 1) * 8 + g * 2, exchange_pack(acc[0], acc[1]));
        exchange_store(rec + (dt & 1) * 8 + g * 2 + 1, exchange_pack(acc[2], acc[3]));
        if ((dt & 1) == 0 && g == 0) exchange_store(rec + 16, exchange_pack(m, l));
    }

    // Gathers this workgroup's slices from every producer, merges them and writes the output
    // rows' channels. Called by all T threads of the workgroup after their last publish;
    // `sm_x` is LDS the workgroup no longer reads (T * NW words at most, NW the words one thread
    // gathers at most: the planner's bound for the kernel).
    //
    // A look at the buffer is a round trip to memory of more than a microsecond, as long as
    // everything else a decode layer does, and the slowest producer of the group decides when
    // the last word turns up: a consumer that looked just too early would lose a whole round
    // trip. So DEPTH looks at every word are kept in flight, spaced a fraction of the round trip
    // apart, and the oldest is examined first; the loop then samples the buffer DEPTH times per
    // round trip. Every look loads all NW words of the thread (those already seen included, at
    // a clamped address) so that the order of loads in flight is fixed and known to the compiler.
    template <uint32_t T, int NW, int DEPTH>
    __device__ __forceinline__ void finish(unsigned long long *sm_x, const AttnParams &p,
                                           const AttnItem &item, uint32_t kv_head, uint32_t group,
                                           uint32_t group_magic, const float *gate,
                                           unsigned long long *gathered_at = nullptr) const {
        const uint32_t tid = threadIdx.x;
        const uint32_t S = splits;
        const uint32_t n_my = split < slices ? __umulhi(slices - split + S - 1, magic) : 0;
        const uint32_t my_words = n_my * S * kExchangeWords;
        unsigned long long *const src = base + uint64_t(split) * max_local * S * kExchangeWords;
        unsigned long long got[NW];
        if (my_words) {
            uint32_t at[NW];
            uint32_t pending = 0;
#pragma unroll
            for (int u = 0; u < NW; ++u) {
                at[u] = min(tid + u * T, my_words - 1);
                if (tid + u * T < my_words) pending |= 1u << u;
            }
            unsigned long long look[DEPTH][NW];
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
#pragma unroll
                for (int u = 0; u < NW; ++u)
                    if (DEPTH > 1 || u * T < my_words) look[d][u] = exchange_load(src + at[u]);
                if (d + 1 < DEPTH) {
                    __builtin_amdgcn_sched_barrier(0);
                    __builtin_amdgcn_s_sleep(10);  // 640 cycles: about a quarter of the round trip
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            uint32_t polls = 0;
            while (pending) {
#pragma unroll
                for (int d = 0; d < DEPTH; ++d) {
#pragma unroll
                    for (int u = 0; u < NW; ++u)
                        if ((pending >> u & 1) && uint32_t(look[d][u]) != 0xffffffffu &&
                            uint32_t(look[d][u] >> 32) != 0xffffffffu) {
                            got[u] = look[d][u];
                            pending &= ~(1u << u);
                        }
                    if (!pending) break;
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int u = 0; u < NW; ++u)
                        if (DEPTH > 1 || u * T < my_words) look[d][u] = exchange_load(src + at[u]);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (pending && (polls += DEPTH) > p.spin_limit) {  // a producer never arrived: give up, loudly
#pragma unroll
                    for (int u = 0; u < NW; ++u)
                        if (pending >> u & 1) got[u] = 0x7fc000007fc00000ull;
                    atomicAdd(reinterpret_cast<uint32_t *>(p.ws), 1u);
                    break;
                }
            }
        }
        if (gathered_at) *gathered_at = wall_clock64();  // the timeline build's mark
        // The wavefronts are done with their own merge: its LDS now takes the gathered words.
        // What was read is given back to the buffer as empty at once, so that those stores are
        // under way while the slices are summed.
        lds_barrier();
#pragma unroll
        for (int u = 0; u < NW; ++u)
            if (tid + u * T < my_words) {
                sm_x[tid + u * T] = got[u];
                exchange_store(src + tid + u * T, kExchangeEmpty);
            }
        lds_barrier();
        // A team of 256 threads per slice: thread = (channel pair k, producer lane pl); the
        // producers pl, pl + 16, .. fold into the thread's own (m, l, a), and the 16 lanes of a
        // pair meet through DPP.
        const uint32_t k = (tid & 255u) >> 4, pl = tid & 15u;
        for (uint32_t ls = tid >> 8; ls < n_my; ls += T / 256) {
            const unsigned long long *rec = sm_x + uint64_t(ls) * S * kExchangeWords;
            float m_run = -INFINITY, l_run = 0.0f, a0 = 0.0f, a1 = 0.0f;
            for (uint32_t pr = pl; pr < S; pr += 16) {
                const unsigned long long ml = rec[pr * kExchangeWords + 16];
                const unsigned long long xv = rec[pr * kExchangeWords + k];
                const float mp = __uint_as_float(uint32_t(ml)), lp = __uint_as_float(uint32_t(ml >> 32));
                // (A producer that saw nothing finite has m = -inf: weight zero against a
                // stand-in reference, and no branch around it, so that an l or a sum that is NaN
                // there, from a key that is not finite, stays in the result.)
                const float m_new = fmaxf(m_run, mp);
                const float ref = m_new == -INFINITY ? 0.0f : m_new;
                const float keep = fast_exp2(m_run - ref), w = fast_exp2(mp - ref);  // exp2(-inf) = 0
                l_run = fmaf(lp, w, l_run * keep);
                a0 = fmaf(__uint_as_float(uint32_t(xv)), w, a0 * keep);
                a1 = fmaf(__uint_as_float(uint32_t(xv >> 32)), w, a1 * keep);
                m_run = m_new;
            }
            const float Mx = row16_max(m_run);
            const float f = m_run == -INFINITY ? 0.0f : fast_exp2(m_run - Mx);
            const float Lx = row16_sum(l_run * f);
            a0 = row16_sum(a0 * f);
            a1 = row16_sum(a1 * f);
            if (pl == 0) {
                const uint32_t slice = split + ls * S;
                const uint32_t j = slice >> 2, row = (j * group_magic) >> 16;
                const uint32_t head = kv_head * group + (j - row * group);
                const uint64_t at =
                    (uint64_t(item.q_row0 + row) * p.q_heads + head) * kD + (slice & 3u) * 32 + k * 2;
                const float inv = 1.0f / Lx;
                float2 o = make_float2(a0 * inv, a1 * inv);
                if (gate) {
                    const float2 gt = *reinterpret_cast<const float2 *>(gate + at);
                    o = make_float2(o.x * sigmoid_fast(gt.x), o.y * sigmoid_fast(gt.y));
                }
                *reinterpret_cast<float2 *>(p.out + at) = o;
            }
        }
    }
};

}  // namespace itak
