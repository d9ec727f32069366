// Fused attention preparation for gfx950: the per-head RMSNorm of Q and K and their RoPE
// rotation in one launch, between the projections and the attention step (the job of the
// reference's K9 dispatch, crates/wgpu-compute/src/kernels/k9_attn_prep.rs:1-60; the append
// K9 also does is fused into the attention launch here). Numerics follow the reference's CPU
// path, not its shader: mean of squares and the scaled product in f64 with one rounding to
// f32 (crates/torch-math/src/norm.rs:40-51), then angles position * base^(-2i/rotary_dim),
// sine, cosine and the rotation in f64 with one rounding to f32
// (rope_interleaved.rs:103-114, rope.rs:99-114) -- an f32 angle is off by 8e-3 rad at
// position 100,000, a thousand times the 1e-5 bar. The work is a few thousand elements per
// token, so f64 costs nothing that shows.
//
// One wavefront serves one head row (lane i holds channels 2i, 2i+1 [, 2i+128, ...], which is
// also the adjacent pair the interleaved rotation joins); the grid covers every Q head row,
// then every K head row of the step. The gate after attention (a * sigmoid(g),
// crates/cpu-compute/src/cpu.rs:657-673, sigmoid :162-169) is an elementwise kernel of its own
// for paths whose final writer does not apply it.
#include "internal.h"

#include <math.h>

namespace itak {

namespace {

constexpr int kPrepWaves = 4;

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

__global__ __launch_bounds__(kPrepWaves * 64) void attn_prep_kernel(PrepArgs a) {
    const uint32_t lane = threadIdx.x & 63;
    const uint64_t head_row = uint64_t(blockIdx.x) * kPrepWaves + (threadIdx.x >> 6);
    const uint64_t q_rows = uint64_t(a.total_rows) * a.q_heads;
    const uint64_t k_rows = uint64_t(a.total_rows) * a.kv_heads;
    if (head_row >= q_rows + k_rows) return;
    const bool is_k = head_row >= q_rows;
    const uint64_t local = is_k ? head_row - q_rows : head_row;
    const uint32_t heads = is_k ? a.kv_heads : a.q_heads;
    const uint32_t row = uint32_t(local / heads);
    const uint32_t D = a.head_dim;
    const float *src = (is_k ? a.k_in : a.q_in) + local * D;
    float *dst = (is_k ? a.k_out : a.q_out) + local * D;
    const float *weight = is_k ? a.k_weight : a.q_weight;

    // The row's position: items are laid out in order, item i owning rows row0[i]..
    uint32_t it = 0;
    while (it + 1 < a.n && row >= a.row0[it + 1]) ++it;
    const double position = double(a.pos0[it] + (row - a.row0[it]));

    const uint32_t pairs = D / 2;
    // 1. RMSNorm (norm.rs:40-51).
    double inv_rms = 1.0;
    if (weight) {
        double sum = 0.0;
        for (uint32_t p = lane; p < pairs; p += 64) {
            const float2 v = *reinterpret_cast<const float2 *>(src + 2 * p);
            sum += double(v.x) * double(v.x) + double(v.y) * double(v.y);
        }
        sum = wave_sum(sum);
        inv_rms = 1.0 / sqrt(sum / double(D) + double(a.eps));
    }
    auto normed = [&](uint32_t c) -> float {
        const float v = src[c];
        return weight ? float(double(v) * inv_rms * double(weight[c])) : v;
    };
    // 2. RoPE on the normed row (rounded to f32 first, as the reference's two calls do).
    const uint32_t rot = a.rope_base > 1.0f ? a.rotary_dim : 0;
    const uint32_t half = rot / 2;
    for (uint32_t p = lane; p < pairs; p += 64) {
        uint32_t c0, c1;
        bool turn;
        if (a.interleaved) {  // pair p joins channels 2p and 2p+1
            c0 = 2 * p;
            c1 = 2 * p + 1;
            turn = p < half;
        } else if (p < half) {  // pair p joins channels p and p + rotary_dim/2
            c0 = p;
            c1 = p + half;
            turn = true;
        } else {  // the tail beyond rotary_dim, two channels per lane
            c0 = rot + 2 * (p - half);
            c1 = c0 + 1;
            turn = false;
        }
        const float x = normed(c0), y = normed(c1);
        if (turn) {
            const double exponent = -double(2 * p) / double(rot);
            const double freq = a.rope_freq ? a.rope_freq[p] : pow(double(a.rope_base), exponent);
            const double angle = position * freq;
            double s, c;
            sincos(angle, &s, &c);
            // Two products and a sum, each rounded, as the reference's compiler emits them: a
            // fused multiply-add here would differ from it in the last bit of the f64 result,
            // which shows in the f32 row where the rotation cancels to something tiny.
            {
#pragma clang fp contract(off)
                const double xc = double(x) * c, ys = double(y) * s;
                const double xs = double(x) * s, yc = double(y) * c;
                dst[c0] = float(xc - ys);
                dst[c1] = float(xs + yc);
            }
        } else {
            dst[c0] = x;
            dst[c1] = y;
        }
    }
}

__global__ __launch_bounds__(256) void attn_gate_kernel(float *__restrict__ out,
                                                        const float *__restrict__ gate,
                                                        uint64_t count) {
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < count; i += gridDim.x * 256ull)
        out[i] = out[i] * sigmoid_ref(gate[i]);
}

}  // namespace

hipError_t launch_attn_prep(const PrepArgs &a, hipStream_t stream) {
    const uint64_t head_rows = uint64_t(a.total_rows) * (a.q_heads + a.kv_heads);
    if (head_rows == 0) return hipSuccess;
    const uint64_t blocks = (head_rows + kPrepWaves - 1) / kPrepWaves;
    attn_prep_kernel<<<uint32_t(blocks), kPrepWaves * 64, 0, stream>>>(a);
    return hipGetLastError();
}

hipError_t launch_attn_gate(float *out, const float *gate, uint64_t count, hipStream_t stream) {
    if (count == 0) return hipSuccess;
    uint64_t blocks = (count + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    attn_gate_kernel<<<uint32_t(blocks), 256, 0, stream>>>(out, gate, count);
    return hipGetLastError();
}

}  // namespace itak
