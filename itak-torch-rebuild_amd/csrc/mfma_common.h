// Small pieces shared by the MFMA attention kernels (f16 KV, head_dim 128).
#pragma once

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

namespace itak {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kD = 128;          // head_dim this kernel is written for
constexpr int kBlockKeys = 32;   // keys per block (= value plane block)
constexpr int kQStride = kD + 8; // LDS row stride of the staged queries (halves)
constexpr int kMaxNewRows = 8;   // rows one item may append in a fused step
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// A mask over the eight halves of an operand register group (a lane's eight keys of a value
// piece) that keeps the first n. Element-wise conditional stores into such a vector compile to
// a permute and a shift per half under execution masks, hundreds of instructions on a path that
// every workgroup holding a last or oldest block takes once, cold: rows are dropped with an AND.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x4 first_halves(uint32_t n) {
    u32x4 m;
#pragma unroll
    for (int j = 0; j < 4; ++j) m[j] = n > 2u * j + 1 ? 0xffffffffu : n > 2u * j ? 0x0000ffffu : 0u;
    return m;
}
// Zeroes the halves of v whose mask bits are clear.
__device__ __forceinline__ half8 keep_halves(half8 v, u32x4 keep) {
    return __builtin_bit_cast(half8, __builtin_bit_cast(u32x4, v) & keep);
}

// True when some half of the N operand register groups is an infinity or a NaN (exponent field
// all ones), in any lane of the wavefront.
template <int N>
__device__ __forceinline__ bool any_not_finite(const half8 (&v)[N]) {
    uint32_t seen = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const u32x4 x = __builtin_bit_cast(u32x4, v[i]);
#pragma unroll
        for (int c = 0; c < 4; ++c) seen |= (x[c] & 0x7c007c00u) + 0x04000400u;  // 0x7c00 + 0x0400 = 0x8000
    }
    return __builtin_amdgcn_ballot_w64((seen & 0x80008000u) != 0) != 0;
}

// The value of another lane of the same 16-lane row, chosen by a DPP control word.
template <int CTRL>
__device__ __forceinline__ float dpp_lane(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

// cap * tanh(x / cap) * log2(e); x is a scaled score in natural units.
// tanh(y) = 1 - 2 / (exp(2y) + 1) with the hardware's exp2 and reciprocal (each within one
// unit in the last place; exp2 saturates to inf / 0 at the tails, giving +-1): a multiply, an
// add and a fused multiply-add around two transcendental instructions. An IEEE division
// here costs four times as much vector work, on every score of a block.
// `shift` is subtracted from the result inside the same fused multiply-add (a caller that keeps
// scores relative to a reference passes the reference).
__device__ __forceinline__ float softcap_log2(float x, float cap, float inv_cap, float shift = 0.0f) {
    const float e = fast_exp2(x * (inv_cap * (2.0f * kLog2e)));
    const float r = __builtin_amdgcn_rcpf(e + 1.0f);
    const float c = cap * kLog2e;
    return __builtin_fmaf(r, -2.0f * c, c - shift);
}

// The same for a score that arrives as the exponential's argument, a = 2 * log2(e) * x / cap
// (the factor folded into whatever scaled x), with c = cap * log2(e).
__device__ __forceinline__ float softcap_of_exp2_arg(float a, float c, float shift) {
    const float r = __builtin_amdgcn_rcpf(fast_exp2(a) + 1.0f);
    return __builtin_fmaf(r, -2.0f * c, c - shift);
}

}  // namespace itak
