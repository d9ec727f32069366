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

// cap * tanh(x / cap) * log2(e), via exp2; x is a scaled score in natural units.
__device__ __forceinline__ float softcap_log2(float x, float cap, float inv_cap) {
    const float y = x * inv_cap;
    // tanh(y) = 1 - 2 / (exp(2y) + 1); exp2 saturates to inf/0 at the tails, giving +-1.
    const float e = fast_exp2(y * (2.0f * kLog2e));
    const float t = 1.0f - 2.0f / (e + 1.0f);
    return cap * kLog2e * t;
}

}  // namespace itak
