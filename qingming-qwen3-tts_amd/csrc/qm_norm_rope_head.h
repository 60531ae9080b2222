// qm_norm_rope_head.h — QK-RMSNorm + RoPE of one 128-wide head by one 64-lane wave (shared by the
// append kernels and the fused decode step).  Lane l holds dimensions l and l+64, the rotate_half
// partners; every bf16 rounding and the summation order of R17:15365-15526 are kept.
#pragma once

#include "qm_device.h"

namespace qm {

// Sum of squares of the 128 values held as (x0 = dim lane, x1 = dim lane + 64).
// Groups of 32 dims are reduced by value += shfl_down(value, offset) trees; the four
// group sums w0..w3 are combined as (w0 + w2) + (w1 + w3), which is what the
// reference's second-level tree over wave sums evaluates to.
__device__ __forceinline__ float head_sum_squares(float x0, float x1) {
    const float s0 = half_wave_tree_sum(x0 * x0);    // lane 0: w0 (dims 0..31), lane 32: w1 (dims 32..63)
    const float s1 = half_wave_tree_sum(x1 * x1);    // lane 0: w2 (dims 64..95), lane 32: w3
    const float t = s0 + s1;                         // lane 0: w0 + w2, lane 32: w1 + w3
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(t), 0)) + __int_as_float(__builtin_amdgcn_readlane(__float_as_int(t), 32));
}

struct HeadPair {
    uint16_t lo;  // dimension lane
    uint16_t hi;  // dimension lane + 64
};

// RMSNorm (optional) + RoPE of one head from operands already in registers (gamma, cosine and sine at
// dimensions lane and lane + 64 as bf16 bits); returns the two output bit patterns.
__device__ __forceinline__ HeadPair norm_rope_head_values(uint16_t x0b, uint16_t x1b, bool has_gamma,
                                                          uint16_t gamma0, uint16_t gamma1, uint16_t cos0, uint16_t cos1,
                                                          uint16_t sin0, uint16_t sin1, float epsilon) {
    float w0 = bf2f(x0b);
    float w1 = bf2f(x1b);
    if (has_gamma) {
        const float sum = head_sum_squares(w0, w1);
        const float r = 1.0f / sqrtf(sum / 128.0f + epsilon);
        const float n0 = bf2f(f2bf(w0 * r));
        const float n1 = bf2f(f2bf(w1 * r));
        w0 = bf2f(f2bf(n0 * bf2f(gamma0)));
        w1 = bf2f(f2bf(n1 * bf2f(gamma1)));
    }
    // rotate_half(x) = (-x2, +x1): dimension d < 64 pairs with -x[d+64], d >= 64 with +x[d-64].
    const float first0 = bf2f(f2bf(w0 * bf2f(cos0)));
    const float second0 = bf2f(f2bf((-w1) * bf2f(sin0)));
    const float first1 = bf2f(f2bf(w1 * bf2f(cos1)));
    const float second1 = bf2f(f2bf(w0 * bf2f(sin1)));
    HeadPair out;
    out.lo = f2bf(first0 + second0);
    out.hi = f2bf(first1 + second1);
    return out;
}

// The same with gamma (NULL: no RMSNorm), cosine and sine read from memory.
__device__ __forceinline__ HeadPair norm_rope_head(uint16_t x0b, uint16_t x1b,
                                                   const uint16_t* __restrict__ gamma,
                                                   const uint16_t* __restrict__ cosv,
                                                   const uint16_t* __restrict__ sinv,
                                                   float epsilon, int lane) {
    return norm_rope_head_values(x0b, x1b, gamma != nullptr, gamma ? gamma[lane] : static_cast<uint16_t>(0),
                                 gamma ? gamma[lane + 64] : static_cast<uint16_t>(0), cosv[lane], cosv[lane + 64],
                                 sinv[lane], sinv[lane + 64], epsilon);
}

}  // namespace qm
