// qm_predictor_chain.h — pieces of the code predictor's exact attention chain shared by its kernels: the bf16
// round trip, the reference's summation tree, and the P.V sum of one output column.
#pragma once

#include "qm_device.h"
#include "qm_predictor_params.h"

namespace qm {

// bf16 round trip with the hardware converter (round to nearest even; same bits as the integer
// formula of R17:8172-8187 for every non-NaN input).
__device__ __forceinline__ float rbf(float x) { return round_bf16(x); }

// Sum of x[0..N-1], N <= 16, in the shape of the reference's 32-lane shuffle tree (value += shfl_down(value,
// offset) for offset 16, 8, 4, 2, 1, result in lane 0) whose leaves N..31 are exact +0: adding +0 to a value
// that is not -0 is the identity, so absent leaves are dropped instead of added.  X(i) must never be -0
// (fmaf(p, v, +0) and exp() are not).  TreeSum<N, I, S> is what lane I holds once the offsets 16 .. S have been
// applied: lane I's value before offset S plus that of lane I + S — so the innermost additions pair x[i] with
// x[i + 8] and the last one adds the even and the odd lanes' sums.  Use TreeSum<N, 0, 1>.
template <int N, int I, int STRIDE>
struct TreeSum {
    template <class X>
    static __device__ __forceinline__ float eval(const X& x) {
        if constexpr (STRIDE >= 16) {
            return x(I);
        } else if constexpr (I + STRIDE < N) {
            return TreeSum<N, I, 2 * STRIDE>::eval(x) + TreeSum<N, I + STRIDE, 2 * STRIDE>::eval(x);
        } else {
            return TreeSum<N, I, 2 * STRIDE>::eval(x);
        }
    }
};

// The same sum for a runtime number of keys: the full 16-leaf tree whose leaves at and beyond
// `limit` are +0 (never read from V, whose cache slots there may hold anything).
__device__ __forceinline__ float pv_limited(const float* pr, const float* vcol, int limit) {
    return TreeSum<kPredRows, 0, 1>::eval([&](int j) { return j < limit ? fmaf(pr[j], vcol[j], 0.0f) : 0.0f; });
}

}  // namespace qm
