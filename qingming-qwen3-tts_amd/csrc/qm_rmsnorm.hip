// qm_rmsnorm.hip — hidden-state RMSNorm (any rows) and the fused residual add + post-attention
// RMSNorm of one decode step, for gfx950, bit-identical to the reference's kernels.
//
// Both reference kernels run 256 threads per row: thread t accumulates the squares of columns
// t, t+256, ... with fmaf, and the block sum is eight 32-lane shfl_down trees followed by one tree
// over the eight results (R17:8233-8274, 15102-15148).  The same thread layout and the same trees
// are used here — __shfl_down with width 32 inside the 64-lane waves — so the statistic has the
// reference's bits; the inverse RMS is a correctly rounded 1 / sqrt.  A row is a few KB: the
// kernels are bound by launch and load latency, not by bandwidth.

#include "qm_device.h"
#include "qm_host.h"

namespace qm {

constexpr int kNormThreads = 256;

// rmsnorm_kernel (R17:8276-8338): one block per row.
__global__ __launch_bounds__(kNormThreads) void rmsnorm_rows_kernel(const uint16_t* input, const uint16_t* weight,
                                                                    uint16_t* output, int dimension, float epsilon) {
    __shared__ float sh_waves[8];
    __shared__ float sh_total;
    const int64_t base = static_cast<int64_t>(blockIdx.x) * dimension;
    float sum_squares = 0.0f;
    for (int c = threadIdx.x; c < dimension; c += kNormThreads) {
        const float v = bf2f(input[base + c]);
        sum_squares = fmaf(v, v, sum_squares);
    }
    const float total = block_sum_256_like_reference(sum_squares, sh_waves, &sh_total);
    const float inverse_rms = 1.0f / sqrtf(total / static_cast<float>(dimension) + epsilon);
    for (int c = threadIdx.x; c < dimension; c += kNormThreads) {
        const float normalized = round_bf16(bf2f(input[base + c]) * inverse_rms);
        output[base + c] = f2bf(normalized * bf2f(weight[c]));
    }
}

// talker_add_postnorm_fused_kernel (R17:16205-16286): one block.
__global__ __launch_bounds__(kNormThreads) void add_postnorm_kernel(const uint16_t* hidden, const uint16_t* attention,
                                                                    const uint16_t* norm_weight, uint16_t* residual,
                                                                    uint16_t* normalized, int dimension, float epsilon) {
    extern __shared__ uint16_t sh_residual[];
    __shared__ float sh_waves[8];
    __shared__ float sh_total;
    float local_sum = 0.0f;
    for (int c = threadIdx.x; c < dimension; c += kNormThreads) {
        const uint16_t value = f2bf(bf2f(hidden[c]) + bf2f(attention[c]));
        residual[c] = value;
        sh_residual[c] = value;
        const float x = bf2f(value);
        local_sum = fmaf(x, x, local_sum);
    }
    const float total = block_sum_256_like_reference(local_sum, sh_waves, &sh_total);
    const float inverse_rms = 1.0f / sqrtf(total / static_cast<float>(dimension) + epsilon);
    for (int c = threadIdx.x; c < dimension; c += kNormThreads) {
        const float n = round_bf16(bf2f(sh_residual[c]) * inverse_rms);
        normalized[c] = f2bf(n * bf2f(norm_weight[c]));
    }
}

}  // namespace qm

extern "C" int32_t qm_rmsnorm_rows(const uint16_t* input, const uint16_t* weight, uint16_t* output, int32_t rows,
                                   int32_t dimension, float epsilon, void* hip_stream) {
    using namespace qm;
    if (!input || !weight || !output) return QM_ERR_NULL;
    if (rows < 0 || dimension <= 0) return QM_ERR_ARGUMENT;
    if (rows == 0) return QM_OK;
    hipLaunchKernelGGL(rmsnorm_rows_kernel, dim3(static_cast<unsigned>(rows)), dim3(kNormThreads), 0,
                       static_cast<hipStream_t>(hip_stream), input, weight, output, dimension, epsilon);
    return launch_status();
}

extern "C" int32_t qm_add_postnorm_m1(const uint16_t* hidden, const uint16_t* attention, const uint16_t* norm_weight,
                                      uint16_t* residual, uint16_t* normalized, int32_t dimension, float epsilon,
                                      void* hip_stream) {
    using namespace qm;
    if (!hidden || !attention || !norm_weight || !residual || !normalized) return QM_ERR_NULL;
    if (dimension <= 0) return QM_ERR_ARGUMENT;
    if (dimension > 32768) return QM_ERR_GEOMETRY;   // the rounded residual is kept in 64 KB of LDS
    hipLaunchKernelGGL(add_postnorm_kernel, dim3(1), dim3(kNormThreads), static_cast<size_t>(dimension) * 2,
                       static_cast<hipStream_t>(hip_stream), hidden, attention, norm_weight, residual, normalized,
                       dimension, epsilon);
    return launch_status();
}
