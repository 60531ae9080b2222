// qm_linear.hip — M = 1 weight-streaming linears (fused Q/K/V projection, o_proj / down_proj with
// bias and residual) for gfx950, bit-identical to the reference's kernels.
//
// What fixes the design.  The reference computes one output scalar per 32-lane wave: lane l
// accumulates the products k = l, l+32, l+64, ... with fmaf in increasing k, the 32 lane sums go
// through a shuffle tree, lane 0 adds the bias and rounds to bf16 (R17:15239-15266, 15340-15360).
// fp32 addition does not associate, so to reproduce those bits every one of the 32 chains of an
// output must be evaluated in its own order by one lane.  Here 16 lanes (one DPP row) own an
// output: lane q keeps two accumulators, for the chains 2q and 2q+1, and reads the two adjacent
// weights k = 32j + 2q, 32j + 2q + 1 of step j with one 32-bit load — the 16 lanes of a row read
// 64 contiguous bytes of one weight row per step, a wave four such rows.  The shuffle tree of the
// reference becomes four DPP row rotations (lanes q+8, q+4, q+2, q+1) and one add inside lane 0.
// A wider load would put more chains into one lane and leave fewer lanes per output: with 4 096
// outputs of 2 048 weights, 16 lanes per output is what gives one wave to every SIMD of the chip.
//
// Memory.  Weights are read exactly once, 32 loads per lane in flight in each of two register
// batches (all 64 steps of a 2 048-wide reduction are requested before the first is consumed);
// the input vector is converted to fp32 once per block into LDS and read from there as
// broadcast 8-byte pairs.  Algorithmic HBM bytes: 2 * outputs * reduction (weights) + input +
// outputs (+ bias, residual); bound: HBM bandwidth.

#include "qm_device.h"
#include "qm_host.h"

namespace qm {

constexpr int kLinThreads = 256;
constexpr int kLinRowsPerBlock = kLinThreads / 16;
constexpr int kLinBatch = 32;          // loads per register batch
constexpr int kLinMaxReduction = 16384;   // fp32 input vector must fit in 64 KB of LDS

struct LinearParams {
    const uint16_t* input;        // [reduction]
    const uint16_t* weight[3];    // [rows_i][reduction] each
    const uint16_t* bias[3];      // [rows_i] or NULL
    uint16_t* output[3];          // [rows_i]
    const uint16_t* residual;     // [rows_0] or NULL (single-matrix form only)
    int rows[3];
    int reduction;
};

__global__ __launch_bounds__(kLinThreads) void linear_m1_kernel(LinearParams prm) {
    extern __shared__ __attribute__((aligned(16))) float lin_x[];   // the input vector, fp32

    const int tid = threadIdx.x;
    const int q = tid & 15;                                         // lane within the output's row
    const int reduction = prm.reduction;
    const int steps = (reduction + 31) >> 5;

    // This lane's output: global row index over the concatenation of the (up to) three matrices.
    int row = static_cast<int>(blockIdx.x) * kLinRowsPerBlock + (tid >> 4);
    int m = 0;
    if (row >= prm.rows[0]) {
        row -= prm.rows[0];
        m = 1;
        if (row >= prm.rows[1]) {
            row -= prm.rows[1];
            m = 2;
        }
    }
    const bool live = row < prm.rows[m];
    const uint16_t* wrow = prm.weight[m] + static_cast<int64_t>(live ? row : 0) * reduction;

    // Steps [j0, j0 + kLinBatch) of this lane's weight row: elements 32j + 2q, 32j + 2q + 1.
    // Unpredicated: a lane without an output reads row 0, a step past the end the last pair.
    auto load_batch = [&](uint32_t (&w)[kLinBatch], int j0) {
#pragma unroll
        for (int u = 0; u < kLinBatch; ++u) {
            const int k = min(32 * (j0 + u) + 2 * q, reduction - 2);
            w[u] = *reinterpret_cast<const uint32_t*>(wrow + k);
        }
    };
    uint32_t wa[kLinBatch], wb[kLinBatch];
    load_batch(wa, 0);
    if (kLinBatch < steps) load_batch(wb, kLinBatch);

    // fp32 input vector, zero-padded to whole steps of 32.
    for (int k = tid; k < 32 * steps; k += kLinThreads) lin_x[k] = k < reduction ? bf2f(prm.input[k]) : 0.0f;
    __syncthreads();

    float acc0 = 0.0f, acc1 = 0.0f;
    // A whole batch is straight-line code (the LDS reads of its 32 input pairs are requested ahead
    // of the multiply-adds); a batch cut by the end of the reduction takes the per-step test, and
    // in a ragged last step the pairs past the end are multiplied as 0 * 0, which leaves the
    // accumulators (never -0) unchanged.
    auto consume_batch = [&](const uint32_t (&w)[kLinBatch], int j0) {
        const float* xs = lin_x + 32 * j0 + 2 * q;
        if (j0 + kLinBatch <= steps && 32 * steps == reduction) {
            float2 x[kLinBatch];
#pragma unroll
            for (int u = 0; u < kLinBatch; ++u) x[u] = *reinterpret_cast<const float2*>(xs + 32 * u);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < kLinBatch; ++u) {
                acc0 = fmaf(x[u].x, lo_bf16(w[u]), acc0);
                acc1 = fmaf(x[u].y, hi_bf16(w[u]), acc1);
            }
        } else {
#pragma unroll
            for (int u = 0; u < kLinBatch; ++u) {
                if (j0 + u < steps) {
                    const float2 x = *reinterpret_cast<const float2*>(xs + 32 * u);
                    const uint32_t wu = 32 * (j0 + u) + 2 * q < reduction ? w[u] : 0u;
                    acc0 = fmaf(x.x, lo_bf16(wu), acc0);
                    acc1 = fmaf(x.y, hi_bf16(wu), acc1);
                }
            }
        }
    };
    for (int j0 = 0; j0 < steps; j0 += 2 * kLinBatch) {
        consume_batch(wa, j0);
        if (j0 + 2 * kLinBatch < steps) load_batch(wa, j0 + 2 * kLinBatch);
        if (j0 + kLinBatch < steps) consume_batch(wb, j0 + kLinBatch);
        if (j0 + 3 * kLinBatch < steps) load_batch(wb, j0 + 3 * kLinBatch);
    }

    // The reference's tree over its 32 lanes, v += shfl_down(v, 16 / 8 / 4 / 2 / 1): chain c lives in
    // lane c/2, accumulator c%2, so +16, +8, +4, +2 are lanes q+8, q+4, q+2, q+1 (row_ror by
    // 8, 12, 14, 15 brings lane q+n to lane q) and +1 is the other accumulator of lane 0.
    acc0 += row_ror<8>(acc0);
    acc1 += row_ror<8>(acc1);
    acc0 += row_ror<12>(acc0);
    acc1 += row_ror<12>(acc1);
    acc0 += row_ror<14>(acc0);
    acc1 += row_ror<14>(acc1);
    acc0 += row_ror<15>(acc0);
    acc1 += row_ror<15>(acc1);
    if (q == 0 && live) {
        float a = acc0 + acc1;
        if (prm.bias[m]) a += bf2f(prm.bias[m][row]);
        uint16_t v = f2bf(a);
        if (prm.residual) v = f2bf(bf2f(prm.residual[row]) + bf2f(v));
        prm.output[m][row] = v;
    }
}

inline int32_t launch_linear(const LinearParams& prm, hipStream_t s) {
    const int64_t total = static_cast<int64_t>(prm.rows[0]) + prm.rows[1] + prm.rows[2];
    if (total == 0) return QM_OK;
    const size_t smem = static_cast<size_t>((prm.reduction + 31) / 32 * 32) * sizeof(float);
    static bool attr_set = false;
    if (!attr_set) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(linear_m1_kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 kLinMaxReduction * static_cast<int>(sizeof(float)));
        if (e != hipSuccess) return hip_code(e);
        attr_set = true;
    }
    const unsigned blocks = static_cast<unsigned>((total + kLinRowsPerBlock - 1) / kLinRowsPerBlock);
    hipLaunchKernelGGL(linear_m1_kernel, dim3(blocks), dim3(kLinThreads), smem, s, prm);
    return launch_status();
}

inline int32_t check_reduction(int32_t reduction) {
    if (reduction <= 0) return QM_ERR_ARGUMENT;
    // 32-bit weight loads of element pairs; the fp32 copy of the input lives in LDS.
    if ((reduction & 1) || reduction > kLinMaxReduction) return QM_ERR_GEOMETRY;
    return QM_OK;
}

}  // namespace qm

extern "C" int32_t qm_linear_m1(const uint16_t* input, const uint16_t* weight, const uint16_t* bias,
                                const uint16_t* residual, uint16_t* output, int32_t output_columns,
                                int32_t reduction_columns, void* hip_stream) {
    using namespace qm;
    if (!input || !weight || !output) return QM_ERR_NULL;
    if (output_columns < 0) return QM_ERR_ARGUMENT;
    const int32_t rc = check_reduction(reduction_columns);
    if (rc != QM_OK) return rc;
    if ((reinterpret_cast<uintptr_t>(weight) & 3)) return QM_ERR_GEOMETRY;
    LinearParams prm = {};
    prm.input = input;
    prm.weight[0] = weight;
    prm.bias[0] = bias;
    prm.output[0] = output;
    prm.residual = residual;
    prm.rows[0] = output_columns;
    prm.reduction = reduction_columns;
    prm.weight[1] = prm.weight[2] = weight;   // never read: rows[1] = rows[2] = 0
    prm.output[1] = prm.output[2] = output;
    return launch_linear(prm, static_cast<hipStream_t>(hip_stream));
}

extern "C" int32_t qm_qkv_m1(const uint16_t* input, const uint16_t* q_weight, const uint16_t* q_bias,
                             const uint16_t* k_weight, const uint16_t* k_bias, const uint16_t* v_weight,
                             const uint16_t* v_bias, uint16_t* q_output, uint16_t* k_output,
                             uint16_t* v_output, int32_t hidden, int32_t q_dim, int32_t kv_dim,
                             void* hip_stream) {
    using namespace qm;
    if (!input || !q_weight || !k_weight || !v_weight || !q_output || !k_output || !v_output) return QM_ERR_NULL;
    if (q_dim < 0 || kv_dim < 0) return QM_ERR_ARGUMENT;
    const int32_t rc = check_reduction(hidden);
    if (rc != QM_OK) return rc;
    if ((reinterpret_cast<uintptr_t>(q_weight) | reinterpret_cast<uintptr_t>(k_weight)
         | reinterpret_cast<uintptr_t>(v_weight)) & 3)
        return QM_ERR_GEOMETRY;
    LinearParams prm = {};
    prm.input = input;
    prm.weight[0] = q_weight; prm.weight[1] = k_weight; prm.weight[2] = v_weight;
    prm.bias[0] = q_bias; prm.bias[1] = k_bias; prm.bias[2] = v_bias;
    prm.output[0] = q_output; prm.output[1] = k_output; prm.output[2] = v_output;
    prm.residual = nullptr;
    prm.rows[0] = q_dim; prm.rows[1] = kv_dim; prm.rows[2] = kv_dim;
    prm.reduction = hidden;
    return launch_linear(prm, static_cast<hipStream_t>(hip_stream));
}
