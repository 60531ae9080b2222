// qm_linear.hip — M = 1 weight-streaming linears (fused Q/K/V projection, o_proj / down_proj with
// bias and residual, gate/up projection with SwiGLU) for gfx950, bit-identical to the reference's
// kernels.
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
    // Fused prologue of the staged kernel (pre != 0): the input vector is produced in the block.
    int pre;                      // 1: RMSNorm(input) * norm_weight; 2: RMSNorm(bf16(input + addend)) * norm_weight
    const uint16_t* addend;       // pre == 2: the attention output added to the hidden state
    const uint16_t* norm_weight;  // [reduction]
    uint16_t* residual_out;       // pre == 2: bf16(input + addend), written by block 0
    float epsilon;
    int rows_per_block;           // staged kernel: outputs (channels) per block, 1..8
    // Order of a row's 32 chains (staged kernel).  0: lane l takes k = l, l + 32, ... (the talker's
    // kernels).  1: lane l takes the pairs k = 2l, 2l + 1, then 2l + 64, 2l + 65, ..., first
    // element first (the code predictor's kernels, R17:12110-12120, in their portable form: two
    // fmaf per pair; the gfx1100 build of the reference uses that chip's dot2 instruction).
    int pairs;
};

// DUAL: weight[0] / weight[1] are the gate and up matrices of one SwiGLU channel per output
// (talker_gate_up_swiglu_fused_kernel, R17:16289-16362): two dot products in the same order, each
// rounded to bf16, then act = bf16(g / (1 + expf(-g))) and out = bf16(act * u).
template <bool DUAL>
__global__ __launch_bounds__(kLinThreads) void linear_m1_kernel(LinearParams prm) {
    request_arguments(prm);
    extern __shared__ __attribute__((aligned(16))) float lin_x[];   // the input vector, fp32
    constexpr int kBatch = DUAL ? kLinBatch / 2 : kLinBatch;        // loads per matrix and register batch

    const int tid = threadIdx.x;
    const int q = tid & 15;                                         // lane within the output's row
    const int reduction = prm.reduction;
    const int steps = (reduction + 31) >> 5;

    // This lane's output: global row index over the concatenation of the (up to) three matrices.
    int row = static_cast<int>(blockIdx.x) * kLinRowsPerBlock + (tid >> 4);
    int m = 0;
    if (!DUAL && row >= prm.rows[0]) {
        row -= prm.rows[0];
        m = 1;
        if (row >= prm.rows[1]) {
            row -= prm.rows[1];
            m = 2;
        }
    }
    const bool live = row < prm.rows[m];
    const int64_t row_off = static_cast<int64_t>(live ? row : 0) * reduction;
    const uint16_t* wrow = prm.weight[m] + row_off;
    const uint16_t* urow = prm.weight[1] + row_off;   // DUAL only

    // Steps [j0, j0 + kBatch) of this lane's weight row(s): elements 32j + 2q, 32j + 2q + 1.
    // Unpredicated: a lane without an output reads row 0, a step past the end the last pair.
    auto load_batch = [&](uint32_t (&w)[kBatch], uint32_t (&u)[kBatch], int j0) {
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            const int k = min(32 * (j0 + i) + 2 * q, reduction - 2);
            w[i] = *reinterpret_cast<const uint32_t*>(wrow + k);
            if (DUAL) u[i] = *reinterpret_cast<const uint32_t*>(urow + k);
        }
    };
    uint32_t wa[kBatch], wb[kBatch], ua[kBatch], ub[kBatch];
    load_batch(wa, ua, 0);
    if (kBatch < steps) load_batch(wb, ub, kBatch);

    // fp32 input vector, zero-padded to whole steps of 32.
    for (int k = tid; k < 32 * steps; k += kLinThreads) lin_x[k] = k < reduction ? bf2f(prm.input[k]) : 0.0f;
    __syncthreads();

    float acc0 = 0.0f, acc1 = 0.0f, up0 = 0.0f, up1 = 0.0f;
    // A whole batch is straight-line code (the LDS reads of its input pairs are requested ahead of
    // the multiply-adds); a batch cut by the end of the reduction takes the per-step test, and in
    // a ragged last step the pairs past the end are multiplied as 0 * 0, which leaves the
    // accumulators (never -0) unchanged.
    auto consume_batch = [&](const uint32_t (&w)[kBatch], const uint32_t (&u)[kBatch], int j0) {
        const float* xs = lin_x + 32 * j0 + 2 * q;
        if (j0 + kBatch <= steps && 32 * steps == reduction) {
            float2 x[kBatch];
#pragma unroll
            for (int i = 0; i < kBatch; ++i) x[i] = *reinterpret_cast<const float2*>(xs + 32 * i);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                acc0 = fmaf(x[i].x, lo_bf16(w[i]), acc0);
                acc1 = fmaf(x[i].y, hi_bf16(w[i]), acc1);
                if (DUAL) {
                    up0 = fmaf(x[i].x, lo_bf16(u[i]), up0);
                    up1 = fmaf(x[i].y, hi_bf16(u[i]), up1);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                if (j0 + i < steps) {
                    const float2 x = *reinterpret_cast<const float2*>(xs + 32 * i);
                    const bool inside = 32 * (j0 + i) + 2 * q < reduction;
                    const uint32_t wi = inside ? w[i] : 0u;
                    acc0 = fmaf(x.x, lo_bf16(wi), acc0);
                    acc1 = fmaf(x.y, hi_bf16(wi), acc1);
                    if (DUAL) {
                        const uint32_t ui = inside ? u[i] : 0u;
                        up0 = fmaf(x.x, lo_bf16(ui), up0);
                        up1 = fmaf(x.y, hi_bf16(ui), up1);
                    }
                }
            }
        }
    };
    for (int j0 = 0; j0 < steps; j0 += 2 * kBatch) {
        consume_batch(wa, ua, j0);
        if (j0 + 2 * kBatch < steps) load_batch(wa, ua, j0 + 2 * kBatch);
        if (j0 + kBatch < steps) consume_batch(wb, ub, j0 + kBatch);
        if (j0 + 3 * kBatch < steps) load_batch(wb, ub, j0 + 3 * kBatch);
    }

    // The reference's tree over its 32 lanes, v += shfl_down(v, 16 / 8 / 4 / 2 / 1): chain c lives in
    // lane c/2, accumulator c%2, so +16, +8, +4, +2 are lanes q+8, q+4, q+2, q+1 (row_ror by
    // 8, 12, 14, 15 brings lane q+n to lane q) and +1 is the other accumulator of lane 0.
    auto tree = [&](float a0, float a1) {
        a0 += row_ror<8>(a0);
        a1 += row_ror<8>(a1);
        a0 += row_ror<12>(a0);
        a1 += row_ror<12>(a1);
        a0 += row_ror<14>(a0);
        a1 += row_ror<14>(a1);
        a0 += row_ror<15>(a0);
        a1 += row_ror<15>(a1);
        return a0 + a1;
    };
    const float a = tree(acc0, acc1);
    const float u_sum = DUAL ? tree(up0, up1) : 0.0f;
    if (q == 0 && live) {
        if (DUAL) {
            const float gv = bf2f(f2bf(a));
            const uint16_t act = f2bf(gv / (1.0f + expf(-gv)));
            prm.output[0][row] = f2bf(bf2f(act) * bf2f(f2bf(u_sum)));
        } else {
            float r = a;
            if (prm.bias[m]) r += bf2f(prm.bias[m][row]);
            uint16_t v = f2bf(r);
            if (prm.residual) v = f2bf(bf2f(prm.residual[row]) + bf2f(v));
            prm.output[m][row] = v;
        }
    }
}

template <bool DUAL>
inline int32_t launch_linear(const LinearParams& prm, hipStream_t s) {
    const int64_t total = DUAL ? prm.rows[0] : static_cast<int64_t>(prm.rows[0]) + prm.rows[1] + prm.rows[2];
    if (total == 0) return QM_OK;
    const size_t smem = static_cast<size_t>((prm.reduction + 31) / 32 * 32) * sizeof(float);
    static std::atomic<bool> lds_raised[kMaxDevices];
    const int32_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(linear_m1_kernel<DUAL>),
                                          kLinMaxReduction * static_cast<int>(sizeof(float)), lds_raised);
    if (rc != QM_OK) return rc;
    const unsigned blocks = static_cast<unsigned>((total + kLinRowsPerBlock - 1) / kLinRowsPerBlock);
    hipLaunchKernelGGL(linear_m1_kernel<DUAL>, dim3(blocks), dim3(kLinThreads), smem, s, prm);
    return launch_status();
}

// ---- the staged kernel ---------------------------------------------------------------------------------
// The register path above can keep at most 64 loads of a lane in flight (the hardware's counter
// of outstanding vector memory instructions), which is 4 KB per output whatever the lane layout, and
// the order of a chain's additions forbids splitting one output over more lanes: 2 048 outputs of a
// 6 144-wide reduction moved 1.1 TB/s.  Here the memory traffic is decoupled from the summation
// order: a block copies the weight rows of its (up to) eight outputs straight from HBM into LDS
// with 16-byte global_load_lds instructions — every byte of the matrix is requested at once
// across the chip, no registers held — and only then do 8 x 32 threads walk their chains, one
// reference lane each, reading 2-byte weights and the fp32 input from LDS.  LDS rows are padded by
// 64 bytes so the two rows a wave reads in one instruction fall on different banks.
// The block may also produce its input vector itself (RMSNorm of the hidden state, or residual
// add + post-norm), in the reference kernels' own thread layout and summation order, while the
// weights are in flight; that removes two single-block launches from a decode layer.
// (Measured and dropped: blocks that loop over several output groups through two LDS stages, the
// next group's rows streaming in while the current chains run — gate/up 24 us instead of 26 us, but
// the halved group size it needs cost the down projection 18 us instead of 15.5 us and Q/K/V 12 us
// instead of 11 us: a launch here is start + first HBM latency + tail around its streaming time.)
constexpr int kStagedThreads = 256;
constexpr int kStagedMaxRows = 8;
constexpr int kStagedXPerThread = 24;    // input columns a thread can hold in registers (reductions up to 6144)
constexpr int kStagedLdsBudget = 156 * 1024;

__host__ __device__ inline int staged_row_stride(int reduction) { return 2 * reduction + 64; }   // bytes
__host__ __device__ inline int staged_x_floats(int reduction) { return (reduction + 31) / 32 * 32; }

template <bool DUAL>
__global__ __launch_bounds__(kStagedThreads) void linear_m1_staged_kernel(LinearParams prm) {
    request_arguments(prm);
    extern __shared__ __attribute__((aligned(16))) unsigned char st_smem[];
    __shared__ float sh_waves[8];
    __shared__ float sh_total;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int K = prm.reduction;
    const int R = prm.rows_per_block;
    const int row_stride = staged_row_stride(K);
    float* lin_x = reinterpret_cast<float*>(st_smem);
    unsigned char* lds_w = st_smem + staged_x_floats(K) * sizeof(float);
    const int first = static_cast<int>(blockIdx.x) * R;     // first output (channel) of the block

    // Kernel arguments indexed by a run-time matrix number would be fetched again from the argument buffer at
    // every use (a scalar load and its wait each: 4 500 cycles for the eight rows of a block, measured); the three
    // entries are picked by selects instead.
    const int rows0 = prm.rows[0], rows1 = prm.rows[1], rows2 = prm.rows[2];
    const uint16_t* const weight0 = prm.weight[0];
    const uint16_t* const weight1 = prm.weight[1];
    const uint16_t* const weight2 = prm.weight[2];
    auto matrix_of = [&](int& out) {                        // global output -> (matrix, row in it)
        int m = 0;
        if (out >= rows0) {
            out -= rows0;
            m = 1;
            if (out >= rows1) {
                out -= rows1;
                m = 2;
            }
        }
        return m;
    };

    // ---- request the weight rows: LDS row i of the block <- row (first + i) of its matrix ----------
    // (DUAL: LDS rows 2c, 2c+1 are the gate and up rows of channel first + c)
    // The block's rows nearly always lie in one matrix and inside it: then they are requested by straight-line
    // code (eight rows found one by one, with the matrix looked up per row, took 3 200 cycles of scalar branches
    // before the first byte was even asked for).
    const int row_bytes = 2 * K;
    auto request_row = [&](const unsigned char* src, int i) {
        unsigned char* dst = lds_w + i * row_stride;
        for (int off = wave * 1024; off < row_bytes; off += 4 * 1024) {
            if (off + lane * 16 < row_bytes) {
                __builtin_amdgcn_global_load_lds(src + off + lane * 16,
                                                 (__attribute__((address_space(3))) void*)(dst + off),
                                                 16, 0, 0);
            }
        }
    };
    {
        int first_row = first;
        const int first_matrix = DUAL ? 0 : matrix_of(first_row);
        const int matrix_rows = first_matrix == 0 ? rows0 : (first_matrix == 1 ? rows1 : rows2);
        if (first_row + R <= matrix_rows) {
            const uint16_t* matrix = first_matrix == 0 ? weight0 : (first_matrix == 1 ? weight1 : weight2);
            const unsigned char* src = reinterpret_cast<const unsigned char*>(matrix + static_cast<int64_t>(first_row) * K);   // (advances row by row)
            const unsigned char* src_up = reinterpret_cast<const unsigned char*>(weight1 + static_cast<int64_t>(first_row) * K);
            // (a rolled loop: after its first turn the instructions come from the cache)
#pragma unroll 1
            for (int i = 0; i < R; ++i) {
                if (DUAL) {
                    request_row(src, 2 * i);
                    request_row(src_up, 2 * i + 1);
                    src_up += row_bytes;
                } else {
                    request_row(src, i);
                }
                src += row_bytes;
            }
        } else {
            const int lds_rows = DUAL ? 2 * R : R;
            for (int i = 0; i < lds_rows; ++i) {
                int out = first + (DUAL ? i >> 1 : i);
                const int m = DUAL ? (i & 1) : matrix_of(out);
                if (out >= (DUAL ? rows0 : (m == 0 ? rows0 : (m == 1 ? rows1 : rows2)))) break;   // past the last output (wave-uniform)
                const uint16_t* matrix = m == 0 ? weight0 : (m == 1 ? weight1 : weight2);
                request_row(reinterpret_cast<const unsigned char*>(matrix + static_cast<int64_t>(out) * K), i);
            }
        }
    }

    // ---- the input vector, requested at once: thread t holds columns t, t + 256, ... (up to kStagedXPerThread of
    // them; longer inputs take the loops below) ----
    const bool x_in_registers = K <= kStagedThreads * kStagedXPerThread;
    // (32-bit holders: two 16-bit values sharing a register would make the second load wait for the first)
    uint32_t x_raw[kStagedXPerThread], add_raw[kStagedXPerThread], norm_raw[kStagedXPerThread];
    // A kernel starts with a cold instruction cache: every instruction it executes for the first time costs tens
    // of cycles of fetch (measured: this kernel's timeline follows the number of distinct instructions on its
    // path far more than its arithmetic), so the columns are stepped through in batches of four with one test per
    // batch, nothing is initialised that is not used, and `each_column` below visits exactly what was loaded.
    auto fetch_columns = [&](const uint16_t* src, uint32_t (&dst)[kStagedXPerThread]) {
#pragma unroll
        for (int i0 = 0; i0 < kStagedXPerThread; i0 += 4) {
            if (kStagedThreads * i0 < K) {
#pragma unroll
                for (int i = i0; i < i0 + 4; ++i) dst[i] = src[min(tid + kStagedThreads * i, K - 1)];
            }
        }
    };
    // f(i, k) for this thread's columns k = tid + 256 i < K
    auto each_column = [&](auto&& f) {
#pragma unroll
        for (int i0 = 0; i0 < kStagedXPerThread; i0 += 4) {
            if (kStagedThreads * i0 < K) {
#pragma unroll
                for (int i = i0; i < i0 + 4; ++i) {
                    const int k = tid + kStagedThreads * i;
                    if (k < K) f(i, k);
                }
            }
        }
    };
    if (x_in_registers) {
        fetch_columns(prm.input, x_raw);
        if (prm.pre != 0) fetch_columns(prm.norm_weight, norm_raw);
        if (prm.pre == 2) fetch_columns(prm.addend, add_raw);
    }

    // ---- what the epilogue adds (bias, residual) is requested now as well, by the lane that will use it ----
    const int c = tid >> 5;             // output (channel) within the block
    const int l = tid & 31;             // reference lane
    const bool live = c < R && first + c < (DUAL ? rows0 : rows0 + rows1 + rows2);
    int out_row = first + c;
    int out_matrix = 0;
    uint32_t bias_raw = 0, residual_raw = 0;
    bool has_bias = false;
    if (!DUAL && live && l == 0) {
        out_matrix = matrix_of(out_row);
        const uint16_t* bias = out_matrix == 0 ? prm.bias[0] : (out_matrix == 1 ? prm.bias[1] : prm.bias[2]);
        has_bias = bias != nullptr;
        if (has_bias) bias_raw = bias[out_row];
        if (prm.residual) residual_raw = prm.residual[out_row];
    }

    // ---- the input vector as fp32, zero-padded to whole steps of 32 -----------------------------------
    const int steps = (K + 31) >> 5;
    if (prm.pre == 0) {
        if (x_in_registers) {
            each_column([&](int i, int k) { lin_x[k] = bf2f(static_cast<uint16_t>(x_raw[i])); });
            if (tid < 32 * steps - K) lin_x[K + tid] = 0.0f;     // the padding of the last step
        } else {
            // (eight loads at a time: one load per turn would wait for each in turn)
            for (int k0 = tid; k0 < 32 * steps; k0 += 8 * kStagedThreads) {
                uint32_t raw[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) raw[u] = prm.input[min(k0 + kStagedThreads * u, K - 1)];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int k = k0 + kStagedThreads * u;
                    if (k < 32 * steps) lin_x[k] = k < K ? bf2f(static_cast<uint16_t>(raw[u])) : 0.0f;
                }
            }
        }
    } else {
        // rmsnorm_kernel (R17:8276-8338) / talker_add_postnorm_fused_kernel (R17:16205-16286): thread t
        // sums the squares of columns t, t+256, ... with fmaf; block tree; two roundings per element.
        float local_sum = 0.0f;
        auto take = [&](int k, uint16_t x_bits, uint16_t add_bits) {
            float v = bf2f(x_bits);
            if (prm.pre == 2) {
                const uint16_t r = f2bf(v + bf2f(add_bits));
                if (blockIdx.x == 0) prm.residual_out[k] = r;
                v = bf2f(r);
            }
            lin_x[k] = v;
            local_sum = fmaf(v, v, local_sum);
        };
        if (x_in_registers) {
            each_column([&](int i, int k) {
                take(k, static_cast<uint16_t>(x_raw[i]), prm.pre == 2 ? static_cast<uint16_t>(add_raw[i]) : static_cast<uint16_t>(0));
            });
        } else {
            for (int k = tid; k < K; k += kStagedThreads) take(k, prm.input[k], prm.pre == 2 ? prm.addend[k] : static_cast<uint16_t>(0));
        }
        const float total = block_sum_256_like_reference(local_sum, sh_waves, &sh_total);
        const float inverse_rms = 1.0f / sqrtf(total / static_cast<float>(K) + prm.epsilon);
        if (x_in_registers) {
            each_column([&](int i, int k) {
                lin_x[k] = round_bf16(round_bf16(lin_x[k] * inverse_rms) * bf2f(static_cast<uint16_t>(norm_raw[i])));
            });
            if (tid < 32 * steps - K) lin_x[K + tid] = 0.0f;     // the padding of the last step
        } else {
            for (int k = tid; k < 32 * steps; k += kStagedThreads) {
                float y = 0.0f;
                if (k < K) y = round_bf16(round_bf16(lin_x[k] * inverse_rms) * bf2f(prm.norm_weight[k]));
                lin_x[k] = y;
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(0);      // this wave's global_load_lds writes have landed
    __syncthreads();

    // ---- 32 chains per output, one thread each: k = l, l+32, ... in increasing k ----------------------
    const uint16_t* w0 = reinterpret_cast<const uint16_t*>(lds_w + (DUAL ? 2 * c : c) * row_stride) + l;
    const uint16_t* w1 = reinterpret_cast<const uint16_t*>(lds_w + (2 * c + 1) * row_stride) + l;   // DUAL only
    const float* xs = lin_x + l;
    float acc = 0.0f, up = 0.0f;
    if (live && prm.pairs) {
        const uint32_t* p0 = reinterpret_cast<const uint32_t*>(lds_w + (DUAL ? 2 * c : c) * row_stride) + l;
        const uint32_t* p1 = reinterpret_cast<const uint32_t*>(lds_w + (2 * c + 1) * row_stride) + l;   // DUAL only
        const float2* xp = reinterpret_cast<const float2*>(lin_x) + l;
        const int full = K >> 6;        // steps of 32 pairs in which every lane has a pair
        const int pair_steps = (K + 63) >> 6;
        int j = 0;
        for (; j + 8 <= full; j += 8) {
            float2 x[8];
            uint32_t a[8], b[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                x[u] = xp[32 * (j + u)];
                a[u] = p0[32 * (j + u)];
                if (DUAL) b[u] = p1[32 * (j + u)];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                acc = fmaf(x[u].x, lo_bf16(a[u]), acc);
                acc = fmaf(x[u].y, hi_bf16(a[u]), acc);
                if (DUAL) {
                    up = fmaf(x[u].x, lo_bf16(b[u]), up);
                    up = fmaf(x[u].y, hi_bf16(b[u]), up);
                }
            }
        }
        for (; j < pair_steps; ++j) {
            if (64 * j + 2 * l + 1 < K) {
                const float2 x = xp[32 * j];
                const uint32_t a = p0[32 * j];
                acc = fmaf(x.x, lo_bf16(a), acc);
                acc = fmaf(x.y, hi_bf16(a), acc);
                if (DUAL) {
                    const uint32_t b = p1[32 * j];
                    up = fmaf(x.x, lo_bf16(b), up);
                    up = fmaf(x.y, hi_bf16(b), up);
                }
            }
        }
    } else if (live) {
        const int full = K >> 5;        // steps in which every lane has an element
        int j = 0;
        for (; j + 8 <= full; j += 8) {
            float x[8], a[8], b[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                x[u] = xs[32 * (j + u)];
                a[u] = bf2f(w0[32 * (j + u)]);
                if (DUAL) b[u] = bf2f(w1[32 * (j + u)]);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                acc = fmaf(x[u], a[u], acc);
                if (DUAL) up = fmaf(x[u], b[u], up);
            }
        }
        for (; j < steps; ++j) {
            if (32 * j + l < K) {
                acc = fmaf(xs[32 * j], bf2f(w0[32 * j]), acc);
                if (DUAL) up = fmaf(xs[32 * j], bf2f(w1[32 * j]), up);
            }
        }
    }
    // the reference's shuffle tree over its 32 lanes; lane 0 holds the sum
    acc = half_wave_tree_sum(acc);
    if (DUAL) up = half_wave_tree_sum(up);
    if (l == 0 && live) {
        if (DUAL) {
            const float gv = bf2f(f2bf(acc));
            const uint16_t act = f2bf(gv / (1.0f + expf(-gv)));
            prm.output[0][out_row] = f2bf(bf2f(act) * bf2f(f2bf(up)));
        } else {
            float r = acc;
            if (has_bias) r += bf2f(static_cast<uint16_t>(bias_raw));
            uint16_t v = f2bf(r);
            if (prm.residual) v = f2bf(bf2f(static_cast<uint16_t>(residual_raw)) + bf2f(v));
            uint16_t* output = out_matrix == 0 ? prm.output[0] : (out_matrix == 1 ? prm.output[1] : prm.output[2]);
            output[out_row] = v;
        }
    }
}

// Outputs per block of the staged kernel for this reduction length, 0 if even one row does not fit.
template <bool DUAL>
inline int staged_rows_per_block(int reduction) {
    for (int r = kStagedMaxRows; r >= 1; r >>= 1) {
        const int64_t bytes = static_cast<int64_t>(staged_x_floats(reduction)) * 4
                            + static_cast<int64_t>(DUAL ? 2 * r : r) * staged_row_stride(reduction);
        if (bytes <= kStagedLdsBudget) return r;
    }
    return 0;
}

// The staged kernel needs 16-byte pieces: reduction % 8 == 0 and 16-byte aligned weight rows.
inline bool staged_ok(const LinearParams& prm, bool dual) {
    if (prm.reduction & 7) return false;
    const int n = dual ? 2 : 3;
    for (int i = 0; i < n; ++i)
        if (reinterpret_cast<uintptr_t>(prm.weight[i]) & 15) return false;
    return true;
}

template <bool DUAL>
inline int32_t launch_staged(LinearParams prm, hipStream_t s) {
    const int64_t total = DUAL ? prm.rows[0] : static_cast<int64_t>(prm.rows[0]) + prm.rows[1] + prm.rows[2];
    if (total == 0 && prm.pre != 2) return QM_OK;
    const int r = staged_rows_per_block<DUAL>(prm.reduction);
    prm.rows_per_block = r;
    const size_t smem = static_cast<size_t>(staged_x_floats(prm.reduction)) * 4
                      + static_cast<size_t>(DUAL ? 2 * r : r) * staged_row_stride(prm.reduction);
    static std::atomic<bool> lds_raised[kMaxDevices];
    const int32_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(linear_m1_staged_kernel<DUAL>), kStagedLdsBudget,
                                          lds_raised);
    if (rc != QM_OK) return rc;
    const int64_t blocks = total == 0 ? 1 : (total + r - 1) / r;
    hipLaunchKernelGGL(linear_m1_staged_kernel<DUAL>, dim3(static_cast<unsigned>(blocks)), dim3(kStagedThreads), smem, s, prm);
    return launch_status();
}

inline int32_t check_reduction(int32_t reduction) {
    if (reduction <= 0) return QM_ERR_ARGUMENT;
    // 32-bit weight loads of element pairs; the fp32 copy of the input lives in LDS.
    if ((reduction & 1) || reduction > kLinMaxReduction) return QM_ERR_GEOMETRY;
    return QM_OK;
}

// ---- the entry points' bodies; `pairs` selects the order of the chains (LinearParams::pairs) ------------
inline int32_t linear_entry(int pairs, const uint16_t* input, const uint16_t* weight, const uint16_t* bias,
                            const uint16_t* residual, uint16_t* output, int32_t output_columns,
                            int32_t reduction_columns, void* hip_stream) {
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
    prm.pairs = pairs;
    if (staged_ok(prm, false) && staged_rows_per_block<false>(prm.reduction) > 0)
        return launch_staged<false>(prm, static_cast<hipStream_t>(hip_stream));
    if (pairs) return QM_ERR_GEOMETRY;        // the pair order exists in the staged kernel only
    return launch_linear<false>(prm, static_cast<hipStream_t>(hip_stream));
}

// pre: 0 = the input is given; 1 = RMSNorm(input) * norm_weight is computed in the kernel
inline int32_t qkv_entry(int pairs, int pre, const uint16_t* input, const uint16_t* norm_weight, float epsilon,
                         const uint16_t* q_weight, const uint16_t* q_bias, const uint16_t* k_weight,
                         const uint16_t* k_bias, const uint16_t* v_weight, const uint16_t* v_bias,
                         uint16_t* q_output, uint16_t* k_output, uint16_t* v_output, int32_t hidden,
                         int32_t q_dim, int32_t kv_dim, void* hip_stream) {
    if (!input || !q_weight || !k_weight || !v_weight || !q_output || !k_output || !v_output) return QM_ERR_NULL;
    if (pre && !norm_weight) return QM_ERR_NULL;
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
    prm.pairs = pairs;
    prm.pre = pre; prm.norm_weight = norm_weight; prm.epsilon = epsilon;
    if (staged_ok(prm, false) && staged_rows_per_block<false>(prm.reduction) > 0)
        return launch_staged<false>(prm, static_cast<hipStream_t>(hip_stream));
    if (pairs || pre) return QM_ERR_GEOMETRY;  // the pair order and the fused prologue exist in the staged kernel only
    return launch_linear<false>(prm, static_cast<hipStream_t>(hip_stream));
}

// pre: 0 = the input is given; 2 = residual = bf16(input + attention), RMSNorm(residual) * norm_weight
inline int32_t gate_up_entry(int pairs, int pre, const uint16_t* input, const uint16_t* attention,
                             const uint16_t* norm_weight, float epsilon, uint16_t* residual,
                             const uint16_t* gate_weight, const uint16_t* up_weight, uint16_t* output,
                             int32_t hidden, int32_t intermediate, void* hip_stream) {
    if (!input || !gate_weight || !up_weight || !output) return QM_ERR_NULL;
    if (pre && (!attention || !norm_weight || !residual)) return QM_ERR_NULL;
    if (intermediate < 0) return QM_ERR_ARGUMENT;
    const int32_t rc = check_reduction(hidden);
    if (rc != QM_OK) return rc;
    if ((reinterpret_cast<uintptr_t>(gate_weight) | reinterpret_cast<uintptr_t>(up_weight)) & 3) return QM_ERR_GEOMETRY;
    LinearParams prm = {};
    prm.input = input;
    prm.weight[0] = gate_weight; prm.weight[1] = up_weight; prm.weight[2] = gate_weight;
    prm.output[0] = prm.output[1] = prm.output[2] = output;
    prm.rows[0] = intermediate;
    prm.reduction = hidden;
    prm.pairs = pairs;
    prm.pre = pre; prm.addend = attention; prm.norm_weight = norm_weight; prm.epsilon = epsilon;
    prm.residual_out = residual;
    if (staged_ok(prm, true) && staged_rows_per_block<true>(prm.reduction) > 0)
        return launch_staged<true>(prm, static_cast<hipStream_t>(hip_stream));
    if (pairs || pre) return QM_ERR_GEOMETRY;
    return launch_linear<true>(prm, static_cast<hipStream_t>(hip_stream));
}

}  // namespace qm

extern "C" int32_t qm_linear_m1(const uint16_t* input, const uint16_t* weight, const uint16_t* bias,
                                const uint16_t* residual, uint16_t* output, int32_t output_columns,
                                int32_t reduction_columns, void* hip_stream) {
    return qm::linear_entry(0, input, weight, bias, residual, output, output_columns, reduction_columns, hip_stream);
}

extern "C" int32_t qm_qkv_m1(const uint16_t* input, const uint16_t* q_weight, const uint16_t* q_bias,
                             const uint16_t* k_weight, const uint16_t* k_bias, const uint16_t* v_weight,
                             const uint16_t* v_bias, uint16_t* q_output, uint16_t* k_output,
                             uint16_t* v_output, int32_t hidden, int32_t q_dim, int32_t kv_dim,
                             void* hip_stream) {
    return qm::qkv_entry(0, 0, input, nullptr, 0.0f, q_weight, q_bias, k_weight, k_bias, v_weight, v_bias,
                         q_output, k_output, v_output, hidden, q_dim, kv_dim, hip_stream);
}

extern "C" int32_t qm_gate_up_swiglu_m1(const uint16_t* input, const uint16_t* gate_weight, const uint16_t* up_weight,
                                        uint16_t* output, int32_t hidden, int32_t intermediate, void* hip_stream) {
    return qm::gate_up_entry(0, 0, input, nullptr, nullptr, 0.0f, nullptr, gate_weight, up_weight, output, hidden,
                             intermediate, hip_stream);
}

// ---- fusions of two reference launches each (staged kernel only) -------------------------------------
extern "C" int32_t qm_rmsnorm_qkv_m1(const uint16_t* hidden_state, const uint16_t* norm_weight, float epsilon,
                                     const uint16_t* q_weight, const uint16_t* q_bias,
                                     const uint16_t* k_weight, const uint16_t* k_bias,
                                     const uint16_t* v_weight, const uint16_t* v_bias,
                                     uint16_t* q_output, uint16_t* k_output, uint16_t* v_output,
                                     int32_t hidden, int32_t q_dim, int32_t kv_dim, void* hip_stream) {
    return qm::qkv_entry(0, 1, hidden_state, norm_weight, epsilon, q_weight, q_bias, k_weight, k_bias, v_weight,
                         v_bias, q_output, k_output, v_output, hidden, q_dim, kv_dim, hip_stream);
}

extern "C" int32_t qm_add_postnorm_gate_up_swiglu_m1(const uint16_t* hidden_state, const uint16_t* attention,
                                                     const uint16_t* norm_weight, float epsilon, uint16_t* residual,
                                                     const uint16_t* gate_weight, const uint16_t* up_weight,
                                                     uint16_t* output, int32_t hidden, int32_t intermediate,
                                                     void* hip_stream) {
    if (!attention || !norm_weight || !residual) return QM_ERR_NULL;
    return qm::gate_up_entry(0, 2, hidden_state, attention, norm_weight, epsilon, residual, gate_weight, up_weight,
                             output, hidden, intermediate, hip_stream);
}

// ---- the code predictor's twins: the pair order of the chains, no bias ---------------------------------
extern "C" int32_t qm_predictor_linear_m1(const uint16_t* input, const uint16_t* weight, const uint16_t* residual,
                                          uint16_t* output, int32_t output_columns, int32_t reduction_columns,
                                          void* hip_stream) {
    return qm::linear_entry(1, input, weight, nullptr, residual, output, output_columns, reduction_columns, hip_stream);
}

extern "C" int32_t qm_predictor_qkv_m1(const uint16_t* input, const uint16_t* q_weight, const uint16_t* k_weight,
                                       const uint16_t* v_weight, uint16_t* q_output, uint16_t* k_output,
                                       uint16_t* v_output, int32_t hidden, int32_t q_dim, int32_t kv_dim,
                                       void* hip_stream) {
    return qm::qkv_entry(1, 0, input, nullptr, 0.0f, q_weight, nullptr, k_weight, nullptr, v_weight, nullptr,
                         q_output, k_output, v_output, hidden, q_dim, kv_dim, hip_stream);
}

extern "C" int32_t qm_predictor_gate_up_swiglu_m1(const uint16_t* input, const uint16_t* gate_weight,
                                                  const uint16_t* up_weight, uint16_t* output, int32_t hidden,
                                                  int32_t intermediate, void* hip_stream) {
    return qm::gate_up_entry(1, 0, input, nullptr, nullptr, 0.0f, nullptr, gate_weight, up_weight, output, hidden,
                             intermediate, hip_stream);
}

extern "C" int32_t qm_predictor_rmsnorm_qkv_m1(const uint16_t* hidden_state, const uint16_t* norm_weight, float epsilon,
                                               const uint16_t* q_weight, const uint16_t* k_weight,
                                               const uint16_t* v_weight, uint16_t* q_output, uint16_t* k_output,
                                               uint16_t* v_output, int32_t hidden, int32_t q_dim, int32_t kv_dim,
                                               void* hip_stream) {
    return qm::qkv_entry(1, 1, hidden_state, norm_weight, epsilon, q_weight, nullptr, k_weight, nullptr, v_weight,
                         nullptr, q_output, k_output, v_output, hidden, q_dim, kv_dim, hip_stream);
}

extern "C" int32_t qm_predictor_add_postnorm_gate_up_swiglu_m1(const uint16_t* hidden_state, const uint16_t* attention,
                                                               const uint16_t* norm_weight, float epsilon,
                                                               uint16_t* residual, const uint16_t* gate_weight,
                                                               const uint16_t* up_weight, uint16_t* output,
                                                               int32_t hidden, int32_t intermediate, void* hip_stream) {
    if (!attention || !norm_weight || !residual) return QM_ERR_NULL;
    return qm::gate_up_entry(1, 2, hidden_state, attention, norm_weight, epsilon, residual, gate_weight, up_weight,
                             output, hidden, intermediate, hip_stream);
}
