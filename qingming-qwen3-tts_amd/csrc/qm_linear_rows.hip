// qm_linear_rows.hip — linears over many token rows (the prompt pass), every output scalar
// bit-identical to the reference's one-wave-per-output kernel, for gfx950.
//
// Reference: native_ops::linear_wave32_bf16_f32acc_kernel (R17:126-196, reached through
// NativeTalkerEngine::linear_generic, R17:17453-17472, in ::prefill, R17:16620-16790), add_bf16_kernel
// and swiglu_kernel (R17:8729-8770).  An output (row r, column n) is 32 lane-strided fmaf chains
// over k = l, l + 32, ..., the shuffle tree, bias in fp32, one rounding to bf16 — the order of the
// M = 1 kernels, so a prompt row and a decode step of the same vector agree to the bit.
//
// That order rules out the matrix cores (an MFMA adds in its own order); this is a VALU kernel.
// A block owns up to eight output columns: their weight rows go from HBM into LDS once
// (global_load_lds), then the block walks the token rows eight at a time — the eight input
// rows are put into LDS as [k][8 rows] (an 8 x 8 register transpose on the way in, the next pass's
// pieces already requested) so that a thread, which is one chain (column c, lane l), fetches the
// eight inputs of a step with one 16-byte read and feeds eight accumulators with one weight.
// Weights are read from HBM once per launch, inputs once per block from L2.
// Optional epilogues fold the reference's next launch: residual add (add_bf16_kernel: the sum of
// two bf16 values, rounded) and, for the gate/up pair, SwiGLU (swiglu_kernel).

#include <type_traits>

#include "qm_device.h"
#include "qm_host.h"
#include "qm_linear_rows_params.h"

namespace qm {

constexpr int kRowsThreads = 256;
constexpr int kRowsTile = 8;                   // token rows per pass
constexpr int kRowsLdsBudget = 156 * 1024;
constexpr int kRowsMaxReduction = 16384;

__host__ __device__ inline int rows_w_stride(int reduction) { return 2 * reduction + 64; }   // bytes

// SPAN: token rows per thread and pass (8 with eight columns per block, 4 with four)
template <bool DUAL, int SPAN>
__global__ __launch_bounds__(kRowsThreads) void linear_rows_kernel(LinearRowsParams prm) {
    request_arguments(prm);
    extern __shared__ __attribute__((aligned(16))) unsigned char lr_smem[];
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int K = prm.reduction;
    constexpr int C = SPAN == 8 ? 8 : 4;
    const int w_stride = rows_w_stride(K);
    const int w_rows = DUAL ? 2 * C : C;
    unsigned char* lds_w = lr_smem;                                            // [w_rows][w_stride]
    uint4* lds_x = reinterpret_cast<uint4*>(lr_smem + w_rows * w_stride);      // [K] x 8 bf16 (one per token row)
    const int first = static_cast<int>(blockIdx.x) * C;

    // ---- this block's weight rows: HBM -> LDS, once (DUAL: rows 2c, 2c + 1 = gate, up of column first + c)
    for (int i = 0; i < w_rows; ++i) {
        const int column = first + (DUAL ? i >> 1 : i);
        if (column >= prm.columns) break;
        const unsigned char* src = reinterpret_cast<const unsigned char*>(prm.weight[DUAL ? (i & 1) : 0]
                                                                          + static_cast<int64_t>(column) * K);
        unsigned char* dst = lds_w + i * w_stride;
        for (int off = wave * 1024; off < 2 * K; off += 4 * 1024)
            if (off + lane * 16 < 2 * K)
                __builtin_amdgcn_global_load_lds(src + off + lane * 16, (__attribute__((address_space(3))) void*)(dst + off), 16, 0, 0);
    }

    // thread = chain (column c, reference lane l) for token rows [sub * span, sub * span + span) of a pass
    const int l = tid & 31;
    constexpr int span = SPAN;
    const int c = C == 8 ? tid >> 5 : (tid >> 5) & 3;
    const int sub = C == 8 ? 0 : tid >> 7;
    const int column = first + c;
    const bool live = column < prm.columns;
    const uint16_t* w0 = reinterpret_cast<const uint16_t*>(lds_w + (DUAL ? 2 * c : c) * w_stride) + l;
    const uint16_t* w1 = reinterpret_cast<const uint16_t*>(lds_w + (2 * c + 1) * w_stride) + l;   // DUAL only
    const int steps = (K + 31) >> 5;

    // Staging of a pass's eight token rows as [k][row]: a thread owns blocks of eight consecutive k
    // (block b = tid, tid + 256, ...), fetches that 16-byte piece of each of the eight rows,
    // transposes the 8 x 8 bf16 values in registers (v_perm) and writes eight 16-byte [k] entries.
    // The pieces of the next pass are requested before this pass is computed.
    const int k_blocks = K >> 3;
    auto fetch = [&](int row0, int b, uint4 (&piece)[8]) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const int row = min(row0 + r, prm.rows - 1);   // a row past the end repeats the last one (never stored)
            piece[r] = *reinterpret_cast<const uint4*>(prm.input + static_cast<int64_t>(row) * K + 8 * b);
        }
    };
    auto deposit = [&](int b, const uint4 (&piece)[8]) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {                      // k = 8 b + 2 e (low halves) and 8 b + 2 e + 1 (high halves)
            uint32_t word[8];
#pragma unroll
            for (int r = 0; r < 8; ++r) word[r] = e == 0 ? piece[r].x : e == 1 ? piece[r].y : e == 2 ? piece[r].z : piece[r].w;
            uint4 lo, hi;
            lo.x = __builtin_amdgcn_perm(word[1], word[0], 0x05040100U); hi.x = __builtin_amdgcn_perm(word[1], word[0], 0x07060302U);
            lo.y = __builtin_amdgcn_perm(word[3], word[2], 0x05040100U); hi.y = __builtin_amdgcn_perm(word[3], word[2], 0x07060302U);
            lo.z = __builtin_amdgcn_perm(word[5], word[4], 0x05040100U); hi.z = __builtin_amdgcn_perm(word[5], word[4], 0x07060302U);
            lo.w = __builtin_amdgcn_perm(word[7], word[6], 0x05040100U); hi.w = __builtin_amdgcn_perm(word[7], word[6], 0x07060302U);
            lds_x[8 * b + 2 * e] = lo;
            lds_x[8 * b + 2 * e + 1] = hi;
        }
    };
    // (the first block of a thread is kept in registers across the pass; further blocks, when K > 2048, are fetched late)
    uint4 ahead[8];
    if (tid < k_blocks) fetch(0, tid, ahead);

    for (int row0 = 0; row0 < prm.rows; row0 += kRowsTile) {
        __syncthreads();                                   // the pass before has read its inputs
        if (tid < k_blocks) deposit(tid, ahead);
        for (int b = tid + kRowsThreads; b < k_blocks; b += kRowsThreads) {
            uint4 piece[8];
            fetch(row0, b, piece);
            deposit(b, piece);
        }
        if (row0 + kRowsTile < prm.rows && tid < k_blocks) fetch(row0 + kRowsTile, tid, ahead);
        if (row0 == 0) __builtin_amdgcn_s_waitcnt(0);      // this wave's weight rows have landed
        __syncthreads();

        float acc[SPAN], up[SPAN];
#pragma unroll
        for (int r = 0; r < SPAN; ++r) acc[r] = up[r] = 0.0f;
        if (live) {
            typedef typename std::conditional<SPAN == 8, uint4, uint2>::type xrow_t;      // SPAN bf16 values of one k
            const xrow_t* xs = reinterpret_cast<const xrow_t*>(lds_x) + (SPAN == 8 ? 0 : sub);
            constexpr int x_stride = SPAN == 8 ? 1 : 2;                                    // entries of xrow_t per k
            auto step = [&](float a, float b, const xrow_t& x) {
                uint32_t words[SPAN / 2];
                __builtin_memcpy(words, &x, sizeof(x));
#pragma unroll
                for (int e = 0; e < SPAN / 2; ++e) {
                    const float x0 = lo_bf16(words[e]), x1 = hi_bf16(words[e]);
                    acc[2 * e] = fmaf(x0, a, acc[2 * e]);
                    acc[2 * e + 1] = fmaf(x1, a, acc[2 * e + 1]);
                    if (DUAL) {
                        up[2 * e] = fmaf(x0, b, up[2 * e]);
                        up[2 * e + 1] = fmaf(x1, b, up[2 * e + 1]);
                    }
                }
            };
            const int full = K >> 5;                       // steps in which every lane has an element
            int j = 0;
            for (; j + 4 <= full; j += 4) {                // four steps' operands are requested before the first is used
                float a[4], b[4];
                xrow_t x[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    a[u] = bf2f(w0[32 * (j + u)]);
                    b[u] = DUAL ? bf2f(w1[32 * (j + u)]) : 0.0f;
                    x[u] = xs[(32 * (j + u) + l) * x_stride];
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) step(a[u], b[u], x[u]);
            }
            // (a chain's last step may lie past the end of a row when K is not a multiple of 32)
            for (; j < steps; ++j) {
                const int k = 32 * j + l;
                if (k >= K) break;
                step(bf2f(w0[32 * j]), DUAL ? bf2f(w1[32 * j]) : 0.0f, xs[k * x_stride]);
            }
        }
        // the reference's shuffle tree over its 32 lanes, per token row; lane 0 holds the sums
#pragma unroll
        for (int r = 0; r < SPAN; ++r) {
            acc[r] = half_wave_tree_sum(acc[r]);
            if (DUAL) up[r] = half_wave_tree_sum(up[r]);
        }
        if (l == 0 && live) {
#pragma unroll
            for (int r = 0; r < SPAN; ++r) {
                const int row = row0 + sub * span + r;
                if (row < prm.rows) {
                    const int64_t at = static_cast<int64_t>(row) * prm.columns + column;
                    uint16_t v;
                    if (DUAL) {
                        const float gv = bf2f(f2bf(acc[r]));
                        const uint16_t act = f2bf(gv / (1.0f + expf(-gv)));
                        v = f2bf(bf2f(act) * bf2f(f2bf(up[r])));
                    } else {
                        float s = acc[r];
                        if (prm.bias) s += bf2f(prm.bias[column]);
                        v = f2bf(s);
                        if (prm.residual) v = f2bf(bf2f(prm.residual[at]) + bf2f(v));
                    }
                    prm.output[at] = v;
                }
            }
        }
    }
}

template <bool DUAL>
inline int32_t launch_rows(LinearRowsParams prm, hipStream_t s) {
    if (prm.rows == 0 || prm.columns == 0) return QM_OK;
    int columns_per_block = 0;
    size_t smem = 0;
    for (int c = 8; c >= 4; c >>= 1) {
        const size_t bytes = static_cast<size_t>(DUAL ? 2 * c : c) * rows_w_stride(prm.reduction)
                           + static_cast<size_t>(prm.reduction) * 16;
        if (bytes <= static_cast<size_t>(kRowsLdsBudget)) {
            columns_per_block = c;
            smem = bytes;
            break;
        }
    }
    if (!columns_per_block) return QM_ERR_GEOMETRY;
    prm.columns_per_block = columns_per_block;
    const unsigned blocks = static_cast<unsigned>((prm.columns + columns_per_block - 1) / columns_per_block);
    static std::atomic<bool> lds_raised[2][kMaxDevices];
    if (columns_per_block == 8) {
        const int32_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(linear_rows_kernel<DUAL, 8>), kRowsLdsBudget,
                                              lds_raised[0]);
        if (rc != QM_OK) return rc;
        hipLaunchKernelGGL((linear_rows_kernel<DUAL, 8>), dim3(blocks), dim3(kRowsThreads), smem, s, prm);
    } else {
        const int32_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(linear_rows_kernel<DUAL, 4>), kRowsLdsBudget,
                                              lds_raised[1]);
        if (rc != QM_OK) return rc;
        hipLaunchKernelGGL((linear_rows_kernel<DUAL, 4>), dim3(blocks), dim3(kRowsThreads), smem, s, prm);
    }
    return launch_status();
}

inline int32_t check_rows(const LinearRowsParams& prm, bool dual) {
    if (prm.rows < 0 || prm.columns < 0 || prm.reduction <= 0) return QM_ERR_ARGUMENT;
    // 16-byte pieces of the rows on both sides
    if ((prm.reduction & 7) || prm.reduction > kRowsMaxReduction) return QM_ERR_GEOMETRY;
    uintptr_t align = reinterpret_cast<uintptr_t>(prm.input) | reinterpret_cast<uintptr_t>(prm.weight[0]);
    if (dual) align |= reinterpret_cast<uintptr_t>(prm.weight[1]);
    if (align & 15) return QM_ERR_GEOMETRY;
    return QM_OK;
}

// QM_OPT_LINEAR_ROWS_KERNEL: 0 = the matrix cores from kRowsMatrixMinimum token rows on, where the shape fits their tiles
// (columns % 128 == 0, reduction % 128 == 0, 8-byte aligned rows of bias / residual / output); 1 = always the exact chain.
constexpr int kRowsMatrixMinimum = 16;
inline int32_t rows_on_matrix_cores(const LinearRowsParams& prm, int32_t* yes) {
    const int32_t choice = option_value(QM_OPT_LINEAR_ROWS_KERNEL);
    if (choice < 0 || choice > 1) return QM_ERR_ARGUMENT;
    const uintptr_t align = reinterpret_cast<uintptr_t>(prm.bias) | reinterpret_cast<uintptr_t>(prm.residual)
                          | reinterpret_cast<uintptr_t>(prm.output);
    *yes = choice == 0 && prm.rows >= kRowsMatrixMinimum && prm.columns % 128 == 0 && prm.reduction % 128 == 0 && (align & 7) == 0;
    return QM_OK;
}

}  // namespace qm

namespace qm {

// With a workspace the matrix-core path may cut the reduction (few token rows); the exact chain never uses it.
inline int32_t rows_entry(LinearRowsParams prm, bool dual, void* workspace, int64_t workspace_bytes, void* hip_stream) {
    if (workspace_bytes < 0 || (workspace_bytes > 0 && !workspace)) return QM_ERR_ARGUMENT;
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return QM_ERR_GEOMETRY;
    const int32_t rc = check_rows(prm, dual);
    if (rc != QM_OK) return rc;
    int32_t matrix_cores = 0;
    const int32_t rc_kernel = rows_on_matrix_cores(prm, &matrix_cores);
    if (rc_kernel != QM_OK) return rc_kernel;
    prm.reduction_parts = 1;
    prm.partials = nullptr;
    prm.groups = 1;
    if (!matrix_cores) return dual ? launch_rows<true>(prm, static_cast<hipStream_t>(hip_stream))
                                   : launch_rows<false>(prm, static_cast<hipStream_t>(hip_stream));
    if (workspace) {
        const size_t need = rows_mfma_workspace_bytes(prm.rows, prm.columns, prm.reduction, dual);
        if (need > 0) {
            if (static_cast<size_t>(workspace_bytes) < need) return QM_ERR_WORKSPACE;
            prm.reduction_parts = rows_mfma_reduction_parts(prm.rows, prm.columns, prm.reduction, dual);
            prm.partials = static_cast<float*>(workspace);
        }
    }
    return launch_rows_mfma(prm, dual, static_cast<hipStream_t>(hip_stream));
}

}  // namespace qm

extern "C" int32_t qm_linear_rows(const uint16_t* input, const uint16_t* weight, const uint16_t* bias,
                                  const uint16_t* residual, uint16_t* output, int32_t rows, int32_t output_columns,
                                  int32_t reduction_columns, void* hip_stream) {
    return qm_linear_rows_split(input, weight, bias, residual, output, rows, output_columns, reduction_columns, nullptr, 0, hip_stream);
}

extern "C" int32_t qm_gate_up_swiglu_rows(const uint16_t* input, const uint16_t* gate_weight, const uint16_t* up_weight,
                                          uint16_t* output, int32_t rows, int32_t hidden, int32_t intermediate,
                                          void* hip_stream) {
    return qm_gate_up_swiglu_rows_split(input, gate_weight, up_weight, output, rows, hidden, intermediate, nullptr, 0, hip_stream);
}

extern "C" int64_t qm_linear_rows_split_workspace_bytes(int32_t rows, int32_t output_columns, int32_t reduction_columns, int32_t gate_up_pair) {
    using namespace qm;
    if (rows < kRowsMatrixMinimum || output_columns <= 0 || reduction_columns <= 0 || output_columns % 128 || reduction_columns % 128) return 0;
    return static_cast<int64_t>(rows_mfma_workspace_bytes(rows, output_columns, reduction_columns, gate_up_pair != 0));
}

extern "C" int32_t qm_linear_rows_split(const uint16_t* input, const uint16_t* weight, const uint16_t* bias,
                                        const uint16_t* residual, uint16_t* output, int32_t rows, int32_t output_columns,
                                        int32_t reduction_columns, void* workspace, int64_t workspace_bytes, void* hip_stream) {
    using namespace qm;
    if (!input || !weight || !output) return QM_ERR_NULL;
    LinearRowsParams prm = {};
    prm.input = input; prm.weight[0] = weight; prm.weight[1] = weight; prm.bias = bias; prm.residual = residual;
    prm.output = output; prm.rows = rows; prm.columns = output_columns; prm.reduction = reduction_columns;
    return rows_entry(prm, false, workspace, workspace_bytes, hip_stream);
}

// Three linears of one input.  On the matrix cores: one grid over the column tiles of all three (the same sums and
// roundings as three calls: an output's k blocks are added in the same order whatever the tile); otherwise three calls.
extern "C" int32_t qm_qkv_rows_split(const uint16_t* input, const uint16_t* q_weight, const uint16_t* k_weight, const uint16_t* v_weight,
                                     const uint16_t* q_bias, const uint16_t* k_bias, const uint16_t* v_bias,
                                     uint16_t* q_output, uint16_t* k_output, uint16_t* v_output, int32_t rows, int32_t q_columns,
                                     int32_t kv_columns, int32_t reduction_columns, void* workspace, int64_t workspace_bytes,
                                     void* hip_stream) {
    using namespace qm;
    if (!input || !q_weight || !k_weight || !v_weight || !q_output || !k_output || !v_output) return QM_ERR_NULL;
    if (workspace_bytes < 0 || (workspace_bytes > 0 && !workspace)) return QM_ERR_ARGUMENT;
    LinearRowsParams prm = {};
    prm.input = input; prm.weight[0] = q_weight; prm.weight[1] = q_weight; prm.bias = q_bias; prm.output = q_output;
    prm.rows = rows; prm.columns = q_columns; prm.reduction = reduction_columns;
    LinearRowsParams other = prm;
    other.weight[0] = other.weight[1] = k_weight; other.bias = k_bias; other.output = k_output; other.columns = kv_columns;
    int32_t fused = 0, fused_other = 0;
    int32_t rc = check_rows(prm, false);
    if (rc == QM_OK) rc = check_rows(other, false);
    if (rc == QM_OK) rc = rows_on_matrix_cores(prm, &fused);
    if (rc == QM_OK) rc = rows_on_matrix_cores(other, &fused_other);
    if (rc != QM_OK) return rc;
    const uintptr_t align = reinterpret_cast<uintptr_t>(v_weight) | reinterpret_cast<uintptr_t>(v_bias) | reinterpret_cast<uintptr_t>(v_output);
    // (the one grid is never cut: at 128 rows it takes 11 us where three cut calls take 31)
    if (!fused || !fused_other || q_columns == 0 || kv_columns == 0 || (align & 15)) {
        rc = qm_linear_rows_split(input, q_weight, q_bias, nullptr, q_output, rows, q_columns, reduction_columns, workspace, workspace_bytes, hip_stream);
        if (rc == QM_OK)
            rc = qm_linear_rows_split(input, k_weight, k_bias, nullptr, k_output, rows, kv_columns, reduction_columns, workspace, workspace_bytes, hip_stream);
        if (rc == QM_OK)
            rc = qm_linear_rows_split(input, v_weight, v_bias, nullptr, v_output, rows, kv_columns, reduction_columns, workspace, workspace_bytes, hip_stream);
        return rc;
    }
    prm.reduction_parts = 1;
    prm.groups = 3;
    prm.group_first_tile[0] = q_columns / 128;
    prm.group_first_tile[1] = (q_columns + kv_columns) / 128;
    prm.group_weight[0] = k_weight; prm.group_bias[0] = k_bias; prm.group_output[0] = k_output; prm.group_columns[0] = kv_columns;
    prm.group_weight[1] = v_weight; prm.group_bias[1] = v_bias; prm.group_output[1] = v_output; prm.group_columns[1] = kv_columns;
    return launch_rows_mfma(prm, false, static_cast<hipStream_t>(hip_stream));
}

extern "C" int32_t qm_qkv_rows(const uint16_t* input, const uint16_t* q_weight, const uint16_t* k_weight, const uint16_t* v_weight,
                               const uint16_t* q_bias, const uint16_t* k_bias, const uint16_t* v_bias,
                               uint16_t* q_output, uint16_t* k_output, uint16_t* v_output, int32_t rows, int32_t q_columns,
                               int32_t kv_columns, int32_t reduction_columns, void* hip_stream) {
    return qm_qkv_rows_split(input, q_weight, k_weight, v_weight, q_bias, k_bias, v_bias, q_output, k_output, v_output, rows, q_columns,
                             kv_columns, reduction_columns, nullptr, 0, hip_stream);
}

extern "C" int32_t qm_gate_up_swiglu_rows_split(const uint16_t* input, const uint16_t* gate_weight, const uint16_t* up_weight,
                                                uint16_t* output, int32_t rows, int32_t hidden, int32_t intermediate,
                                                void* workspace, int64_t workspace_bytes, void* hip_stream) {
    using namespace qm;
    if (!input || !gate_weight || !up_weight || !output) return QM_ERR_NULL;
    LinearRowsParams prm = {};
    prm.input = input; prm.weight[0] = gate_weight; prm.weight[1] = up_weight;
    prm.output = output; prm.rows = rows; prm.columns = intermediate; prm.reduction = hidden;
    return rows_entry(prm, true, workspace, workspace_bytes, hip_stream);
}
