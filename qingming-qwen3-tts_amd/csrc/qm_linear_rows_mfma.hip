// qm_linear_rows_mfma.hip — the prompt pass's linears over many token rows on the bf16 matrix cores (gfx950).
//
// out[m][n] = bf16(sum_k x[m][k] w[n][k] + bias[n]) (+ residual, or the SwiGLU of a gate/up pair): what
// native_ops::linear_bf16 computes per (row, column) (R17:126-245, reached through NativeTalkerEngine::linear_generic,
// R17:17453-17472, in ::prefill, R17:16620-16790), with the fp32 sum taken by v_mfma_f32_32x32x16_bf16 in its own order
// instead of the reference's 32 lane-strided chains: bf16 inputs, fp32 accumulation, the same roundings after the sum,
// results within the operators' tolerance of the exact-chain kernel (qm_linear_rows.hip), not bit-identical to it.
//
// A block of four waves owns 128 token rows x 128 output columns; a wave 64 x 64 as 2 x 2 MFMA tiles.  Both operands
// are K-contiguous rows (x [m][k], w [n][k]), so one tile layout serves both: 64 k per step, a row of a tile is eight
// 16-byte pieces in LDS, piece q of row r stored in slot q ^ (r % 8) so that the 32 rows a fragment read touches spread
// over all banks.  An MFMA takes the weight rows as its A operand and the token rows as B (D = W X^T): a lane then
// holds, for one token row, runs of four consecutive output columns — 8-byte stores.  The tiles of step t + 2 are
// requested into registers before step t's MFMAs and written to LDS (three stages) an iteration later: one barrier
// per step, two steps of arithmetic for a request to come back.  Bound: bf16 MFMA (2.5 PFLOP/s); algorithmic flops 2 m n k (x 2 for the gate/up pair).

#include "qm_device.h"
#include "qm_host.h"
#include "qm_linear_rows_params.h"

namespace qm {
namespace {

constexpr int kGmThreads = 256;
constexpr int kGmTile = 128;                 // token rows and output columns per block
constexpr int kGmStep = 64;                  // k per step
constexpr int kGmTileBytes = kGmTile * kGmStep * 2;   // 16 KiB per operand tile

typedef float f32x16_t __attribute__((ext_vector_type(16)));

// LDS byte offset of piece `piece` (16 bytes = 8 k) of row `row` inside a tile
__device__ __forceinline__ int tile_slot(int row, int piece) { return (row * 8 + (piece ^ (row & 7))) * 16; }

// A thread's share of one step's tiles on its way from memory to LDS: four 16-byte pieces per operand, kept as
// vectors with constant element numbers (arrays carried round the loop end up in scratch memory).
typedef uint32_t u32x16_t __attribute__((ext_vector_type(16)));
struct GmStaged {
    u32x16_t x, w, u;
};
__device__ __forceinline__ void gm_take(u32x16_t& to, const uint16_t* const (&src)[4], int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint4 v = *reinterpret_cast<const uint4*>(src[i] + k0);
        to[4 * i] = v.x; to[4 * i + 1] = v.y; to[4 * i + 2] = v.z; to[4 * i + 3] = v.w;
    }
}
__device__ __forceinline__ void gm_put(const u32x16_t& from, const int (&dst)[4], unsigned char* tile) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
        *reinterpret_cast<uint4*>(tile + dst[i]) = make_uint4(from[4 * i], from[4 * i + 1], from[4 * i + 2], from[4 * i + 3]);
}
template <bool DUAL>
__device__ __forceinline__ void gm_request(GmStaged& st, const uint16_t* const (&sx)[4], const uint16_t* const (&sw)[4],
                                           const uint16_t* const (&su)[4], int k0) {
    gm_take(st.x, sx, k0);
    gm_take(st.w, sw, k0);
    if (DUAL) gm_take(st.u, su, k0);
}
template <bool DUAL>
__device__ __forceinline__ void gm_deposit(const GmStaged& st, const int (&dst)[4], unsigned char* stage) {
    gm_put(st.x, dst, stage);
    gm_put(st.w, dst, stage + kGmTileBytes);
    if (DUAL) gm_put(st.u, dst, stage + 2 * kGmTileBytes);
}

template <bool DUAL>
__global__ __launch_bounds__(kGmThreads) void linear_rows_mfma_kernel(LinearRowsParams prm) {
    extern __shared__ __attribute__((aligned(16))) unsigned char gm_smem[];
    constexpr int kOperands = DUAL ? 3 : 2;                      // x, w (, up)
    constexpr int kStageBytes = kOperands * kGmTileBytes;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_n = wave & 1, wave_m = wave >> 1;
    const int K = prm.reduction;
    const int n0 = static_cast<int>(blockIdx.x) * kGmTile;
    const int m0 = static_cast<int>(blockIdx.y) * kGmTile;

    // ---- this thread's pieces of a step's tiles: piece index p = tid + 256 i (i < 4) of 1024 per tile; row p / 8,
    // global piece (p % 8) ^ (row % 8) lands in slot p % 8 ----
    const uint16_t* src_x[4];
    const uint16_t* src_w[4];
    const uint16_t* src_u[4];
    int dst[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int p = tid + kGmThreads * i;
        const int row = p >> 3, slot = p & 7;
        const int piece = slot ^ (row & 7);
        dst[i] = p * 16;
        const int m = min(m0 + row, prm.rows - 1);                // rows past the end repeat the last one (never stored)
        src_x[i] = prm.input + static_cast<int64_t>(m) * K + 8 * piece;
        src_w[i] = prm.weight[0] + static_cast<int64_t>(n0 + row) * K + 8 * piece;
        src_u[i] = prm.weight[DUAL ? 1 : 0] + static_cast<int64_t>(n0 + row) * K + 8 * piece;
    }
    GmStaged staged_a, staged_b;

    f32x16_t acc[2][2], acc_up[DUAL ? 2 : 1][DUAL ? 2 : 1];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                acc[a][b][r] = 0.0f;
                if (DUAL) acc_up[a][b][r] = 0.0f;
            }
        }

    // fragment of tile rows [32 t, 32 t + 32), k block kb (16 k): lane l takes row l % 32, piece 2 kb + l / 32
    const int frag_row = lane & 31, frag_half = lane >> 5;
    auto fragment = [&](const unsigned char* tile, int t, int kb) __attribute__((always_inline)) {
        const int row = 32 * t + frag_row;
        return *reinterpret_cast<const bf16x8_t*>(tile + tile_slot(row, 2 * kb + frag_half));
    };

    // Two sets of staging registers: the tiles of step t + 2 are requested while step t is multiplied, and written to
    // LDS (three stages) an iteration later, so that a request has two steps of arithmetic to come back.
    const int steps = K / kGmStep;
    // the MFMAs of k blocks [kb0, kb0 + 2) of a step
    auto multiply = [&](int step, int kb0) __attribute__((always_inline)) {
        const unsigned char* stage = gm_smem + (step % 3) * kStageBytes;
        const unsigned char* x_tile = stage;
        const unsigned char* w_tile = stage + kGmTileBytes;
        const unsigned char* u_tile = stage + 2 * kGmTileBytes;
#pragma unroll
        for (int kb = kb0; kb < kb0 + 2; ++kb) {
            bf16x8_t wf[2], xf[2], uf[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                wf[t] = fragment(w_tile, 2 * wave_n + t, kb);
                xf[t] = fragment(x_tile, 2 * wave_m + t, kb);
                if (DUAL) uf[t] = fragment(u_tile, 2 * wave_n + t, kb);
            }
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int b = 0; b < 2; ++b) {
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[a], xf[b], acc[a][b], 0, 0, 0);
                    if (DUAL) acc_up[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(uf[a], xf[b], acc_up[a][b], 0, 0, 0);
                }
        }
    };
    // (requests past the last step repeat it and their tiles land in a stage nobody reads again: staging that is
    // conditional on the step makes the compiler keep the staged registers in scratch memory)
    auto k_of = [&](int step) { return min(step, steps - 1) * kGmStep; };
    gm_request<DUAL>(staged_a, src_x, src_w, src_u, k_of(0));
    gm_request<DUAL>(staged_b, src_x, src_w, src_u, k_of(1));
    gm_deposit<DUAL>(staged_a, dst, gm_smem);
    __syncthreads();
    for (int step = 0; step < steps; step += 2) {
        // (the next step's tiles are written to LDS between the two halves of a step's MFMAs, which hide the writes)
        gm_request<DUAL>(staged_a, src_x, src_w, src_u, k_of(step + 2));
        multiply(step, 0);
        gm_deposit<DUAL>(staged_b, dst, gm_smem + ((step + 1) % 3) * kStageBytes);
        multiply(step, 2);
        __syncthreads();
        gm_request<DUAL>(staged_b, src_x, src_w, src_u, k_of(step + 3));
        multiply(step + 1, 0);                          // (the number of steps is even: reduction % 128 == 0)
        gm_deposit<DUAL>(staged_a, dst, gm_smem + ((step + 2) % 3) * kStageBytes);
        multiply(step + 1, 2);
        __syncthreads();
    }

    // ---- epilogue: accumulator register r of a lane is output column 8 (r / 4) + 4 (lane / 32) + r % 4 of the MFMA
    // tile's 32, token row lane % 32 ----
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const int m = m0 + 64 * wave_m + 32 * b + (lane & 31);
            const bool inside = m < prm.rows;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                if (!inside) break;
                const int n = n0 + 64 * wave_n + 32 * a + 8 * g + 4 * (lane >> 5);
                uint16_t bits[4];
                uint2 res = make_uint2(0, 0);
                if (!DUAL && prm.residual) res = *reinterpret_cast<const uint2*>(prm.residual + static_cast<int64_t>(m) * prm.columns + n);
                uint2 bias = make_uint2(0, 0);
                if (!DUAL && prm.bias) bias = *reinterpret_cast<const uint2*>(prm.bias + n);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float sum = acc[a][b][4 * g + e];
                    if (DUAL) {
                        // swiglu_kernel (R17:8746-8770) on the rounded gate and up values
                        const float gv = bf2f(f2bf(sum));
                        const uint16_t act = f2bf(gv / (1.0f + expf(-gv)));
                        bits[e] = f2bf(bf2f(act) * bf2f(f2bf(acc_up[a][b][4 * g + e])));
                    } else {
                        float r = sum;
                        if (prm.bias) r += bf2f(static_cast<uint16_t>((e < 2 ? bias.x : bias.y) >> (16 * (e & 1))));
                        uint16_t v = f2bf(r);
                        if (prm.residual) v = f2bf(bf2f(static_cast<uint16_t>((e < 2 ? res.x : res.y) >> (16 * (e & 1)))) + bf2f(v));
                        bits[e] = v;
                    }
                }
                *reinterpret_cast<uint2*>(prm.output + static_cast<int64_t>(m) * prm.columns + n) =
                    make_uint2(bits[0] | (static_cast<uint32_t>(bits[1]) << 16), bits[2] | (static_cast<uint32_t>(bits[3]) << 16));
            }
        }
    }
}

}  // namespace

int32_t launch_rows_mfma(const LinearRowsParams& prm, bool dual, hipStream_t stream) {
    if (prm.rows == 0 || prm.columns == 0) return QM_OK;
    const dim3 grid(static_cast<unsigned>(prm.columns / kGmTile), static_cast<unsigned>((prm.rows + kGmTile - 1) / kGmTile));
    if (grid.y > 65535u) return QM_ERR_ARGUMENT;
    static std::atomic<bool> lds_raised[2][kMaxDevices];
    if (dual) {
        const int smem = 3 * 3 * kGmTileBytes;
        const int32_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(linear_rows_mfma_kernel<true>), smem, lds_raised[1]);
        if (rc != QM_OK) return rc;
        hipLaunchKernelGGL(linear_rows_mfma_kernel<true>, grid, dim3(kGmThreads), smem, stream, prm);
    } else {
        const int smem = 3 * 2 * kGmTileBytes;
        const int32_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(linear_rows_mfma_kernel<false>), smem, lds_raised[0]);
        if (rc != QM_OK) return rc;
        hipLaunchKernelGGL(linear_rows_mfma_kernel<false>, grid, dim3(kGmThreads), smem, stream, prm);
    }
    return launch_status();
}

}  // namespace qm
