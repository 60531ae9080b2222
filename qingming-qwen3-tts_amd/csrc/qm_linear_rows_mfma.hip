// qm_linear_rows_mfma.hip — the prompt pass's linears over many token rows on the bf16 matrix cores (gfx950).
//
// out[m][n] = bf16(sum_k x[m][k] w[n][k] + bias[n]) (+ residual, or the SwiGLU of a gate/up pair): what
// native_ops::linear_bf16 computes per (row, column) (R17:126-245, reached through NativeTalkerEngine::linear_generic,
// R17:17453-17472, in ::prefill, R17:16620-16790), with the fp32 sum taken by v_mfma_f32_32x32x16_bf16 in its own order
// instead of the reference's 32 lane-strided chains: bf16 inputs, fp32 accumulation, the same roundings after the sum,
// results within the operators' tolerance of the exact-chain kernel (qm_linear_rows.hip), not bit-identical to it.
//
// A block of four waves owns 128 output columns x 128 token rows (waves 2 x 2, each 64 x 64 as 2 x 2 MFMA tiles) or, for
// calls whose grid would leave CUs empty, x 64 token rows (waves 4 x 1, each 32 columns x 64 rows).  Both operands are
// K-contiguous rows (x [m][k], w [n][k]), so one tile layout serves both: 64 k per step, a row of a tile is eight 16-byte
// pieces in LDS, piece q of row r stored in slot q ^ ((r / 2) % 8) so that the sixteen rows a fragment read touches in a
// cycle spread over all 64 banks.  An MFMA takes the weight rows as its A operand and the token rows as B (D = W X^T): a lane then holds, for one
// token row, runs of four consecutive output columns — 8-byte stores.
// The tiles go from memory straight into a ring of LDS stages (global_load_lds, no registers, the swizzle chosen by which
// piece a lane fetches), up to four steps ahead (three for the gate/up pair, whose stage is 48 KiB).  A step's one barrier
// stands between the MFMAs of its last two k blocks, where a wave has read all it needs of the step's stage and waits
// (vmcnt counts the later stages' pieces still in flight) for its own pieces of the next; the requests for the stage
// just freed go out a piece at a time between the MFMAs that follow (issued in a bunch, the four waves' requests keep
// the CU's address path and the waves busy for 700 cycles of a 1024-cycle step), and the next step's first fragments
// are read behind the barrier while the last k block's MFMAs run.  The fragment reads are inline assembly: the compiler makes every LDS read of its own wait
// for all global_load_lds in flight, which would expose the memory latency in every step.
// Bound: bf16 MFMA (2.5 PFLOP/s); algorithmic flops 2 m n k (x 2 for the gate/up pair).

#include "qm_device.h"
#include "qm_host.h"
#include "qm_linear_rows_params.h"

#include <type_traits>

namespace qm {

constexpr int kGmThreads = 256;
constexpr int kGmTile = 128;                 // token rows and output columns per block
constexpr int kGmStep = 64;                  // k per step
constexpr int kGmTileBytes = kGmTile * kGmStep * 2;   // 16 KiB per operand tile

typedef float f32x16_t __attribute__((ext_vector_type(16)));

// LDS byte offset of piece `piece` (16 bytes = 8 k) of row `row` inside a tile
// (the LDS has 64 banks of four bytes: a row of 128 bytes covers half of them, which half by the row's parity, and the
// sixteen lanes served in a cycle read sixteen consecutive rows: the eight rows of one parity take eight different slots)
__device__ __forceinline__ int slot_key(int row) { return (row >> 1) & 7; }

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// s_waitcnt that waits until at most N vector-memory operations are outstanding (nothing else)
template <int N>
__device__ __forceinline__ void gm_wait_vm() {
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// What follows the fp32 sums of two neighbouring output columns, as a packed bf16 pair.  Every rounding is one half of a
// v_cvt_pk_bf16_f32 (round to nearest even, a NaN quieted with its payload kept: the bits f2bf gives for every fp32 input).
// Linear: bf16(sum + bias), then bf16(residual + that) (linear_bf16 and add_bf16, R17:126-245, 8772-8790).
__device__ __forceinline__ uint32_t finish_pair(float s0, float s1, bool has_bias, uint32_t bias, bool has_residual, uint32_t residual) {
    if (has_bias) {
        s0 += lo_bf16(bias);
        s1 += hi_bf16(bias);
    }
    uint32_t v = pack_bf16_pair(s0, s1);
    if (has_residual) v = pack_bf16_pair(lo_bf16(residual) + lo_bf16(v), hi_bf16(residual) + hi_bf16(v));
    return v;
}

// Gate/up: swiglu_kernel (R17:8746-8770) on the rounded gate and up values.
__device__ __forceinline__ uint32_t swiglu_pair(float g0, float g1, float u0, float u1) {
    float gv0, gv1, uv0, uv1, a0, a1;
    round_bf16_pair(g0, g1, gv0, gv1);
    round_bf16_pair(u0, u1, uv0, uv1);
    round_bf16_pair(gv0 / (1.0f + expf(-gv0)), gv1 / (1.0f + expf(-gv1)), a0, a1);
    return pack_bf16_pair(a0 * uv0, a1 * uv1);
}

// 16 bytes per lane from `from` to LDS: lane l's land at `to` + 16 l
__device__ __forceinline__ void gm_to_lds(const uint16_t* from, unsigned char* to) {
    __builtin_amdgcn_global_load_lds(from, (__attribute__((address_space(3))) void*)to, 16, 0, 0);
}

template <bool DUAL, int BM>
__global__ __launch_bounds__(kGmThreads) void linear_rows_mfma_kernel(LinearRowsParams prm) {
    extern __shared__ __attribute__((aligned(16))) unsigned char gm_smem[];
    constexpr int kStages = DUAL ? 3 : 4;
    constexpr int kXBytes = BM * kGmStep * 2;
    constexpr int kWeights = DUAL ? 2 : 1;
    constexpr int kStageBytes = kXBytes + kWeights * kGmTileBytes;
    constexpr int kTn = BM == 128 ? 2 : 1;                        // MFMA tiles of a wave along the output columns
    constexpr int kTm = 2;                                        // and along the token rows
    // pieces of 1 KiB (one instruction of a wave) per stage: x, w (, up); dealt to the four waves in turn
    constexpr int kPiecesX = kXBytes / 1024, kPiecesW = kGmTileBytes / 1024;
    constexpr int kPerWave = (kPiecesX + kWeights * kPiecesW) / 4;
    static_assert((kPiecesX + kWeights * kPiecesW) % 4 == 0, "pieces are dealt evenly to four waves");
    static_assert(kPerWave * (kStages - 1) <= 63, "the waits count the later stages' pieces");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_n = BM == 128 ? (wave & 1) : wave;
    const int wave_m = BM == 128 ? (wave >> 1) : 0;
    const int K = prm.reduction;
    const int n0 = static_cast<int>(blockIdx.x) * kGmTile;
    const int m0 = static_cast<int>(blockIdx.y) * BM;

    // ---- this wave's pieces of a stage: instruction q = wave + 4 i covers LDS bytes [1024 q, 1024 q + 1024) of the
    // stage (x tile, then w, then up); its lane l fills slot l % 8 of tile row 8 (q within the tile) + l / 8 with
    // global piece slot ^ slot_key(row) ----
    const uint16_t* src[kPerWave];
#pragma unroll
    for (int i = 0; i < kPerWave; ++i) {
        const int q = wave + 4 * i;
        const int operand = q < kPiecesX ? 0 : (q < kPiecesX + kPiecesW ? 1 : 2);
        const int qt = q - (operand == 0 ? 0 : (operand == 1 ? kPiecesX : kPiecesX + kPiecesW));
        const int row = 8 * qt + (lane >> 3), slot = lane & 7;
        const int piece = slot ^ slot_key(row);
        if (operand == 0) {
            const int m = min(m0 + row, prm.rows - 1);            // rows past the end repeat the last one (never stored)
            src[i] = prm.input + static_cast<int64_t>(m) * K + 8 * piece;
        } else {
            src[i] = prm.weight[operand - 1] + static_cast<int64_t>(n0 + row) * K + 8 * piece;
        }
    }
    // (a block takes piece blockIdx.z of the reduction: all of it unless the launch cut it)
    const int steps = K / kGmStep / prm.reduction_parts;
    const int first_step = static_cast<int>(blockIdx.z) * steps;
    // Piece `i` of this wave's pieces of step `step_`, into stage step_ % kStages.  (Requests past the last step repeat it
    // and land in a stage nobody reads again: the wait before the barrier counts pieces.)
    auto request_piece = [&](int step_, int i) __attribute__((always_inline)) {
        const int k0 = (first_step + min(step_, steps - 1)) * kGmStep;
        gm_to_lds(src[i] + k0, gm_smem + (step_ % kStages) * kStageBytes + 1024 * wave + 4096 * i);
    };

    f32x16_t acc[kTn][kTm], acc_up[DUAL ? kTn : 1][DUAL ? kTm : 1];
#pragma unroll
    for (int a = 0; a < kTn; ++a)
#pragma unroll
        for (int b = 0; b < kTm; ++b) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                acc[a][b][r] = 0.0f;
                if (DUAL) acc_up[a][b][r] = 0.0f;
            }
        }

    // fragment of tile rows [32 t, 32 t + 32), k block kb (16 k): lane l takes row l % 32, piece 2 kb + l / 32.  The LDS
    // address of (tile 0 row, k block 0) per lane; tile t adds 32 rows = 4096 bytes, k block kb flips the slot by 2 kb.
    const int frag_row = lane & 31, frag_half = lane >> 5;
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) unsigned char*)gm_smem));
    uint32_t at_kb[4];                                            // byte offset inside a tile for each k block (row part included)
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) at_kb[kb] = static_cast<uint32_t>(frag_row * 128 + (((2 * kb + frag_half) ^ slot_key(frag_row)) * 16));
    struct Frags {
        u32x4_t w[kTn], x[kTm], u[DUAL ? kTn : 1];
    };
    auto read_frags = [&](Frags& f, uint32_t stage_at, int kb) __attribute__((always_inline)) {
        const uint32_t x_at = stage_at + at_kb[kb] + static_cast<uint32_t>(wave_m * kTm * 4096);
        const uint32_t w_at = stage_at + kXBytes + at_kb[kb] + static_cast<uint32_t>(wave_n * kTn * 4096);
        // (offsets are literal: tile t of an operand lies 32 rows = 4096 bytes further on)
        asm volatile("ds_read_b128 %0, %1" : "=v"(f.w[0]) : "v"(w_at));
        if (DUAL) asm volatile("ds_read_b128 %0, %1 offset:16384" : "=v"(f.u[0]) : "v"(w_at));
        if (kTn == 2) {
            asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(f.w[kTn - 1]) : "v"(w_at));
            if (DUAL) asm volatile("ds_read_b128 %0, %1 offset:20480" : "=v"(f.u[kTn - 1]) : "v"(w_at));
        }
        asm volatile("ds_read_b128 %0, %1" : "=v"(f.x[0]) : "v"(x_at));
        asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(f.x[1]) : "v"(x_at));
    };
    static_assert(kGmTileBytes == 16384 && kTm == 2, "the literal offsets of the fragment reads");
    constexpr int kReads = kTn * (DUAL ? 2 : 1) + kTm;            // LDS reads per k block and lane
    // the results of read_frags(f, ...) may be used once at most `later` reads issued after them are outstanding
    auto arrived = [&](Frags& f, auto later) __attribute__((always_inline)) {
        if constexpr (kTn == 2 && DUAL) {
            asm volatile("s_waitcnt lgkmcnt(%6)" : "+v"(f.w[0]), "+v"(f.w[1]), "+v"(f.u[0]), "+v"(f.u[1]), "+v"(f.x[0]), "+v"(f.x[1])
                         : "n"(decltype(later)::value) : "memory");
        } else if constexpr (kTn == 2) {
            asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(f.w[0]), "+v"(f.w[1]), "+v"(f.x[0]), "+v"(f.x[1]) : "n"(decltype(later)::value) : "memory");
        } else if constexpr (DUAL) {
            asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(f.w[0]), "+v"(f.u[0]), "+v"(f.x[0]), "+v"(f.x[1]) : "n"(decltype(later)::value) : "memory");
        } else {
            asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(f.w[0]), "+v"(f.x[0]), "+v"(f.x[1]) : "n"(decltype(later)::value) : "memory");
        }
    };
    // The MFMAs of one k block, with this wave's pieces [P0, P1) of step `req_step` requested between them: a request
    // takes the CU's one address path about 16 cycles a piece (64 bytes a cycle), and issued in a bunch by four waves at
    // once they leave the matrix cores idle for that long; between MFMAs they are issued in the shadow of the 32 cycles
    // each MFMA takes.
    constexpr int kMfmas = kTn * kTm * (DUAL ? 2 : 1);
    auto multiply = [&](const Frags& f, int req_step, auto p0, auto p1) __attribute__((always_inline)) {
        constexpr int P0 = decltype(p0)::value, P1 = decltype(p1)::value;
        int done = 0, piece = P0;
#pragma unroll
        for (int a = 0; a < kTn; ++a)
#pragma unroll
            for (int b = 0; b < kTm; ++b) {
                acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, f.w[a]), __builtin_bit_cast(bf16x8_t, f.x[b]),
                                                                    acc[a][b], 0, 0, 0);
                if (DUAL)
                    acc_up[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, f.u[a]),
                                                                           __builtin_bit_cast(bf16x8_t, f.x[b]), acc_up[a][b], 0, 0, 0);
                done += DUAL ? 2 : 1;
                // (as many pieces behind this MFMA as keep them evenly spread over the k block's MFMAs)
                while (piece < P1 && (piece - P0 + 1) * kMfmas <= done * (P1 - P0)) {
                    __builtin_amdgcn_sched_barrier(0);
                    request_piece(req_step, piece);
                    __builtin_amdgcn_sched_barrier(0);
                    ++piece;
                }
            }
    };
    using std::integral_constant;
    constexpr int kQ1 = kPerWave / 4, kQ2 = kPerWave / 2, kQ3 = 3 * kPerWave / 4;

    // A step's schedule.  The stage of step s is complete for everybody at the barrier of step s - 1; k blocks 0 and 1 of
    // it are read right behind that barrier, while the MFMAs of the last k block of step s - 1 run.  The barrier of step s
    // stands between the MFMAs of k blocks 2 and 3, at a point where this wave has read all it needs of stage s (its last
    // reads have landed): behind it stage s is free, and the pieces of step s + kStages are requested into it, spread over
    // the four k blocks that follow.  The wait in front of the barrier lets the pieces of the steps after s + 1 be in flight.
#pragma unroll
    for (int ahead = 0; ahead < kStages; ++ahead)
#pragma unroll
        for (int i = 0; i < (ahead == kStages - 1 ? kQ1 : kPerWave); ++i) request_piece(ahead, i);
    gm_wait_vm<kPerWave * (kStages - 2) + kQ1>();
    asm volatile("s_barrier" ::: "memory");
    Frags f0, f1;
    read_frags(f0, lds_base, 0);
    read_frags(f1, lds_base, 1);
    for (int step = 0; step < steps; ++step) {
        const uint32_t stage_at = lds_base + static_cast<uint32_t>((step % kStages) * kStageBytes);
        const uint32_t next_at = lds_base + static_cast<uint32_t>(((step + 1) % kStages) * kStageBytes);
        const int req = step - 1 + kStages;                       // (its first quarter went out behind the last barrier)
        arrived(f0, integral_constant<int, kReads>{});
        multiply(f0, req, integral_constant<int, kQ1>{}, integral_constant<int, kQ2>{});
        read_frags(f0, stage_at, 2);
        arrived(f1, integral_constant<int, kReads>{});
        multiply(f1, req, integral_constant<int, kQ2>{}, integral_constant<int, kQ3>{});
        read_frags(f1, stage_at, 3);
        arrived(f0, integral_constant<int, kReads>{});
        multiply(f0, req, integral_constant<int, kQ3>{}, integral_constant<int, kPerWave>{});
        arrived(f1, integral_constant<int, 0>{});
        gm_wait_vm<kPerWave * (kStages - 2)>();                   // this wave's pieces of the next step's stage have landed
        asm volatile("s_barrier" ::: "memory");                   // everybody's have; and everybody has read this step's stage
        if (step + 1 < steps) read_frags(f0, next_at, 0);
        multiply(f1, step + kStages, integral_constant<int, 0>{}, integral_constant<int, kQ1>{});
        if (step + 1 < steps) read_frags(f1, next_at, 1);
    }
    gm_wait_vm<0>();                                              // (the requests past the last step, before the block's LDS goes)

    // ---- epilogue: accumulator register r of a lane is output column 8 (r / 4) + 4 (lane / 32) + r % 4 of the MFMA
    // tile's 32, token row lane % 32 ----
    if (prm.reduction_parts > 1) {
        // a piece of the reduction: the sums as they are, for linear_rows_parts_kernel
        const int64_t plane = static_cast<int64_t>(prm.rows) * prm.columns;
        float* const part = prm.partials + static_cast<int64_t>(blockIdx.z) * (DUAL ? 2 : 1) * plane;
#pragma unroll
        for (int a = 0; a < kTn; ++a) {
#pragma unroll
            for (int b = 0; b < kTm; ++b) {
                const int m = m0 + 32 * (kTm * wave_m + b) + (lane & 31);
                if (m >= prm.rows) continue;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int n = n0 + 32 * (kTn * wave_n + a) + 8 * g + 4 * (lane >> 5);
                    float* at = part + static_cast<int64_t>(m) * prm.columns + n;
                    *reinterpret_cast<float4*>(at) = make_float4(acc[a][b][4 * g], acc[a][b][4 * g + 1], acc[a][b][4 * g + 2], acc[a][b][4 * g + 3]);
                    if (DUAL)
                        *reinterpret_cast<float4*>(at + plane) =
                            make_float4(acc_up[a][b][4 * g], acc_up[a][b][4 * g + 1], acc_up[a][b][4 * g + 2], acc_up[a][b][4 * g + 3]);
                }
            }
        }
        return;
    }
#pragma unroll
    for (int a = 0; a < kTn; ++a) {
#pragma unroll
        for (int b = 0; b < kTm; ++b) {
            const int m = m0 + 32 * (kTm * wave_m + b) + (lane & 31);
            const bool inside = m < prm.rows;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                if (!inside) break;
                const int n = n0 + 32 * (kTn * wave_n + a) + 8 * g + 4 * (lane >> 5);
                uint2 res = make_uint2(0, 0);
                if (!DUAL && prm.residual) res = *reinterpret_cast<const uint2*>(prm.residual + static_cast<int64_t>(m) * prm.columns + n);
                uint2 bias = make_uint2(0, 0);
                if (!DUAL && prm.bias) bias = *reinterpret_cast<const uint2*>(prm.bias + n);
                uint32_t packed[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const float s0 = acc[a][b][4 * g + 2 * e], s1 = acc[a][b][4 * g + 2 * e + 1];
                    if (DUAL) {
                        packed[e] = swiglu_pair(s0, s1, acc_up[a][b][4 * g + 2 * e], acc_up[a][b][4 * g + 2 * e + 1]);
                    } else {
                        packed[e] = finish_pair(s0, s1, prm.bias != nullptr, e == 0 ? bias.x : bias.y, prm.residual != nullptr,
                                                e == 0 ? res.x : res.y);
                    }
                }
                *reinterpret_cast<uint2*>(prm.output + static_cast<int64_t>(m) * prm.columns + n) = make_uint2(packed[0], packed[1]);
            }
        }
    }
}

// The pieces of a cut reduction added in order, then what the epilogue above does: thread = four output columns of a row.
template <bool DUAL>
__global__ __launch_bounds__(256) void linear_rows_parts_kernel(LinearRowsParams prm) {
    const int64_t quad = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int quads_per_row = prm.columns / 4;
    if (quad >= static_cast<int64_t>(prm.rows) * quads_per_row) return;
    const int m = static_cast<int>(quad / quads_per_row);
    const int n = 4 * static_cast<int>(quad % quads_per_row);
    const int64_t plane = static_cast<int64_t>(prm.rows) * prm.columns;
    const float* at = prm.partials + static_cast<int64_t>(m) * prm.columns + n;
    float4 sum = make_float4(0.0f, 0.0f, 0.0f, 0.0f), up = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    for (int z = 0; z < prm.reduction_parts; ++z) {
        const float4 v = *reinterpret_cast<const float4*>(at + static_cast<int64_t>(z) * (DUAL ? 2 : 1) * plane);
        sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
        if (DUAL) {
            const float4 u = *reinterpret_cast<const float4*>(at + static_cast<int64_t>(z) * 2 * plane + plane);
            up.x += u.x; up.y += u.y; up.z += u.z; up.w += u.w;
        }
    }
    uint2 res = make_uint2(0, 0), bias = make_uint2(0, 0);
    if (!DUAL && prm.residual) res = *reinterpret_cast<const uint2*>(prm.residual + static_cast<int64_t>(m) * prm.columns + n);
    if (!DUAL && prm.bias) bias = *reinterpret_cast<const uint2*>(prm.bias + n);
    uint2 packed;
    if (DUAL) {
        packed.x = swiglu_pair(sum.x, sum.y, up.x, up.y);
        packed.y = swiglu_pair(sum.z, sum.w, up.z, up.w);
    } else {
        packed.x = finish_pair(sum.x, sum.y, prm.bias != nullptr, bias.x, prm.residual != nullptr, res.x);
        packed.y = finish_pair(sum.z, sum.w, prm.bias != nullptr, bias.y, prm.residual != nullptr, res.y);
    }
    *reinterpret_cast<uint2*>(prm.output + static_cast<int64_t>(m) * prm.columns + n) = packed;
}

template <bool DUAL, int BM>
int32_t launch_rows_mfma_as(const LinearRowsParams& prm, hipStream_t stream) {
    constexpr int kStages = DUAL ? 3 : 4;
    constexpr int smem = kStages * (BM * kGmStep * 2 + (DUAL ? 2 : 1) * kGmTileBytes);
    const dim3 grid(static_cast<unsigned>(prm.columns / kGmTile), static_cast<unsigned>((prm.rows + BM - 1) / BM),
                    static_cast<unsigned>(prm.reduction_parts));
    if (grid.y > 65535u) return QM_ERR_ARGUMENT;
    static std::atomic<bool> lds_raised[kMaxDevices];
    const int32_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(linear_rows_mfma_kernel<DUAL, BM>), smem, lds_raised);
    if (rc != QM_OK) return rc;
    hipLaunchKernelGGL((linear_rows_mfma_kernel<DUAL, BM>), grid, dim3(kGmThreads), smem, stream, prm);
    int32_t status = launch_status();
    if (status == QM_OK && prm.reduction_parts > 1) {
        const int64_t quads = static_cast<int64_t>(prm.rows) * (prm.columns / 4);
        hipLaunchKernelGGL((linear_rows_parts_kernel<DUAL>), dim3(static_cast<unsigned>((quads + 255) / 256)), dim3(256), 0, stream, prm);
        status = launch_status();
    }
    return status;
}

// Few token rows leave most CUs without a block (128 rows of a 2048-column linear: 32 blocks), and a block's time is its
// chain of 64-k steps.  With a workspace the reduction is cut so that the grid comes to about one block per CU: pieces of
// four steps at least, as many as divide the steps evenly, at most eight.
int rows_mfma_reduction_parts(int rows, int columns, int reduction, bool dual) {
    (void)dual;
    if (rows <= 0 || columns < kGmTile || reduction < kGmStep) return 1;
    const int64_t blocks = static_cast<int64_t>(columns / kGmTile) * ((rows + 63) / 64);
    const int steps = reduction / kGmStep;
    int parts = 1;
    for (int p = 2; p <= 8; p *= 2)
        if (blocks * p <= 256 && steps % p == 0 && steps / p >= 4) parts = p;
    return parts;
}

size_t rows_mfma_workspace_bytes(int rows, int columns, int reduction, bool dual) {
    const int parts = rows_mfma_reduction_parts(rows, columns, reduction, dual);
    if (parts <= 1) return 0;
    return static_cast<size_t>(parts) * (dual ? 2 : 1) * rows * columns * sizeof(float);
}

int32_t launch_rows_mfma(const LinearRowsParams& prm, bool dual, hipStream_t stream) {
    if (prm.rows == 0 || prm.columns == 0) return QM_OK;
    // blocks of 64 token rows where blocks of 128 would leave CUs without one (one block per CU either way)
    const int64_t blocks_128 = static_cast<int64_t>(prm.columns / kGmTile) * ((prm.rows + 127) / 128);
    const bool small = blocks_128 < 200;
    if (dual) return small ? launch_rows_mfma_as<true, 64>(prm, stream) : launch_rows_mfma_as<true, 128>(prm, stream);
    return small ? launch_rows_mfma_as<false, 64>(prm, stream) : launch_rows_mfma_as<false, 128>(prm, stream);
}

}  // namespace qm
