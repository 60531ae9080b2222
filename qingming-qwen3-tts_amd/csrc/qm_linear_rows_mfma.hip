// qm_linear_rows_mfma.hip — the prompt pass's linears over many token rows on the bf16 matrix cores (gfx950).
//
// out[m][n] = bf16(sum_k x[m][k] w[n][k] + bias[n]) (+ residual, or the SwiGLU of a gate/up pair): what
// native_ops::linear_bf16 computes per (row, column) (R17:126-245, reached through NativeTalkerEngine::linear_generic,
// R17:17453-17472, in ::prefill, R17:16620-16790), with the fp32 sum taken by v_mfma_f32_32x32x16_bf16 in its own order
// instead of the reference's 32 lane-strided chains: bf16 inputs, fp32 accumulation, the same roundings after the sum,
// results within the operators' tolerance of the exact-chain kernel (qm_linear_rows.hip), not bit-identical to it.
//
// A block of four waves owns a tile of BM token rows x BN output columns: 128 x 128 (waves 2 x 2, each 64 x 64 as 2 x 2
// MFMA tiles); 64 x 128 for calls whose grid of 128-row tiles would leave CUs empty (waves 4 x 1, each 32 columns x 64
// rows); 128 x 192 for a gate/up pair whose 128-column tiles come to between one and two rounds of the CUs and whose
// 192-column tiles fit in one (1024 tokens x 6144 channels: 256 blocks).  Several linears of one input (q, k, v) share a
// grid: a column tile's number says which of them it belongs to.  Both operands are K-contiguous rows (x [m][k],
// w [n][k]), so one tile layout serves both: KSTEP (64, or 128 for 64-row tiles with a long reduction) k per step, a row
// of a tile is KSTEP / 8 16-byte pieces in LDS, piece q of row r stored in slot q ^ key(r), the key chosen so that the
// sixteen rows a fragment read touches in a cycle spread over all 64 banks.  An MFMA takes the weight rows as its A
// operand and the token rows as B (D = W X^T): a lane then holds, for one token row, runs of four consecutive output
// columns — 8-byte stores.
// The tiles go from memory straight into a ring of LDS stages (buffer_load ... lds, no registers, the swizzle chosen by
// which piece a lane fetches): four stages where they fit in 128 KiB, else three, two for the 192-column tile (64 KiB a
// stage).  A step's one barrier stands between the MFMAs of its last two k blocks, where a wave has read all it needs of
// the step's stage and waits (vmcnt counts the later stages' pieces still in flight) for its own pieces of the next.
// Nothing but MFMAs is issued in a bunch: a k block's LDS reads and the requests for the stage just freed stand one or
// two to a slot between its MFMAs (GmSchedule), because the wave issues in order and an MFMA hides 32 cycles of other
// issue and no more — bunched, the four waves' requests of a step keep the CU's one address path (64 bytes a cycle) and
// with it the waves busy for 700 cycles of a 1024-cycle step.  The fragment reads are inline assembly: the compiler makes
// every LDS read of its own wait for all requests in flight, which would expose the memory latency in every step.
// Bound: bf16 MFMA (2.5 PFLOP/s at 2.4 GHz; under these kernels the clock settles at 1.8 to 1.9 GHz); algorithmic flops
// 2 m n k (x 2 for the gate/up pair).

#include "qm_device.h"
#include "qm_host.h"
#include "qm_linear_rows_params.h"

#include <type_traits>

namespace qm {

constexpr int kGmThreads = 256;
constexpr int kGmTile = 128;                 // output columns per block (192 for a gate/up pair that it divides), token rows 128 or 64
constexpr int kGmStep = 64;                  // k per step (32 with the 192-column tile)

typedef float f32x16_t __attribute__((ext_vector_type(16)));

// LDS byte offset of piece `piece` (16 bytes = 8 k) of row `row` inside a tile
// The LDS has 64 banks of four bytes, and the sixteen lanes served in a cycle read the same piece of sixteen consecutive
// rows.  A row of ROW_BYTES covers ROW_BYTES / 4 banks, which of them by the row's number within 256 bytes; the rows that
// share banks take different slots for the same piece: slot = piece ^ key(row).
template <int ROW_BYTES>
__device__ __forceinline__ int slot_key(int row) { return (row / (256 / ROW_BYTES)) & (ROW_BYTES / 16 - 1); }

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

// A block's tile: BM token rows x BN output columns (x 2 for a gate/up pair), KSTEP k per step, a ring of kStages stages.
template <bool DUAL, int BM, int BN, int KSTEP>
struct GmShape {
    static constexpr int kStageBytes = (BM + (DUAL ? 2 : 1) * BN) * KSTEP * 2;
    static constexpr int kStages = kStageBytes * 4 <= 128 * 1024 ? 4 : (kStageBytes * 3 <= 144 * 1024 ? 3 : 2);
    static_assert(kStageBytes * kStages <= 160 * 1024 - 1024, "the CU's LDS");
};

// Where the side operations of a k block stand among its MFMAs.  The MFMAs of a k block run over the wave's tiles (a, b),
// a the weight tile and b the token tile, b fastest, and for a gate/up pair the gate MFMA before the up MFMA; MFMA number i
// is followed by slot i.  A matrix-core instruction takes 32 cycles and the wave issues in order, so whatever else the wave
// has to issue (LDS reads, requests to memory) goes one or two to a slot, in the shadow of the MFMA before it.
template <bool DUAL, int TN, int TM>
struct GmSchedule {
    static constexpr int kD = DUAL ? 2 : 1;
    static constexpr int kMfmas = TN * TM * kD;
    static constexpr int kReads = TN * kD + TM;                   // fragments (LDS reads) of a k block
    // the slot behind the last MFMA that takes a fragment: from there on its registers can be read into again
    static constexpr int w_slot(int a) { return (a * TM + TM - 1) * kD; }
    static constexpr int u_slot(int a) { return (a * TM + TM - 1) * kD + 1; }
    static constexpr int x_slot(int b) { return ((TN - 1) * TM + b) * kD + kD - 1; }
    static constexpr int own_at(int slot) {
        int n = 0;
        for (int a = 0; a < TN; ++a) n += (w_slot(a) == slot) + (DUAL && u_slot(a) == slot);
        for (int b = 0; b < TM; ++b) n += x_slot(b) == slot;
        return n;
    }
    static constexpr int own_from(int slot) {
        int n = 0;
        for (int s = slot; s < kMfmas; ++s) n += own_at(s);
        return n;
    }
    // the other buffer's fragments, read ahead of their k block: from slot 0 on, this many to a slot
    static constexpr int kEarlyPerSlot = (kReads + kMfmas - 1) / kMfmas;
    static constexpr int kLastEarlySlot = (kReads - 1) / kEarlyPerSlot;
    // `pieces` requests over the slots: one more to a slot at a time, the slots with fewer reads of their own first
    static constexpr int requests_at(int slot, int pieces) {
        int given[kMfmas] = {};
        for (int p = 0; p < pieces; ++p) {
            int best = 0;
            for (int s = 1; s < kMfmas; ++s)
                if (own_at(s) + given[s] < own_at(best) + given[best]) best = s;
            ++given[best];
        }
        return given[slot];
    }
    static constexpr int requests_before(int slot, int pieces) {
        int n = 0;
        for (int s = 0; s < slot; ++s) n += requests_at(s, pieces);
        return n;
    }
};

template <bool DUAL, int BM, int BN, int KSTEP>
__global__ __launch_bounds__(kGmThreads) void linear_rows_mfma_kernel(LinearRowsParams prm) {
    request_arguments(prm);
    extern __shared__ __attribute__((aligned(16))) unsigned char gm_smem[];
    constexpr int kStages = GmShape<DUAL, BM, BN, KSTEP>::kStages;
    constexpr int kRowBytes = KSTEP * 2, kSlots = kRowBytes / 16, kKb = KSTEP / 16;
    constexpr int kRowsPerPiece = 64 / kSlots;                    // tile rows one instruction of a wave fills
    constexpr int kXBytes = BM * kRowBytes, kWBytes = BN * kRowBytes;
    constexpr int kWeights = DUAL ? 2 : 1;
    constexpr int kStageBytes = kXBytes + kWeights * kWBytes;
    static_assert(kStageBytes == GmShape<DUAL, BM, BN, KSTEP>::kStageBytes, "");
    constexpr int kTn = BM == 128 ? BN / 64 : BN / 128;           // MFMA tiles of a wave along the output columns
    constexpr int kTm = 2;                                        // and along the token rows
    constexpr int kFragTile = 32 * kRowBytes;                     // LDS bytes from an operand's MFMA tile to its next
    using Schedule = GmSchedule<DUAL, kTn, kTm>;
    // pieces of 1 KiB (one instruction of a wave) per stage: x, w (, up); dealt to the four waves in turn
    constexpr int kPiecesX = kXBytes / 1024, kPiecesW = kWBytes / 1024;
    constexpr int kPerWave = (kPiecesX + kWeights * kPiecesW) / 4;
    static_assert(kPiecesX % 4 == 0 && kPiecesW % 4 == 0, "a wave's piece i is of the same operand in every wave");
    static_assert(kPerWave * (kStages - 2) <= 63 && kStages >= 2, "the waits count the later stages' pieces");
    static_assert(kKb == 4 || kKb == 8, "the step schedule lists the k blocks");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_n = BM == 128 ? (wave & 1) : wave;
    const int wave_m = BM == 128 ? (wave >> 1) : 0;
    const int K = prm.reduction;
    const int m0 = static_cast<int>(blockIdx.y) * BM;
    // (several linears of one input in one grid: which of them this block's column tile belongs to)
    int tile = static_cast<int>(blockIdx.x);
    const uint16_t* weight0 = prm.weight[0];
    const uint16_t* bias = prm.bias;
    uint16_t* output = prm.output;
    int columns = prm.columns;
    if (!DUAL && prm.groups > 1) {
        const int g = (tile >= prm.group_first_tile[0]) + (prm.groups > 2 && tile >= prm.group_first_tile[1]);
        if (g > 0) {
            tile -= prm.group_first_tile[g - 1];
            weight0 = prm.group_weight[g - 1];
            bias = prm.group_bias[g - 1];
            output = prm.group_output[g - 1];
            columns = prm.group_columns[g - 1];
        }
    }
    const int n0 = tile * BN;

    // ---- this wave's pieces of a stage: instruction q = wave + 4 i covers LDS bytes [1024 q, 1024 q + 1024) of the
    // stage (x tile, then w, then up); its lane l fills slot l % kSlots of tile row kRowsPerPiece (q within the tile) +
    // l / kSlots with global piece slot ^ slot_key(row).  The tiles are read through buffer descriptors that begin at the
    // block's first row of each operand: a lane's offset is the same for every piece (4 kRowsPerPiece rows further on,
    // the key of a row is the same), what changes from piece to piece and step to step is a scalar; token rows past the
    // last are out of the descriptor's range and read as zero without touching memory (their results are never stored).
    const uint32_t row_bytes = static_cast<uint32_t>(K) * 2u;
    const int x_rows = min(prm.rows - m0, BM);
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(prm.input + static_cast<int64_t>(m0) * K), 0, static_cast<int>(x_rows * row_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(weight0 + static_cast<int64_t>(n0) * K), 0, static_cast<int>(BN * row_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t u_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>((DUAL ? prm.weight[1] : weight0) + static_cast<int64_t>(n0) * K), 0, static_cast<int>(BN * row_bytes), 0x00020000);
    const int lane_row = kRowsPerPiece * wave + lane / kSlots;
    const uint32_t lane_off = static_cast<uint32_t>(lane_row) * row_bytes
                            + 16u * static_cast<uint32_t>((lane % kSlots) ^ slot_key<kRowBytes>(lane_row));
    static_assert((4 * kRowsPerPiece) % (256 / kRowBytes * kSlots) == 0, "a piece further on, a row's key is the same");
    // (a block takes piece blockIdx.z of the reduction: all of it unless the launch cut it)
    const int steps = K / KSTEP / prm.reduction_parts;
    const int first_step = static_cast<int>(blockIdx.z) * steps;
    // Piece `i` of this wave's pieces of step `step_`, into stage step_ % kStages.  (Requests past the last step repeat it
    // and land in a stage nobody reads again: the wait before the barrier counts pieces.)
    auto request_piece = [&](int step_, int i) __attribute__((always_inline)) {
        constexpr int kX = kPiecesX / 4, kW = kPiecesW / 4;
        const int j = i < kX ? i : (i < kX + kW ? i - kX : i - kX - kW);
        const uint32_t k_bytes = static_cast<uint32_t>((first_step + min(step_, steps - 1)) * KSTEP * 2);
        const int scalar = static_cast<int>(k_bytes + static_cast<uint32_t>(4 * kRowsPerPiece * j) * row_bytes);
        auto* to = (__attribute__((address_space(3))) void*)(gm_smem + (step_ % kStages) * kStageBytes + 1024 * wave + 4096 * i);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(i < kX ? x_rsrc : (i < kX + kW ? w_rsrc : u_rsrc), to, 16, static_cast<int>(lane_off),
                                                 scalar, 0, 0);
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
    // address of (tile 0 row, k block 0) per lane; tile t adds 32 rows, k block kb flips the slot by 2 kb.
    const int frag_row = lane & 31, frag_half = lane >> 5;
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) unsigned char*)gm_smem));
    uint32_t x_kb[kKb], w_kb[kKb];                                // this wave's first x / w tile, row and k block included
#pragma unroll
    for (int kb = 0; kb < kKb; ++kb) {
        const uint32_t at = static_cast<uint32_t>(frag_row * kRowBytes + (((2 * kb + frag_half) ^ slot_key<kRowBytes>(frag_row)) * 16));
        x_kb[kb] = at + static_cast<uint32_t>(wave_m * kTm * kFragTile);
        w_kb[kb] = at + static_cast<uint32_t>(kXBytes + wave_n * kTn * kFragTile);
    }
    struct Frags {
        u32x4_t w[kTn], x[kTm], u[DUAL ? kTn : 1];
    };
    // (the reads are inline assembly: the compiler makes every LDS read of its own wait for all requests in flight,
    // which would expose the memory latency in every step; tile t of an operand lies kFragTile bytes further on, the up
    // tile kWBytes behind the gate tile)
    auto read_w = [&](Frags& f, uint32_t stage_at, int kb, auto a) __attribute__((always_inline)) {
        const uint32_t at = stage_at + w_kb[kb];
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f.w[decltype(a)::value]) : "v"(at), "n"(kFragTile * decltype(a)::value));
    };
    auto read_u = [&](Frags& f, uint32_t stage_at, int kb, auto a) __attribute__((always_inline)) {
        const uint32_t at = stage_at + w_kb[kb];
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f.u[decltype(a)::value]) : "v"(at), "n"(kWBytes + kFragTile * decltype(a)::value));
    };
    auto read_x = [&](Frags& f, uint32_t stage_at, int kb, auto b) __attribute__((always_inline)) {
        const uint32_t at = stage_at + x_kb[kb];
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f.x[decltype(b)::value]) : "v"(at), "n"(kFragTile * decltype(b)::value));
    };
    static_assert(kWBytes + kFragTile * kTn <= 65535, "the literal offsets of the fragment reads");
    using std::integral_constant;
    // fragment number `n` of a k block in the order of first use: w0, x0, (u0,) x1 .., then the later weight tiles
    auto read_nth = [&](Frags& f, uint32_t stage_at, int kb, auto n) __attribute__((always_inline)) {
        constexpr int N = decltype(n)::value, kD = DUAL ? 2 : 1;
        if constexpr (N == 0) read_w(f, stage_at, kb, integral_constant<int, 0>{});
        else if constexpr (N == 1) read_x(f, stage_at, kb, integral_constant<int, 0>{});
        else if constexpr (DUAL && N == 2) read_u(f, stage_at, kb, integral_constant<int, 0>{});
        else if constexpr (N < kD + kTm) read_x(f, stage_at, kb, integral_constant<int, N - kD>{});
        else if constexpr (DUAL && (N - kD - kTm) % 2 == 1) read_u(f, stage_at, kb, integral_constant<int, 1 + (N - kD - kTm) / 2>{});
        else read_w(f, stage_at, kb, integral_constant<int, 1 + (N - kD - kTm) / kD>{});
    };
    auto read_all = [&](Frags& f, uint32_t stage_at, int kb) __attribute__((always_inline)) {
        read_nth(f, stage_at, kb, integral_constant<int, 0>{});
        read_nth(f, stage_at, kb, integral_constant<int, 1>{});
        read_nth(f, stage_at, kb, integral_constant<int, 2>{});
        if constexpr (Schedule::kReads > 3) read_nth(f, stage_at, kb, integral_constant<int, 3>{});
        if constexpr (Schedule::kReads > 4) {
            read_nth(f, stage_at, kb, integral_constant<int, 4>{});
            read_nth(f, stage_at, kb, integral_constant<int, 5>{});
        }
        if constexpr (Schedule::kReads > 6) {
            read_nth(f, stage_at, kb, integral_constant<int, 6>{});
            read_nth(f, stage_at, kb, integral_constant<int, 7>{});
        }
    };
    static_assert(Schedule::kReads == 3 || Schedule::kReads == 4 || Schedule::kReads == 6 || Schedule::kReads == 8, "read_all lists them");
    constexpr int kReads = Schedule::kReads;
    // the fragments of f may be used once at most `later` reads issued after them are outstanding
    auto arrived = [&](Frags& f, auto later) __attribute__((always_inline)) {
        if constexpr (kTn == 3 && DUAL) {
            asm volatile("s_waitcnt lgkmcnt(%8)" : "+v"(f.w[0]), "+v"(f.w[1]), "+v"(f.w[kTn - 1]), "+v"(f.u[0]), "+v"(f.u[1]), "+v"(f.u[kTn - 1]),
                         "+v"(f.x[0]), "+v"(f.x[1]) : "n"(decltype(later)::value) : "memory");
        } else if constexpr (kTn == 2 && DUAL) {
            asm volatile("s_waitcnt lgkmcnt(%6)" : "+v"(f.w[0]), "+v"(f.w[1]), "+v"(f.u[0]), "+v"(f.u[1]), "+v"(f.x[0]), "+v"(f.x[1])
                         : "n"(decltype(later)::value) : "memory");
        } else if constexpr (kTn == 2) {
            asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(f.w[0]), "+v"(f.w[1]), "+v"(f.x[0]), "+v"(f.x[1]) : "n"(decltype(later)::value) : "memory");
        } else if constexpr (DUAL) {
            asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(f.w[0]), "+v"(f.u[0]), "+v"(f.x[0]), "+v"(f.x[1]) : "n"(decltype(later)::value) : "memory");
        } else {
            static_assert(kTn <= 2 || DUAL, "");
            asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(f.w[0]), "+v"(f.x[0]), "+v"(f.x[1]) : "n"(decltype(later)::value) : "memory");
        }
    };

    // The MFMAs of one k block from the fragments f, and in the slots between them:
    //  OWN    a fragment of f that has served its last MFMA is read again, for k block own_kb of the stage at own_at;
    //  EARLY  the fragments of g are read for k block 0 of the stage at early_at, from the first slot on;
    //  PIECES this wave's pieces [P0, P0 + PIECES) of step req_step are requested, the emptier slots first.
    auto multiply = [&](Frags& f, Frags& g, auto own, uint32_t own_at, int own_kb, auto early, uint32_t early_at, int req_step, auto p0,
                        auto pieces) __attribute__((always_inline)) {
        constexpr bool OWN = decltype(own)::value, EARLY = decltype(early)::value;
        constexpr int P0 = decltype(p0)::value, PIECES = decltype(pieces)::value;
        auto slot = [&](auto number) __attribute__((always_inline)) {
            constexpr int S = decltype(number)::value;
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (EARLY) {
                if constexpr (S * Schedule::kEarlyPerSlot < kReads) read_nth(g, early_at, 0, integral_constant<int, S * Schedule::kEarlyPerSlot>{});
                if constexpr (Schedule::kEarlyPerSlot == 2 && S * 2 + 1 < kReads) read_nth(g, early_at, 0, integral_constant<int, S * 2 + 1>{});
            }
            if constexpr (OWN) {
                constexpr int kD = Schedule::kD, unit = S / kD, a = unit / kTm, b = unit % kTm;
                if constexpr (Schedule::w_slot(a) == S) read_w(f, own_at, own_kb, integral_constant<int, a>{});
                if constexpr (DUAL && Schedule::u_slot(a) == S) read_u(f, own_at, own_kb, integral_constant<int, a>{});
                if constexpr (Schedule::x_slot(b) == S && a == kTn - 1) read_x(f, own_at, own_kb, integral_constant<int, b>{});
            }
            constexpr int kHere = Schedule::requests_at(S, PIECES), kFirst = P0 + Schedule::requests_before(S, PIECES);
            static_assert(kHere <= 4, "listed below");
            if constexpr (kHere > 0) request_piece(req_step, kFirst);
            if constexpr (kHere > 1) request_piece(req_step, kFirst + 1);
            if constexpr (kHere > 2) request_piece(req_step, kFirst + 2);
            if constexpr (kHere > 3) request_piece(req_step, kFirst + 3);
            __builtin_amdgcn_sched_barrier(0);
        };
        auto unit = [&](auto a_, auto b_) __attribute__((always_inline)) {
            constexpr int a = decltype(a_)::value, b = decltype(b_)::value, first = (a * kTm + b) * Schedule::kD;
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, f.w[a]), __builtin_bit_cast(bf16x8_t, f.x[b]),
                                                                acc[a][b], 0, 0, 0);
            slot(integral_constant<int, first>{});
            if constexpr (DUAL) {
                acc_up[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, f.u[a]), __builtin_bit_cast(bf16x8_t, f.x[b]),
                                                                       acc_up[a][b], 0, 0, 0);
                slot(integral_constant<int, first + 1>{});
            }
        };
        unit(integral_constant<int, 0>{}, integral_constant<int, 0>{});
        unit(integral_constant<int, 0>{}, integral_constant<int, 1>{});
        if constexpr (kTn >= 2) {
            unit(integral_constant<int, 1>{}, integral_constant<int, 0>{});
            unit(integral_constant<int, 1>{}, integral_constant<int, 1>{});
        }
        if constexpr (kTn == 3) {
            unit(integral_constant<int, 2>{}, integral_constant<int, 0>{});
            unit(integral_constant<int, 2>{}, integral_constant<int, 1>{});
        }
    };
    static_assert(kTm == 2 && kTn <= 3, "multiply lists the units");
    using yes = std::true_type;
    using no = std::false_type;

    // A step's schedule.  f0 holds the even k blocks of a stage in turn, f1 the odd ones.  While the MFMAs of a k block
    // run, its fragments are read again as they fall free, for the k block two further on; the last k block's (f1) are
    // read for k block 1 of the next step.  The step's one barrier stands behind the MFMAs of the last k block but one:
    // there this wave's reads of the stage have all landed and its own pieces of the next step's stage have (the wait
    // lets the pieces of the steps after that be in flight); behind it the next stage is complete for everybody and
    // this one free.  f0's fragments for k block 0 of the next step are read in the first slots of the last k block; the
    // pieces of step s + kStages - 1 are requested into the stage freed at the barrier before, spread over the k blocks in
    // front of the barrier (with two stages they must have landed at the step's own barrier and go out as early as one
    // to a slot allows).
    auto piece_begin = [](int j) constexpr {
        if (kStages == 2) return j == 0 ? 0 : (j == 1 ? (kPerWave > Schedule::kMfmas ? Schedule::kMfmas : kPerWave) : kPerWave);
        return j * kPerWave / (kKb - 1);
    };
#pragma unroll
    for (int ahead = 0; ahead < kStages - 1; ++ahead)
#pragma unroll
        for (int i = 0; i < kPerWave; ++i) request_piece(ahead, i);
    gm_wait_vm<kPerWave * (kStages - 2)>();
    asm volatile("s_barrier" ::: "memory");
    Frags f0, f1;
    read_all(f0, lds_base, 0);
    read_all(f1, lds_base, 1);
    for (int step = 0; step < steps; ++step) {
        const uint32_t stage_at = lds_base + static_cast<uint32_t>((step % kStages) * kStageBytes);
        const uint32_t next_at = lds_base + static_cast<uint32_t>(((step + 1) % kStages) * kStageBytes);
        const int req = step + kStages - 1;
        // k block j in front of the barrier: its own fragments go on to k block j + 2 (the last of them reads nothing)
        auto k_block = [&](auto j_) __attribute__((always_inline)) {
            constexpr int j = decltype(j_)::value;
            constexpr int p0 = piece_begin(j), count = piece_begin(j + 1) - p0;
            // (f0's last read for k block 0 was issued in slot kLastEarlySlot of the k block before, f1's own reads of
            // that slot and later behind it)
            constexpr int later = j == 0 ? Schedule::own_from(Schedule::kLastEarlySlot) : kReads;
            using own = std::integral_constant<bool, (j + 2 < kKb)>;
            if constexpr (j % 2 == 0) {
                arrived(f0, integral_constant<int, later>{});
                multiply(f0, f1, own{}, stage_at, j + 2, no{}, 0u, req, integral_constant<int, p0>{}, integral_constant<int, count>{});
            } else {
                arrived(f1, integral_constant<int, later>{});
                multiply(f1, f0, own{}, stage_at, j + 2, no{}, 0u, req, integral_constant<int, p0>{}, integral_constant<int, count>{});
            }
        };
        k_block(integral_constant<int, 0>{});
        k_block(integral_constant<int, 1>{});
        k_block(integral_constant<int, 2>{});
        if constexpr (kKb == 8) {
            k_block(integral_constant<int, 3>{});
            k_block(integral_constant<int, 4>{});
            k_block(integral_constant<int, 5>{});
            k_block(integral_constant<int, 6>{});
        }
        arrived(f1, integral_constant<int, 0>{});
        gm_wait_vm<kPerWave * (kStages - 2)>();                   // this wave's pieces of the next step's stage have landed
        asm volatile("s_barrier" ::: "memory");                   // everybody's have; and everybody has read this step's stage
        multiply(f1, f0, yes{}, next_at, 1, yes{}, next_at, req, integral_constant<int, 0>{}, integral_constant<int, 0>{});
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
                if (!DUAL && prm.residual) res = *reinterpret_cast<const uint2*>(prm.residual + static_cast<int64_t>(m) * columns + n);
                uint2 bias_pair = make_uint2(0, 0);
                if (!DUAL && bias) bias_pair = *reinterpret_cast<const uint2*>(bias + n);
                uint32_t packed[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const float s0 = acc[a][b][4 * g + 2 * e], s1 = acc[a][b][4 * g + 2 * e + 1];
                    if (DUAL) {
                        packed[e] = swiglu_pair(s0, s1, acc_up[a][b][4 * g + 2 * e], acc_up[a][b][4 * g + 2 * e + 1]);
                    } else {
                        packed[e] = finish_pair(s0, s1, bias != nullptr, e == 0 ? bias_pair.x : bias_pair.y, prm.residual != nullptr,
                                                e == 0 ? res.x : res.y);
                    }
                }
                *reinterpret_cast<uint2*>(output + static_cast<int64_t>(m) * columns + n) = make_uint2(packed[0], packed[1]);
            }
        }
    }
}

// The pieces of a cut reduction added in order, then what the epilogue above does: thread = four output columns of a row.
template <bool DUAL>
__global__ __launch_bounds__(256) void linear_rows_parts_kernel(LinearRowsParams prm) {
    request_arguments(prm);
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

template <bool DUAL, int BM, int BN, int KSTEP>
int32_t launch_rows_mfma_as(const LinearRowsParams& prm, hipStream_t stream) {
    using Shape = GmShape<DUAL, BM, BN, KSTEP>;
    constexpr int smem = Shape::kStages * Shape::kStageBytes;
    int column_tiles = prm.columns / BN;
    for (int g = 1; g < prm.groups; ++g) column_tiles += prm.group_columns[g - 1] / BN;
    const dim3 grid(static_cast<unsigned>(column_tiles), static_cast<unsigned>((prm.rows + BM - 1) / BM),
                    static_cast<unsigned>(prm.reduction_parts));
    if (grid.y > 65535u) return QM_ERR_ARGUMENT;
    static std::atomic<bool> lds_raised[kMaxDevices];
    const int32_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(linear_rows_mfma_kernel<DUAL, BM, BN, KSTEP>), smem, lds_raised);
    if (rc != QM_OK) return rc;
    hipLaunchKernelGGL((linear_rows_mfma_kernel<DUAL, BM, BN, KSTEP>), grid, dim3(kGmThreads), smem, stream, prm);
    int32_t status = launch_status();
    if (status == QM_OK && prm.reduction_parts > 1) {
        const int64_t quads = static_cast<int64_t>(prm.rows) * (prm.columns / 4);
        hipLaunchKernelGGL((linear_rows_parts_kernel<DUAL>), dim3(static_cast<unsigned>((quads + 255) / 256)), dim3(256), 0, stream, prm);
        status = launch_status();
    }
    return status;
}

// Few token rows leave most CUs without a block (128 rows of a 2048-column linear: 32 blocks), and a block's time is its
// chain of 64-k steps.  With a workspace a long reduction (64 steps or more: the down projection's 6144) is cut so that
// the grid comes to about one block per CU: as many pieces as divide the steps evenly, at most eight.  A reduction of
// 2048 stays whole: the uncut call takes 10 to 11 us at any number of rows up to 512, and the second launch that adds
// the pieces costs what the shorter chains save (measured: 8 us cut at 16 rows, 12 at 128, 14 at 512).
int rows_mfma_reduction_parts(int rows, int columns, int reduction, bool dual) {
    (void)dual;
    if (rows <= 0 || columns < kGmTile || reduction < kGmStep) return 1;
    const int64_t blocks = static_cast<int64_t>(columns / kGmTile) * ((rows + 63) / 64);
    const int steps = reduction / kGmStep;
    if (steps < 64) return 1;
    int parts = 1;
    for (int p = 2; p <= 8; p *= 2)
        if (blocks * p <= 256 && steps % p == 0) parts = p;
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
    const int64_t row_tiles = (prm.rows + 127) / 128;
    int64_t columns = prm.columns;
    for (int g = 1; g < prm.groups; ++g) columns += prm.group_columns[g - 1];
    const int64_t blocks_128 = columns / kGmTile * row_tiles;
    const bool small = blocks_128 < 200;
    if (dual) {
        // a gate/up pair whose grid of 128-column tiles is more than the CUs take at once and less than twice that: tiles
        // of 192 columns, if those fit in one round (1024 tokens x 6144 channels: 384 blocks of 128, 256 of 192)
        const int64_t blocks_192 = static_cast<int64_t>(prm.columns / 192) * row_tiles;
        if (prm.reduction_parts == 1 && prm.columns % 192 == 0 && blocks_128 > 256 && blocks_128 < 512 && blocks_192 <= 256)
            return launch_rows_mfma_as<true, 128, 192, 64>(prm, stream);
        return small ? launch_rows_mfma_as<true, 64, 128, 64>(prm, stream) : launch_rows_mfma_as<true, 128, 128, 64>(prm, stream);
    }
    // (64 token rows and a long uncut reduction: steps of 128 k, half as many barriers for the same MFMAs; a short one
    // loses more to the larger first stages than it gains)
    if (small && prm.reduction_parts == 1 && prm.reduction >= 4096) return launch_rows_mfma_as<false, 64, 128, 128>(prm, stream);
    return small ? launch_rows_mfma_as<false, 64, 128, 64>(prm, stream) : launch_rows_mfma_as<false, 128, 128, 64>(prm, stream);
}

}  // namespace qm
