// qm_talker_chain.hip — everything between two attentions of the talker's decode step in ONE launch (gfx950):
// o_proj, residual + post-norm + gate/up/SwiGLU, down_proj + residual of a layer and the RMSNorm + Q/K/V of the next.
//
// What the launch replaces.  A decode step of a talker layer (R17:17155-17248) is six launches, each a chain of
// start + first-byte latency + a few microseconds of arithmetic + tail around 8 to 75 MB of weights: memory idles
// while the chains run and the reverse, and a layer's 100 MB move at 2 TB/s.  Four of the six operators depend
// only on the attention's output and on each other.
//
// The design.  256 blocks, one per CU, each owning the same rows of every matrix, turn the four operators into
// one stream of weight UNITS: 8 outputs (a pass of the block: 32 threads per output, one reference lane each) by
// 2048 reduction columns, or 8 SwiGLU channels (gate and up row) by 1024 — 32 KiB either way, 12 units per layer
// and block, through a ring of four LDS slots.  An operator whose reduction is longer than a unit carries its
// accumulators from unit to unit, so every chain still runs in the reference's order.  A block is seven waves:
//   * Waves 4 to 6, the WEIGHT waves, do nothing but copy units from memory straight into free slots
//     (global_load_lds, no registers; a third of a unit's 1 KiB pieces each — one wave issues a piece every 200
//     cycles or so, which alone would cap the chip at 3 TB/s), up to three units ahead of the one being consumed,
//     and never have more than a fixed window of pieces under way.  The window is what keeps the hand-offs short: a
//     memory system asked for more than bandwidth x latency only queues the excess, and everything else — the
//     other blocks' polls — waits in the same queues (all free slots requested at once: 25 MB under way, 9 us per
//     hand-off, measured).
//   * Waves 0 to 3, the COMPUTE waves, wait for an operator's input (tagged words, see below), form the input
//     vector (the fused norms: thread t the columns t, t + 256, ... as the reference's 256-thread blocks) and walk the
//     chains, two outputs per wave.  Nothing they wait for is queued behind weight traffic of their own.
//   The waves meet through counters in LDS, not through the block barrier: units landed (each weight wave), units
//   read into registers (each compute wave; a slot is free when all four have read it), arrivals of the compute
//   waves (their own barrier).
//   * Activations go from all blocks to all blocks as in the predictor's frame kernel: a 16-bit value travels in
//     a 32-bit word whose upper half is the number of the operator instance that produced it (counted on from
//     launch to launch in the workspace), the consumer asks for all its words at once until every tag is the
//     expected one.  While a block waits for an input its ring fills up.
//   * Every wait is bounded; a block that gives up raises the abort word, ORs QM_STATUS_FRAME_TIMEOUT into the
//     status word and returns, and so does every block that sees the abort word: the grid always drains.
// Arithmetic: the operators of qm_linear.hip (R17:15239-15266, 15340-15360, 16205-16362, 8276-8338) chain for
// chain, tree for tree and rounding for rounding — the outputs equal the four launches' bit for bit.
//
// Geometry is that of the 1.7B talker: hidden 2048 (R17:14626), and what its checkpoint gives for the rest
// (R17:14862, 14993-15003): 16 / 8 heads of 128, intermediate 6144.

#include "qm_device.h"
#include "qm_host.h"
#include "qm_resident.h"
#include "qm_decode_step.h"

#include <atomic>
#include <type_traits>

namespace qm {
namespace {

constexpr int kTkThreads = 448;                      // four compute waves + three weight waves
constexpr int kTkComputeThreads = 256;
constexpr int kTkWeightWaves = 3;
constexpr int kTkBlocks = 256;
constexpr int kTkHidden = 2048;
constexpr int kTkQDim = 2048;
constexpr int kTkKvDim = 1024;
constexpr int kTkInter = 6144;
constexpr unsigned kTkSpinLimit = 1u << 17;

// a unit in LDS: 8 rows of 2048 columns or 16 rows (gate, up, gate, ...) of 1024, rows padded by 64 bytes so that
// the rows read by one instruction fall on different banks
constexpr int kTkUnitColumns = 2048;
constexpr int kTkDualColumns = 1024;
constexpr int kTkSingleStride = 2 * kTkUnitColumns + 64;
constexpr int kTkDualStride = 2 * kTkDualColumns + 64;
constexpr int kTkSlotBytes = 16 * kTkDualStride;
static_assert(8 * kTkSingleStride <= kTkSlotBytes, "both kinds of unit fit a slot");
constexpr int kTkSlots = 4;
constexpr int kTkPieces = 32;                        // 1 KiB pieces per unit (one instruction of a wave each)
constexpr int kTkFirstHandoffGate = 3;                 // units requested before o_proj's outputs have been exchanged
constexpr int kTkWindow = 10;                        // pieces a weight wave has under way at most: its share of a unit
constexpr int kTkLdsX = 0;                           // the operator's input vector, fp32 (down_proj: 6144)
constexpr int kTkLdsRing = kTkLdsX + kTkInter * 4;
constexpr int kTkLdsBytes = kTkLdsRing + kTkSlots * kTkSlotBytes;
static_assert(kTkLdsBytes <= 160 * 1024 - 1024, "the LDS map must fit one CU");

// units of a layer and block, in the order of use
constexpr int kTkUnitO = 0;                          // 1: the block's 8 o_proj rows
constexpr int kTkUnitGu = 1;                         // 6: 3 passes of 8 channels x 2 halves of the reduction
constexpr int kTkUnitDown = 7;                       // 3: the block's 8 down_proj rows x 3 thirds of the reduction
constexpr int kTkUnitQkv = 10;                       // 2: 2 passes of the block's 16 Q/K/V rows of the next layer
constexpr int kTkUnits = 12;

// workspace map (32-bit words)
constexpr int kTkWsBase = 0;                         // number of the next launch's first operator instance
constexpr int kTkWsAbort = 1;
constexpr int kTkWsLastContext = 2;                  // operator number in the context words, as the last launch that wrote them left it
constexpr int kTkWsAttn = 64;
constexpr int kTkWsAct = kTkWsAttn + kTkHidden;
constexpr int kTkWsHidden = kTkWsAct + kTkInter;
constexpr int kTkWsContext = kTkWsHidden + kTkHidden;   // the attention's output, when this launch combines its splits
constexpr int kTkWsWords = kTkWsContext + kTkQDim;
constexpr int64_t kTkWsBytes = (static_cast<int64_t>(kTkWsWords) * 4 + 255) / 256 * 256;
constexpr uint32_t kTkTagsPerLaunch = 8;               // 0..3 used; 5: the context's second choice (below)

struct TkParams {
    const uint16_t* context;
    const uint16_t* hidden;
    const uint16_t* o_weight;
    const uint16_t* o_bias;
    const uint16_t* post_norm;
    const uint16_t* gate_weight;
    const uint16_t* up_weight;
    const uint16_t* down_weight;
    uint16_t* hidden_out;
    const uint16_t* next_input_norm;
    const uint16_t* next_weight[3];
    const uint16_t* next_bias[3];
    uint16_t* next_out[3];
    uint32_t* workspace;
    uint32_t* status;
    float epsilon;
    unsigned spin_limit;
    int has_next;
    // The attention ran without its merge launch (qm_talker_layer_step_m1): the first eight blocks combine the split
    // records of one kv head each and hand the context to everybody; NULL: `context` holds it already.
    const float* attention_records;
    int attention_splits;
    int attention_max_splits;
    uint16_t* context_out;
};

struct TkShared {
    // (each of the two counter sets is read with one 16-byte instruction)
    __attribute__((aligned(16))) int landed[4];   // units whose pieces of weight wave 0, 1, 2 are in LDS; [3] unused
    __attribute__((aligned(16))) int done[4];     // units each compute wave has read into registers
    int abort;
    int first_input_seen;       // the compute waves have o_proj's outputs of all blocks
    int arrivals;               // of compute waves at their barrier, counted on
    float groups[8];            // the eight 32-lane sums of a norm
    float residual[8];
    float bias[16];
};

// A compute thread's words tid, tid + 256, ... of a tagged vector, all requested at once, again and again until
// every one carries `tag`.  False when the wait gave up (or another block did).
template <int N>
__device__ __forceinline__ bool poll_words(const uint32_t* words, uint32_t tag, const uint32_t* abort_word, unsigned spin_limit,
                                           uint32_t (&v)[N]) {
    const int tid = threadIdx.x;
    for (unsigned spins = 0;; ++spins) {
#pragma unroll
        for (int u = 0; u < N; ++u) v[u] = agent_load(words + tid + kTkComputeThreads * u);
        bool fresh = true;
#pragma unroll
        for (int u = 0; u < N; ++u) fresh = fresh && (v[u] >> 16) == tag;
        if (fresh) return true;
        if (spins >= spin_limit) return false;
        if ((spins & 255u) == 255u && agent_load(abort_word) != 0u) return false;
        __builtin_amdgcn_s_sleep(1);
    }
}

// A weight wave (`third` = 0, 1, 2): requests its pieces of unit `v` of block `b` into `slot`, one by one, each once
// fewer than kTkWindow of its pieces are under way; `issued` counts its pieces so far.  Returns how many of them are
// known to have landed.
__device__ __forceinline__ int request_unit(const TkParams& p, int v, int b, unsigned char* slot, int third, int& issued) {
    const int lane = threadIdx.x & 63;
    const unsigned char* base;
    const unsigned char* base_up = nullptr;
    int64_t pitch = 2 * kTkHidden;
    bool dual = false;
    if (v == kTkUnitO) {
        base = reinterpret_cast<const unsigned char*>(p.o_weight + static_cast<int64_t>(8 * b) * kTkQDim);
        pitch = 2 * kTkQDim;
    } else if (v < kTkUnitDown) {
        const int pass = (v - kTkUnitGu) >> 1, half = (v - kTkUnitGu) & 1;
        const int64_t at = static_cast<int64_t>(24 * b + 8 * pass) * kTkHidden + kTkDualColumns * half;
        base = reinterpret_cast<const unsigned char*>(p.gate_weight + at);
        base_up = reinterpret_cast<const unsigned char*>(p.up_weight + at);
        dual = true;
    } else if (v < kTkUnitQkv) {
        base = reinterpret_cast<const unsigned char*>(p.down_weight + static_cast<int64_t>(8 * b) * kTkInter + kTkUnitColumns * (v - kTkUnitDown));
        pitch = 2 * kTkInter;
    } else {
        int row = 16 * b;                                  // over [Q | K | V]; a block's rows lie in one matrix
        const uint16_t* matrix = p.next_weight[0];
        if (row >= kTkQDim + kTkKvDim) { matrix = p.next_weight[2]; row -= kTkQDim + kTkKvDim; }
        else if (row >= kTkQDim) { matrix = p.next_weight[1]; row -= kTkQDim; }
        base = reinterpret_cast<const unsigned char*>(matrix + static_cast<int64_t>(row + 8 * (v - kTkUnitQkv)) * kTkHidden);
    }
#pragma unroll 1
    for (int q = third; q < kTkPieces; q += kTkWeightWaves) {
        const unsigned char* src;
        unsigned char* dst;
        if (!dual) {
            const int row = q >> 2, off = (q & 3) << 10;
            src = base + row * pitch + off;
            dst = slot + row * kTkSingleStride + off;
        } else {
            const int row = q >> 1, off = (q & 1) << 10;      // LDS rows 2c, 2c + 1: gate and up row of channel c
            src = ((row & 1) ? base_up : base) + (row >> 1) * pitch + off;
            dst = slot + row * kTkDualStride + off;
        }
        wait_vm_at_most<kTkWindow - 1>();
        __builtin_amdgcn_global_load_lds(src + lane * 16, (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
        ++issued;
    }
    // (requests complete in the order they were made: all but the last kTkWindow have landed)
    return issued > kTkWindow ? issued - kTkWindow : 0;
}
static_assert(kTkWindow <= kTkPieces / kTkWeightWaves, "a unit is known to have landed when the next has been requested");

__global__ __launch_bounds__(kTkThreads, 1) void talker_chain_kernel(TkParams p) {
    request_arguments(p);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ TkShared sh;
    const int tid = threadIdx.x;
    const int b = blockIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    uint32_t* const ws = p.workspace;
    const uint32_t* const abort_word = ws + kTkWsAbort;
    const uint32_t base = agent_load(ws + kTkWsBase);
    // The context words are written only by launches that combine the attention's splits: what they hold may be any
    // number of launches old, and the 16-bit operator numbers repeat.  A launch whose number for them would be the one
    // they were last written with takes its second choice.
    const uint32_t last_context = agent_load(ws + kTkWsLastContext);
    const uint32_t context_number = ((base + 3u) ^ last_context) & 0xffffu ? base + 3u : base + 5u;
    const uint32_t context_tag = context_number & 0xffffu;
    if (tid == 0) {
        sh.abort = agent_load(abort_word) != 0u ? 1 : 0;   // a launch gave up and the workspace was not set up again
        sh.landed[0] = sh.landed[1] = sh.landed[2] = sh.landed[3] = 0;
        sh.done[0] = sh.done[1] = sh.done[2] = sh.done[3] = 0;
        sh.arrivals = 0;
        sh.first_input_seen = 0;
    }
    __syncthreads();
    if (sh.abort) {
        if (tid == 0 && p.status) atomicOr(p.status, QM_STATUS_FRAME_TIMEOUT);
        return;
    }
    const unsigned spin_limit = p.spin_limit;
    const int units = p.has_next ? kTkUnits : kTkUnitQkv;
    unsigned char* const ring = smem + kTkLdsRing;
    float* const lin_x = reinterpret_cast<float*>(smem + kTkLdsX);

    if (tid >= kTkComputeThreads) {
        // ---- a weight wave: every third piece of every unit ----
        const int third = wave - kTkComputeThreads / 64;
        const int my_pieces = (kTkPieces - third + kTkWeightWaves - 1) / kTkWeightWaves;
        int issued = 0, published = 0;                  // pieces requested; units whose pieces are known to have landed
        bool alive = true;
#pragma unroll 1
        for (int r = 0; alive && r < units; ++r) {
            // While the first hand-off is under way only the first three units are requested: the polls for o_proj's
            // outputs travel through the same queues as the requests that fill the ring and come back when those have
            // (gate at unit 1 / 2 / 3 / none: 35.9 / 34.8 / 34.7 / 36.0 us per layer).
            if (r == kTkFirstHandoffGate) {
                while (lds_word(&sh.first_input_seen) == 0u && lds_word(&sh.abort) == 0u) __builtin_amdgcn_s_sleep(1);
            }
            // the slot is free once unit r - kTkSlots has been read by all four compute waves
            if (r >= kTkSlots) {
                for (;;) {
                    const lds_int4 d = lds_four(sh.done);
                    if (min(min(d.x, d.y), min(d.z, d.w)) > r - kTkSlots) break;
                    if (lds_word(&sh.abort) != 0u) { alive = false; break; }
                    if (published < r) {                  // nothing to request: see everything requested land, say so
                        wait_vm_at_most<0>();
                        published = r;
                        if (lane == 0) lds_store(&sh.landed[third], static_cast<uint32_t>(published));
                    }
                    __builtin_amdgcn_s_sleep(1);
                }
                if (!alive) break;
            }
            int landed = request_unit(p, r, b, ring + (r & (kTkSlots - 1)) * kTkSlotBytes, third, issued) / my_pieces;
            if (r == 0) {                                 // the first unit is waited for: say so as soon as it is there
                wait_vm_at_most<0>();
                landed = 1;
            }
            if (landed > published) {
                published = landed;
                if (lane == 0) lds_store(&sh.landed[third], static_cast<uint32_t>(published));
            }
        }
        wait_vm_at_most<0>();
        if (alive && lane == 0) lds_store(&sh.landed[third], static_cast<uint32_t>(units));
    } else {
        // ---- the compute waves ----
        const int l = tid & 31;             // reference lane
        const int c8 = tid >> 5;            // output of the pass
        auto tag = [&](uint32_t phase) { return (base + phase) & 0xffffu; };
        uint32_t* const attn = ws + kTkWsAttn;
        uint32_t* const act = ws + kTkWsAct;
        uint32_t* const hidden_words = ws + kTkWsHidden;
        int unit = 0, arrivals = 0;
        bool alive = true;
        // waits until *counter >= value; false when the launch gave up
        auto wait_for = [&](const int* counter, int value) __attribute__((always_inline)) -> bool {
            for (;;) {
                if (static_cast<int>(lds_word(counter)) >= value) return true;
                if (lds_word(&sh.abort) != 0u) return false;
                __builtin_amdgcn_s_sleep(1);
            }
        };
        // the barrier of the four compute waves (a wave's LDS traffic is performed in order: what it wrote before
        // it arrived is there for whoever sees its arrival); false when the launch gave up
        auto compute_barrier = [&]() __attribute__((always_inline)) -> bool {
            arrivals += kTkComputeThreads / 64;
            if (lane == 0) lds_add_one(&sh.arrivals);
            return wait_for(&sh.arrivals, arrivals);
        };
        auto give_up = [&]() __attribute__((always_inline)) { lds_store(&sh.abort, 1u); };
        // One unit: wait until it has landed, read this thread's input values and weights, say so, then walk the
        // chain segment.  False when the launch gave up.
        auto run_unit = [&](auto dual, int x_first, float& acc, float& up) __attribute__((always_inline)) -> bool {
            constexpr bool kDual = decltype(dual)::value;
            constexpr int kSteps = kDual ? kTkDualColumns / 32 : kTkUnitColumns / 32;
            unsigned char* const slot = ring + (unit & (kTkSlots - 1)) * kTkSlotBytes;
            for (;;) {
                const lds_int4 landed = lds_four(sh.landed);
                if (min(min(landed.x, landed.y), landed.z) > unit) break;
                if (lds_word(&sh.abort) != 0u) return false;
                __builtin_amdgcn_s_sleep(1);
            }
            uint32_t x[kSteps], w[kSteps], wu[kDual ? kSteps : 1];
            lds_read_b32<0, kSteps, 128>(lds_at(lin_x + x_first) + 4u * l, x);
            if constexpr (kDual) {
                lds_read_u16<0, kSteps, 64>(lds_at(slot) + static_cast<uint32_t>(2 * c8 * kTkDualStride) + 2u * l, w);
                lds_read_u16<0, kSteps, 64>(lds_at(slot) + static_cast<uint32_t>((2 * c8 + 1) * kTkDualStride) + 2u * l, wu);
            } else {
                lds_read_u16<0, kSteps, 64>(lds_at(slot) + static_cast<uint32_t>(c8 * kTkSingleStride) + 2u * l, w);
            }
            lds_wait();
            pin<0, kSteps>(x);
            pin<0, kSteps>(w);
            if constexpr (kDual) pin<0, kSteps>(wu);
            ++unit;
            if (lane == 0) lds_store(&sh.done[wave], static_cast<uint32_t>(unit));
#pragma unroll
            for (int j = 0; j < kSteps; ++j) {
                acc = fmaf(__uint_as_float(x[j]), bf2f(static_cast<uint16_t>(w[j])), acc);
                if constexpr (kDual) up = fmaf(__uint_as_float(x[j]), bf2f(static_cast<uint16_t>(wu[j])), up);
            }
            return true;
        };
        // RMSNorm of this thread's eight columns `value` (R17:8276-8338, 16205-16286) into the input vector.  The
        // reference's block of 256 threads sums the squares of columns t, t + 256, ... per thread, adds the threads in
        // eight 32-lane trees and those in a tree over lanes 0..7 (R17:15102-15148).  Between the group sums and the
        // write lies a barrier that every wave reaches after its last read of the input vector before.
        auto norm_into_input = [&](const float (&value)[kTkHidden / kTkComputeThreads], const uint32_t (&norm_raw)[kTkHidden / kTkComputeThreads])
                __attribute__((always_inline)) -> bool {
            float partial = 0.0f;
#pragma unroll
            for (int u = 0; u < kTkHidden / kTkComputeThreads; ++u) partial = fmaf(value[u], value[u], partial);
            const float tree = half_wave_tree_sum(partial);
            if (l == 0) sh.groups[c8] = tree;
            if (!compute_barrier()) return false;
            const float* g = sh.groups;
            const float total = ((g[0] + g[4]) + (g[2] + g[6])) + ((g[1] + g[5]) + (g[3] + g[7]));
            const float inverse_rms = 1.0f / sqrtf(total / static_cast<float>(kTkHidden) + p.epsilon);
#pragma unroll
            for (int u = 0; u < kTkHidden / kTkComputeThreads; ++u)
                lin_x[tid + kTkComputeThreads * u] = round_bf16(round_bf16(value[u] * inverse_rms) * bf2f(static_cast<uint16_t>(norm_raw[u])));
            return compute_barrier();
        };
        const std::true_type dual_unit;
        const std::false_type single_unit;
        float acc = 0.0f, up = 0.0f;
        constexpr int kPerThread = kTkHidden / kTkComputeThreads;     // input columns of a thread: tid, tid + 256, ...
        static_assert(kTkQDim == kTkHidden, "o_proj's input is staged like the hidden state");
        // the block's 16 rows of the next layer's [Q | K | V] lie in one matrix
        int qkv_row = 16 * b;
        const uint16_t* qkv_bias = p.next_bias[0];
        uint16_t* qkv_out = p.next_out[0];
        if (qkv_row >= kTkQDim + kTkKvDim) { qkv_bias = p.next_bias[2]; qkv_out = p.next_out[2]; qkv_row -= kTkQDim + kTkKvDim; }
        else if (qkv_row >= kTkQDim) { qkv_bias = p.next_bias[1]; qkv_out = p.next_out[1]; qkv_row -= kTkQDim; }

        if (p.attention_records && b < kTkKvDim / 128) {
            // ---- the attention's splits, combined as decode_merge_kernel<2> combines them (same statistics, same
            // order, same bits): block h the two query heads of kv head h, thread (g, d) one output ----
            constexpr int kRecord = 2 * 128 + 4;                 // acc[2][128], max[2], sum[2]
            const int g = tid >> 7, d = tid & 127;
            const int n = p.attention_splits;
            const float* records = p.attention_records + static_cast<int64_t>(b) * p.attention_max_splits * kRecord;
            float* const stat_m = lin_x;                            // [32][2]: the input vector is not in use yet
            float* const stat_l = lin_x + 2 * kDecodeMergeRound;
            // (eight records at a time through one small loop: instructions a block executes once cost tens of cycles
            // each to fetch, and this runs while the first weights are still on their way)
            constexpr int kChunk = 8;
            float part[kChunk];
            const float* column = records + g * 128 + d;
#pragma unroll
            for (int u = 0; u < kChunk; ++u) part[u] = u < n ? column[u * kRecord] : 0.0f;
            if (tid < 2 * n) {
                const float* rec = records + (tid >> 1) * kRecord;
                stat_m[tid] = rec[2 * 128 + (tid & 1)];
                stat_l[tid] = rec[2 * 128 + 2 + (tid & 1)];
            }
            alive = compute_barrier();
            if (alive) {
                float mm = -INFINITY;
                for (int s = 0; s < n; ++s) mm = fmaxf(mm, stat_m[2 * s + g]);
                const float m_ref = mm == -INFINITY ? 0.0f : mm;
                float ll = 0.0f, aa = 0.0f;
#pragma unroll 1
                for (int first = 0; first < n; first += kChunk) {
                    if (first > 0) {
#pragma unroll
                        for (int u = 0; u < kChunk; ++u) part[u] = first + u < n ? column[(first + u) * kRecord] : 0.0f;
                    }
#pragma unroll
                    for (int u = 0; u < kChunk; ++u) {
                        if (first + u < n) {
                            const float w = fast_exp2((stat_m[2 * (first + u) + g] - m_ref) * kLog2e);
                            ll = fmaf(stat_l[2 * (first + u) + g], w, ll);
                            aa = fmaf(part[u], w, aa);
                        }
                    }
                }
                const uint16_t bits = f2bf(ll > 0.0f ? aa / ll : 0.0f);
                agent_store(ws + kTkWsContext + 256 * b + tid, (context_tag << 16) | bits);
                if (p.context_out) p.context_out[256 * b + tid] = bits;
                alive = compute_barrier();                          // the statistics have been read: the input vector may be written
            }
        }

        // The units in order, through ONE copy of each piece of code (a kernel's instructions are fetched as they are
        // first executed, tens of cycles each: straight-line code for twelve units ran several times slower than this
        // loop).  Before the first unit of an operator its input vector is formed, after the last the outputs leave.
#pragma unroll 1
        for (int u = 0; alive && u < units; ++u) {
            if (u == kTkUnitO) {
                // ---- o_proj (R17:17203-17210): the attention's output is given ----
                uint32_t raw[kPerThread];
                if (p.attention_records) {
                    alive = poll_words<kPerThread>(ws + kTkWsContext, context_tag, abort_word, spin_limit, raw);
                    if (!alive) give_up();
                } else {
#pragma unroll
                    for (int i = 0; i < kPerThread; ++i) raw[i] = p.context[tid + kTkComputeThreads * i];
                }
                if (!alive) break;
                if (p.o_bias && tid < 8) sh.bias[tid] = bf2f(p.o_bias[8 * b + tid]);
#pragma unroll
                for (int i = 0; i < kPerThread; ++i) lin_x[tid + kTkComputeThreads * i] = bf2f(static_cast<uint16_t>(raw[i]));
                alive = compute_barrier();
            } else if (u == kTkUnitGu || u == kTkUnitQkv) {
                // ---- residual + post-norm in front of gate/up (R17:17215-17229), or the next layer's input norm in
                // front of its Q/K/V (R17:17163-17176) ----
                const bool with_add = u == kTkUnitGu;
                const uint16_t* norm_weight = with_add ? p.post_norm : p.next_input_norm;
                uint32_t raw[kPerThread], plain[kPerThread], norm_raw[kPerThread];
#pragma unroll
                for (int i = 0; i < kPerThread; ++i) {
                    norm_raw[i] = norm_weight[tid + kTkComputeThreads * i];
                    plain[i] = with_add ? p.hidden[tid + kTkComputeThreads * i] : 0u;
                }
                if (!with_add && qkv_bias && tid < 16) sh.bias[tid] = bf2f(qkv_bias[qkv_row + tid]);
                alive = poll_words<kPerThread>(with_add ? attn : hidden_words, with_add ? tag(0) : tag(2), abort_word, spin_limit, raw);
                if (!alive) give_up();
                if (with_add && tid == 0) lds_store(&sh.first_input_seen, 1u);
                float value[kPerThread];
#pragma unroll
                for (int i = 0; i < kPerThread; ++i) {
                    value[i] = bf2f(static_cast<uint16_t>(raw[i]));
                    if (with_add) {
                        // residual = bf16(hidden + attention); the block keeps that of its own down_proj rows
                        value[i] = bf2f(f2bf(bf2f(static_cast<uint16_t>(plain[i])) + value[i]));
                        const int k = tid + kTkComputeThreads * i - 8 * b;
                        if (k >= 0 && k < 8) sh.residual[k] = value[i];
                    }
                }
                alive = alive && norm_into_input(value, norm_raw);
            } else if (u == kTkUnitDown) {
                // ---- down_proj's input (R17:17236-17244) ----
                uint32_t raw[kTkInter / kTkComputeThreads];
                alive = poll_words<kTkInter / kTkComputeThreads>(act, tag(1), abort_word, spin_limit, raw);
                if (!alive) give_up();
                alive = alive && compute_barrier();          // everybody has read the input vector before
                if (alive) {
#pragma unroll
                    for (int i = 0; i < kTkInter / kTkComputeThreads; ++i)
                        lin_x[tid + kTkComputeThreads * i] = bf2f(static_cast<uint16_t>(raw[i]));
                    alive = compute_barrier();
                }
            }
            if (!alive) break;
            const bool is_dual = u >= kTkUnitGu && u < kTkUnitDown;
            const int part = is_dual ? (u - kTkUnitGu) & 1 : (u >= kTkUnitDown && u < kTkUnitQkv ? u - kTkUnitDown : 0);   // of the reduction
            const bool last_part = is_dual ? part == 1 : (u >= kTkUnitDown && u < kTkUnitQkv ? part == 2 : true);
            if (part == 0) {
                acc = 0.0f;
                up = 0.0f;
            }
            alive = is_dual ? run_unit(dual_unit, kTkDualColumns * part, acc, up) : run_unit(single_unit, kTkUnitColumns * part, acc, up);
            if (!alive || !last_part) continue;
            // ---- the outputs of a pass: the reference's shuffle tree over its 32 lanes, lane 0 rounds and stores ----
            acc = half_wave_tree_sum(acc);
            if (is_dual) up = half_wave_tree_sum(up);
            if (l != 0) continue;
            if (u == kTkUnitO) {
                float r = acc;
                if (p.o_bias) r += __uint_as_float(lds_word(&sh.bias[c8]));
                agent_store(attn + 8 * b + c8, (tag(0) << 16) | f2bf(r));
            } else if (is_dual) {
                const int pass = (u - kTkUnitGu) >> 1;
                const float gv = bf2f(f2bf(acc));
                const uint16_t activated = f2bf(gv / (1.0f + expf(-gv)));
                agent_store(act + 24 * b + 8 * pass + c8, (tag(1) << 16) | f2bf(bf2f(activated) * bf2f(f2bf(up))));
            } else if (u < kTkUnitQkv) {
                const uint16_t bits = f2bf(__uint_as_float(lds_word(&sh.residual[c8])) + bf2f(f2bf(acc)));
                agent_store(hidden_words + 8 * b + c8, (tag(2) << 16) | bits);
                p.hidden_out[8 * b + c8] = bits;
            } else {
                const int pass = u - kTkUnitQkv;
                float r = acc;
                if (qkv_bias) r += __uint_as_float(lds_word(&sh.bias[8 * pass + c8]));
                qkv_out[qkv_row + 8 * pass + c8] = f2bf(r);
            }
        }
        if (!alive) give_up();
    }

    __builtin_amdgcn_s_waitcnt(0);                       // (a wave that gave up may still have pieces under way)
    __syncthreads();
    if (sh.abort) {
        if (tid == 0) {
            agent_store(ws + kTkWsAbort, 1u);
            if (p.status) atomicOr(p.status, QM_STATUS_FRAME_TIMEOUT);
        }
        return;
    }
    // (every block has read the base before this one could finish its last operator)
    if (tid == 0 && b == 0) {
        agent_store(ws + kTkWsBase, base + kTkTagsPerLaunch);
        if (p.attention_records) agent_store(ws + kTkWsLastContext, context_number);
    }
}

// Sets a workspace to "nothing produced yet": every tagged word 0, operator numbers from 1 (a kernel, not a
// memset: callers may capture it).
__global__ void talker_chain_clear_kernel(uint32_t* words, int count) {
    const int i = static_cast<int>(blockIdx.x) * static_cast<int>(blockDim.x) + static_cast<int>(threadIdx.x);
    if (i < count) words[i] = i == kTkWsBase ? 1u : 0u;
}

}  // namespace
}  // namespace qm

extern "C" int64_t qm_talker_post_attention_workspace_bytes(void) { return qm::kTkWsBytes; }

extern "C" int32_t qm_talker_post_attention_workspace_init(void* workspace, int64_t workspace_bytes, void* hip_stream) {
    using namespace qm;
    if (!workspace) return QM_ERR_NULL;
    if (workspace_bytes < kTkWsBytes) return QM_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return QM_ERR_GEOMETRY;
    const int count = static_cast<int>(kTkWsBytes / 4);
    hipLaunchKernelGGL(talker_chain_clear_kernel, dim3((count + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(hip_stream),
                       static_cast<uint32_t*>(workspace), count);
    return launch_status();
}

namespace qm {
namespace {

// What a launch asks of its arguments (everything that can be seen from the host without a device call).
int32_t check_chain(const qm_talker_post_attention* op, const void* workspace, int64_t workspace_bytes) {
    if (!op || !workspace) return QM_ERR_NULL;
    if (workspace_bytes < kTkWsBytes) return QM_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return QM_ERR_GEOMETRY;
    if (op->hidden_columns != kTkHidden || op->q_columns != kTkQDim || op->kv_columns != kTkKvDim
        || op->intermediate_columns != kTkInter)
        return QM_ERR_GEOMETRY;                           // the talker's geometry only; other shapes take the operators one by one
    if (!op->context || !op->hidden || !op->o_weight || !op->post_norm || !op->gate_weight || !op->up_weight || !op->down_weight
        || !op->hidden_out)
        return QM_ERR_NULL;
    const bool has_next = op->next_q_weight != nullptr;
    if (has_next && (!op->next_input_norm || !op->next_k_weight || !op->next_v_weight || !op->q_out || !op->k_out || !op->v_out))
        return QM_ERR_NULL;
    uintptr_t align = reinterpret_cast<uintptr_t>(op->o_weight) | reinterpret_cast<uintptr_t>(op->gate_weight)
                    | reinterpret_cast<uintptr_t>(op->up_weight) | reinterpret_cast<uintptr_t>(op->down_weight);
    if (has_next)
        align |= reinterpret_cast<uintptr_t>(op->next_q_weight) | reinterpret_cast<uintptr_t>(op->next_k_weight)
               | reinterpret_cast<uintptr_t>(op->next_v_weight);
    if (align & 15) return QM_ERR_GEOMETRY;               // 16-byte pieces of weight rows
    return QM_OK;
}

// Every block must be resident at once, one per CU: QM_OK if `hip_stream` can hold the launch, QM_ERR_NO_DEVICE if
// the device, or the part of it the stream is confined to by a CU mask, is too small.  (The occupancy is asked of the
// runtime once per device, the stream's mask at every call.)
int32_t chain_residency(void* hip_stream) {
    int device = 0;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return hip_code(err);
    if (device < 0 || device >= kMaxDevices) return QM_ERR_NO_DEVICE;
    static std::atomic<bool> lds_raised[kMaxDevices];
    const int32_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(talker_chain_kernel), kTkLdsBytes, lds_raised);
    if (rc != QM_OK) return rc;
    static std::atomic<int> per_cu_of[kMaxDevices];        // 0: not asked yet; else blocks a CU holds at once (-1: none)
    int per_cu = per_cu_of[device].load(std::memory_order_acquire);
    if (per_cu == 0) {
        err = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, talker_chain_kernel, kTkThreads, kTkLdsBytes);
        if (err != hipSuccess) return hip_code(err);
        if (per_cu <= 0) per_cu = -1;
        per_cu_of[device].store(per_cu, std::memory_order_release);
    }
    bool fits = false;
    const int32_t rc_fit = resident_blocks_fit(hip_stream, device, per_cu > 0 ? per_cu : 0, kTkBlocks, &fits);
    if (rc_fit != QM_OK) return rc_fit;
    return fits ? QM_OK : QM_ERR_NO_DEVICE;
}

// The launch; with `attention` the kernel first combines that decode step's split records into `context_out`.
int32_t launch_chain(const qm_talker_post_attention* op, void* workspace, int64_t workspace_bytes, uint32_t* status_dev,
                     void* hip_stream, const DecodeSplitInfo* attention, uint16_t* context_out) {
    const int32_t bad = check_chain(op, workspace, workspace_bytes);
    if (bad != QM_OK) return bad;
    const bool has_next = op->next_q_weight != nullptr;
    TkParams prm = {};
    prm.context = op->context; prm.hidden = op->hidden; prm.o_weight = op->o_weight; prm.o_bias = op->o_bias;
    prm.post_norm = op->post_norm; prm.gate_weight = op->gate_weight; prm.up_weight = op->up_weight;
    prm.down_weight = op->down_weight; prm.hidden_out = op->hidden_out;
    prm.next_input_norm = op->next_input_norm;
    prm.next_weight[0] = op->next_q_weight; prm.next_weight[1] = op->next_k_weight; prm.next_weight[2] = op->next_v_weight;
    prm.next_bias[0] = op->next_q_bias; prm.next_bias[1] = op->next_k_bias; prm.next_bias[2] = op->next_v_bias;
    prm.next_out[0] = op->q_out; prm.next_out[1] = op->k_out; prm.next_out[2] = op->v_out;
    prm.workspace = static_cast<uint32_t*>(workspace);
    prm.status = status_dev;
    prm.epsilon = op->epsilon;
    prm.has_next = has_next ? 1 : 0;
    if (attention && attention->records) {
        if (attention->splits < 1 || attention->splits > kDecodeMergeRound || attention->splits > attention->max_splits) return QM_ERR_ARGUMENT;
        prm.attention_records = attention->records;
        prm.attention_splits = attention->splits;
        prm.attention_max_splits = attention->max_splits;
        prm.context_out = context_out;
    }
    const int32_t spin_option = option_value(QM_OPT_PREDICTOR_FRAME_SPIN_LIMIT);
    prm.spin_limit = spin_option > 0 ? static_cast<unsigned>(spin_option) : kTkSpinLimit;

    const int32_t rc = chain_residency(hip_stream);
    if (rc != QM_OK) return rc;
    hipLaunchKernelGGL(talker_chain_kernel, dim3(kTkBlocks), dim3(kTkThreads), kTkLdsBytes, static_cast<hipStream_t>(hip_stream), prm);
    return launch_status();
}

}  // namespace
}  // namespace qm

extern "C" int32_t qm_talker_chain_fits(void* hip_stream, int32_t* fits) {
    if (!fits) return QM_ERR_NULL;
    const int32_t rc = qm::chain_residency(hip_stream);
    if (rc != QM_OK && rc != QM_ERR_NO_DEVICE) return rc;
    *fits = rc == QM_OK ? 1 : 0;
    return QM_OK;
}

extern "C" int32_t qm_talker_post_attention_m1(const qm_talker_post_attention* op, void* workspace, int64_t workspace_bytes,
                                               uint32_t* status_dev, void* hip_stream) {
    return qm::launch_chain(op, workspace, workspace_bytes, status_dev, hip_stream, nullptr, nullptr);
}

extern "C" int32_t qm_talker_layer_step_m1(const qm_talker_layer_step* step, void* workspace, int64_t workspace_bytes,
                                           uint32_t* status_dev, void* hip_stream) {
    using namespace qm;
    if (!step || !workspace || !step->context) return QM_ERR_NULL;
    if (step->q_heads != kTkQDim / 128 || !step->cache || step->cache->kv_heads != kTkKvDim / 128) return QM_ERR_GEOMETRY;
    // validate the second launch's arguments before the first is made: a step is made whole or not at all
    qm_talker_post_attention post = step->post;
    post.context = step->context;
    const int32_t bad = check_chain(&post, workspace, workspace_bytes);
    if (bad != QM_OK) return bad;
    const int32_t no_room = chain_residency(hip_stream);
    if (no_room != QM_OK) return no_room;
    DecodeSplitInfo info = {};
    const int32_t rc = decode_step(step->q, step->k, step->v, step->q_norm_w, step->k_norm_w, step->cos_row, step->sin_row,
                                   step->q_rotated_out, step->cache, step->page_table, step->max_pages, step->context, step->q_heads,
                                   step->position, step->sliding_window, step->scale, step->epsilon, step->attention_workspace,
                                   step->attention_workspace_bytes, status_dev, hip_stream, &info);
    if (rc != QM_OK) return rc;
    return launch_chain(&post, workspace, workspace_bytes, status_dev, hip_stream, &info, step->context);
}
