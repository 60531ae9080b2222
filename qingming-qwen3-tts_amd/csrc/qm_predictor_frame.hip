// qm_predictor_frame.hip — the M = 1 steps of one code-predictor frame in ONE launch (gfx950).
//
// What the launch replaces.  A step of the predictor (PersistentPredictor::capture_step, R17:13592-13854) is a chain
// of 28 operators, each of which needs the whole output of the one before it: the input projection, five layers
// of (RMSNorm + Q/K/V, QK-norm + RoPE + append + attention, o_proj, residual + post-norm + gate/up/SwiGLU,
// down_proj + residual), the final norm with that step's head, the top-k sampler and the gather of the sampled
// code's embedding.  Launched one by one they cost 4.5 to 8 us each whatever their 2 to 12 MB of weights: a launch
// is start + first-byte latency + tail around a microsecond of arithmetic.
//
// The design.  256 blocks, one per CU, stay resident for all steps; block b owns the same rows of every matrix
// in every step.
//   * Weights never wait for activations: a block requests its rows of a matrix straight from memory into LDS
//     (global_load_lds, no registers) as soon as the LDS region of that operator has been consumed for the
//     layer before — one whole layer ahead — so when an operator's input arrives its weights are already there.
//     Regions: Q/K/V 16 rows, o_proj 4 rows (time-shared with the input projection's 4 and the head's 8),
//     gate/up 24 rows, down_proj 4 rows; 123 KiB of the CU's 160.
//   * Activations are handed from all blocks to all blocks without a barrier: every 16-bit value travels in a
//     32-bit word whose upper half is the number of the operator instance that produced it (a counter that runs
//     on from launch to launch in the workspace), written with one agent-scope store.  A consumer requests all
//     its words at once and repeats until every tag is the one it expects: the data is its own flag.  Measured
//     on this chip, 256 blocks: 2.3 to 2.7 us per hand-off of 1 024 to 4 096 words, against 5.4 to 8.3 us for
//     store + arrive-counter (or flag array) + load.
//   * The sampler runs in every block: the step's 2 048 scores reach all blocks as any operator's output does and each
//     block draws from them with its own copy of the generator state — the same code everywhere, so the code needs no
//     hand-off of its own on its way into the next step's projection.  The last block alone records the code, gathers
//     its embedding for the caller and stores the generator state at the end.
//   * Every wait is bounded; a block that gives up raises the abort word, ORs QM_STATUS_FRAME_TIMEOUT into the
//     status word and returns, and so does every block that sees the abort word: the grid always drains.
// Arithmetic.  Every operator keeps the reference's summation order and roundings as the one-operator kernels of
// this library do (qm_linear.hip, qm_predictor.hip, qm_sampler.hip): one reference lane per thread for the
// dot products, the same shuffle trees, the same block sums for the norms — the sampled codes are those of the
// operator-by-operator path bit for bit.
//
// Step 0.  The frame's first step has two rows (the talker's hidden state and the embedding of the talker's code) and
// the reference runs it through its row operators (R17:13663-13699).  Row by row those are the talker-order M = 1
// operators — lane l takes k = l, l + 32, ... — and the causal two-row attention is the M = 1 attention at positions
// 0 and 1: step 0 is one more pass of the same loop with that chain order in which every operator takes the first
// row and then the second (each row with its own copy of the handed-over vectors), so it waits for the hand-offs of
// one row; the head and the sampler follow the second row.
//
// Geometry is the predictor's (R17:7951-7964): hidden 1024, 16 / 8 heads of 128, intermediate 3072, outer
// dimension 2048, vocabulary 2048, five layers, cache of 16 positions.

#include "qm_device.h"
#include "qm_host.h"
#include "qm_norm_rope_head.h"
#include "qm_predictor_chain.h"
#include "qm_sampler_block.h"

namespace qm {
namespace {

constexpr int kFrThreads = 256;
constexpr int kFrBlocks = 256;
constexpr int kFrLayers = 5;
constexpr int kFrHidden = 1024;
constexpr int kFrQDim = 2048;
constexpr int kFrKvDim = 1024;
constexpr int kFrInter = 3072;
constexpr int kFrOuter = 2048;
constexpr int kFrVocab = 2048;
constexpr int kFrCache = 16;
constexpr int kFrFirstStep = 0;
constexpr int kFrLastStep = 14;
constexpr int kFrPositions = 16;                     // passes of a whole frame: positions 0 and 1 are step 0
constexpr int kFrPhasesPerStep = 32;                 // tags reserved per step (28 used)
constexpr unsigned kFrSpinLimit = 1u << 17;          // polls of about a microsecond each (FrParams::spin_limit)

// rows of a matrix in LDS are padded by 64 bytes so that two rows read by one instruction fall on different banks
__host__ __device__ constexpr int fr_row_stride(int reduction) { return 2 * reduction + 64; }
__host__ __device__ constexpr int fr_max(int a, int b) { return a > b ? a : b; }

// rows of each operator per block
constexpr int kFrRowsProj = kFrHidden / kFrBlocks;               // 4 of 1024, reduction 2048
constexpr int kFrRowsQkv = (kFrQDim + 2 * kFrKvDim) / kFrBlocks; // 16 of 4096, reduction 1024
constexpr int kFrRowsO = kFrHidden / kFrBlocks;                  // 4, reduction 2048
constexpr int kFrRowsGu = kFrInter / kFrBlocks;                  // 12 channels = 24 rows, reduction 1024
constexpr int kFrRowsDown = kFrHidden / kFrBlocks;               // 4, reduction 3072
constexpr int kFrRowsHead = kFrVocab / kFrBlocks;                // 8, reduction 1024

// LDS map (bytes)
constexpr int kFrLdsScratch = 0;                                  // 16 KiB: an operator's input vector / attention / sampler
constexpr int kFrLdsScratchBytes = 16384;
constexpr int kFrLdsCache = kFrLdsScratch + kFrLdsScratchBytes;   // 8 KiB: K rows, V rows of an attention block's head
constexpr int kFrLdsCacheBytes = 2 * kFrCache * kDim * 2;
constexpr int kFrLdsQkv = kFrLdsCache + kFrLdsCacheBytes;
constexpr int kFrLdsOm = kFrLdsQkv + kFrRowsQkv * fr_row_stride(kFrHidden);
constexpr int kFrLdsOmBytes = fr_max(fr_max(kFrRowsO * fr_row_stride(kFrQDim), kFrRowsProj * fr_row_stride(kFrOuter)),
                                     kFrRowsHead * fr_row_stride(kFrHidden));
constexpr int kFrLdsGu = kFrLdsOm + kFrLdsOmBytes;
constexpr int kFrLdsDown = kFrLdsGu + 2 * kFrRowsGu * fr_row_stride(kFrHidden);
constexpr int kFrLdsBytes = kFrLdsDown + kFrRowsDown * fr_row_stride(kFrInter);
static_assert(kFrLdsBytes <= 160 * 1024 - 1024, "the frame kernel's LDS map must fit one CU");
static_assert(sizeof(SamplerScratch) <= kFrLdsScratchBytes, "the sampler's scratch lives in the scratch region");
static_assert(kFrInter * 4 <= kFrLdsScratchBytes, "the longest input vector as fp32");

// workspace map (32-bit words)
constexpr int kFrWsBase = 0;          // number of the next launch's first operator instance
constexpr int kFrWsAbort = 1;
constexpr int kFrWsLastDual = 2;      // first tag of the last pass that wrote the second row's vectors (step 0)
constexpr int kFrWsHidden = 64;
constexpr int kFrWsQkv = kFrWsHidden + kFrHidden;
constexpr int kFrWsCtx = kFrWsQkv + kFrQDim + 2 * kFrKvDim;
constexpr int kFrWsAttn = kFrWsCtx + kFrQDim;
constexpr int kFrWsAct = kFrWsAttn + kFrHidden;
constexpr int kFrWsLogits = kFrWsAct + kFrInter;
constexpr int kFrWsCode = kFrWsLogits + kFrVocab;        // 16 spare words
// step 0's second row: a second copy of the vectors from kFrWsHidden up to kFrWsLogits, kFrWsRowShift words further on
constexpr int kFrWsRowShift = kFrWsCode + 16 - kFrWsHidden;
constexpr int kFrWsWords = kFrWsHidden + kFrWsRowShift + (kFrWsLogits - kFrWsHidden);
constexpr int64_t kFrWsBytes = (static_cast<int64_t>(kFrWsWords) * 4 + 255) / 256 * 256;

struct FrLayer {
    const uint16_t* input_norm;
    const uint16_t* q_weight;
    const uint16_t* k_weight;
    const uint16_t* v_weight;
    const uint16_t* q_norm;
    const uint16_t* k_norm;
    const uint16_t* o_weight;
    const uint16_t* post_norm;
    const uint16_t* gate_weight;
    const uint16_t* up_weight;
    const uint16_t* down_weight;
    uint16_t* key_cache;
    uint16_t* value_cache;
};

struct FrParams {
    FrLayer layers[kFrLayers];
    const uint16_t* projection_weight;
    const uint16_t* projection_bias;
    const uint16_t* final_norm;
    const uint16_t* heads[kFrLastStep + 1];          // [step]
    const uint16_t* embeddings[kFrLastStep + 1];     // [step]
    const uint16_t* projected[kFrLastStep + 1];      // [step] optional: the projection of every row of embeddings[step]
    const uint16_t* cosine;                          // [16][128]
    const uint16_t* sine;
    const uint16_t* step0_input;                     // [2][2048] (first_step == 0)
    uint16_t* free_input;                            // [2048]
    uint16_t* selected;                              // [16][2048]
    int32_t* codes;                                  // [16]
    unsigned long long* rng_state;
    uint32_t* workspace;
    uint32_t* status;
    float epsilon;
    float temperature;
    int top_k;
    int first_step;
    int last_step;
    unsigned spin_limit;
};

struct FrShared {
    float waves[8];
    float total;
    int abort;
    int code;
    float residual[8];              // [row of the pass][the block's four down_proj rows]
};

__device__ __forceinline__ uint32_t agent_load(const uint32_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void agent_store(uint32_t* p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// This thread's words tid, tid + 256, ... of a tagged vector, all requested at once, again and again until
// every one carries `tag`.  False when the wait gave up (or another block did).
template <int N>
__device__ __forceinline__ bool poll_words(const uint32_t* words, uint32_t tag, const uint32_t* abort_word, unsigned spin_limit,
                                           uint32_t (&v)[N]) {
    const int tid = threadIdx.x;
    for (unsigned spins = 0;; ++spins) {
#pragma unroll
        for (int u = 0; u < N; ++u) v[u] = agent_load(words + tid + kFrThreads * u);
        bool fresh = true;
#pragma unroll
        for (int u = 0; u < N; ++u) fresh = fresh && (v[u] >> 16) == tag;
        if (fresh) return true;
        if (spins >= spin_limit) return false;
        if ((spins & 255u) == 255u && agent_load(abort_word) != 0u) return false;
        __builtin_amdgcn_s_sleep(1);
    }
}

// `rows` consecutive rows of a row-major [.][K] matrix, from `src`, into LDS rows dst, dst + step * stride, ...:
// pieces of 1 KiB (one instruction of a wave, 16 bytes per lane), dealt to the four waves in turn.
template <int K>
__device__ __forceinline__ void request_rows(const uint16_t* src, int rows, unsigned char* dst, int step) {
    constexpr int kPieces = 2 * K / 1024;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6);
    const int lane = threadIdx.x & 63;
    const unsigned char* bytes = reinterpret_cast<const unsigned char*>(src);
    for (int q = wave; q < rows * kPieces; q += 4) {
        const int row = q / kPieces, off = (q % kPieces) * 1024;
        __builtin_amdgcn_global_load_lds(bytes + static_cast<int64_t>(row) * (2 * K) + off + lane * 16,
                                         (__attribute__((address_space(3))) void*)(dst + row * step * fr_row_stride(K) + off),
                                         16, 0, 0);
    }
}

// One M = 1 linear operator, this block's R outputs (channels if DUAL).  The weights are in LDS already (requested
// long before); the input vector arrives as tagged words (or plain bf16 for the step's first operator) and
// becomes fp32 in LDS, through the fused prologue if there is one:
//   PRE 1: RMSNorm(input) * norm_w (rmsnorm_kernel, R17:8276-8338);
//   PRE 2: residual = bf16(input + addend), then RMSNorm(residual) * norm_w (R17:16205-16286), the block keeping
//          the residual of its own down_proj rows.
// Then 32 threads per output walk the reference's 32 chains (PAIRS: lane l takes the pairs k = 2l, 2l + 1, then
// + 64, ... as the predictor's kernels do, R17:12110-12120; else k = l, l + 32, ... as the talker's), the
// reference's shuffle tree adds them and lane 0 rounds, adds what the operator adds and stores the tagged word.
template <bool DUAL, int PRE, bool PAIRS, int K, int R>
__device__ __forceinline__ bool linear_phase(FrShared& sh, unsigned char* smem, int lds_weights,
                                             const uint32_t* x_words, uint32_t x_tag, const uint16_t* x_plain,
                                             const uint32_t* add_words, uint32_t add_tag,
                                             const uint16_t* norm_w, float epsilon, const uint16_t* bias, bool add_residual,
                                             int keep_residual_first, int first_out, uint32_t* out_words, uint32_t out_tag,
                                             const uint32_t* abort_word, unsigned spin_limit, int row = 0) {
    constexpr int N = K / kFrThreads;                   // input columns per thread: tid, tid + 256, ...
    constexpr int kStride = fr_row_stride(K);
    float* lin_x = reinterpret_cast<float*>(smem + kFrLdsScratch);
    const int tid = threadIdx.x;

    uint32_t norm_raw[N];
    if (PRE != 0) {
#pragma unroll
        for (int u = 0; u < N; ++u) norm_raw[u] = norm_w[tid + kFrThreads * u];
    }
    uint32_t bias_raw = 0;
    if (bias && (tid & 31) == 0 && (tid >> 5) < R) bias_raw = bias[first_out + (tid >> 5)];

    uint32_t x_raw[N], add_raw[N];
    bool ok = true;
    if (x_plain) {
#pragma unroll
        for (int u = 0; u < N; ++u) x_raw[u] = x_plain[tid + kFrThreads * u];
    } else {
        ok = poll_words<N>(x_words, x_tag, abort_word, spin_limit, x_raw);
    }
    if (PRE == 2) ok = poll_words<N>(add_words, add_tag, abort_word, spin_limit, add_raw) && ok;
    if (!ok) sh.abort = 1;

    if (PRE == 0) {
#pragma unroll
        for (int u = 0; u < N; ++u) lin_x[tid + kFrThreads * u] = bf2f(static_cast<uint16_t>(x_raw[u]));
    } else {
        float local_sum = 0.0f;
#pragma unroll
        for (int u = 0; u < N; ++u) {
            const int k = tid + kFrThreads * u;
            float v = bf2f(static_cast<uint16_t>(x_raw[u]));
            if (PRE == 2) {
                v = bf2f(f2bf(v + bf2f(static_cast<uint16_t>(add_raw[u]))));
                if (k >= keep_residual_first && k < keep_residual_first + 4) sh.residual[4 * row + k - keep_residual_first] = v;
            }
            lin_x[k] = v;
            local_sum = fmaf(v, v, local_sum);
        }
        const float total = block_sum_256_like_reference(local_sum, sh.waves, &sh.total);
        const float inverse_rms = 1.0f / sqrtf(total / static_cast<float>(K) + epsilon);
#pragma unroll
        for (int u = 0; u < N; ++u) {
            const int k = tid + kFrThreads * u;
            lin_x[k] = round_bf16(round_bf16(lin_x[k] * inverse_rms) * bf2f(static_cast<uint16_t>(norm_raw[u])));
        }
    }
    __builtin_amdgcn_s_waitcnt(0);      // this wave's weight pieces have landed
    __syncthreads();
    if (sh.abort) return false;

    const int l = tid & 31;             // reference lane
    // This lane's share of the input vector, read once for all passes; then per output all of its weights are
    // requested from LDS before the chain starts, so that the chain waits for additions, not for reads.
    constexpr int kSteps = PAIRS ? K / 64 : K / 32;
    float2 x_pair[PAIRS ? kSteps : 1];
    float x_one[PAIRS ? 1 : kSteps];
    if (PAIRS) {
        const float2* xp = reinterpret_cast<const float2*>(lin_x) + l;
#pragma unroll
        for (int j = 0; j < kSteps; ++j) x_pair[j] = xp[32 * j];
    } else {
        const float* xs = lin_x + l;
#pragma unroll
        for (int j = 0; j < kSteps; ++j) x_one[j] = xs[32 * j];
    }
#pragma unroll 1
    for (int c0 = 0; c0 < R; c0 += 8) {
        const int c = c0 + (tid >> 5);
        const bool live = c < R;
        const unsigned char* row0 = smem + lds_weights + (live ? (DUAL ? 2 * c : c) : 0) * kStride;
        const unsigned char* row1 = row0 + kStride;                 // DUAL only: the up row
        float acc = 0.0f, up = 0.0f;
        if (PAIRS) {
            const uint32_t* p0 = reinterpret_cast<const uint32_t*>(row0) + l;
            const uint32_t* p1 = reinterpret_cast<const uint32_t*>(row1) + l;
            uint32_t a[kSteps], b[DUAL ? kSteps : 1];
#pragma unroll
            for (int j = 0; j < kSteps; ++j) {
                a[j] = p0[32 * j];
                if (DUAL) b[j] = p1[32 * j];
            }
#pragma unroll
            for (int j = 0; j < kSteps; ++j) {
                acc = fmaf(x_pair[j].x, lo_bf16(a[j]), acc);
                acc = fmaf(x_pair[j].y, hi_bf16(a[j]), acc);
                if (DUAL) {
                    up = fmaf(x_pair[j].x, lo_bf16(b[j]), up);
                    up = fmaf(x_pair[j].y, hi_bf16(b[j]), up);
                }
            }
        } else {
            const uint16_t* w0 = reinterpret_cast<const uint16_t*>(row0) + l;
            const uint16_t* w1 = reinterpret_cast<const uint16_t*>(row1) + l;
            uint32_t a[kSteps], b[DUAL ? kSteps : 1];
#pragma unroll
            for (int j = 0; j < kSteps; ++j) {
                a[j] = w0[32 * j];
                if (DUAL) b[j] = w1[32 * j];
            }
#pragma unroll
            for (int j = 0; j < kSteps; ++j) {
                acc = fmaf(x_one[j], bf2f(static_cast<uint16_t>(a[j])), acc);
                if (DUAL) up = fmaf(x_one[j], bf2f(static_cast<uint16_t>(b[j])), up);
            }
        }
        // the reference's shuffle tree over its 32 lanes; lane 0 holds the sum
        acc = half_wave_tree_sum(acc);
        if (DUAL) up = half_wave_tree_sum(up);
        if (l == 0 && live) {
            uint16_t bits;
            if (DUAL) {
                const float gv = bf2f(f2bf(acc));
                const uint16_t act = f2bf(gv / (1.0f + expf(-gv)));
                bits = f2bf(bf2f(act) * bf2f(f2bf(up)));
            } else {
                float r = acc;
                if (bias) r += bf2f(static_cast<uint16_t>(bias_raw));
                bits = f2bf(r);
                if (add_residual) bits = f2bf(sh.residual[4 * row + c] + bf2f(bits));
            }
            agent_store(out_words + first_out + c, (out_tag << 16) | bits);
        }
    }
    __syncthreads();                    // every read of the weights and of the input vector is done
    return true;
}

// QK-norm + RoPE + cache append + attention of one kv head for one step (R17:12133-12290, 12314-12575): the head's
// K/V rows of this frame live in LDS for the whole launch (and are written to the caller's caches as they come).
__device__ __forceinline__ bool attention_phase(FrShared& sh, unsigned char* smem, const FrParams& prm, const FrLayer& w, int kvh,
                                                int position, const uint32_t* qkv_words, uint32_t in_tag, uint32_t* ctx_words,
                                                uint32_t out_tag, const uint32_t* abort_word, unsigned spin_limit) {
    uint16_t* xq = reinterpret_cast<uint16_t*>(smem + kFrLdsScratch);   // [2][128] the two heads' projections, then rotated
    uint16_t* xk = xq + 2 * kDim;                                       // [128]
    uint16_t* xv = xk + kDim;                                           // [128]
    float* probs = reinterpret_cast<float*>(xv + kDim);                 // [2][16] scores, then probabilities
    uint16_t* kc = reinterpret_cast<uint16_t*>(smem + kFrLdsCache);     // [16][128]
    uint16_t* vc = kc + kFrCache * kDim;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // what the norm needs besides the projections, requested before the wait
    uint16_t g0 = 0, g1 = 0, c0 = 0, c1 = 0, s0 = 0, s1 = 0;
    if (wave < 3) {
        const uint16_t* gamma = wave < 2 ? w.q_norm : w.k_norm;
        g0 = gamma[lane]; g1 = gamma[lane + 64];
        c0 = prm.cosine[position * kDim + lane]; c1 = prm.cosine[position * kDim + lane + 64];
        s0 = prm.sine[position * kDim + lane]; s1 = prm.sine[position * kDim + lane + 64];
    }
    // this thread's two words: one of the head pair's 256 query values, one of the 128 + 128 key / value values
    const uint32_t* first = qkv_words + 2 * kDim * kvh + tid;
    const uint32_t* second = qkv_words + (tid < kDim ? kFrQDim + kDim * kvh + tid : kFrQDim + kFrKvDim + kDim * kvh + (tid - kDim));
    uint32_t a = 0, b = 0;
    bool ok = false;
    for (unsigned spins = 0;; ++spins) {
        a = agent_load(first);
        b = agent_load(second);
        if ((a >> 16) == in_tag && (b >> 16) == in_tag) { ok = true; break; }
        if (spins >= spin_limit) break;
        if ((spins & 255u) == 255u && agent_load(abort_word) != 0u) break;
        __builtin_amdgcn_s_sleep(1);
    }
    if (!ok) sh.abort = 1;
    xq[tid] = static_cast<uint16_t>(a);
    if (tid < kDim) xk[tid] = static_cast<uint16_t>(b); else xv[tid - kDim] = static_cast<uint16_t>(b);
    __syncthreads();
    if (sh.abort) return false;

    // waves 0, 1: the two query heads; wave 2: the key; wave 3 moves the value row
    const int64_t cache_at = (static_cast<int64_t>(kvh) * kFrCache + position) * kDim;
    if (wave < 3) {
        uint16_t* x = wave < 2 ? xq + kDim * wave : xk;
        const HeadPair r = norm_rope_head_values(x[lane], x[lane + 64], true, g0, g1, c0, c1, s0, s1, prm.epsilon);
        if (wave < 2) {
            x[lane] = r.lo; x[lane + 64] = r.hi;
        } else {
            kc[position * kDim + lane] = r.lo; kc[position * kDim + lane + 64] = r.hi;
            w.key_cache[cache_at + lane] = r.lo; w.key_cache[cache_at + lane + 64] = r.hi;
        }
    } else {
        // V is appended as it is (R17:12279-12288)
        const uint16_t v0 = xv[lane], v1 = xv[lane + 64];
        vc[position * kDim + lane] = v0; vc[position * kDim + lane + 64] = v1;
        w.value_cache[cache_at + lane] = v0; w.value_cache[cache_at + lane + 64] = v1;
    }
    __syncthreads();

    // scores: a 32-lane half wave per (head, key); reference lane l accumulates dims l, l + 32, l + 64, l + 96, then the
    // shuffle tree; bf16(sum), bf16(that * scale) (R17:12386-12418)
    {
        const int half = tid >> 5, l = tid & 31, g = half & 1;
        const float scale = __uint_as_float(0x3db504f3U);   // kAttentionScaleBits, R17:9354-9356
        float q4[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) q4[c] = bf2f(xq[kDim * g + l + 32 * c]);
        for (int j = half >> 1; j <= position; j += 4) {
            float acc = 0.0f;
#pragma unroll
            for (int c = 0; c < 4; ++c) acc = fmaf(q4[c], bf2f(kc[j * kDim + l + 32 * c]), acc);
            acc = half_wave_tree_sum(acc);
            if (l == 0) probs[16 * g + j] = rbf(rbf(acc) * scale);
        }
    }
    __syncthreads();
    // softmax: 16 lanes per head; the sum in the shuffle tree's order (R17:12449-12509)
    if (tid < 32) {
        const int t = tid & 15;
        const bool inside = t <= position;
        const float score = inside ? probs[tid] : -INFINITY;
        float maximum = score;
#pragma unroll
        for (int offset = 8; offset > 0; offset >>= 1) maximum = fmaxf(maximum, __shfl_xor(maximum, offset, 16));
        const float e = inside ? expf(score - maximum) : 0.0f;
        float total = e;
#pragma unroll
        for (int offset = 8; offset > 0; offset >>= 1) total += __shfl_xor(total, offset, 16);
        probs[tid] = inside ? rbf(e / total) : 0.0f;
    }
    __syncthreads();
    // P.V: thread (head, d) (R17:12515-12574)
    {
        const int g = tid >> 7, d = tid & 127;
        float vcol[kFrCache];
#pragma unroll
        for (int j = 0; j < kFrCache; ++j) vcol[j] = bf2f(vc[j * kDim + d]);
        const float o = pv_limited(probs + 16 * g, vcol, position + 1);
        const uint16_t bits = __builtin_bit_cast(uint16_t, static_cast<__bf16>(o));
        agent_store(ctx_words + kDim * (2 * kvh + g) + d, (out_tag << 16) | bits);
    }
    __syncthreads();
    return true;
}

__global__ __launch_bounds__(kFrThreads, 1) void predictor_frame_kernel(FrParams prm) {
    request_arguments(prm);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ FrShared sh;
    const int tid = threadIdx.x;
    const int b = blockIdx.x;
    uint32_t* const ws = prm.workspace;
    const uint32_t* const abort_word = ws + kFrWsAbort;
    const uint32_t base = agent_load(ws + kFrWsBase);
    const uint32_t last_dual = agent_load(ws + kFrWsLastDual);
    uint32_t dual_t0 = last_dual;
    if (tid == 0) sh.abort = agent_load(abort_word) != 0u ? 1 : 0;   // a launch gave up and the workspace was not set up again
    __syncthreads();
    if (sh.abort) {
        if (tid == 0 && prm.status) atomicOr(prm.status, QM_STATUS_FRAME_TIMEOUT);
        return;
    }

    // Passes are numbered by the cache position they write: step s >= 1 is position s + 1, step 0 positions 0 and 1.
    const int first = prm.first_step == 0 ? 0 : prm.first_step + 1, last = prm.last_step + 1;
    const unsigned spin_limit = prm.spin_limit;
    // ---- the weights of the first operators -----------------------------------------------------------------------
    const int qkv_row = kFrRowsQkv * b;                   // this block's Q/K/V rows lie in one matrix
    auto qkv_source = [&](const FrLayer& w) {
        return qkv_row < kFrQDim ? w.q_weight + static_cast<int64_t>(qkv_row) * kFrHidden
             : qkv_row < kFrQDim + kFrKvDim ? w.k_weight + static_cast<int64_t>(qkv_row - kFrQDim) * kFrHidden
             : w.v_weight + static_cast<int64_t>(qkv_row - kFrQDim - kFrKvDim) * kFrHidden;
    };
    auto request_qkv = [&](const FrLayer& w) { request_rows<kFrHidden>(qkv_source(w), kFrRowsQkv, smem + kFrLdsQkv, 1); };
    auto request_o = [&](const FrLayer& w) {
        request_rows<kFrQDim>(w.o_weight + static_cast<int64_t>(kFrRowsO) * b * kFrQDim, kFrRowsO, smem + kFrLdsOm, 1);
    };
    auto request_gu = [&](const FrLayer& w) {
        request_rows<kFrHidden>(w.gate_weight + static_cast<int64_t>(kFrRowsGu) * b * kFrHidden, kFrRowsGu, smem + kFrLdsGu, 2);
        request_rows<kFrHidden>(w.up_weight + static_cast<int64_t>(kFrRowsGu) * b * kFrHidden, kFrRowsGu,
                                smem + kFrLdsGu + fr_row_stride(kFrHidden), 2);
    };
    auto request_down = [&](const FrLayer& w) {
        request_rows<kFrInter>(w.down_weight + static_cast<int64_t>(kFrRowsDown) * b * kFrInter, kFrRowsDown, smem + kFrLdsDown, 1);
    };
    auto request_proj = [&]() {
        request_rows<kFrOuter>(prm.projection_weight + static_cast<int64_t>(kFrRowsProj) * b * kFrOuter, kFrRowsProj, smem + kFrLdsOm, 1);
    };
    auto request_head = [&](int step) {
        request_rows<kFrHidden>(prm.heads[step] + static_cast<int64_t>(kFrRowsHead) * b * kFrHidden, kFrRowsHead, smem + kFrLdsOm, 1);
    };
    request_proj();
    request_qkv(prm.layers[0]);
    request_gu(prm.layers[0]);
    request_down(prm.layers[0]);

    // ---- an attention block's head: layer b / 8, kv head b % 8; its rows before the first step come from the caches ----
    const bool attends = b < 8 * kFrLayers;
    const int my_layer = b >> 3, my_head = b & 7;
    if (attends) {
        uint16_t* kc = reinterpret_cast<uint16_t*>(smem + kFrLdsCache);
        const int rows_before = first;                    // cache positions 0 .. first - 1
        for (int c = tid; c < 2 * kFrCache * 16; c += kFrThreads) {
            const int chunk = c & 15, row = (c >> 4) & 15, is_v = c >> 8;
            uint4 value = make_uint4(0, 0, 0, 0);
            if (row < rows_before) {
                const uint16_t* src = is_v ? prm.layers[my_layer].value_cache : prm.layers[my_layer].key_cache;
                value = *reinterpret_cast<const uint4*>(src + (static_cast<int64_t>(my_head) * kFrCache + row) * kDim + chunk * 8);
            }
            *reinterpret_cast<uint4*>(kc + (is_v * kFrCache + row) * kDim + chunk * 8) = value;
        }
    }
    const bool samples = b == kFrBlocks - 1;
    unsigned long long rng = 0;
    if (tid == 0) rng = *prm.rng_state;        // every block keeps the generator's state: all draw, the last one stores it
    __syncthreads();

    uint32_t* const hidden = ws + kFrWsHidden;
    uint32_t* const qkv = ws + kFrWsQkv;
    uint32_t* const ctx = ws + kFrWsCtx;
    uint32_t* const attn = ws + kFrWsAttn;
    uint32_t* const act = ws + kFrWsAct;
    uint32_t* const logits = ws + kFrWsLogits;

#pragma unroll 1
    for (int position = first; position <= last; ++position) {
        // Step 0's two rows go through every operator one after the other, in ONE pass: an operator's weights are in LDS
        // for both, and the second row's inputs arrive with the first's (its own copy of every handed-over vector,
        // kFrWsRowShift words further on), so the pass costs the hand-offs of one row.  It writes cache positions 0 and 1
        // and ends like position 1: with step 0's head and code.
        const int rows = position == 0 ? 2 : 1;
        const int head_position = position + rows - 1;
        const int step = head_position - 1;               // of the head and of the table of the code sampled after this pass
        const bool pairs = position >= 2;                 // the predictor's chain order; step 0 runs the talker's
        uint32_t t0 = base + static_cast<uint32_t>(position - first) * kFrPhasesPerStep;
        if (rows == 2) {
            // The second row's vectors are written by step 0 only: what they hold may be any number of launches old, and
            // tags repeat after 65 536.  If this pass's tags would be those of the pass that wrote them last, it takes
            // the tags of position 1, which a launch with step 0 does not use otherwise.
            if (((t0 ^ last_dual) & 0xffffu) == 0u) t0 += kFrPhasesPerStep;
            dual_t0 = t0;
        }
        auto tag = [&](int phase) { return (t0 + static_cast<uint32_t>(phase)) & 0xffffu; };
        bool alive = true;
        // the pass's input already projected (a table row of the code just sampled): no projection operator
        const uint16_t* const projected_row = position >= 2 && position != first && prm.projected[step - 1]
            ? prm.projected[step - 1] + static_cast<int64_t>(sh.code) * kFrHidden : nullptr;

        // ---- input projection.  The input of the first pass of a launch is given (step 0: the talker's hidden state
        // and the embedding of the talker's code; otherwise the free input); a later one's is the embedding of the code
        // just sampled (every block has drawn it itself, below) ----
#pragma unroll 1
        for (int r = 0; alive && !projected_row && r < rows; ++r) {
            const uint16_t* x_plain = prm.free_input;
            if (position < 2) x_plain = prm.step0_input + (position + r) * kFrOuter;
            else if (position != first) x_plain = prm.embeddings[step - 1] + static_cast<int64_t>(sh.code) * kFrOuter;
            alive = linear_phase<false, 0, false, kFrOuter, kFrRowsProj>(sh, smem, kFrLdsOm, nullptr, 0, x_plain, nullptr, 0, nullptr, 0.0f,
                                                                         prm.projection_bias, false, 0, kFrRowsProj * b,
                                                                         hidden + r * kFrWsRowShift, tag(0), abort_word, spin_limit, r);
        }
        if (!alive) break;
        if (!projected_row) request_o(prm.layers[0]);       // (else requested when the head had been read)
        uint32_t hidden_tag = tag(0);

#pragma unroll 1
        for (int layer = 0; layer < kFrLayers; ++layer) {
            const FrLayer& w = prm.layers[layer];
            const bool more = layer + 1 < kFrLayers || head_position < last;      // is there a next layer to request weights for
            const FrLayer& next = prm.layers[layer + 1 < kFrLayers ? layer + 1 : 0];
            const int p = 1 + 5 * layer;
            const uint16_t* const x_given = layer == 0 ? projected_row : nullptr;   // in place of `hidden` as handed over
#pragma unroll 1
            for (int r = 0; alive && r < rows; ++r) {
                const int shift = r * kFrWsRowShift;
                alive = pairs
                    ? linear_phase<false, 1, true, kFrHidden, kFrRowsQkv>(sh, smem, kFrLdsQkv, hidden + shift, hidden_tag, x_given, nullptr, 0,
                                                                          w.input_norm, prm.epsilon, nullptr, false, 0, qkv_row, qkv + shift,
                                                                          tag(p), abort_word, spin_limit, r)
                    : linear_phase<false, 1, false, kFrHidden, kFrRowsQkv>(sh, smem, kFrLdsQkv, hidden + shift, hidden_tag, nullptr, nullptr, 0,
                                                                           w.input_norm, prm.epsilon, nullptr, false, 0, qkv_row, qkv + shift,
                                                                           tag(p), abort_word, spin_limit, r);
            }
            if (!alive) break;
            if (more) request_qkv(next);
            if (attends && my_layer == layer) {
#pragma unroll 1
                for (int r = 0; alive && r < rows; ++r)
                    alive = attention_phase(sh, smem, prm, w, my_head, position + r, qkv + r * kFrWsRowShift, tag(p), ctx + r * kFrWsRowShift,
                                            tag(p + 1), abort_word, spin_limit);
                if (!alive) break;
            }
#pragma unroll 1
            for (int r = 0; alive && r < rows; ++r) {
                const int shift = r * kFrWsRowShift;
                alive = pairs
                    ? linear_phase<false, 0, true, kFrQDim, kFrRowsO>(sh, smem, kFrLdsOm, ctx + shift, tag(p + 1), nullptr, nullptr, 0, nullptr, 0.0f,
                                                                      nullptr, false, 0, kFrRowsO * b, attn + shift, tag(p + 2), abort_word,
                                                                      spin_limit, r)
                    : linear_phase<false, 0, false, kFrQDim, kFrRowsO>(sh, smem, kFrLdsOm, ctx + shift, tag(p + 1), nullptr, nullptr, 0, nullptr, 0.0f,
                                                                       nullptr, false, 0, kFrRowsO * b, attn + shift, tag(p + 2), abort_word,
                                                                       spin_limit, r);
            }
            if (!alive) break;
            // (the region after the last o_proj holds the pass's head)
            if (layer + 1 < kFrLayers) request_o(next);
            else request_head(step);
#pragma unroll 1
            for (int r = 0; alive && r < rows; ++r) {
                const int shift = r * kFrWsRowShift;
                alive = pairs
                    ? linear_phase<true, 2, true, kFrHidden, kFrRowsGu>(sh, smem, kFrLdsGu, hidden + shift, hidden_tag, x_given, attn + shift,
                                                                        tag(p + 2), w.post_norm, prm.epsilon, nullptr, false, kFrRowsDown * b,
                                                                        kFrRowsGu * b, act + shift, tag(p + 3), abort_word, spin_limit, r)
                    : linear_phase<true, 2, false, kFrHidden, kFrRowsGu>(sh, smem, kFrLdsGu, hidden + shift, hidden_tag, nullptr, attn + shift,
                                                                         tag(p + 2), w.post_norm, prm.epsilon, nullptr, false, kFrRowsDown * b,
                                                                         kFrRowsGu * b, act + shift, tag(p + 3), abort_word, spin_limit, r);
            }
            if (!alive) break;
            if (more) request_gu(next);
#pragma unroll 1
            for (int r = 0; alive && r < rows; ++r) {
                const int shift = r * kFrWsRowShift;
                alive = pairs
                    ? linear_phase<false, 0, true, kFrInter, kFrRowsDown>(sh, smem, kFrLdsDown, act + shift, tag(p + 3), nullptr, nullptr, 0, nullptr,
                                                                          0.0f, nullptr, true, 0, kFrRowsDown * b, hidden + shift, tag(p + 4),
                                                                          abort_word, spin_limit, r)
                    : linear_phase<false, 0, false, kFrInter, kFrRowsDown>(sh, smem, kFrLdsDown, act + shift, tag(p + 3), nullptr, nullptr, 0, nullptr,
                                                                           0.0f, nullptr, true, 0, kFrRowsDown * b, hidden + shift, tag(p + 4),
                                                                           abort_word, spin_limit, r);
            }
            if (!alive) break;
            if (more) request_down(next);
            hidden_tag = tag(p + 4);
        }
        if (!alive) break;
        uint32_t* const last_hidden = hidden + (rows - 1) * kFrWsRowShift;   // step 0's head reads its second row
        position = head_position;

        // ---- final norm + this step's head ----
        if (!linear_phase<false, 1, false, kFrHidden, kFrRowsHead>(sh, smem, kFrLdsOm, last_hidden, hidden_tag, nullptr, nullptr, 0, prm.final_norm,
                                                                   prm.epsilon, nullptr, false, 0, kFrRowsHead * b, logits, tag(26), abort_word, spin_limit))
            break;
        // the region is free again: the next pass's projection, or — if its input comes projected — its first o_proj
        if (position < last) {
            if (prm.projected[step]) request_o(prm.layers[0]);
            else request_proj();
        }

        // ---- the sampler: EVERY block draws the code, from the same scores and the same generator state — the same code
        // everywhere, and one hand-off fewer per step than one block that samples and tells the others; the last block
        // also records the code and gathers its embedding (what the host reads and the next launch starts from) ----
        {
            uint32_t raw[kFrVocab / kFrThreads];
            if (!poll_words<kFrVocab / kFrThreads>(logits, tag(26), abort_word, spin_limit, raw)) sh.abort = 1;
            float score[kSmpPerThread];
#pragma unroll
            for (int j = 0; j < kSmpPerThread; ++j) score[j] = j < kFrVocab / kFrThreads ? bf2f(static_cast<uint16_t>(raw[j])) : 0.0f;
            __syncthreads();
            if (sh.abort) break;
            SamplerParams sp = {};
            sp.vocab = kFrVocab;
            sp.top_k = prm.top_k;
            sp.temperature = prm.temperature;
            const int32_t chosen = sampler_block(sp, *reinterpret_cast<SamplerScratch*>(smem + kFrLdsScratch), score, rng);
            if (tid == 0) {
                sh.code = chosen;
                if (samples) prm.codes[step + 1] = chosen;
            }
            __syncthreads();
            if (samples) {
                const uint4 row = reinterpret_cast<const uint4*>(prm.embeddings[step] + static_cast<int64_t>(sh.code) * kFrOuter)[tid];
                reinterpret_cast<uint4*>(prm.selected + static_cast<int64_t>(step + 1) * kFrOuter)[tid] = row;
                reinterpret_cast<uint4*>(prm.free_input)[tid] = row;
            }
            __syncthreads();
        }
    }

    if (sh.abort) {
        if (tid == 0) {
            agent_store(ws + kFrWsAbort, 1u);
            if (prm.status) atomicOr(prm.status, QM_STATUS_FRAME_TIMEOUT);
        }
        return;
    }
    if (tid == 0) {
        if (samples) *prm.rng_state = rng;
        // (every block has read the base before this one could finish its last operator)
        if (b == 0) {
            agent_store(ws + kFrWsBase, base + static_cast<uint32_t>(kFrPositions) * kFrPhasesPerStep);
            if (dual_t0 != last_dual) agent_store(ws + kFrWsLastDual, dual_t0);
        }
    }
}

// Sets a frame workspace to "nothing produced yet": every tagged word 0, operator numbers from 1 (a kernel, not
// a memset: callers may capture it).
__global__ void predictor_frame_clear_kernel(uint32_t* words, int count) {
    const int i = static_cast<int>(blockIdx.x) * static_cast<int>(blockDim.x) + static_cast<int>(threadIdx.x);
    if (i < count) words[i] = i == kFrWsBase ? 1u : 0u;
}

// Every block must be resident at once, one per CU: QM_OK if `hip_stream` can hold the launch, QM_ERR_NO_DEVICE if
// the device, or the part of it the stream is confined to by a CU mask, is too small.  (The occupancy is asked of the
// runtime once per device, the stream's mask at every call.)
int32_t frame_residency(void* hip_stream) {
    int device = 0;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return hip_code(err);
    if (device < 0 || device >= kMaxDevices) return QM_ERR_NO_DEVICE;
    static std::atomic<bool> lds_raised[kMaxDevices];
    const int32_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(predictor_frame_kernel), kFrLdsBytes, lds_raised);
    if (rc != QM_OK) return rc;
    static std::atomic<int> per_cu_of[kMaxDevices];        // 0: not asked yet; else blocks a CU holds at once (-1: none)
    int per_cu = per_cu_of[device].load(std::memory_order_acquire);
    if (per_cu == 0) {
        err = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, predictor_frame_kernel, kFrThreads, kFrLdsBytes);
        if (err != hipSuccess) return hip_code(err);
        if (per_cu <= 0) per_cu = -1;
        per_cu_of[device].store(per_cu, std::memory_order_release);
    }
    bool fits = false;
    const int32_t rc_fit = resident_blocks_fit(hip_stream, device, per_cu > 0 ? per_cu : 0, kFrBlocks, &fits);
    if (rc_fit != QM_OK) return rc_fit;
    return fits ? QM_OK : QM_ERR_NO_DEVICE;
}

}  // namespace
}  // namespace qm

extern "C" int64_t qm_predictor_frame_workspace_bytes(void) { return qm::kFrWsBytes; }

extern "C" int32_t qm_predictor_frame_fits(void* hip_stream, int32_t* fits) {
    if (!fits) return QM_ERR_NULL;
    const int32_t rc = qm::frame_residency(hip_stream);
    if (rc != QM_OK && rc != QM_ERR_NO_DEVICE) return rc;
    *fits = rc == QM_OK ? 1 : 0;
    return QM_OK;
}

extern "C" int32_t qm_predictor_frame_workspace_init(void* workspace, int64_t workspace_bytes, void* hip_stream) {
    using namespace qm;
    if (!workspace) return QM_ERR_NULL;
    if (workspace_bytes < kFrWsBytes) return QM_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return QM_ERR_GEOMETRY;
    const int count = static_cast<int>(kFrWsBytes / 4);
    hipLaunchKernelGGL(predictor_frame_clear_kernel, dim3((count + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(hip_stream),
                       static_cast<uint32_t*>(workspace), count);
    return launch_status();
}

extern "C" int32_t qm_predictor_frame_steps(const qm_predictor_frame* frame, int32_t first_step, int32_t last_step, int32_t top_k,
                                            float temperature, void* workspace, int64_t workspace_bytes, uint32_t* status_dev,
                                            void* hip_stream) {
    using namespace qm;
    if (!frame || !workspace) return QM_ERR_NULL;
    if (first_step < kFrFirstStep || last_step > kFrLastStep || first_step > last_step) return QM_ERR_ARGUMENT;
    if (top_k > kSmpMaxKeep || (top_k > 0 && !(temperature > 0.0f))) return QM_ERR_ARGUMENT;
    if (workspace_bytes < kFrWsBytes) return QM_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return QM_ERR_GEOMETRY;
    FrParams prm = {};
    uintptr_t align = 0;
    auto take = [&](const void* p) {
        align |= reinterpret_cast<uintptr_t>(p);
        return p != nullptr;
    };
    bool all = true;
    for (int i = 0; i < kFrLayers; ++i) {
        const qm_predictor_frame_layer& src = frame->layers[i];
        FrLayer& dst = prm.layers[i];
        dst.input_norm = src.input_norm; dst.q_weight = src.q_weight; dst.k_weight = src.k_weight; dst.v_weight = src.v_weight;
        dst.q_norm = src.q_norm; dst.k_norm = src.k_norm; dst.o_weight = src.o_weight; dst.post_norm = src.post_norm;
        dst.gate_weight = src.gate_weight; dst.up_weight = src.up_weight; dst.down_weight = src.down_weight;
        dst.key_cache = src.key_cache; dst.value_cache = src.value_cache;
        all = take(src.input_norm) && take(src.q_weight) && take(src.k_weight) && take(src.v_weight) && take(src.q_norm)
           && take(src.k_norm) && take(src.o_weight) && take(src.post_norm) && take(src.gate_weight) && take(src.up_weight)
           && take(src.down_weight) && take(src.key_cache) && take(src.value_cache) && all;
    }
    prm.projection_weight = frame->projection_weight; prm.projection_bias = frame->projection_bias; prm.final_norm = frame->final_norm;
    all = take(frame->projection_weight) && take(frame->final_norm) && take(frame->cosine) && take(frame->sine)
       && take(frame->free_input) && take(frame->selected) && all;
    if (!frame->projection_bias || !frame->codes || !frame->rng_state) all = false;
    for (int step = first_step; step <= last_step; ++step) {
        prm.heads[step] = frame->heads[step];
        prm.embeddings[step] = frame->embeddings[step];
        prm.projected[step] = frame->projected[step];
        all = take(frame->heads[step]) && take(frame->embeddings[step]) && all;
    }
    if (!all) return QM_ERR_NULL;
    if (align & 15) return QM_ERR_GEOMETRY;               // 16-byte pieces of weight rows, cache rows and embedding rows
    prm.cosine = frame->cosine; prm.sine = frame->sine;
    if (first_step == 0 && !frame->step0_input) return QM_ERR_NULL;
    prm.step0_input = frame->step0_input;
    prm.free_input = frame->free_input; prm.selected = frame->selected; prm.codes = frame->codes;
    prm.rng_state = reinterpret_cast<unsigned long long*>(frame->rng_state);
    prm.workspace = static_cast<uint32_t*>(workspace);
    prm.status = status_dev;
    prm.epsilon = frame->epsilon; prm.temperature = temperature; prm.top_k = top_k;
    prm.first_step = first_step; prm.last_step = last_step;
    const int32_t spin_option = option_value(QM_OPT_PREDICTOR_FRAME_SPIN_LIMIT);
    prm.spin_limit = spin_option > 0 ? static_cast<unsigned>(spin_option) : kFrSpinLimit;

    const int32_t rc = qm::frame_residency(hip_stream);
    if (rc != QM_OK) return rc;
    hipLaunchKernelGGL(predictor_frame_kernel, dim3(kFrBlocks), dim3(kFrThreads), kFrLdsBytes, static_cast<hipStream_t>(hip_stream), prm);
    return launch_status();
}
