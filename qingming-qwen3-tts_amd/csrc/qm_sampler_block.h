// qm_sampler_block.h — the top-k categorical sampler (and arg-max) as the work of one block, shared by the
// sampler's own kernel and the predictor's frame kernel.
//
// Reference: gpu_sample_topk_f32_kernel / gpu_sample_topk_bf16_kernel (R17:7407-7518) and the final-head score
// processing in front of it (R17:14025-14143).
//
// What fixes the result.  The reference sorts all scores by (score descending, id ascending)
// with a 4 096-wide sorting network in LDS; that order is total (no two entries compare equal),
// so the first `keep` entries of the sorted sequence are a property of the scores, not of the
// sorting algorithm.  Thread 0 then sums exp(score / T - maximum) over them in double, in that
// order, draws one SplitMix64 number and walks the running sum.  Here the first `keep` entries
// are found without sorting the rest: every score becomes a 64-bit key (order-preserving image
// of the float above, inverted id below), the keep-th largest key is found by a radix select
// over the key's 44 significant bits (histogram passes of 8 bits, one bin per thread, ended as
// soon as the bin of the keep-th key is wanted whole: two passes for typical scores), the
// `keep` keys at or above it are gathered and ranked by counting.  The exponentials are computed
// by `keep` threads at once; the sums stay one thread's, in the reference's order: the running
// sum of the second loop repeats the partial sums of the first, so one pass gives both.
// One block of 256 threads; vocab <= 4096 (the reference's sort size), top_k <= 256.
#pragma once

#include "qm_device.h"

namespace qm {

constexpr int kSmpThreads = 256;
constexpr int kSmpMaxVocab = 4096;                       // kGpuSamplerSortSize, R17:7336
constexpr int kSmpPerThread = kSmpMaxVocab / kSmpThreads;
constexpr int kSmpMaxKeep = 256;
constexpr int kSmpReplicas = 8;                          // counters per histogram bin (a power of two)

struct SamplerParams {
    const void* logits;          // float or bf16 bits
    int is_bf16;
    int offset;                  // first element (last_row_offset of the bf16 kernel)
    int vocab;
    int top_k;                   // <= 0: arg-max
    float temperature;
    unsigned long long* rng_state;
    int32_t* output_id;
    // final-head processing in front of the selection (process != 0; logits are bf16)
    int process;
    int32_t* history;            // read [0, history_count); the code is appended at [append_index] if >= 0
    int history_count;
    int append_index;
    int generation_index;
    int eos;
    int suppressed_tail;
    float penalty;
    float reciprocal;            // float(1) / float(penalty)
    float* scores_out;           // processed scores, or NULL
    int process_only;            // stop after writing scores_out
};

// Order-preserving image of a float: a > b  <=>  image(a) > image(b)  (-0 counted as +0).
__device__ __forceinline__ uint32_t ordered_bits(float v) {
    const uint32_t bits = __float_as_uint(v + 0.0f);
    return (bits & 0x80000000U) ? ~bits : (bits | 0x80000000U);
}
__device__ __forceinline__ float from_ordered_bits(uint32_t image) {
    return __uint_as_float((image & 0x80000000U) ? (image & 0x7fffffffU) : ~image);
}

__device__ __forceinline__ unsigned long long splitmix64_next(unsigned long long* state) {
    unsigned long long z = *state + 0x9e3779b97f4a7c15ULL;
    *state = z;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
    return z ^ (z >> 31);
}

// Inclusive prefix sum over the 64 lanes of a wave: four DPP row shifts inside the 16-lane rows, then the
// three row totals (no LDS traffic; a shuffle-based scan costs an LDS round trip per step).
__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);   // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);   // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);   // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);   // row_shr:8
    const int t0 = __builtin_amdgcn_readlane(v, 15);
    const int t1 = __builtin_amdgcn_readlane(v, 31);
    const int t2 = __builtin_amdgcn_readlane(v, 47);
    if (lane >= 16) v += t0;
    if (lane >= 32) v += t1;
    if (lane >= 48) v += t2;
    return v;
}

// The block's scratch memory (LDS): 14.6 KiB.
struct SamplerScratch {
    uint32_t seen[kSmpMaxVocab / 32];                    // tokens present in the history
    __attribute__((aligned(16))) int hist[256 * kSmpReplicas];   // [bin][replica]
    int wave_total[4], wave_first[4];
    int digit, remaining, done, count;
    unsigned long long cand[kSmpMaxKeep];
    unsigned long long sorted[kSmpMaxKeep];
    __attribute__((aligned(16))) double exp_terms[kSmpMaxKeep];  // the terms, then their running sums
    double target;
};

// The selection by one block of kSmpThreads threads, all of which call it: score[j] is the score of id
// tid + 256 j (ids beyond the vocabulary are ignored), rng the generator's state (read and advanced by thread 0
// only, when a draw happens).  Returns the chosen id in thread 0 (anything in the others), or -2 in every
// thread when prm.process_only stops after the processed scores.  Nothing is read from prm.logits or
// prm.rng_state and nothing written to prm.output_id / prm.history / prm.rng_state: that is the caller's.
// `sync` is the barrier of the kSmpThreads calling threads (the block's barrier where they are the whole block).
template <class Sync>
__device__ __forceinline__ int32_t sampler_block(const SamplerParams& prm, SamplerScratch& sh, const float (&score)[kSmpPerThread],
                                                 unsigned long long& rng, Sync&& sync) {
    uint32_t* const sh_seen = sh.seen;
    int* const sh_hist = sh.hist;
    int* const sh_wave_total = sh.wave_total;
    int* const sh_wave_first = sh.wave_first;
    int& sh_digit = sh.digit;
    int& sh_remaining = sh.remaining;
    int& sh_done = sh.done;
    int& sh_count = sh.count;
    unsigned long long* const sh_cand = sh.cand;
    unsigned long long* const sh_sorted = sh.sorted;
    double* const sh_exp = sh.exp_terms;
    double& sh_target = sh.target;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int vocab = prm.vocab;
#pragma unroll
    for (int r = 0; r < kSmpReplicas; ++r) sh_hist[tid * kSmpReplicas + r] = 0;   // (a thread only ever reads and clears its own bin)

    // ---- which tokens were generated before (R17:14046-14052, as a bitmap) -----------------------------
    if (prm.process) {
        for (int i = tid; i < kSmpMaxVocab / 32; i += kSmpThreads) sh_seen[i] = 0;
        sync();
        for (int i = tid; i < prm.history_count; i += kSmpThreads) {
            const int token = prm.history[i];
            if (token >= 0 && token < vocab) atomicOr(&sh_seen[token >> 5], 1U << (token & 31));
        }
        sync();
    }

    // ---- the scores as keys: larger key = earlier in the order -------------------------------------------
    unsigned long long key[kSmpPerThread];
#pragma unroll
    for (int j = 0; j < kSmpPerThread; ++j) {
        const int id = tid + kSmpThreads * j;
        key[j] = 0;                                        // below every real key
        if (id < vocab) {
            float value = score[j];
            if (prm.process) {
                if ((sh_seen[id >> 5] >> (id & 31)) & 1U) value = value < 0.0f ? value * prm.penalty : value * prm.reciprocal;
                if (id == prm.eos && prm.generation_index < 2) value = -INFINITY;
                if (id >= vocab - prm.suppressed_tail && id != prm.eos) value = -INFINITY;
                if (prm.scores_out) prm.scores_out[id] = value;
            }
            key[j] = (static_cast<unsigned long long>(ordered_bits(value)) << 32) | (0xffffffffU - static_cast<uint32_t>(id));
        }
    }

    if (prm.process_only) return -2;
    const int keep = prm.top_k <= 0 ? 1 : min(prm.top_k, vocab);

    // ---- radix select of the keep-th largest key: digits of 8 bits, most significant first -------------
    // The significant bits are the 32 of the score and the low 12 of the inverted id (ids < 4096).  A bin of
    // the histogram has kSmpReplicas counters, a lane adds to counter lane % kSmpReplicas: scores share
    // their leading bits, and LDS additions to one address take turns.  The passes end as soon as the bin
    // that holds the keep-th key is wanted whole.
    unsigned long long prefix = 0, prefix_mask = 0;
    int remaining = keep;
    bool whole_bin = false;
    // (kept as a loop: unrolled, the compiler computes the digits of all passes ahead and runs out of registers)
#pragma unroll 1
    for (int pass = 0; pass < 6 && !whole_bin; ++pass) {
        const int shift = pass < 4 ? 56 - 8 * pass : (pass == 4 ? 4 : 0);       // 56, 48, 40, 32, 4, 0
        const int width = pass < 5 ? 8 : 4;
        const unsigned digit_mask = (1U << width) - 1U;
        sync();                                   // the bins are clear (and, later, the last pass's results read)
#pragma unroll
        for (int j = 0; j < kSmpPerThread; ++j)
            if (key[j] != 0 && (key[j] & prefix_mask) == prefix)
                atomicAdd(&sh_hist[(static_cast<unsigned>(key[j] >> shift) & digit_mask) * kSmpReplicas + (lane & (kSmpReplicas - 1))], 1);
        sync();
        // keys in bins above this thread's bin: inside the wave from a prefix sum, then the waves above
        int own = 0;
#pragma unroll
        for (int r = 0; r < kSmpReplicas; ++r) {
            own += sh_hist[tid * kSmpReplicas + r];
            sh_hist[tid * kSmpReplicas + r] = 0;
        }
        const int upto = wave_inclusive_scan(own, lane);
        const int wave_sum = __builtin_amdgcn_readlane(upto, 63);
        if (lane == 0) sh_wave_total[wave] = wave_sum;
        sync();
        int above = wave_sum - upto;
        for (int w = wave + 1; w < 4; ++w) above += sh_wave_total[w];
        if (above < remaining && remaining <= above + own) {       // exactly one bin
            sh_digit = tid;
            sh_remaining = remaining - above;
            sh_done = remaining == above + own ? 1 : 0;
        }
        sync();
        prefix |= static_cast<unsigned long long>(sh_digit) << shift;
        prefix_mask |= static_cast<unsigned long long>(digit_mask) << shift;
        remaining = sh_remaining;
        whole_bin = sh_done != 0;
    }
    // The keep-th largest key starts with the digits in `prefix`; the digits of passes not run are free (zero
    // here), and bits 12..31 of an inverted id, which no pass looks at, are all ones in every key.
    const unsigned long long threshold = prefix | 0x00000000fffff000ULL;

    // ---- gather the keep keys at or above it, rank them by counting -------------------------------------
    // (each thread counts its own, a prefix sum over the block gives it its place: no counter to queue at)
    {
        int mine = 0;
#pragma unroll
        for (int j = 0; j < kSmpPerThread; ++j) mine += (key[j] != 0 && key[j] >= threshold) ? 1 : 0;
        const int upto = wave_inclusive_scan(mine, lane);
        sync();                                   // (the select's last reads of sh_wave_total are done)
        if (lane == 63) sh_wave_total[wave] = upto;
        sync();
        int at = upto - mine;
        for (int w = 0; w < wave; ++w) at += sh_wave_total[w];
#pragma unroll
        for (int j = 0; j < kSmpPerThread; ++j)
            if (key[j] != 0 && key[j] >= threshold) sh_cand[at++] = key[j];
        sync();
    }
    if (tid < keep) {
        const unsigned long long mine = sh_cand[tid];
        int rank = 0;
        for (int j = 0; j < keep; ++j) rank += sh_cand[j] > mine ? 1 : 0;
        sh_sorted[rank] = mine;
    }
    sync();

    // ---- sample (R17:7431-7460) ----------------------------------------------------------------------------
    const double inv_t = 1.0 / static_cast<double>(prm.temperature);
    if (prm.top_k > 0 && tid < keep) {
        const double maximum = static_cast<double>(from_ordered_bits(static_cast<uint32_t>(sh_sorted[0] >> 32))) * inv_t;
        const double value = static_cast<double>(from_ordered_bits(static_cast<uint32_t>(sh_sorted[tid] >> 32)));
        sh_exp[tid] = exp(value * inv_t - maximum);
    } else if (tid < ((keep + 7) & ~7)) {
        sh_exp[tid] = 0.0;                                 // (padding of the last batch of eight below: x + 0 is x)
    }
    sync();
    auto id_of = [&](int i) { return static_cast<int32_t>(0xffffffffU - static_cast<uint32_t>(sh_sorted[i])); };
    // The running sums, added by one thread in the reference's order (its second loop repeats
    // the partial sums of its first: one pass serves both); the terms come eight at a time, the next
    // eight already on their way, so that the chain waits for additions, not for LDS.
    if (prm.top_k > 0 && tid == 0) {
        typedef double f64x2_t __attribute__((ext_vector_type(2)));
        const f64x2_t* terms = reinterpret_cast<const f64x2_t*>(sh_exp);
        f64x2_t* sums = reinterpret_cast<f64x2_t*>(sh_exp);
        double running = 0.0;
        f64x2_t next[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) next[u] = terms[u];
        for (int i0 = 0; i0 < keep; i0 += 8) {
            f64x2_t term[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) term[u] = next[u];
            if (i0 + 8 < keep) {
#pragma unroll
                for (int u = 0; u < 4; ++u) next[u] = terms[(i0 + 8) / 2 + u];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                running += term[u].x;
                term[u].x = running;
                running += term[u].y;
                term[u].y = running;
                sums[i0 / 2 + u] = term[u];
            }
        }
        const double total = running;
        sh_count = -1;                                     // no draw
        if (total > 0.0) {
            const double uniform = static_cast<double>(splitmix64_next(&rng) >> 11) * (1.0 / 9007199254740992.0);
            sh_target = uniform * total;
            sh_count = keep - 1;                           // the answer if no running sum exceeds the target
        }
    }
    sync();
    // first index whose running sum exceeds the target: the lowest such lane of each wave, then the lowest wave
    {
        const bool beyond = prm.top_k > 0 && sh_count >= 0 && tid < keep && sh_target < sh_exp[tid];
        const unsigned long long lanes = __builtin_amdgcn_ballot_w64(beyond);
        if (lane == 0) sh_wave_first[wave] = lanes ? 64 * wave + __builtin_ctzll(lanes) : 0x7fffffff;
    }
    sync();
    int32_t chosen = id_of(0);
    if (tid == 0 && prm.top_k > 0 && sh_count >= 0) {
        const int first = min(min(sh_wave_first[0], sh_wave_first[1]), min(sh_wave_first[2], sh_wave_first[3]));
        chosen = id_of(min(first, sh_count));              // sh_count = keep - 1: the answer if no sum exceeds the target
    }
    return chosen;
}

struct WholeBlockBarrier {
    __device__ __forceinline__ void operator()() const { __syncthreads(); }
};
__device__ __forceinline__ int32_t sampler_block(const SamplerParams& prm, SamplerScratch& sh, const float (&score)[kSmpPerThread],
                                                 unsigned long long& rng) {
    return sampler_block(prm, sh, score, rng, WholeBlockBarrier());
}

}  // namespace qm
