// qm_sampler.hip — the per-frame tail of generation on the device: final-head score processing
// (repetition penalty, suppressed tokens), the top-k categorical sampler with its SplitMix64
// state, arg-max, and the append to the code history, for gfx950.
//
// Reference: gpu_sample_topk_f32_kernel / gpu_sample_topk_bf16_kernel (R17:7407-7518),
// cast_final_head_logits / repetition_penalty / suppress_tokens / argmax_final_head
// (R17:14025-14143), append_sampled_code_history_kernel (R17:7530-7543) and their sequence in
// NativeFinalHead::run_fast_device (R17:14456-14545).
//
// What fixes the result.  The reference sorts all scores by (score descending, id ascending)
// with a 4 096-wide sorting network in LDS; that order is total (no two entries compare equal),
// so the first `keep` entries of the sorted sequence are a property of the scores, not of the
// sorting algorithm.  Thread 0 then sums exp(score / T - maximum) over them in double, in that
// order, draws one SplitMix64 number and walks the running sum.  Here the first `keep` entries
// are found without sorting the rest: every score becomes a 64-bit key (order-preserving image
// of the float above, inverted id below), the keep-th largest key is found by a radix select
// over the key's 44 significant bits (six histogram passes of 8 bits, one bin per thread), the
// `keep` keys at or above it are gathered and ranked by counting.  The exponentials are computed
// by `keep` threads at once; the sums stay one thread's, in the reference's order: the running
// sum of the second loop repeats the partial sums of the first, so one pass gives both.
// One block of 256 threads; vocab <= 4096 (the reference's sort size), top_k <= 256.
//
// Scores with NaN have no defined place in the reference's order either; -0.0 is taken as +0.0
// (they compare equal there).

#include "qm_device.h"
#include "qm_host.h"

namespace qm {

constexpr int kSmpThreads = 256;
constexpr int kSmpMaxVocab = 4096;                       // kGpuSamplerSortSize, R17:7336
constexpr int kSmpPerThread = kSmpMaxVocab / kSmpThreads;
constexpr int kSmpMaxKeep = 256;

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

__global__ __launch_bounds__(kSmpThreads) void sampler_kernel(SamplerParams prm) {
    __shared__ uint32_t sh_seen[kSmpMaxVocab / 32];      // tokens present in the history
    __shared__ int sh_hist[256];
    __shared__ int sh_wave_total[4];
    __shared__ int sh_digit, sh_remaining, sh_count;
    __shared__ unsigned long long sh_cand[kSmpMaxKeep];
    __shared__ unsigned long long sh_sorted[kSmpMaxKeep];
    __shared__ double sh_exp[kSmpMaxKeep];                // the terms, then their running sums
    __shared__ double sh_target;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int vocab = prm.vocab;

    // ---- which tokens were generated before (R17:14046-14052, as a bitmap) -----------------------------
    if (prm.process) {
        for (int i = tid; i < kSmpMaxVocab / 32; i += kSmpThreads) sh_seen[i] = 0;
        __syncthreads();
        for (int i = tid; i < prm.history_count; i += kSmpThreads) {
            const int token = prm.history[i];
            if (token >= 0 && token < vocab) atomicOr(&sh_seen[token >> 5], 1U << (token & 31));
        }
        __syncthreads();
    }

    // ---- this thread's scores (ids tid, tid + 256, ...) as keys: larger key = earlier in the order -----
    unsigned long long key[kSmpPerThread];
#pragma unroll
    for (int j = 0; j < kSmpPerThread; ++j) {
        const int id = tid + kSmpThreads * j;
        key[j] = 0;                                        // below every real key
        if (id < vocab) {
            float score = prm.is_bf16 ? bf2f(static_cast<const uint16_t*>(prm.logits)[prm.offset + id])
                                      : static_cast<const float*>(prm.logits)[prm.offset + id];
            if (prm.process) {
                if ((sh_seen[id >> 5] >> (id & 31)) & 1U) score = score < 0.0f ? score * prm.penalty : score * prm.reciprocal;
                if (id == prm.eos && prm.generation_index < 2) score = -INFINITY;
                if (id >= vocab - prm.suppressed_tail && id != prm.eos) score = -INFINITY;
                if (prm.scores_out) prm.scores_out[id] = score;
            }
            key[j] = (static_cast<unsigned long long>(ordered_bits(score)) << 32) | (0xffffffffU - static_cast<uint32_t>(id));
        }
    }

    if (prm.process_only) return;
    const int keep = prm.top_k <= 0 ? 1 : min(prm.top_k, vocab);

    // ---- radix select of the keep-th largest key: digits of 8 bits, most significant first -------------
    // The significant bits are the 32 of the score and the low 12 of the inverted id (ids < 4096).
    unsigned long long prefix = 0, prefix_mask = 0;
    int remaining = keep;
    const int shifts[6] = {56, 48, 40, 32, 4, 0};
    const int widths[6] = {8, 8, 8, 8, 8, 4};
#pragma unroll
    for (int pass = 0; pass < 6; ++pass) {
        const int shift = shifts[pass];
        const unsigned digit_mask = (1U << widths[pass]) - 1U;
        sh_hist[tid] = 0;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < kSmpPerThread; ++j)
            if (key[j] != 0 && (key[j] & prefix_mask) == prefix)
                atomicAdd(&sh_hist[static_cast<unsigned>(key[j] >> shift) & digit_mask], 1);
        __syncthreads();
        // keys in bins above this thread's bin: suffix sum inside the wave, then the waves above
        const int own = sh_hist[tid];
        int sum = own;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int other = __shfl_down(sum, d, 64);
            if (lane + d < 64) sum += other;
        }
        if (lane == 0) sh_wave_total[wave] = sum;
        __syncthreads();
        int above = sum - own;
        for (int w = wave + 1; w < 4; ++w) above += sh_wave_total[w];
        if (above < remaining && remaining <= above + own) {       // exactly one bin
            sh_digit = tid;
            sh_remaining = remaining - above;
        }
        __syncthreads();
        prefix |= static_cast<unsigned long long>(sh_digit) << shift;
        prefix_mask |= static_cast<unsigned long long>(digit_mask) << shift;
        remaining = sh_remaining;
        __syncthreads();
    }
    // prefix now holds every significant bit of the keep-th largest key; the other bits of a key
    // (bits 12..31 of the inverted id) are all ones
    const unsigned long long threshold = prefix | 0x00000000fffff000ULL;

    // ---- gather the keep keys at or above it, rank them by counting -------------------------------------
    if (tid == 0) sh_count = 0;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kSmpPerThread; ++j)
        if (key[j] >= threshold) sh_cand[atomicAdd(&sh_count, 1)] = key[j];
    __syncthreads();
    if (tid < keep) {
        const unsigned long long mine = sh_cand[tid];
        int rank = 0;
        for (int j = 0; j < keep; ++j) rank += sh_cand[j] > mine ? 1 : 0;
        sh_sorted[rank] = mine;
    }
    __syncthreads();

    // ---- sample (R17:7431-7460) ----------------------------------------------------------------------------
    const double inv_t = 1.0 / static_cast<double>(prm.temperature);
    if (prm.top_k > 0 && tid < keep) {
        const double maximum = static_cast<double>(from_ordered_bits(static_cast<uint32_t>(sh_sorted[0] >> 32))) * inv_t;
        const double value = static_cast<double>(from_ordered_bits(static_cast<uint32_t>(sh_sorted[tid] >> 32)));
        sh_exp[tid] = exp(value * inv_t - maximum);
    }
    __syncthreads();
    auto id_of = [&](int i) { return static_cast<int32_t>(0xffffffffU - static_cast<uint32_t>(sh_sorted[i])); };
    // The running sums, added by one thread in the reference's order (its second loop repeats
    // the partial sums of its first: one pass serves both); the terms are fetched eight at a
    // time so that the chain waits for additions, not for LDS.
    if (prm.top_k > 0 && tid == 0) {
        double running = 0.0;
        for (int i0 = 0; i0 < keep; i0 += 8) {
            double term[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) term[u] = i0 + u < keep ? sh_exp[i0 + u] : 0.0;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (i0 + u < keep) {
                    running += term[u];
                    sh_exp[i0 + u] = running;
                }
            }
        }
        const double total = running;
        sh_count = -1;                                     // no draw
        if (total > 0.0) {
            const double uniform = static_cast<double>(splitmix64_next(prm.rng_state) >> 11) * (1.0 / 9007199254740992.0);
            sh_target = uniform * total;
            sh_count = keep - 1;                           // the answer if no running sum exceeds the target
        }
    }
    __syncthreads();
    // first index whose running sum exceeds the target: the smallest such index over all threads
    if (prm.top_k > 0 && sh_count >= 0 && tid < keep && sh_target < sh_exp[tid]) atomicMin(&sh_count, tid);
    __syncthreads();
    if (tid != 0) return;
    int32_t chosen = id_of(0);
    if (prm.top_k > 0 && sh_count >= 0) chosen = id_of(sh_count);
    prm.output_id[0] = chosen;
    if (prm.history && prm.append_index >= 0) prm.history[prm.append_index] = chosen;
}

// gather_predictor_embedding_kernel (R17:11998-12030): the embedding row of the code just sampled
// becomes the next step's input and is kept for the frame's sum.  A code outside the table
// (which the reference would read out of bounds) moves nothing.
__global__ void gather_embedding_kernel(const uint16_t* table, int table_rows, const int32_t* codes, int group,
                                        int dimension, uint16_t* selected, uint16_t* next_input) {
    const int d = static_cast<int>(blockIdx.x) * static_cast<int>(blockDim.x) + static_cast<int>(threadIdx.x);
    if (d >= dimension) return;
    const int token = codes[group];
    if (token < 0 || token >= table_rows) return;
    const uint16_t value = table[static_cast<int64_t>(token) * dimension + d];
    selected[static_cast<int64_t>(group) * dimension + d] = value;
    next_input[d] = value;
}

inline int32_t launch_sampler(const SamplerParams& prm, void* hip_stream) {
    if (prm.vocab <= 0 || prm.offset < 0) return QM_ERR_ARGUMENT;
    if (prm.vocab > kSmpMaxVocab || prm.top_k > kSmpMaxKeep) return QM_ERR_GEOMETRY;
    if (prm.top_k > 0 && !(prm.temperature > 0.0f)) return QM_ERR_ARGUMENT;
    hipLaunchKernelGGL(sampler_kernel, dim3(1), dim3(kSmpThreads), 0, static_cast<hipStream_t>(hip_stream), prm);
    return launch_status();
}

}  // namespace qm

extern "C" int32_t qm_sample_topk(const void* logits, int32_t logits_are_bf16, int32_t offset, int32_t vocab,
                                  int32_t top_k, float temperature, uint64_t* rng_state, int32_t* output_id,
                                  void* hip_stream) {
    using namespace qm;
    if (!logits || !output_id || (top_k > 0 && !rng_state)) return QM_ERR_NULL;
    SamplerParams prm = {};
    prm.logits = logits; prm.is_bf16 = logits_are_bf16 != 0; prm.offset = offset; prm.vocab = vocab;
    prm.top_k = top_k; prm.temperature = temperature;
    prm.rng_state = reinterpret_cast<unsigned long long*>(rng_state);
    prm.output_id = output_id;
    prm.append_index = -1;
    return launch_sampler(prm, hip_stream);
}

extern "C" int32_t qm_final_head_process(const uint16_t* logits, const int32_t* history, int32_t history_count,
                                         int32_t generation_index, int32_t vocab, int32_t eos,
                                         int32_t suppressed_tail, float penalty, float* scores, void* hip_stream) {
    using namespace qm;
    if (!logits || !scores || (history_count > 0 && !history)) return QM_ERR_NULL;
    if (history_count < 0 || suppressed_tail < 0) return QM_ERR_ARGUMENT;
    SamplerParams prm = {};
    prm.logits = logits; prm.is_bf16 = 1; prm.vocab = vocab;
    prm.process = 1; prm.process_only = 1;
    prm.history = const_cast<int32_t*>(history); prm.history_count = history_count; prm.append_index = -1;
    prm.generation_index = generation_index; prm.eos = eos; prm.suppressed_tail = suppressed_tail;
    prm.penalty = penalty; prm.reciprocal = 1.0f / penalty;
    prm.scores_out = scores;
    return launch_sampler(prm, hip_stream);
}

extern "C" int32_t qm_final_head_sample(const uint16_t* logits, int32_t* history, int32_t generation_index,
                                        int32_t vocab, int32_t eos, int32_t suppressed_tail, float penalty,
                                        int32_t top_k, float temperature, uint64_t* rng_state, int32_t* code_out,
                                        float* scores_out, void* hip_stream) {
    using namespace qm;
    if (!logits || !history || !code_out || (top_k > 0 && !rng_state)) return QM_ERR_NULL;
    if (generation_index < 0 || suppressed_tail < 0) return QM_ERR_ARGUMENT;
    SamplerParams prm = {};
    prm.logits = logits; prm.is_bf16 = 1; prm.offset = 0; prm.vocab = vocab;
    prm.top_k = top_k; prm.temperature = temperature;
    prm.rng_state = reinterpret_cast<unsigned long long*>(rng_state);
    prm.output_id = code_out;
    prm.process = 1;
    prm.history = history; prm.history_count = generation_index; prm.append_index = generation_index;
    prm.generation_index = generation_index; prm.eos = eos; prm.suppressed_tail = suppressed_tail;
    prm.penalty = penalty; prm.reciprocal = 1.0f / penalty;
    prm.scores_out = scores_out;
    return launch_sampler(prm, hip_stream);
}

extern "C" int32_t qm_gather_embedding(const uint16_t* table, int32_t table_rows, const int32_t* codes, int32_t group,
                                       int32_t dimension, uint16_t* selected_embeddings, uint16_t* next_step_input,
                                       void* hip_stream) {
    if (!table || !codes || !selected_embeddings || !next_step_input) return QM_ERR_NULL;
    if (table_rows <= 0 || group < 0 || dimension <= 0) return QM_ERR_ARGUMENT;
    hipLaunchKernelGGL(qm::gather_embedding_kernel, dim3(static_cast<unsigned>((dimension + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(hip_stream), table, table_rows, codes, group, dimension,
                       selected_embeddings, next_step_input);
    return qm::launch_status();
}
