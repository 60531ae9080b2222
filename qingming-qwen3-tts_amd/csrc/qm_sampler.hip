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
// over the key's 44 significant bits (histogram passes of 8 bits, one bin per thread, ended as
// soon as the bin of the keep-th key is wanted whole: two passes for typical scores), the
// `keep` keys at or above it are gathered and ranked by counting.  The exponentials are computed
// by `keep` threads at once; the sums stay one thread's, in the reference's order: the running
// sum of the second loop repeats the partial sums of the first, so one pass gives both.
// One block of 256 threads; vocab <= 4096 (the reference's sort size), top_k <= 256.
//
// The kernel is a chain of short dependent steps, so what costs is latency.  Measured with cycle
// stamps, 2048 bf16 scores, top 50 (21 us at first, 7.5 us now, of which about 5 are the launch):
// a load per element inside the arithmetic waits for each in turn (16 x 1 100 cycles; now all
// requested at once: 1 900); LDS additions to one address take turns (a pass 2 400 cycles;
// with eight counters per bin, prefix sums by DPP instead of shuffles and three barriers: 1 000);
// a counter handed round for the gather (3 000; now a prefix sum over per-thread counts); the
// unrolled pass loop made the compiler compute all passes' digits ahead and spill (40 000).
//
// Scores with NaN have no defined place in the reference's order either; -0.0 is taken as +0.0
// (they compare equal there).

#include "qm_device.h"
#include "qm_host.h"
#include "qm_sampler_block.h"

namespace qm {

__global__ __launch_bounds__(kSmpThreads) void sampler_kernel(SamplerParams prm) {
    request_arguments(prm);
    __shared__ SamplerScratch scratch;
    const int tid = threadIdx.x;
    const int vocab = prm.vocab;
    // ---- everything that comes from global memory is requested first, in one go (a load per element
    // inside the arithmetic would wait for each one in turn): the scores of ids tid, tid + 256, ...
    // (an id beyond the vocabulary reads the last score and is dropped later), the generator's state ----
    float score[kSmpPerThread];
    if (prm.is_bf16) {
        const uint16_t* src = static_cast<const uint16_t*>(prm.logits) + prm.offset;
        uint16_t raw[kSmpPerThread];
#pragma unroll
        for (int j = 0; j < kSmpPerThread; ++j) raw[j] = src[min(tid + kSmpThreads * j, vocab - 1)];
#pragma unroll
        for (int j = 0; j < kSmpPerThread; ++j) score[j] = bf2f(raw[j]);
    } else {
        const float* src = static_cast<const float*>(prm.logits) + prm.offset;
#pragma unroll
        for (int j = 0; j < kSmpPerThread; ++j) score[j] = src[min(tid + kSmpThreads * j, vocab - 1)];
    }
    unsigned long long rng = 0;
    if (tid == 0 && prm.top_k > 0 && !prm.process_only) rng = *prm.rng_state;
    const unsigned long long before = rng;
    const int32_t chosen = sampler_block(prm, scratch, score, rng);
    if (tid != 0 || chosen == -2) return;
    if (rng != before) *prm.rng_state = rng;
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

// prepare_group0_input_kernel (R17:11963-11996): the talker's code of the frame selects a row of the talker's
// codec embedding table: it is the frame's first selected embedding, the second row of the predictor's two-row
// input (the first is the talker's hidden vector) and the frame's first code.  A code outside the table
// stores code 0 and moves nothing, as the reference does.
__global__ void prepare_group0_kernel(const uint16_t* table, int table_rows, const int32_t* code0, int dimension,
                                      uint16_t* free_input, uint16_t* selected, int32_t* codes) {
    const int d = static_cast<int>(blockIdx.x) * static_cast<int>(blockDim.x) + static_cast<int>(threadIdx.x);
    const int token = code0[0];
    if (token < 0 || token >= table_rows) {
        if (d == 0) codes[0] = 0;
        return;
    }
    if (d < dimension) {
        const uint16_t value = table[static_cast<int64_t>(token) * dimension + d];
        selected[d] = value;
        free_input[dimension + d] = value;
    }
    if (d == 0) codes[0] = token;
}

// sum_codec_embeddings_kernel (R17:8877-8906) followed by add (R17:8729-8744) with the context embedding:
// sum = bf16(e_0 + e_1 + ... in fp32, in group order), next = bf16(sum + context).
__global__ void next_talker_input_kernel(const uint16_t* selected, int groups, const uint16_t* context, int dimension,
                                         uint16_t* sum_out, uint16_t* next_out) {
    const int d = static_cast<int>(blockIdx.x) * static_cast<int>(blockDim.x) + static_cast<int>(threadIdx.x);
    if (d >= dimension) return;
    float accumulation = 0.0f;
    for (int group = 0; group < groups; ++group) accumulation += bf2f(selected[static_cast<int64_t>(group) * dimension + d]);
    const uint16_t sum = f2bf(accumulation);
    if (sum_out) sum_out[d] = sum;
    next_out[d] = f2bf(bf2f(sum) + bf2f(context[d]));
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

extern "C" int32_t qm_predictor_prepare_group0(const uint16_t* codec_table, int32_t table_rows, const int32_t* code0,
                                               int32_t dimension, uint16_t* free_input, uint16_t* selected_embeddings,
                                               int32_t* generated_codes, void* hip_stream) {
    if (!codec_table || !code0 || !free_input || !selected_embeddings || !generated_codes) return QM_ERR_NULL;
    if (table_rows <= 0 || dimension <= 0) return QM_ERR_ARGUMENT;
    hipLaunchKernelGGL(qm::prepare_group0_kernel, dim3(static_cast<unsigned>((dimension + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(hip_stream), codec_table, table_rows, code0, dimension, free_input,
                       selected_embeddings, generated_codes);
    return qm::launch_status();
}

extern "C" int32_t qm_predictor_next_talker_input(const uint16_t* selected_embeddings, int32_t groups,
                                                  const uint16_t* context_embedding, int32_t dimension,
                                                  uint16_t* embedding_sum, uint16_t* next_talker_input, void* hip_stream) {
    if (!selected_embeddings || !context_embedding || !next_talker_input) return QM_ERR_NULL;
    if (groups <= 0 || dimension <= 0) return QM_ERR_ARGUMENT;
    hipLaunchKernelGGL(qm::next_talker_input_kernel, dim3(static_cast<unsigned>((dimension + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(hip_stream), selected_embeddings, groups, context_embedding, dimension,
                       embedding_sum, next_talker_input);
    return qm::launch_status();
}
