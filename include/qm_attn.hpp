// qm_attn.hpp — C++ host adapters over the C ABI of qm_attn.h.
//
// These free functions keep the names, argument order and error behaviour of the reference
// engine's private launch wrappers (devices/rx7900xtx-24g/qwen3_tts_1_7b.cpp, "R17"), so that an
// engine written against them needs no other change:
//   - device pointers are raw, bf16 is uint16_t bit patterns, the KV cache is the flat
//     [kv_head][max_cache][128] LayerCache (R17:16371-16390);
//   - every call is asynchronous on the given stream and never synchronises;
//   - failures throw std::runtime_error with a label, like hip_check / PRED_HIP_CHECK
//     (R17:7941-7949, 17603-17605) and the host overflow guards (R17:16844-16847).
// Paged callers use the C ABI (or the *_paged overloads below) directly.
#ifndef QM_ATTN_HPP
#define QM_ATTN_HPP

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>

#include "qm_attn.h"

namespace qm_attn {

inline void check(int32_t code, const char* label) {
    if (code != QM_OK) {
        throw std::runtime_error(std::string(label) + ": " + qm_error_string(code) + " ("
                                 + std::to_string(code) + ")");
    }
}

// View of the reference's LayerCache as a one-page qm_kv_cache.
inline qm_kv_cache flat_cache(std::uint16_t* key_cache, std::uint16_t* value_cache, int kv_heads,
                              int head_dim, int max_cache) {
    qm_kv_cache c;
    c.k_pool = key_cache;
    c.v_pool = value_cache;
    c.stride_page = 0;
    c.stride_head = static_cast<std::int64_t>(max_cache) * head_dim;
    c.stride_token = head_dim;
    c.page_size = max_cache;
    c.n_pages = 1;
    c.kv_heads = kv_heads;
    c.head_dim = head_dim;
    return c;
}

// Native paged layout [page][kv_head][16][128].
inline qm_kv_cache paged_cache(std::uint16_t* k_pool, std::uint16_t* v_pool, int n_pages, int kv_heads) {
    qm_kv_cache c;
    c.k_pool = k_pool;
    c.v_pool = v_pool;
    c.stride_page = static_cast<std::int64_t>(kv_heads) * 16 * 128;
    c.stride_head = 16 * 128;
    c.stride_token = 128;
    c.page_size = 16;
    c.n_pages = n_pages;
    c.kv_heads = kv_heads;
    c.head_dim = 128;
    return c;
}

// ≙ NativeTalkerEngine::launch_qk_norm_rope_cache_m1 (R17:17569-17606) with the argument list of
// talker_qk_norm_rope_cache_fused_kernel (R17:15365-15381); also the predictor's
// qk_norm_rope_cache_m1 (R17:13432-13471) with q_heads 16, kv_heads 8, max_cache 16.
inline void launch_qk_norm_rope_cache_m1(
    const std::uint16_t* q, const std::uint16_t* k, const std::uint16_t* v,
    const std::uint16_t* q_norm_weight, const std::uint16_t* k_norm_weight,
    const std::uint16_t* cosine, const std::uint16_t* sine,
    std::uint16_t* q_rotated, std::uint16_t* key_cache, std::uint16_t* value_cache,
    int q_heads, int kv_heads, int head_dim, int max_cache, int cache_position, float epsilon,
    void* stream) {
    if (cache_position >= max_cache) throw std::runtime_error("Talker decode cache overflow.");
    const qm_kv_cache c = flat_cache(key_cache, value_cache, kv_heads, head_dim, max_cache);
    check(qm_qk_norm_rope_kv_append(q, k, v, q_norm_weight, k_norm_weight, cosine, sine, q_rotated, &c,
                                    nullptr, 1, q_heads, cache_position, epsilon, stream),
          "Qingming QK norm/RoPE/cache launch");
}

// Bytes of split-K workspace launch_attention needs for contexts up to max_cache tokens: query_length 1, and
// query_length > 1 where the call goes to the row-by-row operator (any cache_before, window or group).
inline std::size_t attention_workspace_bytes(int q_heads, int kv_heads, int max_cache, int query_length = 1) {
    return qm_attention_rows_workspace_bytes(query_length, q_heads, kv_heads, max_cache);
}

// ≙ NativeTalkerEngine::launch_attention (R17:17723-17814).  query_length == 1 is decode over
// keys [key_start, cache_before + 1).  query_length > 1 attends the rows that scatter_prefill_cache has
// already placed in the cache: with two query heads per kv head and no sliding window on the matrix cores (a whole
// prompt from an empty cache, as in NativeTalkerEngine::prefill R17:16710-16717, or rows that continue a sequence —
// those also with one or four query heads per kv head); every other case of the reference's generic kernel (a sliding
// window, another group) row by row.
// The reference sizes dynamic LDS from the context; here the caller passes a workspace sized by
// attention_workspace_bytes instead (the matrix-core cases need none).
inline void launch_attention(
    const std::uint16_t* query, std::uint16_t* key_cache, std::uint16_t* value_cache,
    std::uint16_t* context, int query_length, int cache_before,
    int q_heads, int kv_heads, int head_dim, int max_cache, int sliding_window, float scale,
    void* workspace, std::size_t workspace_bytes, void* stream) {
    const qm_kv_cache c = flat_cache(key_cache, value_cache, kv_heads, head_dim, max_cache);
    if (query_length == 1) {
        check(qm_decode_attention(query, &c, nullptr, 1, context, q_heads, cache_before, sliding_window,
                                  scale, workspace, workspace_bytes, stream),
              "Talker GQA M1 attention launch");
        return;
    }
    if (cache_before + query_length > max_cache) throw std::runtime_error("Talker prefill cache overflow.");
    const bool matrix_group = q_heads == kv_heads || q_heads == 2 * kv_heads || q_heads == 4 * kv_heads;
    if (sliding_window <= 0 && matrix_group && (cache_before != 0 || q_heads != 2 * kv_heads)) {
        // (the caller's workspace lets the keys be shared between blocks, if it is large enough for that)
        const std::int64_t split = qm_prefill_chunk_workspace_bytes(1, query_length, cache_before, kv_heads);
        const bool fits = split > 0 && workspace && static_cast<std::int64_t>(workspace_bytes) >= split
                       && (reinterpret_cast<std::uintptr_t>(workspace) & 255) == 0;
        check(qm_prefill_attention_chunk(query, key_cache, value_cache, context, 1, query_length, cache_before, q_heads,
                                         kv_heads, scale, head_dim, static_cast<std::int64_t>(max_cache) * head_dim, 0,
                                         fits ? workspace : nullptr, fits ? split : 0, stream),
              "Talker generic fused attention launch");
        return;
    }
    if (cache_before != 0 || sliding_window > 0 || q_heads != 2 * kv_heads) {
        check(qm_attention_rows(query, &c, nullptr, 1, context, query_length, cache_before, q_heads, sliding_window,
                                scale, workspace, workspace_bytes, nullptr, stream),
              "Talker generic fused attention launch");
        return;
    }
    check(qm_prefill_attention_causal(query, key_cache, value_cache, context, nullptr, nullptr, 0, 1,
                                      query_length, q_heads, kv_heads, scale, head_dim,
                                      static_cast<std::int64_t>(max_cache) * head_dim, 0, nullptr, stream),
          "Talker generic fused attention launch");
}

// launch_attention over this library's paged cache (no counterpart in the reference, whose cache is flat): the same
// choice between the decode kernels, the matrix cores and the row-by-row operator.
inline void launch_attention_paged(
    const std::uint16_t* query, const qm_kv_cache& cache, const std::int32_t* page_table, int max_pages,
    std::uint16_t* context, int query_length, int cache_before,
    int q_heads, int kv_heads, int sliding_window, float scale,
    void* workspace, std::size_t workspace_bytes, std::uint32_t* status_dev, void* stream) {
    if (query_length == 1) {
        check(qm_decode_attention(query, &cache, page_table, max_pages, context, q_heads, cache_before, sliding_window,
                                  scale, workspace, workspace_bytes, stream),
              "Talker GQA M1 attention launch");
        return;
    }
    const bool matrix_group = q_heads == kv_heads || q_heads == 2 * kv_heads || q_heads == 4 * kv_heads;
    if (sliding_window <= 0 && matrix_group && page_table && cache.page_size % 16 == 0) {
        const std::int64_t split = qm_prefill_chunk_workspace_bytes(1, query_length, cache_before, kv_heads);
        const bool fits = split > 0 && workspace && static_cast<std::int64_t>(workspace_bytes) >= split
                       && (reinterpret_cast<std::uintptr_t>(workspace) & 255) == 0;
        check(qm_prefill_attention_chunk_paged(query, &cache, page_table, max_pages, context, 1, query_length, cache_before,
                                               q_heads, kv_heads, scale, fits ? workspace : nullptr, fits ? split : 0,
                                               status_dev, stream),
              "Talker generic fused attention launch");
        return;
    }
    check(qm_attention_rows(query, &cache, page_table, max_pages, context, query_length, cache_before, q_heads,
                            sliding_window, scale, workspace, workspace_bytes, status_dev, stream),
          "Talker generic fused attention launch");
}

// ≙ launch_rope_rows (R17:17608-17644).
inline void launch_rope_rows(const std::uint16_t* input, const std::uint16_t* cosine,
                             const std::uint16_t* sine, std::uint16_t* output, int sequence_length,
                             int heads, int head_dim, void* stream) {
    if (head_dim != 128) throw std::runtime_error("Talker RoPE rows launch: head_dim must be 128");
    check(qm_norm_rope_rows(input, nullptr, cosine, sine, output, sequence_length, heads, 0.0f, stream),
          "Talker RoPE rows launch");
}

// Per-head RMSNorm over rows = S*heads, dim 128 (rmsnorm_kernel R17:8276, called R17:16673-16689)
// fused with launch_rope_rows: one launch instead of two plus a global round trip.
inline void launch_norm_rope_rows(const std::uint16_t* input, const std::uint16_t* norm_weight,
                                  const std::uint16_t* cosine, const std::uint16_t* sine,
                                  std::uint16_t* output, int sequence_length, int heads, float epsilon,
                                  void* stream) {
    check(qm_norm_rope_rows(input, norm_weight, cosine, sine, output, sequence_length, heads, epsilon,
                            stream),
          "Talker norm/RoPE rows launch");
}

// ≙ scatter_prefill_cache (R17:17646-17682).
inline void scatter_prefill_cache(const std::uint16_t* key, const std::uint16_t* value,
                                  std::uint16_t* key_cache, std::uint16_t* value_cache,
                                  int sequence_length, int kv_heads, int head_dim, int max_cache,
                                  void* stream) {
    const qm_kv_cache c = flat_cache(key_cache, value_cache, kv_heads, head_dim, max_cache);
    check(qm_scatter_kv(key, value, &c, nullptr, 1, sequence_length, 0, nullptr, stream),
          "Talker prefill KV scatter launch");
}

// ≙ scatter_decode_cache (R17:17684-17720).
inline void scatter_decode_cache(const std::uint16_t* key, const std::uint16_t* value,
                                 std::uint16_t* key_cache, std::uint16_t* value_cache, int kv_heads,
                                 int head_dim, int max_cache, int cache_position, void* stream) {
    if (cache_position >= max_cache) throw std::runtime_error("Talker decode cache overflow.");
    const qm_kv_cache c = flat_cache(key_cache, value_cache, kv_heads, head_dim, max_cache);
    check(qm_scatter_kv(key, value, &c, nullptr, 1, 1, cache_position, nullptr, stream),
          "Talker decode KV scatter launch");
}

// ≙ PersistentPredictor::attention_m1 (R17:13473-13497): cache [8][16][128], key_length <= 16.
// Served by the exact-chain kernel (bf16(QK), bf16(* scale), full-row softmax, bf16(P), the reference's
// summation order): with at most 16 keys an online-softmax result can differ from the reference chain by a
// bf16 ulp of the output, which is more than the operator's tolerance when outputs exceed 2.
inline void predictor_attention_m1(const std::uint16_t* query_rotated, std::uint16_t* key_cache,
                                   std::uint16_t* value_cache, std::uint16_t* attention_context,
                                   int key_length, void* stream) {
    if (key_length < 1 || key_length > 16) throw std::runtime_error("Predictor attention: key_length out of range");
    // one query row: [16][1][128] (BHSD) and [1][16][128] are the same bytes as [16][128]
    check(qm_predictor_attention_staged(query_rotated, key_cache, value_cache, attention_context, 1, key_length, 0,
                                        stream),
          "Predictor M1 attention launch");
}

// One launch for all frames x layers x steps of the predictor loop (no reference counterpart as a
// single call; replaces the attention-path nodes of capture_step R17:13592-13707).
inline void predictor_attention_loop(
    const std::uint16_t* q, const std::uint16_t* k, const std::uint16_t* v,
    const std::uint16_t* q_norm_weight, const std::uint16_t* k_norm_weight,
    const std::uint16_t* cosine, const std::uint16_t* sine, std::uint16_t* context,
    std::uint16_t* key_cache_out, std::uint16_t* value_cache_out,
    int units, int layers, int rows, int first_rows, float epsilon, void* stream) {
    check(qm_predictor_attention_loop(q, k, v, q_norm_weight, k_norm_weight, cosine, sine, context,
                                      key_cache_out, value_cache_out, units, layers, rows, first_rows,
                                      epsilon, stream),
          "Predictor attention loop launch");
}

// PersistentPredictor::attention (R17:13300-13386): the staged attention of step 0.
inline void predictor_attention(
    const std::uint16_t* query, const std::uint16_t* key_cache, const std::uint16_t* value_cache,
    std::uint16_t* output, int rows, int key_length, bool causal_prefill, void* stream) {
    check(qm_predictor_attention_staged(query, key_cache, value_cache, output, rows, key_length,
                                        causal_prefill ? 1 : 0, stream),
          "Predictor attention launch");
}

// PersistentPredictor::transpose (R17:13222-13236): [rows][heads][128] -> [heads][rows][128].
inline void predictor_transpose(const std::uint16_t* input, std::uint16_t* output, int rows, int heads,
                                void* stream) {
    check(qm_predictor_transpose(input, output, rows, heads, stream), "Predictor transpose launch");
}

// PersistentPredictor::rope (R17:13238-13254): RoPE of a BHSD tensor [heads][rows][128], head h row s
// rotated with table row s; no norm.
inline void predictor_rope(
    const std::uint16_t* input, const std::uint16_t* cosine, const std::uint16_t* sine, std::uint16_t* output,
    int rows, int heads, void* stream) {
    check(qm_predictor_rope_bhsd(input, cosine, sine, output, rows, heads, stream), "Predictor rope launch");
}

// PersistentPredictor::update_cache (R17:13256-13270): BHSD source [8][rows][128] into one
// [8][16][128] cache at positions start..start+rows-1; called once per cache like the reference.
inline void predictor_update_cache(
    const std::uint16_t* source, std::uint16_t* cache, int rows, int start, void* stream) {
    check(qm_predictor_update_cache(source, cache, rows, start, stream), "Predictor update_cache launch");
}

// launch_qk_norm_rope_cache_m1 + launch_attention of one decode step (R17:17181-17195) in one launch.
inline void decode_step_m1(
    const std::uint16_t* q, const std::uint16_t* k, const std::uint16_t* v,
    const std::uint16_t* q_norm_weight, const std::uint16_t* k_norm_weight,
    const std::uint16_t* cosine, const std::uint16_t* sine, std::uint16_t* q_rotated,
    std::uint16_t* key_cache, std::uint16_t* value_cache, std::uint16_t* context,
    int q_heads, int kv_heads, int head_dim, int max_cache, int cache_position, int sliding_window,
    float scale, float epsilon, void* workspace, std::size_t workspace_bytes, void* stream) {
    if (head_dim != 128) throw std::runtime_error("Talker decode step: head_dim must be 128.");
    if (cache_position < 0 || cache_position >= max_cache) throw std::runtime_error("Talker decode cache overflow.");
    const qm_kv_cache cache = flat_cache(key_cache, value_cache, kv_heads, head_dim, max_cache);
    check(qm_decode_step_fused(q, k, v, q_norm_weight, k_norm_weight, cosine, sine, q_rotated, &cache, nullptr, 1,
                               context, q_heads, cache_position, sliding_window, scale, epsilon, workspace,
                               workspace_bytes, nullptr, stream),
          "Talker fused decode step launch");
}

// launch_linear_m1 (R17:17473-17511), same argument order and label.
inline void launch_linear_m1(
    const std::uint16_t* input, const std::uint16_t* weight, const std::uint16_t* bias,
    const std::uint16_t* residual, std::uint16_t* output, int output_columns, int reduction_columns,
    void* stream) {
    check(qm_linear_m1(input, weight, bias, residual, output, output_columns, reduction_columns, stream),
          "Qingming M1 linear launch");
}

// launch_qkv_m1 (R17:17513-17567) with the layer's parameters spelled out.
inline void launch_qkv_m1(
    const std::uint16_t* input,
    const std::uint16_t* q_weight, const std::uint16_t* q_bias,
    const std::uint16_t* k_weight, const std::uint16_t* k_bias,
    const std::uint16_t* v_weight, const std::uint16_t* v_bias,
    std::uint16_t* q, std::uint16_t* k, std::uint16_t* v,
    int hidden, int q_dim, int kv_dim, void* stream) {
    check(qm_qkv_m1(input, q_weight, q_bias, k_weight, k_bias, v_weight, v_bias, q, k, v, hidden, q_dim,
                    kv_dim, stream),
          "Qingming fused QKV launch");
}

// launch_gate_up_swiglu_m1 (R17:17848-17890).
inline void launch_gate_up_swiglu_m1(
    const std::uint16_t* input, const std::uint16_t* gate_weight, const std::uint16_t* up_weight,
    std::uint16_t* output, int hidden, int intermediate, void* stream) {
    check(qm_gate_up_swiglu_m1(input, gate_weight, up_weight, output, hidden, intermediate, stream),
          "Qingming gate/up/SwiGLU launch");
}

// code_predictor::launch_rmsnorm (R17:8908-8929); epsilon is the reference's kRmsEpsilon.
inline void launch_rmsnorm(
    const std::uint16_t* input, const std::uint16_t* weight, std::uint16_t* output, int rows, int dimension,
    void* stream) {
    check(qm_rmsnorm_rows(input, weight, output, rows, dimension, 1.0e-6f, stream), "rmsnorm launch");
}

// launch_add_postnorm_m1 (R17:17817-17846).
inline void launch_add_postnorm_m1(
    const std::uint16_t* hidden, const std::uint16_t* attention, const std::uint16_t* norm_weight,
    std::uint16_t* residual, std::uint16_t* normalized, int dimension, void* stream) {
    check(qm_add_postnorm_m1(hidden, attention, norm_weight, residual, normalized, dimension, 1.0e-6f, stream),
          "Qingming add/postnorm launch");
}

// PersistentPredictor::linear_m1 (R17:13499-13533).
inline void predictor_linear_m1(
    const std::uint16_t* input, const std::uint16_t* weight, const std::uint16_t* residual, std::uint16_t* output,
    int output_columns, int reduction_columns, void* stream) {
    check(qm_predictor_linear_m1(input, weight, residual, output, output_columns, reduction_columns, stream),
          "predictor linear_m1 launch");
}

// PersistentPredictor::qkv_m1 (R17:13389-13430); the geometry the reference bakes in
// (kHidden 1024, kQueryDim 2048, kKvDim 1024, R17:7951-7959) is passed by the caller.
inline void predictor_qkv_m1(
    const std::uint16_t* input, const std::uint16_t* q_weight, const std::uint16_t* k_weight,
    const std::uint16_t* v_weight, std::uint16_t* q_output, std::uint16_t* k_output, std::uint16_t* v_output,
    int hidden, int q_dim, int kv_dim, void* stream) {
    check(qm_predictor_qkv_m1(input, q_weight, k_weight, v_weight, q_output, k_output, v_output, hidden, q_dim,
                              kv_dim, stream),
          "predictor qkv_m1 launch");
}

// PersistentPredictor::gate_up_swiglu_m1 (R17:13558-13589).
inline void predictor_gate_up_swiglu_m1(
    const std::uint16_t* input, const std::uint16_t* gate_weight, const std::uint16_t* up_weight,
    std::uint16_t* output, int hidden, int intermediate, void* stream) {
    check(qm_predictor_gate_up_swiglu_m1(input, gate_weight, up_weight, output, hidden, intermediate, stream),
          "predictor gate_up_swiglu_m1 launch");
}

// PersistentPredictor::add_postnorm_m1 (R17:13535-13556): the talker's arithmetic.
inline void predictor_add_postnorm_m1(
    const std::uint16_t* hidden, const std::uint16_t* attention, const std::uint16_t* norm_weight,
    std::uint16_t* residual, std::uint16_t* normalized, int dimension, void* stream) {
    check(qm_add_postnorm_m1(hidden, attention, norm_weight, residual, normalized, dimension, 1.0e-6f, stream),
          "predictor add_postnorm_m1 launch");
}

// The sampler launches of NativeFinalHead::run_fast_device (R17:14500-14526) and
// PersistentPredictor::capture_step (R17:13814-13843): top-k sampling when `sampling_enabled`
// (the reference's g_sampling_enabled), else the arg-max kernels.
inline void sample_topk_f32(const float* logits, int vocab, int top_k, float temperature,
                            std::uint64_t* rng_state, std::int32_t* output_id, bool sampling_enabled, void* stream) {
    check(qm_sample_topk(logits, 0, 0, vocab, sampling_enabled ? top_k : 0, temperature, rng_state, output_id, stream),
          "GPU sampler launch");
}
inline void sample_topk_bf16(const std::uint16_t* logits, int last_row_offset, int vocab, int top_k, float temperature,
                             std::uint64_t* rng_state, std::int32_t* output_id, bool sampling_enabled, void* stream) {
    check(qm_sample_topk(logits, 1, last_row_offset, vocab, sampling_enabled ? top_k : 0, temperature, rng_state,
                         output_id, stream),
          "GPU sampler launch");
}

// The device side of NativeFinalHead::run_fast_device after the head projection
// (R17:14456-14545; constants R17:13958-13961, 7338-7339): cast, repetition penalty, suppressed
// tokens, sampling or arg-max, history append — one launch.  The caller keeps the 4-byte
// read-back and the stream synchronisation (R17:14548-14562), and throws for a generation
// index beyond its history capacity as the reference does (R17:14433-14440).
inline void final_head_sample(const std::uint16_t* logits, std::int32_t* history, int generation_index,
                              std::uint64_t* rng_state, std::int32_t* code, bool sampling_enabled, void* stream) {
    if (generation_index < 0) throw std::runtime_error("FinalHead generation index exceeds GPU history capacity");
    check(qm_final_head_sample(logits, history, generation_index, 3072, 2150, 1024, 1.05f, sampling_enabled ? 50 : 0,
                               0.9f, rng_state, code, nullptr, stream),
          "FinalHead sample launch");
}

}  // namespace qm_attn

#endif  // QM_ATTN_HPP
