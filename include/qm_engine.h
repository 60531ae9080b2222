/*
 * qm_engine.h — C ABI of the host-side engine shell around the attention / KV-cache path:
 * safetensors reader, talker weights, the decode layer loop, RoPE rows, the trajectory hash.
 *
 * Reference: devices/rx7900xtx-24g/qwen3_tts_1_7b.cpp ("R17") — SafeFile / ModelWeights
 * (R17:3987-4101), TalkerWeights (R17:14710-15021), NativeTalkerEngine::decode_device
 * (R17:17097-17262), make_talker_rope (R17:21576-21590), fnv1a64 (R17:833-842).
 *
 * Every function returns QM_OK (0) or a negative code of qm_attn.h; the text of the last
 * failure of the calling thread is kept in qm_engine_last_error().  Nothing throws across
 * this boundary.  The library is built on libqm_attn.so (the kernels) and the HIP runtime.
 */
#ifndef QM_ENGINE_H
#define QM_ENGINE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QM_ERR_IO     (-7)   /* a file could not be opened, mapped or is malformed */
#define QM_ERR_TENSOR (-8)   /* a tensor is missing, ambiguous, of the wrong dtype or shape */

const char* qm_engine_last_error(void);

/* fnv1a64 (R17:833-842), the engine's trajectory hash: FNV-1a's xor-then-multiply recurrence with
 * the 64-bit FNV prime over `bytes` bytes, from the reference's offset basis 1469598103934665603
 * (the published basis 14695981039346656037 lacks its last digit there; hashes are compared with
 * the reference's, so its constant is kept). */
uint64_t qm_fnv1a64(const void* data, size_t bytes);

/*
 * make_talker_rope (R17:21576-21590): rows [start, start + rows) of the RoPE tables as bf16,
 * inv_i = theta^(-2i/head_dim) and the angle in double, cos/sin cast to float then to bf16,
 * the half table duplicated into both halves.  cos_out, sin_out: [rows][head_dim].
 */
int32_t qm_rope_rows(int32_t rows, int32_t start, int32_t head_dim, double theta,
                     uint16_t* cos_out, uint16_t* sin_out);

/* ---- safetensors (SafeFile, R17:4020-4057) ---------------------------------------- */
typedef struct qm_safefile qm_safefile;
/* Maps the file, parses the JSON header (8-byte little-endian length, then the header) and
 * checks every tensor's byte range against its dtype and shape. */
int32_t qm_safefile_open(const char* path, qm_safefile** out);
void qm_safefile_close(qm_safefile* file);
int32_t qm_safefile_count(const qm_safefile* file);
/* Tensor `index` in name order: name and dtype point into the file object; shape receives up to
 * 8 extents; data points into the mapping. */
int32_t qm_safefile_tensor(const qm_safefile* file, int32_t index, const char** name, const char** dtype,
                           int32_t* rank, int64_t* shape, const void** data, uint64_t* bytes);

/* ---- talker decode engine --------------------------------------------------------- */
typedef struct qm_talker qm_talker;
/*
 * TalkerWeights + the decode side of NativeTalkerEngine: reads every *.safetensors of model_dir
 * (ModelWeights, R17:4059-4099: tensors are found by name suffix, duplicates and ambiguous
 * suffixes are errors), uploads talker.model.layers.N.* for N = 0, 1, ... until a layer is
 * missing and talker.model.norm.weight, checks the geometry the reference checks (hidden 2048,
 * head_dim 128, integral GQA; here q_heads == 2 * kv_heads as the attention kernels require) and
 * allocates the per-layer KV caches [kv_heads][max_cache][128], the activations and the
 * split-K workspace.  All tensors must be BF16.  `hip_stream` is the generation stream every
 * later call enqueues on (NULL: the engine creates a non-blocking one).
 */
int32_t qm_talker_create(const char* model_dir, int32_t max_cache, void* hip_stream, qm_talker** out);
void qm_talker_destroy(qm_talker* engine);
/* layer count, q_heads, kv_heads, q_dim, kv_dim, intermediate, max_cache */
int32_t qm_talker_info(const qm_talker* engine, int32_t info[7]);
/* Zeroes the caches (as the reference does per request, R17:16526-16546) and sets the number of
 * prompt tokens already in them; a prompt's K/V can be placed with qm_talker_cache. */
int32_t qm_talker_reset(qm_talker* engine, int32_t prefill_length);
/* Device pointers of layer `layer`'s key and value cache ([kv_heads][max_cache][128] bf16). */
int32_t qm_talker_cache(qm_talker* engine, int32_t layer, uint16_t** key_cache, uint16_t** value_cache);
/*
 * NativeTalkerEngine::decode_device (R17:17097-17262): one token through every layer —
 * RMSNorm, fused Q/K/V, QK-norm + RoPE + append at cache position prefill_length + decode_index,
 * GQA attention, o_proj, residual + post-norm, gate/up/SwiGLU, down_proj + residual — then the
 * final RMSNorm.  input_device: [2048] bf16 on the device; cosine, sine: [128] bf16 on the
 * HOST (that position's RoPE row, as in the reference); *final_hidden_device receives the
 * engine-owned device vector [2048] that the final head reads.  Enqueues only: no
 * synchronisation, the result is ordered on the engine's stream.  QM_ERR_SLOT_RANGE on cache
 * overflow (the reference throws "Talker device decode cache overflow").
 */
int32_t qm_talker_decode(qm_talker* engine, const uint16_t* input_device, const uint16_t* cosine,
                         const uint16_t* sine, int32_t decode_index, const uint16_t** final_hidden_device);
/*
 * NativeTalkerEngine::prefill (R17:16561-16800): zeroes the caches, then sends the prompt's `rows`
 * token rows through every layer — RMSNorm, q/k/v projections, QK-norm + RoPE, causal attention
 * that also writes K/V to the layer's cache, o_proj + residual, post-norm, gate/up/SwiGLU,
 * down_proj + residual — and applies the final RMSNorm to the last row.  Sets the prompt length
 * that qm_talker_decode continues from.  input_device: [rows][2048] bf16 on the device; cosine,
 * sine: [rows][128] bf16 on the HOST (positions 0 .. rows-1); *final_hidden_device: the last
 * row's final hidden vector (engine-owned, [2048]).  Enqueues only.  rows <= max_cache
 * (QM_ERR_SLOT_RANGE).  Every linear is evaluated in the M = 1 kernels' order, so a token gives
 * the same K/V whether it was part of the prompt or decoded.
 */
int32_t qm_talker_prefill(qm_talker* engine, const uint16_t* input_device, const uint16_t* cosine,
                          const uint16_t* sine, int32_t rows, const uint16_t** final_hidden_device);
/* Waits for the engine's stream. */
int32_t qm_talker_synchronize(qm_talker* engine);

#ifdef __cplusplus
}
#endif
#endif /* QM_ENGINE_H */
