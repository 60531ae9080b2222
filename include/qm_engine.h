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
/* The same with the RoPE row of the step's position on the DEVICE (cosine_device, sine_device [128], valid until the
 * step has run): for a loop that uploaded the rows of all its positions once, as qm_generate does, instead of two
 * small host-to-device copies in front of every step. */
int32_t qm_talker_decode_device_rope(qm_talker* engine, const uint16_t* input_device, const uint16_t* cosine_device,
                                     const uint16_t* sine_device, int32_t decode_index,
                                     const uint16_t** final_hidden_device);
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
/* Waits for the engine's stream, then reads the device status word the attention kernels OR their
 * QM_STATUS_* bits into (page or position out of range, a key-split block that gave up waiting): if any is
 * set the word is cleared, the key-split workspace initialised again and QM_ERR_STATUS returned — what was
 * computed since the last synchronisation is not to be used. */
int32_t qm_talker_synchronize(qm_talker* engine);

/* The engine's generation stream (hipStream_t as void*): the final head and the predictor of a generation
 * loop are created on it. */
void* qm_talker_stream(qm_talker* engine);
/* The device word the talker's kernels OR their QM_STATUS_* bits into (read and cleared by qm_talker_synchronize); the
 * generation loop copies it back with every frame's codes, so that a flagged step ends the generation at once. */
const uint32_t* qm_talker_status_device(qm_talker* engine);

/* ---- final head (NativeFinalHead, R17:14145-14570) ----------------------------------------- */
typedef struct qm_final_head qm_final_head;
/*
 * Uploads talker.codec_head.weight [3072][2048] and allocates the logits, the code history of
 * `history_capacity` frames, the sampled code and the SplitMix64 generator state (set to `seed`; the
 * predictor of the same loop draws from the same state, R17:13899).
 */
int32_t qm_final_head_create(const char* model_dir, int32_t history_capacity, uint64_t seed, void* hip_stream,
                             qm_final_head** out);
void qm_final_head_destroy(qm_final_head* head);
/* A new request: history cleared, generator state set to `seed`. */
int32_t qm_final_head_reset(qm_final_head* head, uint64_t seed);
/*
 * run_fast_device (R17:14427-14570): codec_head on the (already final-normed) hidden vector, then cast,
 * repetition penalty over the history of the frames before `frame`, suppressed tokens, top-50 sampling at
 * temperature 0.9 (arg-max if sampling == 0), history append, and the four-byte read-back with the stream
 * synchronisation that is the loop's frame boundary.  QM_ERR_SLOT_RANGE beyond the history capacity.
 */
int32_t qm_final_head_run(qm_final_head* head, const uint16_t* hidden_device, int32_t frame, int32_t sampling,
                          int32_t* code_out);
uint64_t* qm_final_head_rng_state(qm_final_head* head);            /* device */
const int32_t* qm_final_head_device_code(qm_final_head* head);      /* device: the code of the last run */

/* ---- code predictor frame (PersistentPredictor, R17:12817-13901) ---------------------------- */
typedef struct qm_predictor qm_predictor;
/*
 * PredictorWeights from the model's safetensors (R17:10620-10712): talker.code_predictor.
 * small_to_mtp_projection.{weight,bias}, model.layers.N.*, model.norm.weight, lm_head.I.weight and
 * model.codec_embedding.I.weight for I = 0..14, and the talker's codec embedding table
 * talker.model.codec_embedding.weight; geometry of R17:7951-7964 (hidden 1024, 16/8 heads of 128,
 * intermediate 3072, vocabulary 2048, 15 steps, 16 code groups).  rng_state_device: the generator state
 * the samplers advance (qm_final_head_rng_state of the same loop).
 */
int32_t qm_predictor_create(const char* model_dir, uint64_t* rng_state_device, void* hip_stream, qm_predictor** out);
void qm_predictor_destroy(qm_predictor* predictor);
/*
 * run_frame_device (R17:13043-13156) with the fifteen steps of capture_step (R17:13592-13854) enqueued
 * directly: caches, selected embeddings and codes cleared; input rows = (talker hidden, embedding of
 * code0); step 0 as the reference's two-row staged path, steps 1..14 with the M = 1 operators; then
 * next talker input = bf16(bf16(sum of the 16 selected embeddings) + context).  context_host: [2048] bf16
 * on the host.  Synchronises the stream and returns the frame's sixteen codes (codes_out[0] = code0).
 */
int32_t qm_predictor_run_frame(qm_predictor* predictor, const uint16_t* talker_hidden_device, const int32_t* code0_device,
                               const uint16_t* context_host, int32_t sampling, int32_t codes_out[16]);
const uint16_t* qm_predictor_next_input(qm_predictor* predictor);    /* device [2048] */

/*
 * The generation loop of generate_codec_sequence (R17:21887-22538) on a prompt whose embedding rows are
 * already on the device: talker prefill; per frame the final head (stop on the end-of-sequence code 2150
 * from frame 2 on), the predictor frame conditioned on trailing_text_host[frame] (rows of 2048, first
 * trailing_rows frames) or tts_pad_host, and the talker's decode step on the predictor's next input at
 * RoPE position prompt_rows + frame.  codes_out: [maximum_frames][16]; *frames_out: frames emitted;
 * *hash_out (optional): qm_fnv1a64 of the emitted codes.  The three engines share the talker's stream
 * (QM_ERR_ARGUMENT otherwise); the caller resets the final head between requests.
 */
int32_t qm_generate(qm_talker* talker, qm_final_head* head, qm_predictor* predictor, const uint16_t* prompt_device,
                    int32_t prompt_rows, int32_t maximum_frames, const uint16_t* tts_pad_host,
                    const uint16_t* trailing_text_host, int32_t trailing_rows, int32_t sampling, int32_t* codes_out,
                    int32_t* frames_out, uint64_t* hash_out);

#ifdef __cplusplus
}
#endif
#endif /* QM_ENGINE_H */
