/*
 * qm_attn.h — C ABI of the MI355X (gfx950) attention / KV-cache operators.
 *
 * Every entry point replaces one private launch wrapper of the reference engine
 * (devices/rx7900xtx-24g/qwen3_tts_1_7b.cpp, "R17" below).  Conventions kept from
 * the reference (R17:7968-8020, 17259-17262, 13857-13863):
 *   - the caller owns all device memory; operators never allocate, free or retain;
 *   - every operator is enqueued asynchronously on the caller's HIP stream and
 *     performs no host/device synchronisation, so it can be stream-captured;
 *   - bf16 tensors travel as uint16_t bit patterns.
 * Differences: errors are returned as negative codes instead of C++ exceptions
 * (nothing throws across this ABI; qm_attn.hpp re-throws std::runtime_error to
 * match R17:7941-7949), and the KV cache is addressed through a page descriptor
 * of which the reference's flat [kv_head][max_cache][128] buffer (R17:16371-16390)
 * is the one-page special case.
 *
 * All pointers named `*_dev` / documented "device" must be device-accessible.
 * `hip_stream` is a hipStream_t passed as void* (NULL = the null stream).
 */
#ifndef QM_ATTN_H
#define QM_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- error codes (0 = success) ------------------------------------------- */
#define QM_OK                 0
#define QM_ERR_NULL          -1   /* a required pointer is NULL                      */
#define QM_ERR_GEOMETRY      -2   /* head_dim != 128, q_heads not a supported multiple
                                     of kv_heads, bad strides / page size           */
#define QM_ERR_SLOT_RANGE    -3   /* cache position / context beyond page capacity
                                     (the reference's "cache overflow", R17:16844)  */
#define QM_ERR_WORKSPACE     -4   /* caller workspace missing or too small           */
#define QM_ERR_ARGUMENT      -5   /* negative counts, unsupported option             */
#define QM_ERR_NO_DEVICE     -6   /* no gfx950 device / kernel image unusable        */
#define QM_ERR_STATUS        -9   /* (engine) a kernel OR-ed QM_STATUS_* bits into the status word   */
#define QM_ERR_HIP_BASE   -1000   /* -(1000 + hipError_t) for launch failures        */

/* bits OR-ed by kernels into the optional device status word */
#define QM_STATUS_BAD_PAGE      1u /* page table entry outside [0, n_pages)          */
#define QM_STATUS_BAD_POSITION  2u /* position / length beyond max_pages*page_size   */
#define QM_STATUS_SPLIT_TIMEOUT 4u /* key-split prefill: a partner's record never came  */
#define QM_STATUS_FRAME_TIMEOUT 8u /* predictor frame kernel: an operator's input never came */

/* ---- paged KV cache descriptor -------------------------------------------- */
/*
 * Token t of kv head h of a sequence lives at element offset
 *     page_table[t / page_size] * stride_page + h * stride_head
 *       + (t % page_size) * stride_token + d,        d in [0, head_dim)
 * inside k_pool / v_pool.  The native layout is [page][kv_head][16][128]
 * (stride_page = kv_heads*16*128, stride_head = 16*128, stride_token = 128), so one
 * (page, head) block is 4 KiB contiguous.  The reference's LayerCache
 * [kv_head][max_cache][128] (R17:15505-15522) is page_size = max_cache, n_pages = 1,
 * stride_head = max_cache*128, page_table = NULL.
 * Constraints: head_dim == 128, stride_token == 128, page_size % 16 == 0 unless the
 * sequence has a single page; strides are multiples of 8 elements (16-byte loads).
 */
typedef struct qm_kv_cache {
    uint16_t* k_pool;      /* device */
    uint16_t* v_pool;      /* device */
    int64_t   stride_page; /* elements */
    int64_t   stride_head; /* elements */
    int64_t   stride_token;/* elements, must be head_dim */
    int32_t   page_size;   /* tokens per page */
    int32_t   n_pages;     /* physical pages in the pool */
    int32_t   kv_heads;
    int32_t   head_dim;    /* must be 128 */
} qm_kv_cache;

/* ---- library ----------------------------------------------------------------- */
/* ABI version of this header; bumped on any signature change. */
int32_t qm_abi_version(void);
/* Short static description of an error code. */
const char* qm_error_string(int32_t code);
/* Names the architecture the kernels were compiled for ("gfx950"). */
const char* qm_target_arch(void);
/*
 * Self-test of the library's fp32 -> bf16 rounding (no counterpart in the reference): the kernels round with the
 * hardware's v_cvt_pk_bf16_f32 where the reference's float_to_bf16 (R17:15040-15056) is an integer sequence; this
 * compares the two on the device for the `count` fp32 bit patterns from `first_bits` on and ADDS the number of
 * mismatches to *mismatches_dev (device memory, cleared by the caller).  The tests sweep all 2^32 patterns.
 */
int32_t qm_selftest_bf16_rounding(uint32_t first_bits, uint32_t count, uint64_t* mismatches_dev, void* hip_stream);

/* Tuning options; they have no counterpart in the reference, whose kernels have one fixed behaviour.  A call
 * reads the options when it is enqueued: the calling thread's own value where qm_set_thread_option has set one (two
 * engines driven from two threads can differ), else the process-wide value of qm_set_option.
 *   QM_OPT_PREFILL_SCORE_ROUNDING  1 (default): qm_prefill_attention_causal rounds raw and scaled
 *       scores to bf16 like the reference (R17:15879-15890); 0: scores stay fp32 (faster; needs
 *       scale > 0; outputs stay within the 1e-2 tolerance of the fp32 definition).
 *   QM_OPT_DECODE_TILES_PER_BLOCK  0 (default): the split-K decode picks the 16-token tiles per
 *       block from the problem size; > 0 forces it (changes qm_decode_workspace_bytes too).
 *   QM_OPT_PREFILL_KERNEL  0 (default): qm_prefill_attention_causal runs four waves per block,
 *       each one software pipeline that alternates MFMAs with softmax arithmetic; 1: four uniform
 *       waves per block (the compiler's instruction order; also what a negative scale runs).  Same
 *       bits either way; other values make the call return QM_ERR_ARGUMENT.
 *   QM_OPT_DECODE_STREAMING_LOADS  0 (default): the decode kernels read K and V with the
 *       non-temporal hint when the contexts of one call may exceed 512 MiB (twice the last-level
 *       cache: less than that is partly still cached from the step before), and with plain loads
 *       otherwise; 1: always plain; 2: always
 *       non-temporal.  Same bits either way; other values make the call return QM_ERR_ARGUMENT.
 *   QM_OPT_PREDICTOR_LOOP_KERNEL  0 (default): qm_predictor_attention_loop forms Q.K^T and P.V on the
 *       matrix cores (fp32 accumulation, fp32 softmax, bf16(QK), bf16(*scale) and bf16(P) as the
 *       reference); 1: the reference's exact summation chain on the vector ALU (about 2.5x slower).
 *       The rotated K and the cache write-back are bit-identical in both; contexts agree within the
 *       operator's tolerance.  Other values make the call return QM_ERR_ARGUMENT.
 *   QM_OPT_PREDICTOR_FRAME_OPERATORS  0 (default): the engine's predictor frame (qm_engine.h) runs its M = 1
 *       steps as one launch of qm_predictor_frame_steps; 1: operator by operator.  Same bits either way.
 *   QM_OPT_PREDICTOR_FRAME_SPIN_LIMIT  0 (default): a block of qm_predictor_frame_steps repeats the request for
 *       an operator's input up to 131 072 times before it gives up; > 0: that many times (1 makes nearly every
 *       launch give up at once: for tests of the give-up path, whose every block still returns normally).
 *   QM_OPT_LINEAR_ROWS_KERNEL  0 (default): qm_linear_rows / qm_gate_up_swiglu_rows take the sums of calls with 16 or more
 *       token rows on the matrix cores where the shape fits their tiles (output columns % 128 == 0, reduction % 128 == 0):
 *       same roundings after the sum, results within the operators' tolerance of the exact chain; 1: every call in the
 *       reference's summation order (bit-identical to the M = 1 operators; 20 to 60 times slower on long prompts).
 *   QM_OPT_TALKER_LAYER_OPERATORS  how the engine's talker decode step (qm_engine.h) runs a layer where the checkpoint has
 *       the geometry qm_talker_post_attention_m1 serves.  0 (default): two launches, qm_talker_layer_step_m1 (the attention
 *       without its merge launch, then everything up to the next layer's Q/K/V, which combines the attention's splits
 *       first); 2: three launches (qm_decode_step_fused with its merge, qm_talker_post_attention_m1); 1: operator by
 *       operator.  Same bits every way. */
enum {
    QM_OPT_PREFILL_SCORE_ROUNDING = 0,
    QM_OPT_DECODE_TILES_PER_BLOCK = 1,
    QM_OPT_PREFILL_KERNEL = 2,
    QM_OPT_DECODE_STREAMING_LOADS = 3,
    QM_OPT_PREDICTOR_LOOP_KERNEL = 4,
    QM_OPT_PREDICTOR_FRAME_OPERATORS = 5,
    QM_OPT_PREDICTOR_FRAME_SPIN_LIMIT = 6,
    QM_OPT_LINEAR_ROWS_KERNEL = 7,
    QM_OPT_TALKER_LAYER_OPERATORS = 8,
    QM_OPT_COUNT = 9
};
/* Returns QM_ERR_ARGUMENT for an unknown option or a negative value. */
int32_t qm_set_option(int32_t option, int32_t value);
/* The same for calls enqueued by the calling thread only; value -1 removes the thread's own value. */
int32_t qm_set_thread_option(int32_t option, int32_t value);
/* What a call enqueued by the calling thread would read. */
int32_t qm_get_option(int32_t option, int32_t* value);

/* ---- (1) fused QK-RMSNorm + RoPE + KV append ------------------------------------- */
/*
 * Replaces NativeTalkerEngine::launch_qk_norm_rope_cache_m1 (R17:17569-17606, kernel
 * talker_qk_norm_rope_cache_fused_kernel R17:15365-15526) and its predictor twin
 * qk_norm_rope_cache_m1 (R17:13432-13471, kernel R17:12133-12307).
 * q [q_heads][128], k, v [kv_heads][128], q_norm_w, k_norm_w, cos, sin [128] (device).
 * Writes q_rotated [q_heads][128]; K (normed, rotated) and V (raw copy) into the cache
 * slot of token `cache_position`.  page_table: device int32 [max_pages] or NULL
 * (identity).  Rounding chain: bf16 after normalise, after gamma, after each RoPE
 * product and after their sum — exactly the reference's.
 */
int32_t qm_qk_norm_rope_kv_append(
    const uint16_t* q, const uint16_t* k, const uint16_t* v,
    const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_row, const uint16_t* sin_row,
    uint16_t* q_rotated,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    int32_t q_heads, int32_t cache_position, float epsilon,
    void* hip_stream);

/*
 * Multi-stream form of the same operator (no reference counterpart: the reference
 * serves one sequence; R17:17110-17112 computes the single position on the host).
 * q [n][q_heads][128], k, v [n][kv_heads][128]; positions [n] device int32;
 * page_table [n][max_pages] device int32; cos/sin: row s if rope_by_position == 0,
 * row positions[s] otherwise.  A stream whose position or page is out of range is
 * skipped and the bits above are OR-ed into *status_dev (optional, device uint32).
 */
int32_t qm_qk_norm_rope_kv_append_ragged(
    const uint16_t* q, const uint16_t* k, const uint16_t* v,
    const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_rows, const uint16_t* sin_rows, int32_t rope_by_position,
    uint16_t* q_rotated,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    const int32_t* positions, int32_t n_streams,
    int32_t q_heads, float epsilon, uint32_t* status_dev,
    void* hip_stream);

/* ---- (2) GQA decode attention ------------------------------------------------------ */
/*
 * Bytes of caller workspace the split-K decode needs for up to n_streams sequences of
 * at most max_seq_len tokens.  Pure host arithmetic (capture-safe).
 */
size_t qm_decode_workspace_bytes(int32_t n_streams, int32_t q_heads,
                                 int32_t kv_heads, int32_t max_seq_len);

/*
 * Replaces NativeTalkerEngine::launch_attention with query_length == 1
 * (R17:17723-17779, kernel talker_attention_gqa2_m1_locality_kernel R17:16014-16203)
 * and the predictor's attention_m1 (R17:13473-13497).  query, context_out
 * [q_heads][128]; keys [key_start, cache_before+1) with key_start from
 * sliding_window as in R17:16032-16036 (<= 0 disables the window).
 * Scores are rounded to bf16 before and after scaling like the reference
 * (R17:16102-16116); softmax and P·V stay in fp32 (online softmax, split-K).
 * q_heads: any multiple of the cache's kv_heads (query head h reads kv head h / (q_heads / kv_heads); groups of
 * 1, 2 and 4 heads have kernels of their own, another group runs as several blocks per kv head).
 */
int32_t qm_decode_attention(
    const uint16_t* query,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    uint16_t* context_out,
    int32_t q_heads, int32_t cache_before, int32_t sliding_window, float scale,
    void* workspace, size_t workspace_bytes,
    void* hip_stream);

/*
 * One decode step of a layer's attention in one call: qm_qk_norm_rope_kv_append at `position`
 * followed by qm_decode_attention with cache_before = position, i.e. the reference's
 * launch_qk_norm_rope_cache_m1 + launch_attention pair (R17:17181-17195), with the first folded
 * into the attention launch (each attention block norms and rotates its own query heads; the
 * block that owns the new token's tile appends K and V before it reads the tile).
 * q [q_heads][128], k, v [kv_heads][128] are the raw projections; cos_row, sin_row [128] the RoPE
 * row of `position`; q_rotated_out [q_heads][128] receives the rotated query (may be NULL).
 * Results (context, cache contents, q_rotated) are bit-identical to the two separate calls.
 * Workspace as for qm_decode_attention with max_seq_len = position + 1.
 * q_heads / kv_heads must be 1, 2 or 4 here (QM_ERR_GEOMETRY otherwise); qm_decode_attention,
 * qm_decode_attention_ragged and qm_attention_rows take any integral group.
 */
int32_t qm_decode_step_fused(
    const uint16_t* q, const uint16_t* k, const uint16_t* v,
    const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_row, const uint16_t* sin_row,
    uint16_t* q_rotated_out,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    uint16_t* context_out,
    int32_t q_heads, int32_t position, int32_t sliding_window, float scale, float epsilon,
    void* workspace, size_t workspace_bytes, uint32_t* status_dev,
    void* hip_stream);

/*
 * Ragged multi-stream decode (no reference counterpart; one launch for all streams).
 * query, context_out [n][q_heads][128]; seq_lens [n] device int32 (context length of
 * each stream, 0 = produce zeros); page_table [n][max_pages]; max_seq_len: host upper
 * bound on seq_lens used to size the grid and the workspace.
 */
int32_t qm_decode_attention_ragged(
    const uint16_t* query,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    const int32_t* seq_lens, int32_t n_streams, int32_t max_seq_len,
    uint16_t* context_out,
    int32_t q_heads, float scale,
    void* workspace, size_t workspace_bytes, uint32_t* status_dev,
    void* hip_stream);

/*
 * qm_decode_attention_ragged without a workspace argument and without any allocation.  It has no
 * counterpart in the reference; it is for callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The split records live
 * in a device array of QM_DECODE_STATIC_SCRATCH_BYTES that the library itself holds on every GPU it
 * runs on until the process ends (its address on a device is looked up at the first call on that
 * device).  Same arguments, same kernels and the same bits as qm_decode_attention_ragged.
 * A shape whose qm_decode_workspace_bytes exceeds the array returns QM_ERR_WORKSPACE and does
 * nothing (G = 2: n_streams * kv_heads * min(32, max_seq_len/64 + 1) records of 1040 bytes, e.g.
 * 31 streams of 8 kv heads at any length, 64 streams up to 960 tokens).
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two streams,
 * two host threads) race; calls ordered on one stream are safe.  Nothing in the array needs to
 * start at zero.
 */
#define QM_DECODE_STATIC_SCRATCH_BYTES (8u << 20)
int32_t qm_decode_attention_ragged_static(
    const uint16_t* query,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    const int32_t* seq_lens, int32_t n_streams, int32_t max_seq_len,
    uint16_t* context_out,
    int32_t q_heads, float scale, uint32_t* status_dev,
    void* hip_stream);

/* ---- (3) prefill ---------------------------------------------------------------------- */
/*
 * Per-head RMSNorm (optional) + RoPE over rows.  Replaces rmsnorm_kernel with
 * rows = S*heads, dim 128 (R17:8276-8338, called R17:16673-16689) followed by
 * launch_rope_rows (R17:17608-17644, kernel R17:15531-15625).
 * in/out [rows][heads][128]; cos/sin [rows][128]; norm_w [128] or NULL (RoPE only).
 */
int32_t qm_norm_rope_rows(
    const uint16_t* in, const uint16_t* norm_w,
    const uint16_t* cos_rows, const uint16_t* sin_rows,
    uint16_t* out, int32_t rows, int32_t heads, float epsilon,
    void* hip_stream);
/*
 * The same for the prompt pass's query and key tensors in ONE launch (the two rmsnorm + two launch_rope_rows calls of
 * NativeTalkerEngine::prefill, R17:16673-16712): q_in/q_out [rows][q_heads][128], k_in/k_out [rows][kv_heads][128], one
 * norm weight each (or NULL), the same cos/sin rows.  Bit for bit two qm_norm_rope_rows calls.
 */
int32_t qm_qk_norm_rope_rows(
    const uint16_t* q_in, const uint16_t* k_in, const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_rows, const uint16_t* sin_rows, uint16_t* q_out, uint16_t* k_out,
    int32_t rows, int32_t q_heads, int32_t kv_heads, float epsilon, void* hip_stream);

/*
 * Replaces scatter_prefill_cache (R17:17646-17682, kernel R17:15630-15687) and, with
 * rows == 1, scatter_decode_cache (R17:17684-17720).  key/value [rows][kv_heads][128]
 * are copied to tokens first_position .. first_position+rows-1.  A token whose page table entry is outside
 * [0, n_pages) is skipped and QM_STATUS_BAD_PAGE is OR-ed into *status_dev (optional, device uint32); the
 * reference has one flat cache and no such case.
 */
int32_t qm_scatter_kv(
    const uint16_t* key, const uint16_t* value,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    int32_t rows, int32_t first_position, uint32_t* status_dev,
    void* hip_stream);

/*
 * Causal GQA prefill on bf16 MFMA.  Replaces launch_attention with query_length > 1,
 * cache_before == 0 (R17:17782-17813, kernel talker_attention_kernel R17:15744-16006)
 * fused with scatter_prefill_cache.  query, context_out [batch][seq][q_heads][128];
 * key, value [batch][seq][kv_heads][128] already normed/rotated; row i attends keys
 * 0..i of its own batch entry.  If cache != NULL, K/V are also written to the pages of
 * page_table [batch][max_pages] at tokens 0..seq-1.
 * kv_stride_token / kv_stride_head / kv_stride_batch: element strides of key and value; all
 * zero selects the contiguous [batch][seq][kv_heads][128] layout.  The reference's
 * LayerCache [kv_head][max_cache][128] is read in place with (128, max_cache*128, 0), which
 * is how launch_attention(query_length > 1, cache_before = 0) is served.
 * Only q_heads == 2 * kv_heads is supported by this entry point.
 * Later tokens never contribute to a row, whatever they hold (a non-finite K or V of a later row included: where the
 * causal mask cuts a 16-key group the matrix core would multiply the masked V by P = 0, so such a group is checked for
 * non-finite values and, if it holds any, they are taken out of the matrix product and added for the rows that see
 * them as the reference's fmaf chain adds them, R17:15784-15789, 15947-15990).
 */
int32_t qm_prefill_attention_causal(
    const uint16_t* query, const uint16_t* key, const uint16_t* value,
    uint16_t* context_out,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    int32_t batch, int32_t seq, int32_t q_heads, int32_t kv_heads, float scale,
    int64_t kv_stride_token, int64_t kv_stride_head, int64_t kv_stride_batch,
    uint32_t* status_dev,
    void* hip_stream);

/*
 * The same operator with a workspace that lets up to three blocks share the keys of a long query
 * tile.  No counterpart in the reference (its kernel gives one block a (batch, head, query row)).
 * A call of qm_prefill_attention_causal whose grid leaves compute units idle (one prompt of 1024
 * tokens: 128 blocks) lasts as long as the block of the last query tile, which walks over all
 * keys.  With a workspace the long query tiles are each given to two or three blocks (runs of key
 * tiles), whose partial results are combined by whichever finishes last.  Results stay within the
 * operator's tolerance of the unsplit call but are not bit-identical to it (another association
 * of the sums); they do not depend on the order in which blocks finish.  Rows of query tiles
 * that are not split, and calls that do not split at all, carry the unsplit call's bits.
 *   qm_prefill_split_workspace_bytes: bytes needed for (batch, seq, kv_heads) on the current
 *     device; 0 when the call would not split: fewer than 9 query tiles of 64 rows, or no room
 *     for the added blocks at two blocks per compute unit (a negative value is an error code).
 *   qm_prefill_split_workspace_init: once after allocation (a kernel on hip_stream).  Every launch
 *     tags what it writes with a number of its own, so a call never believes what an earlier call
 *     left behind (also one that ended with QM_STATUS_SPLIT_TIMEOUT) and nothing has to be reset
 *     between calls.  A launch captured in a HIP graph is replayed with the number it was captured
 *     with: after QM_STATUS_SPLIT_TIMEOUT initialise the workspace again before the next replay.
 *     workspace: 256-byte aligned device memory.
 *   qm_prefill_attention_causal_split: workspace NULL or a shape that does not split: exactly
 *     qm_prefill_attention_causal; too small for the shape: QM_ERR_WORKSPACE.  Only the default
 *     kernel (QM_OPT_PREFILL_KERNEL 0) splits.  Two calls that overlap in time must not share
 *     a workspace.  QM_STATUS_SPLIT_TIMEOUT in status_dev: a block gave up waiting for a partner's
 *     record (rows of that query tile are then not written).
 */
int64_t qm_prefill_split_workspace_bytes(int32_t batch, int32_t seq, int32_t kv_heads);
int32_t qm_prefill_split_workspace_init(void* workspace, int64_t workspace_bytes, void* hip_stream);
int32_t qm_prefill_attention_causal_split(
    const uint16_t* query, const uint16_t* key, const uint16_t* value,
    uint16_t* context_out,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    int32_t batch, int32_t seq, int32_t q_heads, int32_t kv_heads, float scale,
    int64_t kv_stride_token, int64_t kv_stride_head, int64_t kv_stride_batch,
    void* workspace, int64_t workspace_bytes,
    uint32_t* status_dev,
    void* hip_stream);

/*
 * The causal GQA prefill on bf16 MFMA for rows that CONTINUE a sequence (a prompt fed in chunks): replaces
 * launch_attention with query_length > 1 and cache_before > 0 (R17:17782-17813, kernel talker_attention_kernel
 * R17:15744-16006; cache_before == 0 is accepted too).  query, context_out [batch][rows][q_heads][128]; row i stands
 * at position cache_before + i and attends keys 0 .. cache_before + i of its batch entry.  key, value hold the
 * cache_before + rows keys of every batch entry — those of the rows themselves included, as after
 * scatter_prefill_cache — addressed by element strides like qm_prefill_attention_causal's: the reference's LayerCache
 * [kv_head][max_cache][128] is read in place with (128, max_cache*128, 0); all zero selects contiguous
 * [batch][cache_before + rows][kv_heads][128].  q_heads / kv_heads = 1, 2 or 4 (the reference's generic kernel serves
 * any integral group, R17:15780-15782: a wave's 32 matrix columns are 32 / group query rows x group heads, so that
 * every K and V fragment serves all heads of the group; other groups: qm_attention_rows); no sliding window
 * (qm_attention_rows).  qm_prefill_attention_chunk_paged below is the same operator over a paged cache.
 * Rounding as qm_prefill_attention_causal (bf16 scores before and after
 * scaling unless QM_OPT_PREFILL_SCORE_ROUNDING is 0, fp32 online softmax, bf16 P; P = hi + lo where a query tile's
 * rows see fewer than 64 keys).  The uniform-waves kernel of qm_prefill_attention_causal with the query rows shifted:
 * for cache_before == 0, group 2 and no workspace it leaves that entry point's bits.
 * workspace (optional, 256-byte aligned; nothing to initialise): a chunk is few rows over many keys, so its grid of
 * batch * kv_heads * ceil(rows / (128 / group)) blocks can leave most compute units idle.  With a workspace of
 * qm_prefill_chunk_workspace_bytes (for the current device; 0 when the shape would not split) the key tiles of a query
 * tile are handed to up to 16 blocks in runs of at least four, whose unnormalised results a second launch combines in
 * run order: results then differ from the unsplit call in the association of the sums only (within the operator's
 * tolerance, not bit-identical) and do not depend on timing.  Too small for the shape: QM_ERR_WORKSPACE.
 */
int64_t qm_prefill_chunk_workspace_bytes(int32_t batch, int32_t rows, int32_t cache_before, int32_t kv_heads);
int32_t qm_prefill_attention_chunk(
    const uint16_t* query, const uint16_t* key, const uint16_t* value,
    uint16_t* context_out,
    int32_t batch, int32_t rows, int32_t cache_before, int32_t q_heads, int32_t kv_heads, float scale,
    int64_t kv_stride_token, int64_t kv_stride_head, int64_t kv_stride_batch,
    void* workspace, int64_t workspace_bytes,
    void* hip_stream);
/*
 * The same operator over a PAGED cache (this library's native layout; the reference's cache is flat, so this has no
 * counterpart there): the cache_before + rows keys of batch entry b — those of the rows themselves included, as after
 * qm_scatter_kv — lie in `cache` at the pages page_table[b][0 ..] names (max_pages entries per batch entry; page_size a
 * multiple of 16).  Same rounding, groups and workspace as qm_prefill_attention_chunk, and the same bits as that entry
 * point gives for the same keys in a flat cache.  status_dev (optional): QM_STATUS_BAD_PAGE for a page-table entry
 * outside the pool (read as page 0: nothing outside the pool is touched; the rows that see it are then wrong).
 * More keys than max_pages pages hold: QM_ERR_SLOT_RANGE.
 */
int32_t qm_prefill_attention_chunk_paged(
    const uint16_t* query, const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    uint16_t* context_out,
    int32_t batch, int32_t rows, int32_t cache_before, int32_t q_heads, int32_t kv_heads, float scale,
    void* workspace, int64_t workspace_bytes, uint32_t* status_dev,
    void* hip_stream);

/*
 * Attention of query_length rows of ONE sequence over its cache, for every shape the two entry points
 * above do not serve: replaces NativeTalkerEngine::launch_attention in its generic branch
 * (R17:17782-17813, kernel talker_attention_kernel R17:15744-16006) for any cache_before >= 0 (a prompt
 * continued in chunks), any sliding window and any integral GQA group q_heads / kv_heads.
 * query, context_out [query_length][q_heads][128]; row i attends keys
 * [key_start_i, cache_before + i + 1), key_start_i = max(0, cache_before + i + 1 - sliding_window) for
 * sliding_window > 0, else 0 (R17:15784-15789); query head h reads kv head h / (q_heads / kv_heads)
 * (R17:15780-15782).  The keys and values of the rows themselves must already be in the cache
 * (qm_scatter_kv at first_position = cache_before, as scatter_prefill_cache precedes the reference's call).
 * page_table [max_pages] of that sequence, or NULL for pages in pool order (the flat LayerCache).
 * Every row runs as one stream of the split-K decode kernels: row i carries the bits
 * qm_decode_attention gives for cache_before + i, and the rounding is that entry point's.  K and V are
 * read once per row (from the caches after the first): where they serve the shape (group 1, 2 or 4, no window)
 * qm_prefill_attention_causal, qm_prefill_attention_chunk and qm_prefill_attention_chunk_paged are faster by an order
 * of magnitude.
 * Workspace: qm_attention_rows_workspace_bytes(query_length, q_heads, kv_heads, cache_before + query_length).
 * query_length <= 65535.  status_dev (optional): QM_STATUS_BAD_PAGE for page-table entries out of range.
 */
size_t qm_attention_rows_workspace_bytes(int32_t query_length, int32_t q_heads, int32_t kv_heads, int32_t key_end);
int32_t qm_attention_rows(
    const uint16_t* query,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    uint16_t* context_out,
    int32_t query_length, int32_t cache_before, int32_t q_heads, int32_t sliding_window, float scale,
    void* workspace, size_t workspace_bytes, uint32_t* status_dev,
    void* hip_stream);

/* ---- (4) code-predictor attention loop ---------------------------------------------------- */
/*
 * One launch for the whole per-frame step loop of the code predictor: replaces, per
 * (frame, layer) unit, steps x { qk_norm_rope_cache_m1 (R17:13432) + attention_m1
 * (R17:13473) } and step 0's rope/update_cache/attention (R17:13238-13386), following
 * the schedule of PersistentPredictor::capture_step (R17:13592-13596).
 * q [units][rows][16][128], k, v [units][rows][8][128] (rows <= 16, row r at position r);
 * q_norm_w, k_norm_w [n_layers][128], unit u uses layer u % n_layers;
 * cos/sin [rows][128]; context_out [units][rows][16][128].
 * first_rows: 1 or 2 — the number of rows the first step carries (2 = the reference's
 * causal two-row step 0); it changes the step numbering only, row r always attends keys
 * 0..r.  k_cache_out / v_cache_out: optional [units][8][16][128] write-back of the
 * per-unit cache (R17:10711-10737 layout), NULL to skip.
 * Every bf16 rounding of the reference chain is kept, bf16(P) included.  With
 * QM_OPT_PREDICTOR_LOOP_KERNEL = 1 the fp32 sums are also taken in the reference's order (results
 * differ from a CPU restatement only where expf rounds differently); the default kernel takes the
 * two products on the matrix cores (max abs error <= 1e-2 against the same restatement).  QK-RMSNorm,
 * RoPE and the cache write-back are bit-exact in both.  The default kernel needs 16-byte aligned
 * norm weights and RoPE rows as well (QM_ERR_GEOMETRY).
 */
int32_t qm_predictor_attention_loop(
    const uint16_t* q, const uint16_t* k, const uint16_t* v,
    const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_rows, const uint16_t* sin_rows,
    uint16_t* context_out, uint16_t* k_cache_out, uint16_t* v_cache_out,
    int32_t units, int32_t n_layers, int32_t rows, int32_t first_rows,
    float epsilon,
    void* hip_stream);

/*
 * The predictor's staged attention of step 0: replaces PersistentPredictor::attention and its
 * six kernels (R17:13300-13386, 9369-9745) — bf16(QK), bf16(*scale), the -inf causal mask
 * (key > row, R17:9517-9520), softmax rows, bf16(P), P.V and the transpose to [rows][16][128] —
 * in one launch with the same rounding chain and summation order.
 * query_bhsd [16][rows][128] (already rotated); key_cache, value_cache [8][16][128];
 * output [rows][16][128]; rows, key_length in 1..16; causal_prefill as in the reference.
 */
int32_t qm_predictor_attention_staged(
    const uint16_t* query_bhsd, const uint16_t* key_cache, const uint16_t* value_cache,
    uint16_t* output, int32_t rows, int32_t key_length, int32_t causal_prefill,
    void* hip_stream);

/*
 * One M = 1 step of a predictor layer between the Q/K/V projection and o_proj in one launch: replaces the pair
 * PersistentPredictor::qk_norm_rope_cache_m1 + attention_m1 (R17:13432-13520, call site R17:13633-13645;
 * kernels R17:12133-12290, 12314-12575) with every rounding and summation order of both.  q [16][128], k, v
 * [8][128]: the projections' outputs; q_norm_w, k_norm_w [128]; cos_row, sin_row [128]: the RoPE row of
 * cache_position.  The new K row (normed, rotated) and V row are written to key_cache / value_cache
 * [8][16][128] at cache_position (0..15; QM_ERR_SLOT_RANGE otherwise) and the rotated query attends the
 * keys 0..cache_position; context_out [16][128].  Same bits as qm_qk_norm_rope_kv_append followed by
 * qm_predictor_attention_staged(rows 1, key_length cache_position + 1).  All tensors 16-byte aligned.
 */
int32_t qm_predictor_step_attention_m1(
    const uint16_t* q, const uint16_t* k, const uint16_t* v,
    const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_row, const uint16_t* sin_row,
    uint16_t* key_cache, uint16_t* value_cache, uint16_t* context_out,
    int32_t cache_position, float epsilon, void* hip_stream);

/*
 * The steps first_step .. last_step (0 .. 14) of one code-predictor frame in ONE launch: replaces the graph of
 * PersistentPredictor::capture_step (R17:13592-13854; 46 nodes per step) for those steps — per step the input
 * projection (small_to_mtp_projection with bias, R17:13600-13612), five layers of RMSNorm + Q/K/V, QK-norm +
 * RoPE + cache append + attention at cache position step + 1, o_proj, residual + post-norm + gate/up/SwiGLU,
 * down_proj + residual (R17:13614-13780), the final norm with that step's head, the top-k sampler (top_k <= 0:
 * arg-max) and the gather of the sampled code's embedding (R17:13782-13854) — with every rounding and summation
 * order of the one-operator entry points of this header, whose results it equals bit for bit.  Step 0 (two rows: the
 * talker's hidden state and the embedding of the talker's code, R17:13663-13699) is run as one pass that takes both
 * rows through every operator, at cache positions 0 and 1, with the chain order of the row operators the reference uses
 * there (qm_linear_rows: every row as qm_linear_m1 evaluates it); head and sampler follow the second row: the caches'
 * rows 0 and 1, codes[1], selected[1]
 * and the next input equal, bit for bit, what the reference's step-0 operators leave (qm_linear_rows, qm_rmsnorm_rows,
 * qm_predictor_transpose / _rope_bhsd / _update_cache, qm_predictor_attention_staged, qm_gate_up_swiglu_rows).
 *
 * qm_predictor_frame names the tensors (bf16, 16-byte aligned; geometry of R17:7951-7964: hidden 1024, 16 / 8
 * heads of 128, intermediate 3072, outer dimension 2048, vocabulary 2048, five layers):
 *   layers[i]: input_norm, post_norm [1024]; q_weight [2048][1024], k_weight, v_weight [1024][1024]; q_norm,
 *     k_norm [128]; o_weight [1024][2048]; gate_weight, up_weight [3072][1024]; down_weight [1024][3072];
 *     key_cache, value_cache [8][16][128] holding the frame's positions 0 .. first_step (none when first_step is 0),
 *     appended to in place;
 *   projection_weight [1024][2048], projection_bias [1024], final_norm [1024]; heads[s] [2048][1024] and
 *   embeddings[s] [2048][2048] for the steps s run (other entries are not read); cosine, sine [16][128];
 *   free_input [2048]: in, the input of first_step >= 1 (the embedding gathered at the end of the step before); out, the
 *     embedding of the last code sampled;  step0_input [2][2048] (read when first_step is 0, else may be NULL): the
 *     talker's hidden state and the embedding of the talker's code;  selected [16][2048]: row s + 1 receives the embedding of step s's code;
 *   codes [16]: codes[s + 1] receives step s's code;  rng_state: the SplitMix64 state the draws advance.
 *
 * The launch is 256 blocks that stay resident and hand each operator's output to one another through
 * `workspace` (qm_predictor_frame_workspace_bytes() bytes, 256-byte aligned, set up once by
 * qm_predictor_frame_workspace_init and then carried from call to call: it numbers the operator instances so
 * that a captured launch can be replayed).  It needs the WHOLE CHIP for its duration: 256 compute units all of
 * which can hold one of its blocks, on a stream that may use them all.  The call returns QM_ERR_NO_DEVICE, before
 * anything is launched, if the device is smaller or if `hip_stream` was created with a CU mask of fewer compute
 * units (hipExtStreamCreateWithCUMask, as the reference's generation stream is, R17:7733-7792):
 * qm_predictor_frame_fits(stream, &fits) asks the same question without launching, and a caller on such a stream
 * takes the operators one by one (same bits).  What the call cannot see are kernels of OTHER streams that occupy
 * compute units while it runs, and another launch of this kind: each would keep out blocks the other waits for,
 * so nothing else may run on the device at the same time.  Every wait is bounded: if an input never comes the
 * blocks OR QM_STATUS_FRAME_TIMEOUT into status_dev (optional) and return; the outputs are then not to be used
 * and the workspace must be initialised again before the next call.
 */
typedef struct qm_predictor_frame_layer {
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
} qm_predictor_frame_layer;

typedef struct qm_predictor_frame {
    qm_predictor_frame_layer layers[5];
    const uint16_t* projection_weight;
    const uint16_t* projection_bias;
    const uint16_t* final_norm;
    const uint16_t* heads[15];        /* [step] */
    const uint16_t* embeddings[15];   /* [step] */
    const uint16_t* cosine;
    const uint16_t* sine;
    uint16_t* free_input;
    uint16_t* selected;
    int32_t* codes;
    uint64_t* rng_state;
    float epsilon;
    const uint16_t* step0_input;      /* [2][2048], first_step == 0 only */
    /* Optional.  projected[s] [2048][1024]: row c = the input projection (with its bias, as qm_linear_m1 evaluates it)
     * of row c of embeddings[s].  Where it is given, the step after s starts from that row instead of computing the
     * projection of the embedding of the code just sampled — one operator fewer per step, same bits.  NULL: computed. */
    const uint16_t* projected[15];
} qm_predictor_frame;

int64_t qm_predictor_frame_workspace_bytes(void);
int32_t qm_predictor_frame_workspace_init(void* workspace, int64_t workspace_bytes, void* hip_stream);
/* *fits = 1 if qm_predictor_frame_steps can run on `hip_stream` (device and stream CU mask hold 256 blocks), else 0.
 * No counterpart in the reference, which has no kernel of this kind. */
int32_t qm_predictor_frame_fits(void* hip_stream, int32_t* fits);
int32_t qm_predictor_frame_steps(
    const qm_predictor_frame* frame, int32_t first_step, int32_t last_step,
    int32_t top_k, float temperature,
    void* workspace, int64_t workspace_bytes, uint32_t* status_dev, void* hip_stream);

/*
 * Everything between two attentions of the talker's decode step in one launch: the four launches
 * launch_linear_m1 (o_proj, R17:17203-17210), launch_add_postnorm_m1 + launch_gate_up_swiglu_m1 (R17:17215-17229),
 * launch_linear_m1 (down_proj + residual, R17:17236-17244) of a layer and launch_rmsnorm + launch_qkv_m1
 * (R17:17163-17176) of the next one, i.e. qm_linear_m1, qm_add_postnorm_gate_up_swiglu_m1, qm_linear_m1 and
 * qm_rmsnorm_qkv_m1 of this library, with bit-identical outputs: hidden_out = the layer's output, q_out / k_out /
 * v_out = the next layer's raw projections (what qm_decode_step_fused takes).  After the last layer the next_* and
 * *_out pointers are all NULL and the launch ends with hidden_out.  Biases may be NULL.  The talker's geometry only
 * (hidden 2048, q 2048, kv 1024, intermediate 6144; anything else: QM_ERR_GEOMETRY, take the operators one by one);
 * weight matrices 16-byte aligned.  256 blocks stay resident and stream the weights through LDS while they hand the
 * activations to each other through `workspace` (qm_talker_post_attention_workspace_bytes bytes, 256-byte aligned,
 * set up once with qm_talker_post_attention_workspace_init; launches that share a workspace must not overlap).
 * Like qm_predictor_frame_steps it needs the whole chip for its duration: QM_ERR_NO_DEVICE, before anything is
 * launched, if the device cannot hold 256 blocks at once or `hip_stream` is confined by a CU mask to fewer compute
 * units (qm_talker_chain_fits asks without launching; such a caller takes the operators one by one, same bits), and
 * no other stream's kernels may occupy compute units while it runs.  Waits are bounded
 * (QM_OPT_PREDICTOR_FRAME_SPIN_LIMIT applies here too): a launch that gives up ORs QM_STATUS_FRAME_TIMEOUT into
 * *status_dev, every block returns, outputs are undefined and the workspace must be initialised again.
 */
typedef struct qm_talker_post_attention {
    const uint16_t* context;          /* [q_columns] the layer's attention output */
    const uint16_t* hidden;           /* [hidden_columns] the layer's input */
    const uint16_t* o_weight;         /* [hidden_columns][q_columns] */
    const uint16_t* o_bias;           /* [hidden_columns] or NULL */
    const uint16_t* post_norm;        /* [hidden_columns] */
    const uint16_t* gate_weight;      /* [intermediate_columns][hidden_columns] */
    const uint16_t* up_weight;
    const uint16_t* down_weight;      /* [hidden_columns][intermediate_columns] */
    uint16_t* hidden_out;             /* [hidden_columns] */
    const uint16_t* next_input_norm;  /* [hidden_columns] */
    const uint16_t* next_q_weight;    /* [q_columns][hidden_columns] */
    const uint16_t* next_q_bias;
    const uint16_t* next_k_weight;    /* [kv_columns][hidden_columns] */
    const uint16_t* next_k_bias;
    const uint16_t* next_v_weight;
    const uint16_t* next_v_bias;
    uint16_t* q_out;                  /* [q_columns] */
    uint16_t* k_out;                  /* [kv_columns] */
    uint16_t* v_out;
    int32_t hidden_columns;
    int32_t q_columns;
    int32_t kv_columns;
    int32_t intermediate_columns;
    float epsilon;
} qm_talker_post_attention;

int64_t qm_talker_post_attention_workspace_bytes(void);
int32_t qm_talker_post_attention_workspace_init(void* workspace, int64_t workspace_bytes, void* hip_stream);
/* *fits = 1 if qm_talker_post_attention_m1 / qm_talker_layer_step_m1 can run on `hip_stream`, else 0.  No counterpart
 * in the reference. */
int32_t qm_talker_chain_fits(void* hip_stream, int32_t* fits);
int32_t qm_talker_post_attention_m1(
    const qm_talker_post_attention* op,
    void* workspace, int64_t workspace_bytes, uint32_t* status_dev, void* hip_stream);

/*
 * A talker layer's decode step after its Q/K/V projections in TWO launches: qm_decode_step_fused without its merge
 * launch, then qm_talker_post_attention_m1, whose first eight blocks combine the attention's split records (one kv head
 * each, the statistics, order and bits of the merge launch) and hand the context to all blocks while the weights of
 * o_proj and gate/up are already on their way into LDS.  Replaces launch_qk_norm_rope_cache_m1 + launch_attention +
 * the four launches named above (R17:17181-17244, and 17163-17176 of the next layer).  `context` [q_heads][128] receives
 * the attention's output; `post.context` is ignored.  Results (context, cache, q_rotated, hidden_out, q/k/v_out) are
 * bit-identical to qm_decode_step_fused followed by qm_talker_post_attention_m1.  The attention's arguments and
 * attention_workspace are those of qm_decode_step_fused; q_heads 16 over 8 kv heads only (the talker's geometry);
 * workspace, status word, bounded waits and QM_ERR_* as for qm_talker_post_attention_m1.
 */
typedef struct qm_talker_layer_step {
    const uint16_t* q;                /* [q_heads][128] raw projections of the new token */
    const uint16_t* k;                /* [kv_heads][128] */
    const uint16_t* v;
    const uint16_t* q_norm_w;         /* [128] */
    const uint16_t* k_norm_w;
    const uint16_t* cos_row;          /* [128] RoPE row of `position` */
    const uint16_t* sin_row;
    uint16_t* q_rotated_out;          /* [q_heads][128] or NULL */
    const qm_kv_cache* cache;
    const int32_t* page_table;
    void* attention_workspace;        /* qm_decode_workspace_bytes(1, q_heads, kv_heads, position + 1) */
    size_t attention_workspace_bytes;
    uint16_t* context;                /* [q_heads][128] the attention's output */
    int32_t max_pages;
    int32_t q_heads;
    int32_t position;
    int32_t sliding_window;
    float scale;
    float epsilon;
    qm_talker_post_attention post;
} qm_talker_layer_step;

int32_t qm_talker_layer_step_m1(
    const qm_talker_layer_step* step,
    void* workspace, int64_t workspace_bytes, uint32_t* status_dev, void* hip_stream);

/*
 * The three layout operators in front of the staged attention at the predictor's step 0 (call site
 * R17:13663-13699), each with the reference wrapper's per-tensor argument list:
 * qm_predictor_transpose replaces PersistentPredictor::transpose (R17:13222-13236, kernel
 *   transpose_bshd_to_bhsd_kernel :8366-8400): input [rows][heads][128] -> output [heads][rows][128].
 * qm_predictor_rope_bhsd replaces PersistentPredictor::rope (R17:13238-13254, kernel apply_rope_kernel
 *   :8403-8488): input, output [heads][rows][128] (BHSD); head h, row s is rotated with cos/sin row s
 *   ([rows][128]): bf16(bf16(x*cos) + bf16(rotate_half(x)*sin)), no norm.
 * qm_predictor_update_cache replaces PersistentPredictor::update_cache (R17:13256-13270, kernel
 *   update_cache_kernel :8491-8529): source [8][rows][128] (BHSD) is copied to
 *   cache[(h*16 + start + s)*128 ..] of ONE [8][16][128] cache (the reference calls it once for the
 *   key and once for the value cache).  start + rows > 16 is QM_ERR_SLOT_RANGE (the reference has no
 *   guard).  Tensors 16-byte aligned for transpose and update_cache (QM_ERR_GEOMETRY).
 */
int32_t qm_predictor_transpose(
    const uint16_t* input, uint16_t* output, int32_t rows, int32_t heads, void* hip_stream);
int32_t qm_predictor_rope_bhsd(
    const uint16_t* input, const uint16_t* cos_rows, const uint16_t* sin_rows, uint16_t* output,
    int32_t rows, int32_t heads, void* hip_stream);
int32_t qm_predictor_update_cache(
    const uint16_t* source, uint16_t* cache, int32_t rows, int32_t start, void* hip_stream);

/* --- (5) M = 1 weight-streaming linears around the path ----------------------------------- */
/*
 * qm_linear_m1 replaces launch_linear_m1 / talker_linear_fused_kernel (R17:17473-17511,
 * 15201-15268): output[o] = bf16(sum_k input[k] * weight[o][k] + bias[o]); with a residual the
 * stored value is bf16(residual[o] + bf16(that)).  weight is [output_columns][reduction_columns]
 * row-major bf16; bias and residual may be NULL; output must not alias input.
 * qm_qkv_m1 replaces launch_qkv_m1 / talker_qkv_fused_kernel (R17:17513-17567, 15272-15362):
 * the three projections of one decode step over one read of the normalised hidden vector;
 * weights [q_dim][hidden], [kv_dim][hidden], [kv_dim][hidden]; biases may be NULL.
 * Both reproduce the reference's fp32 summation order (32 strided fmaf chains per output, then
 * its shuffle tree), so outputs are bit-identical to the reference kernels'.
 * reduction_columns / hidden must be even and <= 16384 (QM_ERR_GEOMETRY otherwise); weight
 * pointers 4-byte aligned.
 */
int32_t qm_linear_m1(
    const uint16_t* input, const uint16_t* weight, const uint16_t* bias, const uint16_t* residual,
    uint16_t* output, int32_t output_columns, int32_t reduction_columns,
    void* hip_stream);
int32_t qm_qkv_m1(
    const uint16_t* input,
    const uint16_t* q_weight, const uint16_t* q_bias,
    const uint16_t* k_weight, const uint16_t* k_bias,
    const uint16_t* v_weight, const uint16_t* v_bias,
    uint16_t* q_output, uint16_t* k_output, uint16_t* v_output,
    int32_t hidden, int32_t q_dim, int32_t kv_dim,
    void* hip_stream);

/*
 * qm_gate_up_swiglu_m1 replaces launch_gate_up_swiglu_m1 / talker_gate_up_swiglu_fused_kernel
 * (R17:17848-17890, 16289-16362): per channel c, g = bf16(input . gate_weight[c]),
 * u = bf16(input . up_weight[c]) in the M = 1 linear's summation order,
 * output[c] = bf16(bf16(g / (1 + expf(-g))) * u).  Weights [intermediate][hidden]; same limits
 * as qm_linear_m1.  Bit-identical up to the device's expf.
 */
int32_t qm_gate_up_swiglu_m1(
    const uint16_t* input, const uint16_t* gate_weight, const uint16_t* up_weight,
    uint16_t* output, int32_t hidden, int32_t intermediate,
    void* hip_stream);
/*
 * qm_rmsnorm_rows replaces launch_rmsnorm / rmsnorm_kernel (R17:8908-8929, 8276-8338):
 * output[r][c] = bf16(bf16(input[r][c] * inverse_rms_r) * weight[c]), the statistic summed in the
 * reference's 256-thread order.  qm_add_postnorm_m1 replaces launch_add_postnorm_m1 /
 * talker_add_postnorm_fused_kernel (R17:17817-17846, 16205-16286): residual = bf16(hidden +
 * attention), normalized = the RMSNorm of that rounded residual.  dimension <= 32768 there.
 */
int32_t qm_rmsnorm_rows(
    const uint16_t* input, const uint16_t* weight, uint16_t* output,
    int32_t rows, int32_t dimension, float epsilon,
    void* hip_stream);
int32_t qm_add_postnorm_m1(
    const uint16_t* hidden, const uint16_t* attention, const uint16_t* norm_weight,
    uint16_t* residual, uint16_t* normalized, int32_t dimension, float epsilon,
    void* hip_stream);

/*
 * Two fusions of consecutive reference launches of a decode layer; the fused results are
 * bit-identical to running the two operators one after the other:
 * qm_rmsnorm_qkv_m1 = launch_rmsnorm(hidden_state, input_norm) (R17:17163-17169) followed by
 * launch_qkv_m1 (R17:17174-17176): every block normalises the hidden state itself while its
 * weights are in flight, the normalised vector never goes to memory.
 * qm_add_postnorm_gate_up_swiglu_m1 = launch_add_postnorm_m1 (R17:17215-17220) followed by
 * launch_gate_up_swiglu_m1 (R17:17226-17229); `residual` (= bf16(hidden_state + attention), which
 * down_proj adds later) is written, the post-norm vector is not.
 * Both need hidden % 8 == 0, hidden <= 16384 and 16-byte aligned weight matrices
 * (QM_ERR_GEOMETRY otherwise).
 */
int32_t qm_rmsnorm_qkv_m1(
    const uint16_t* hidden_state, const uint16_t* norm_weight, float epsilon,
    const uint16_t* q_weight, const uint16_t* q_bias,
    const uint16_t* k_weight, const uint16_t* k_bias,
    const uint16_t* v_weight, const uint16_t* v_bias,
    uint16_t* q_output, uint16_t* k_output, uint16_t* v_output,
    int32_t hidden, int32_t q_dim, int32_t kv_dim,
    void* hip_stream);
int32_t qm_add_postnorm_gate_up_swiglu_m1(
    const uint16_t* hidden_state, const uint16_t* attention, const uint16_t* norm_weight, float epsilon,
    uint16_t* residual,
    const uint16_t* gate_weight, const uint16_t* up_weight, uint16_t* output,
    int32_t hidden, int32_t intermediate,
    void* hip_stream);

/*
 * The code predictor's M = 1 linears.  Replace PersistentPredictor::linear_m1 (R17:13499-13533,
 * kernel predictor_linear_m1_fused_kernel :12579-12654), ::qkv_m1 (R17:13389-13430, kernel
 * predictor_qkv_m1_fused_kernel :12046-12130) and ::gate_up_swiglu_m1 (R17:13558-13589, kernel
 * :12736-12815).  Same layouts as the talker's linears above, no bias, and another order of the
 * sum, reproduced bit for bit: lane l of the row's 32 chains takes the element pairs
 * k = 2l, 2l + 64, ..., first element of a pair first, each product added with one fmaf
 * (predictor_bf16_dot2_accumulate in its portable form, R17:8216-8228; the gfx1100 build of the
 * reference uses that chip's dot2 instruction, whose rounding is not restated here).
 * qm_predictor_rmsnorm_qkv_m1 and qm_predictor_add_postnorm_gate_up_swiglu_m1 fuse the launch
 * before (rmsnorm R17:13210-13220; add_postnorm_m1 :13535-13556, kernel :12658-12733, the talker's
 * arithmetic) like their talker counterparts.  All five need reduction % 8 == 0,
 * reduction <= 16384 and 16-byte aligned weight matrices (QM_ERR_GEOMETRY otherwise).
 */
int32_t qm_predictor_linear_m1(
    const uint16_t* input, const uint16_t* weight, const uint16_t* residual, uint16_t* output,
    int32_t output_columns, int32_t reduction_columns, void* hip_stream);
int32_t qm_predictor_qkv_m1(
    const uint16_t* input, const uint16_t* q_weight, const uint16_t* k_weight, const uint16_t* v_weight,
    uint16_t* q_output, uint16_t* k_output, uint16_t* v_output,
    int32_t hidden, int32_t q_dim, int32_t kv_dim, void* hip_stream);
int32_t qm_predictor_gate_up_swiglu_m1(
    const uint16_t* input, const uint16_t* gate_weight, const uint16_t* up_weight, uint16_t* output,
    int32_t hidden, int32_t intermediate, void* hip_stream);
int32_t qm_predictor_rmsnorm_qkv_m1(
    const uint16_t* hidden_state, const uint16_t* norm_weight, float epsilon,
    const uint16_t* q_weight, const uint16_t* k_weight, const uint16_t* v_weight,
    uint16_t* q_output, uint16_t* k_output, uint16_t* v_output,
    int32_t hidden, int32_t q_dim, int32_t kv_dim, void* hip_stream);
int32_t qm_predictor_add_postnorm_gate_up_swiglu_m1(
    const uint16_t* hidden_state, const uint16_t* attention, const uint16_t* norm_weight, float epsilon,
    uint16_t* residual,
    const uint16_t* gate_weight, const uint16_t* up_weight, uint16_t* output,
    int32_t hidden, int32_t intermediate, void* hip_stream);

/* ---- linears over token rows (the prompt pass) ------------------------------------ */
/*
 * qm_linear_rows replaces NativeTalkerEngine::linear_generic -> native_ops::linear_bf16
 * (R17:17453-17472, 198-245; kernel linear_wave32_bf16_f32acc_kernel :126-196) as the prompt pass
 * uses it (R17:16646-16790): output[r][n] = bf16(sum_k input[r][k] * weight[n][k] (+ bias[n])), each
 * sum in the order of qm_linear_m1, so a prompt row and a decode step of the same vector agree to
 * the bit.  A non-NULL residual [rows][output_columns] folds the launch_add behind it
 * (add_bf16_kernel R17:8729-8744: bf16(residual + output)).
 * qm_gate_up_swiglu_rows = the two linear_generic calls on gate and up and launch_swiglu
 * (R17:16742-16768, swiglu_kernel :8745-8770): qm_gate_up_swiglu_m1 row by row.
 * reduction % 8 == 0, reduction <= 16384, input and weights 16-byte aligned (QM_ERR_GEOMETRY).  The exact chain
 * (calls of fewer than 16 rows, shapes off the 128-wide matrix tiles, QM_OPT_LINEAR_ROWS_KERNEL = 1) keeps eight token
 * rows and its weight rows in LDS: there reduction <= 6640 for a linear and hidden <= 4976 for a gate/up pair
 * (QM_ERR_GEOMETRY beyond; the talker's largest are 6144 and 2048).
 */
int32_t qm_linear_rows(
    const uint16_t* input, const uint16_t* weight, const uint16_t* bias, const uint16_t* residual,
    uint16_t* output, int32_t rows, int32_t output_columns, int32_t reduction_columns, void* hip_stream);
int32_t qm_gate_up_swiglu_rows(
    const uint16_t* input, const uint16_t* gate_weight, const uint16_t* up_weight, uint16_t* output,
    int32_t rows, int32_t hidden, int32_t intermediate, void* hip_stream);
/*
 * The same two operators with a workspace for SHORT prompts (no counterpart in the reference, whose kernel gives every
 * output its own wave).  On the matrix cores a block owns 128 output columns of 64 or 128 token rows and walks the whole
 * reduction: 128 rows of a 2048-column linear are 32 blocks on 256 compute units, and the call lasts as long as one
 * block's chain.  With a workspace of qm_linear_rows_split_workspace_bytes (0 where the shape is not cut: enough blocks
 * already, a reduction below 4096, or the exact chain) the reduction is cut into 2, 4 or 8 pieces, a block each, whose
 * fp32 sums a second launch adds in order before the same roundings.  Results differ from the uncut call in the association of the sum only
 * (within the matrix-core path's tolerance of the exact chain) and are the same on every call.  workspace: 256-byte
 * aligned, nothing to initialise; NULL: exactly qm_linear_rows / qm_gate_up_swiglu_rows; too small: QM_ERR_WORKSPACE.
 */
int64_t qm_linear_rows_split_workspace_bytes(int32_t rows, int32_t output_columns, int32_t reduction_columns, int32_t gate_up_pair);
int32_t qm_linear_rows_split(
    const uint16_t* input, const uint16_t* weight, const uint16_t* bias, const uint16_t* residual,
    uint16_t* output, int32_t rows, int32_t output_columns, int32_t reduction_columns,
    void* workspace, int64_t workspace_bytes, void* hip_stream);
int32_t qm_gate_up_swiglu_rows_split(
    const uint16_t* input, const uint16_t* gate_weight, const uint16_t* up_weight, uint16_t* output,
    int32_t rows, int32_t hidden, int32_t intermediate,
    void* workspace, int64_t workspace_bytes, void* hip_stream);
/*
 * The q, k and v projections of the prompt pass (the first three linear_generic calls of a layer, R17:16646-16672) as one
 * call: output for output what three qm_linear_rows calls on the same input give, bit for bit (on the matrix cores an
 * output's sum does not depend on the tile it is computed in).  Where all three run on the matrix cores they share
 * one grid (1024 tokens: 256 blocks, one per compute unit, instead of 256 + 128 + 128 in three launches) and no
 * reduction is cut; otherwise the call is the three calls.  _split: the workspace of qm_linear_rows_split (the larger of
 * the two shapes' sizes), used by the three calls only.
 */
int32_t qm_qkv_rows(
    const uint16_t* input, const uint16_t* q_weight, const uint16_t* k_weight, const uint16_t* v_weight,
    const uint16_t* q_bias, const uint16_t* k_bias, const uint16_t* v_bias,
    uint16_t* q_output, uint16_t* k_output, uint16_t* v_output,
    int32_t rows, int32_t q_columns, int32_t kv_columns, int32_t reduction_columns, void* hip_stream);
int32_t qm_qkv_rows_split(
    const uint16_t* input, const uint16_t* q_weight, const uint16_t* k_weight, const uint16_t* v_weight,
    const uint16_t* q_bias, const uint16_t* k_bias, const uint16_t* v_bias,
    uint16_t* q_output, uint16_t* k_output, uint16_t* v_output,
    int32_t rows, int32_t q_columns, int32_t kv_columns, int32_t reduction_columns,
    void* workspace, int64_t workspace_bytes, void* hip_stream);

/* ---- final head: score processing, top-k sampler, history ------------------------ */
/*
 * qm_sample_topk replaces gpu_sample_topk_f32_kernel and gpu_sample_topk_bf16_kernel
 * (R17:7407-7518; callers NativeFinalHead::run_fast_device :14500-14512 and
 * PersistentPredictor::capture_step :13814-13833): over the `vocab` scores starting at element
 * `offset` of `logits` (float, or bf16 bit patterns if logits_are_bf16), ordered by score
 * descending and id ascending, the first keep = min(top_k, vocab) are sampled with probability
 * proportional to exp(score / temperature) — sums in double in that order, one SplitMix64 draw
 * from *rng_state (advanced in place, R17:7353-7371), the first index whose running sum exceeds
 * uniform * total; without a positive total the first id is returned and nothing is drawn.
 * top_k <= 0 is the arg-max (argmax_final_head R17:14099-14143, argmax_bf16_kernel): highest
 * score, lowest id among equals; rng_state may then be NULL.
 * One block; vocab <= 4096 (the reference's sort size), top_k <= 256 (QM_ERR_GEOMETRY beyond),
 * temperature > 0.  Same chosen id as the reference for scores without NaN.
 */
int32_t qm_sample_topk(
    const void* logits, int32_t logits_are_bf16, int32_t offset, int32_t vocab,
    int32_t top_k, float temperature, uint64_t* rng_state, int32_t* output_id,
    void* hip_stream);

/*
 * qm_final_head_process = cast_final_head_logits + repetition_penalty + suppress_tokens
 * (R17:14025-14097) in one launch: scores[t] = f32(logits[t]); a token found in
 * history[0 .. history_count) is multiplied by `penalty` if negative, else by
 * float(1) / float(penalty) (the reference's constant 0x3f73cf3e for 1.05); token `eos` is -inf
 * while generation_index < 2; the last `suppressed_tail` tokens other than eos are -inf.
 * qm_final_head_sample is the device side of NativeFinalHead::run_fast_device after the head
 * projection (R17:14456-14545) in one launch instead of five: that processing with
 * history_count = generation_index, then qm_sample_topk over the processed scores, then
 * history[generation_index] = code (append_sampled_code_history_kernel R17:7530-7543).
 * `scores_out` (NULL or [vocab] floats) receives the processed scores.  The head projection
 * itself is qm_linear_m1 (native_ops::linear_bf16 at one row has the talker linear's order,
 * R17:126-196).  The reference's constants: vocab 3072, eos 2150, suppressed_tail 1024,
 * penalty 1.05, top_k 50, temperature 0.9 (R17:13958-13961, 7338-7339).
 */
int32_t qm_final_head_process(
    const uint16_t* logits, const int32_t* history, int32_t history_count, int32_t generation_index,
    int32_t vocab, int32_t eos, int32_t suppressed_tail, float penalty, float* scores,
    void* hip_stream);
int32_t qm_final_head_sample(
    const uint16_t* logits, int32_t* history, int32_t generation_index,
    int32_t vocab, int32_t eos, int32_t suppressed_tail, float penalty,
    int32_t top_k, float temperature, uint64_t* rng_state, int32_t* code_out, float* scores_out,
    void* hip_stream);

/*
 * Replaces gather_predictor_embedding_kernel (R17:11998-12030; launched in
 * PersistentPredictor::capture_step :13845-13853): with token = codes[group],
 * selected_embeddings[group][d] = next_step_input[d] = table[token][d] for d < dimension
 * (the reference's kOuterHidden = 2048).  A token outside [0, table_rows) moves nothing
 * (the reference has no such guard).
 */
int32_t qm_gather_embedding(
    const uint16_t* table, int32_t table_rows, const int32_t* codes, int32_t group, int32_t dimension,
    uint16_t* selected_embeddings, uint16_t* next_step_input, void* hip_stream);

/*
 * The two ends of a code-predictor frame (PersistentPredictor::run_frame_device R17:13043-13156, capture_graph
 * :13856-13896).
 * qm_predictor_prepare_group0 replaces prepare_group0_input_kernel (R17:11963-11996): with token = code0[0] (the
 *   talker's code of the frame, on the device), row `token` of the talker's codec embedding table becomes
 *   selected_embeddings[0][*] and the second row of the two-row input free_input[1][*]; generated_codes[0] =
 *   token.  A token outside [0, table_rows) stores code 0 and moves nothing, as in the reference.
 * qm_predictor_next_talker_input replaces sum_codec_embeddings_kernel (R17:8877-8906) and the add behind it
 *   (R17:13872-13875): embedding_sum = bf16(sum over the `groups` selected embeddings, fp32, in group order),
 *   next_talker_input = bf16(embedding_sum + context_embedding).  embedding_sum may be NULL.
 */
int32_t qm_predictor_prepare_group0(
    const uint16_t* codec_table, int32_t table_rows, const int32_t* code0, int32_t dimension,
    uint16_t* free_input, uint16_t* selected_embeddings, int32_t* generated_codes, void* hip_stream);
int32_t qm_predictor_next_talker_input(
    const uint16_t* selected_embeddings, int32_t groups, const uint16_t* context_embedding, int32_t dimension,
    uint16_t* embedding_sum, uint16_t* next_talker_input, void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* QM_ATTN_H */
