// qm_frame_engine.cpp — the per-frame generation loop of the engine shell: the final head (codec_head +
// score processing + sampler + history), the code predictor's 15-step frame, and the loop that alternates
// talker decode, final head and predictor frame and hashes the codec trajectory.
//
// Reference: NativeFinalHead::run_fast_device (R17:14427-14570), PredictorWeights (R17:10411-10712),
// PersistentPredictor::run_frame_device (R17:13043-13156), capture_step (R17:13592-13854), capture_graph
// (R17:13856-13896), generate_codec_sequence (R17:21887-22538).  Every device operation is a C-ABI operator of
// libqm_attn on the talker's generation stream; the host reads back four bytes per frame after the final head
// and sixty-four after the predictor, as the reference does.
#include "qm_engine_common.hpp"

#include <array>
#include <cstring>
#include <memory>

namespace qm_engine {

constexpr int kOuter = kHidden;            // kOuterHidden, R17:7951: the talker's width
constexpr int kPredHidden = 1024;          // kHidden, R17:7952
constexpr int kPredIntermediate = 3072;    // R17:7953
constexpr int kPredQueryHeads = 16;        // R17:7955
constexpr int kPredKvHeads = 8;            // R17:7956
constexpr int kPredQueryDim = kPredQueryHeads * kHeadDim;
constexpr int kPredKvDim = kPredKvHeads * kHeadDim;
constexpr int kPredVocab = 2048;           // R17:7960
constexpr int kPredSteps = 15;             // R17:7961
constexpr int kCodeGroups = 16;            // R17:7962
constexpr int kPredMaxCache = 16;          // R17:7964
constexpr int kHeadVocab = 3072;           // final head, R17:14444
constexpr int kCodecEos = 2150;            // R17:13958-13961
constexpr int kSuppressedTail = 1024;
constexpr float kPenalty = 1.05f;
constexpr int kTopK = 50;                  // kGpuSamplerTopK, R17:7338
constexpr float kTemperature = 0.9f;       // kGpuSamplerTemperature, R17:7339

static void expect_shape(const Param& p, std::vector<int64_t> shape, const std::string& what) {
    if (p.shape != shape) throw TensorError("unexpected shape of " + what);
}

// A part of a device allocation that another object owns.
struct DeviceSlice {
    void* pointer = nullptr;
    size_t size = 0;
    uint16_t* u16() const { return static_cast<uint16_t*>(pointer); }
    void* raw() const { return pointer; }
    size_t bytes() const { return size; }
};

struct PredictorLayer {
    Param input_norm, q_weight, k_weight, v_weight, q_norm, k_norm, o_weight, post_norm, gate_weight, up_weight, down_weight;
    DeviceSlice key_cache, value_cache;    // [8][16][128], parts of qm_predictor::frame_state
};

}  // namespace qm_engine

using namespace qm_engine;

struct qm_final_head {
    Param weight;                          // talker.codec_head.weight [3072][2048]
    DeviceBuffer logits, history, code, rng, rng_after_head;
    int capacity = 0;
    hipStream_t stream = nullptr;
};

struct qm_predictor {
    Param projection_weight, projection_bias, final_norm, codec0_table;
    std::vector<PredictorLayer> layers;
    std::vector<Param> heads, embeddings;
    std::vector<DeviceBuffer> projected;   // [step][code][1024]: the input projection of every row of embeddings[step]
    hipStream_t stream = nullptr;
    uint64_t* rng_state = nullptr;         // device, shared with the final head
    DeviceBuffer cosine, sine;             // [16][128], positions 0..15
    DeviceBuffer free_input, context_embedding, hidden_a, hidden_b, norm, q_linear, k_linear, v_linear, q_normed, k_normed,
        q_bhsd, k_bhsd, v_bhsd, q_rotated, k_rotated, context, attention, residual, post_norm, swiglu, logits,
        embedding_sum, next_input;
    // What run_frame_device clears at the start of a frame (R17:13043-13070) — the layers' caches, the selected
    // embeddings, the codes — lies in one allocation, so that one fill clears it.
    DeviceBuffer frame_state;
    DeviceSlice selected, codes;
    // the M = 1 steps as one launch (qm_predictor_frame_steps): only for the five-layer geometry it is built for
    bool one_launch = false;
    qm_predictor_frame frame = {};
    DeviceBuffer frame_workspace, status;
};

namespace qm_engine {

static std::unique_ptr<qm_final_head> create_final_head(const std::string& model_dir, int capacity, uint64_t seed,
                                                        hipStream_t stream) {
    if (capacity <= 0) throw ApiError(QM_ERR_ARGUMENT, "history capacity must be positive");
    ModelDirectory host(model_dir);
    StreamDrain drain(stream);             // (uploads read the mapped files: they finish before `host` goes, also on an error)
    auto head = std::make_unique<qm_final_head>();
    head->stream = stream;
    head->weight = Param(host.suffix("talker.codec_head.weight"), stream);
    expect_shape(head->weight, {kHeadVocab, kHidden}, "talker.codec_head.weight");
    head->logits = DeviceBuffer(kHeadVocab * 2);
    head->history = DeviceBuffer(static_cast<size_t>(capacity) * sizeof(int32_t));
    head->code = DeviceBuffer(sizeof(int32_t));
    head->rng = DeviceBuffer(sizeof(uint64_t));
    head->rng_after_head = DeviceBuffer(sizeof(uint64_t));
    head->capacity = capacity;
    hip_check(hipMemcpyAsync(head->rng.raw(), &seed, sizeof seed, hipMemcpyHostToDevice, stream), "generator seed upload");
    hip_check(hipMemsetAsync(head->history.raw(), 0, head->history.bytes(), stream), "history reset");
    hip_check(hipStreamSynchronize(stream), "final head upload synchronize");
    return head;
}

// run_fast_device (R17:14427-14570): codec_head, then cast + repetition penalty + suppressed tokens + sampler (or
// arg-max) + history append in one launch, then the four-byte read-back that is the frame boundary.
static void final_head_launch(qm_final_head& h, const uint16_t* hidden_device, int frame, bool sampling) {
    if (frame < 0 || frame >= h.capacity) throw ApiError(QM_ERR_SLOT_RANGE, "FinalHead generation index exceeds GPU history capacity");
    op_check(qm_linear_m1(hidden_device, h.weight.data(), nullptr, nullptr, h.logits.u16(), kHeadVocab, kHidden, h.stream),
             "final head projection");
    op_check(qm_final_head_sample(h.logits.u16(), static_cast<int32_t*>(h.history.raw()), frame, kHeadVocab, kCodecEos,
                                  kSuppressedTail, kPenalty, sampling ? kTopK : 0, kTemperature,
                                  static_cast<uint64_t*>(h.rng.raw()), static_cast<int32_t*>(h.code.raw()), nullptr, h.stream),
             "final head sampler");
}

static int32_t final_head_run(qm_final_head& h, const uint16_t* hidden_device, int frame, bool sampling) {
    final_head_launch(h, hidden_device, frame, sampling);
    int32_t code = 0;
    hip_check(hipMemcpyAsync(&code, h.code.raw(), sizeof code, hipMemcpyDeviceToHost, h.stream), "code read-back");
    hip_check(hipStreamSynchronize(h.stream), "frame boundary synchronize");
    return code;
}

static std::unique_ptr<qm_predictor> create_predictor(const std::string& model_dir, uint64_t* rng_state, hipStream_t stream) {
    if (!rng_state) throw ApiError(QM_ERR_NULL, "the predictor samples from the final head's generator state");
    ModelDirectory host(model_dir);
    StreamDrain drain(stream);             // (uploads read the mapped files: they finish before `host` goes, also on an error)
    auto p = std::make_unique<qm_predictor>();
    p->stream = stream;
    p->rng_state = rng_state;
    const std::string root = "talker.code_predictor.";
    p->projection_weight = Param(host.suffix(root + "small_to_mtp_projection.weight"), stream);
    p->projection_bias = Param(host.suffix(root + "small_to_mtp_projection.bias"), stream);
    expect_shape(p->projection_weight, {kPredHidden, kOuter}, "small_to_mtp_projection.weight");
    expect_shape(p->projection_bias, {kPredHidden}, "small_to_mtp_projection.bias");
    for (int index = 0;; ++index) {
        const std::string lr = root + "model.layers." + std::to_string(index) + ".";
        const TensorView* first = host.maybe_suffix(lr + "input_layernorm.weight");
        if (!first) break;
        PredictorLayer w;
        w.input_norm = Param(*first, stream);
        w.q_weight = Param(host.suffix(lr + "self_attn.q_proj.weight"), stream);
        w.k_weight = Param(host.suffix(lr + "self_attn.k_proj.weight"), stream);
        w.v_weight = Param(host.suffix(lr + "self_attn.v_proj.weight"), stream);
        w.o_weight = Param(host.suffix(lr + "self_attn.o_proj.weight"), stream);
        w.q_norm = Param(host.suffix(lr + "self_attn.q_norm.weight"), stream);
        w.k_norm = Param(host.suffix(lr + "self_attn.k_norm.weight"), stream);
        w.post_norm = Param(host.suffix(lr + "post_attention_layernorm.weight"), stream);
        w.gate_weight = Param(host.suffix(lr + "mlp.gate_proj.weight"), stream);
        w.up_weight = Param(host.suffix(lr + "mlp.up_proj.weight"), stream);
        w.down_weight = Param(host.suffix(lr + "mlp.down_proj.weight"), stream);
        expect_shape(w.input_norm, {kPredHidden}, lr + "input_layernorm.weight");
        expect_shape(w.q_weight, {kPredQueryDim, kPredHidden}, lr + "self_attn.q_proj.weight");
        expect_shape(w.k_weight, {kPredKvDim, kPredHidden}, lr + "self_attn.k_proj.weight");
        expect_shape(w.v_weight, {kPredKvDim, kPredHidden}, lr + "self_attn.v_proj.weight");
        expect_shape(w.o_weight, {kPredHidden, kPredQueryDim}, lr + "self_attn.o_proj.weight");
        expect_shape(w.q_norm, {kHeadDim}, lr + "self_attn.q_norm.weight");
        expect_shape(w.k_norm, {kHeadDim}, lr + "self_attn.k_norm.weight");
        expect_shape(w.post_norm, {kPredHidden}, lr + "post_attention_layernorm.weight");
        expect_shape(w.gate_weight, {kPredIntermediate, kPredHidden}, lr + "mlp.gate_proj.weight");
        expect_shape(w.up_weight, {kPredIntermediate, kPredHidden}, lr + "mlp.up_proj.weight");
        expect_shape(w.down_weight, {kPredHidden, kPredIntermediate}, lr + "mlp.down_proj.weight");
        p->layers.push_back(std::move(w));
    }
    if (p->layers.empty()) throw TensorError("no code predictor layers in " + model_dir);
    p->final_norm = Param(host.suffix(root + "model.norm.weight"), stream);
    expect_shape(p->final_norm, {kPredHidden}, "code_predictor.model.norm.weight");
    for (int index = 0; index < kPredSteps; ++index) {
        p->heads.emplace_back(host.suffix(root + "lm_head." + std::to_string(index) + ".weight"), stream);
        p->embeddings.emplace_back(host.suffix(root + "model.codec_embedding." + std::to_string(index) + ".weight"), stream);
        expect_shape(p->heads.back(), {kPredVocab, kPredHidden}, "code_predictor.lm_head weight");
        expect_shape(p->embeddings.back(), {kPredVocab, kOuter}, "code_predictor.model.codec_embedding weight");
    }
    p->codec0_table = Param(host.suffix("talker.model.codec_embedding.weight"), stream);
    if (p->codec0_table.shape.size() != 2 || p->codec0_table.shape[1] != kOuter || p->codec0_table.shape[0] <= 0
        || p->codec0_table.shape[0] > 0x7fffffff)
        throw TensorError("unexpected shape of talker.model.codec_embedding.weight");

    // RoPE rows of positions 0..15 (PersistentPredictor::make_rope, R17:13161-13197: the talker's table rule)
    std::vector<uint16_t> cos_host(kPredMaxCache * kHeadDim), sin_host(kPredMaxCache * kHeadDim);
    op_check(qm_rope_rows(kPredMaxCache, 0, kHeadDim, 1000000.0, cos_host.data(), sin_host.data()), "predictor rope rows");
    p->cosine = DeviceBuffer(cos_host.size() * 2);
    p->sine = DeviceBuffer(sin_host.size() * 2);
    hip_check(hipMemcpyAsync(p->cosine.raw(), cos_host.data(), cos_host.size() * 2, hipMemcpyHostToDevice, stream), "rope upload");
    hip_check(hipMemcpyAsync(p->sine.raw(), sin_host.data(), sin_host.size() * 2, hipMemcpyHostToDevice, stream), "rope upload");

    auto rows2 = [](int width) { return DeviceBuffer(static_cast<size_t>(2) * width * 2); };
    p->free_input = rows2(kOuter); p->context_embedding = DeviceBuffer(kOuter * 2);
    p->hidden_a = rows2(kPredHidden); p->hidden_b = rows2(kPredHidden); p->norm = rows2(kPredHidden);
    p->q_linear = rows2(kPredQueryDim); p->k_linear = rows2(kPredKvDim); p->v_linear = rows2(kPredKvDim);
    p->q_normed = rows2(kPredQueryDim); p->k_normed = rows2(kPredKvDim);
    p->q_bhsd = rows2(kPredQueryDim); p->k_bhsd = rows2(kPredKvDim); p->v_bhsd = rows2(kPredKvDim);
    p->q_rotated = rows2(kPredQueryDim); p->k_rotated = rows2(kPredKvDim); p->context = rows2(kPredQueryDim);
    p->attention = rows2(kPredHidden); p->residual = rows2(kPredHidden); p->post_norm = rows2(kPredHidden);
    p->swiglu = rows2(kPredIntermediate); p->logits = rows2(kPredVocab);
    {
        const size_t cache_bytes = static_cast<size_t>(kPredKvHeads) * kPredMaxCache * kHeadDim * 2;     // a multiple of 256
        const size_t selected_bytes = static_cast<size_t>(kCodeGroups) * kOuter * 2;
        p->frame_state = DeviceBuffer(2 * cache_bytes * p->layers.size() + selected_bytes + 256);
        unsigned char* at = static_cast<unsigned char*>(p->frame_state.raw());
        for (PredictorLayer& w : p->layers) {
            w.key_cache = DeviceSlice{at, cache_bytes};
            w.value_cache = DeviceSlice{at + cache_bytes, cache_bytes};
            at += 2 * cache_bytes;
        }
        p->selected = DeviceSlice{at, selected_bytes};
        p->codes = DeviceSlice{at + selected_bytes, kCodeGroups * sizeof(int32_t)};
    }
    p->embedding_sum = DeviceBuffer(kOuter * 2); p->next_input = DeviceBuffer(kOuter * 2);
    hip_check(hipStreamSynchronize(stream), "predictor upload synchronize");   // the mapped files go away with `host`
    p->status = DeviceBuffer(256);
    hip_check(hipMemsetAsync(p->status.raw(), 0, p->status.bytes(), stream), "predictor status word");
    if (p->layers.size() == 5) {
        qm_predictor_frame& f = p->frame;
        for (size_t i = 0; i < 5; ++i) {
            PredictorLayer& w = p->layers[i];
            qm_predictor_frame_layer& d = f.layers[i];
            d.input_norm = w.input_norm.data(); d.q_weight = w.q_weight.data(); d.k_weight = w.k_weight.data(); d.v_weight = w.v_weight.data();
            d.q_norm = w.q_norm.data(); d.k_norm = w.k_norm.data(); d.o_weight = w.o_weight.data(); d.post_norm = w.post_norm.data();
            d.gate_weight = w.gate_weight.data(); d.up_weight = w.up_weight.data(); d.down_weight = w.down_weight.data();
            d.key_cache = w.key_cache.u16(); d.value_cache = w.value_cache.u16();
        }
        f.projection_weight = p->projection_weight.data(); f.projection_bias = p->projection_bias.data(); f.final_norm = p->final_norm.data();
        for (int step = 0; step < kPredSteps; ++step) {
            f.heads[step] = p->heads[static_cast<size_t>(step)].data();
            f.embeddings[step] = p->embeddings[static_cast<size_t>(step)].data();
        }
        f.cosine = p->cosine.u16(); f.sine = p->sine.u16();
        f.free_input = p->free_input.u16(); f.selected = p->selected.u16(); f.codes = static_cast<int32_t*>(p->codes.raw());
        f.step0_input = p->free_input.u16();              // the two rows of step 0 (its first row is also the later steps' input)
        f.rng_state = rng_state; f.epsilon = kEpsilon;
        // The input projection of every row of the embedding tables of steps 0..13, once: a step of the frame kernel then
        // starts from a table row instead of projecting the embedding of the code just sampled (one operator fewer).
        // Eight rows per call: below sixteen rows qm_linear_rows takes the exact chain, row by row what qm_linear_m1 gives.
        p->projected.reserve(static_cast<size_t>(kPredSteps - 1));
        for (int step = 0; step + 1 < kPredSteps; ++step) {
            const int64_t codes = p->embeddings[static_cast<size_t>(step)].shape[0];
            p->projected.emplace_back(static_cast<size_t>(codes) * kPredHidden * 2);
            uint16_t* table = p->projected.back().u16();
            for (int64_t row = 0; row < codes; row += 8) {
                const int32_t n = static_cast<int32_t>(std::min<int64_t>(8, codes - row));
                op_check(qm_linear_rows(p->embeddings[static_cast<size_t>(step)].data() + row * kOuter, p->projection_weight.data(),
                                        p->projection_bias.data(), nullptr, table + row * kPredHidden, n, kPredHidden, kOuter, stream),
                         "projected embedding table");
            }
            f.projected[step] = table;
        }
        hip_check(hipStreamSynchronize(stream), "projected embedding tables synchronize");
        p->frame_workspace = DeviceBuffer(static_cast<size_t>(qm_predictor_frame_workspace_bytes()));
        op_check(qm_predictor_frame_workspace_init(p->frame_workspace.raw(), static_cast<int64_t>(p->frame_workspace.bytes()), stream),
                 "predictor frame workspace");
        // (that launch needs every compute unit of the chip at once: not on a stream confined by a CU mask)
        int32_t fits = 0;
        op_check(qm_predictor_frame_fits(stream, &fits), "predictor frame launch residency");
        p->one_launch = fits != 0;
    }
    return p;
}

// Step 0 of capture_step (R17:13597-13854 with rows = 2): the two-row "staged" path — generic linears in the
// talker linear's order, per-head RMSNorm over rows * heads vectors, BHSD transpose / RoPE / cache update and the
// staged causal attention.  o_proj + add and down_proj + add are one launch each (the residual is folded in), gate,
// up and SwiGLU one.
static void predictor_step0(qm_predictor& p, bool sampling) {
    hipStream_t s = p.stream;
    const int rows = 2;
    op_check(qm_linear_rows(p.free_input.u16(), p.projection_weight.data(), p.projection_bias.data(), nullptr, p.hidden_a.u16(),
                            rows, kPredHidden, kOuter, s), "predictor input projection");
    DeviceBuffer* current = &p.hidden_a;
    DeviceBuffer* next = &p.hidden_b;
    for (PredictorLayer& w : p.layers) {
        op_check(qm_rmsnorm_rows(current->u16(), w.input_norm.data(), p.norm.u16(), rows, kPredHidden, kEpsilon, s), "predictor rmsnorm");
        op_check(qm_linear_rows(p.norm.u16(), w.q_weight.data(), nullptr, nullptr, p.q_linear.u16(), rows, kPredQueryDim, kPredHidden, s), "predictor q_proj");
        op_check(qm_linear_rows(p.norm.u16(), w.k_weight.data(), nullptr, nullptr, p.k_linear.u16(), rows, kPredKvDim, kPredHidden, s), "predictor k_proj");
        op_check(qm_linear_rows(p.norm.u16(), w.v_weight.data(), nullptr, nullptr, p.v_linear.u16(), rows, kPredKvDim, kPredHidden, s), "predictor v_proj");
        op_check(qm_rmsnorm_rows(p.q_linear.u16(), w.q_norm.data(), p.q_normed.u16(), rows * kPredQueryHeads, kHeadDim, kEpsilon, s), "predictor q_norm");
        op_check(qm_rmsnorm_rows(p.k_linear.u16(), w.k_norm.data(), p.k_normed.u16(), rows * kPredKvHeads, kHeadDim, kEpsilon, s), "predictor k_norm");
        op_check(qm_predictor_transpose(p.q_normed.u16(), p.q_bhsd.u16(), rows, kPredQueryHeads, s), "predictor transpose");
        op_check(qm_predictor_transpose(p.k_normed.u16(), p.k_bhsd.u16(), rows, kPredKvHeads, s), "predictor transpose");
        op_check(qm_predictor_transpose(p.v_linear.u16(), p.v_bhsd.u16(), rows, kPredKvHeads, s), "predictor transpose");
        op_check(qm_predictor_rope_bhsd(p.q_bhsd.u16(), p.cosine.u16(), p.sine.u16(), p.q_rotated.u16(), rows, kPredQueryHeads, s), "predictor rope");
        op_check(qm_predictor_rope_bhsd(p.k_bhsd.u16(), p.cosine.u16(), p.sine.u16(), p.k_rotated.u16(), rows, kPredKvHeads, s), "predictor rope");
        op_check(qm_predictor_update_cache(p.k_rotated.u16(), w.key_cache.u16(), rows, 0, s), "predictor update_cache");
        op_check(qm_predictor_update_cache(p.v_bhsd.u16(), w.value_cache.u16(), rows, 0, s), "predictor update_cache");
        op_check(qm_predictor_attention_staged(p.q_rotated.u16(), w.key_cache.u16(), w.value_cache.u16(), p.context.u16(), rows, 2, 1, s),
                 "predictor attention");
        op_check(qm_linear_rows(p.context.u16(), w.o_weight.data(), nullptr, current->u16(), p.residual.u16(), rows, kPredHidden,
                                kPredQueryDim, s), "predictor o_proj");
        op_check(qm_rmsnorm_rows(p.residual.u16(), w.post_norm.data(), p.post_norm.u16(), rows, kPredHidden, kEpsilon, s), "predictor post norm");
        op_check(qm_gate_up_swiglu_rows(p.post_norm.u16(), w.gate_weight.data(), w.up_weight.data(), p.swiglu.u16(), rows, kPredHidden,
                                        kPredIntermediate, s), "predictor gate/up");
        op_check(qm_linear_rows(p.swiglu.u16(), w.down_weight.data(), nullptr, p.residual.u16(), next->u16(), rows, kPredHidden,
                                kPredIntermediate, s), "predictor down_proj");
        std::swap(current, next);
    }
    op_check(qm_rmsnorm_rows(current->u16(), p.final_norm.data(), p.norm.u16(), rows, kPredHidden, kEpsilon, s), "predictor final norm");
    op_check(qm_linear_rows(p.norm.u16(), p.heads[0].data(), nullptr, nullptr, p.logits.u16(), rows, kPredVocab, kPredHidden, s), "predictor head");
    int32_t* codes = static_cast<int32_t*>(p.codes.raw());
    op_check(qm_sample_topk(p.logits.u16(), 1, (rows - 1) * kPredVocab, kPredVocab, sampling ? kTopK : 0, kTemperature, p.rng_state,
                            codes + 1, s), "predictor sampler");
    op_check(qm_gather_embedding(p.embeddings[0].data(), kPredVocab, codes, 1, kOuter, p.selected.u16(), p.free_input.u16(), s),
             "predictor embedding gather");
}

// Steps 1..14 of capture_step (rows = 1): the M = 1 operators in the predictor's own summation order; the attention
// over at most 16 keys is the exact-chain kernel (the reference's attention_m1 arithmetic).
static void predictor_step_m1(qm_predictor& p, int step, bool sampling) {
    hipStream_t s = p.stream;
    const int position = step + 1;                     // cache_before, R17:13594-13595
    const uint16_t* cos_row = p.cosine.u16() + position * kHeadDim;
    const uint16_t* sin_row = p.sine.u16() + position * kHeadDim;
    op_check(qm_linear_m1(p.free_input.u16(), p.projection_weight.data(), p.projection_bias.data(), nullptr, p.hidden_a.u16(),
                          kPredHidden, kOuter, s), "predictor input projection");
    DeviceBuffer* current = &p.hidden_a;
    DeviceBuffer* next = &p.hidden_b;
    for (PredictorLayer& w : p.layers) {
        op_check(qm_predictor_rmsnorm_qkv_m1(current->u16(), w.input_norm.data(), kEpsilon, w.q_weight.data(), w.k_weight.data(),
                                             w.v_weight.data(), p.q_linear.u16(), p.k_linear.u16(), p.v_linear.u16(), kPredHidden,
                                             kPredQueryDim, kPredKvDim, s), "predictor qkv_m1");
        op_check(qm_predictor_step_attention_m1(p.q_linear.u16(), p.k_linear.u16(), p.v_linear.u16(), w.q_norm.data(), w.k_norm.data(),
                                                cos_row, sin_row, w.key_cache.u16(), w.value_cache.u16(), p.context.u16(), position,
                                                kEpsilon, s), "predictor qk_norm_rope_cache_m1 + attention_m1");
        op_check(qm_predictor_linear_m1(p.context.u16(), w.o_weight.data(), nullptr, p.attention.u16(), kPredHidden, kPredQueryDim, s),
                 "predictor o_proj");
        op_check(qm_predictor_add_postnorm_gate_up_swiglu_m1(current->u16(), p.attention.u16(), w.post_norm.data(), kEpsilon,
                                                             p.residual.u16(), w.gate_weight.data(), w.up_weight.data(), p.swiglu.u16(),
                                                             kPredHidden, kPredIntermediate, s), "predictor gate/up");
        op_check(qm_predictor_linear_m1(p.swiglu.u16(), w.down_weight.data(), p.residual.u16(), next->u16(), kPredHidden,
                                        kPredIntermediate, s), "predictor down_proj");
        std::swap(current, next);
    }
    // final RMSNorm + this step's head in the talker linear's order, no bias: the fused norm + Q/K/V entry with no K/V rows
    const uint16_t* head = p.heads[static_cast<size_t>(step)].data();
    op_check(qm_rmsnorm_qkv_m1(current->u16(), p.final_norm.data(), kEpsilon, head, nullptr, head, nullptr, head, nullptr, p.logits.u16(),
                               p.logits.u16(), p.logits.u16(), kPredHidden, kPredVocab, 0, s), "predictor head");
    int32_t* codes = static_cast<int32_t*>(p.codes.raw());
    op_check(qm_sample_topk(p.logits.u16(), 1, 0, kPredVocab, sampling ? kTopK : 0, kTemperature, p.rng_state, codes + step + 1, s),
             "predictor sampler");
    op_check(qm_gather_embedding(p.embeddings[static_cast<size_t>(step)].data(), kPredVocab, codes, step + 1, kOuter, p.selected.u16(),
                                 p.free_input.u16(), s), "predictor embedding gather");
}

// run_frame_device (R17:13043-13156): reset of the caches and of the frame's selected embeddings and codes, the
// two input rows, the fifteen steps, the next talker input, and the 64-byte read-back of the frame's sixteen codes.
// What a frame sends back to the host: its codes, the code it started from, the frame kernel's status word.
struct FrameResult {
    int32_t codes[kCodeGroups];
    int32_t code0;
    uint32_t status;
    uint32_t talker_status;     // the talker's status word as of this frame (generation loop), else 0
};

// Queues a frame; `result` is filled when everything queued here has run (the caller waits for the stream, or — with
// `result` in pinned memory — for an event it records right after this returns, and may queue more work meanwhile).
static void predictor_frame_launch(qm_predictor& p, const uint16_t* talker_hidden_device, const int32_t* code0_device,
                                   const uint16_t* context_host, bool sampling, FrameResult* result,
                                   const uint32_t* talker_status_device = nullptr) {
    if (!talker_hidden_device || !code0_device || !context_host || !result) throw ApiError(QM_ERR_NULL, "predictor frame input is null");
    hipStream_t s = p.stream;
    hip_check(hipMemsetAsync(p.frame_state.raw(), 0, p.frame_state.bytes(), s), "predictor caches, selected embeddings and codes reset");
    hip_check(hipMemcpyAsync(p.free_input.raw(), talker_hidden_device, kOuter * 2, hipMemcpyDeviceToDevice, s), "talker hidden copy");
    hip_check(hipMemcpyAsync(p.context_embedding.raw(), context_host, kOuter * 2, hipMemcpyHostToDevice, s), "context embedding upload");
    op_check(qm_predictor_prepare_group0(p.codec0_table.data(), static_cast<int32_t>(p.codec0_table.shape[0]), code0_device, kOuter,
                                         p.free_input.u16(), p.selected.u16(), static_cast<int32_t*>(p.codes.raw()), s),
             "predictor group 0 input");
    int32_t by_operators = 0;
    op_check(qm_get_option(QM_OPT_PREDICTOR_FRAME_OPERATORS, &by_operators), "predictor frame option");
    bool one_launch = p.one_launch && by_operators == 0;
    if (one_launch) {
        // all fifteen steps in one launch (step 0 as two passes of the talker-order chain: same bits as predictor_step0)
        const int32_t rc = qm_predictor_frame_steps(&p.frame, 0, kPredSteps - 1, sampling ? kTopK : 0, kTemperature, p.frame_workspace.raw(),
                                                    static_cast<int64_t>(p.frame_workspace.bytes()), static_cast<uint32_t*>(p.status.raw()), s);
        if (rc == QM_ERR_NO_DEVICE) {
            // the stream cannot hold that launch (nothing of it was queued): operator by operator, now and from now on
            p.one_launch = false;
            one_launch = false;
        } else {
            op_check(rc, "predictor frame steps");
        }
    }
    if (!one_launch) {
        predictor_step0(p, sampling);
        for (int step = 1; step < kPredSteps; ++step) predictor_step_m1(p, step, sampling);
    }
    op_check(qm_predictor_next_talker_input(p.selected.u16(), kCodeGroups, p.context_embedding.u16(), kOuter, p.embedding_sum.u16(),
                                            p.next_input.u16(), s), "next talker input");
    hip_check(hipMemcpyAsync(result->codes, p.codes.raw(), kCodeGroups * sizeof(int32_t), hipMemcpyDeviceToHost, s), "codes read-back");
    hip_check(hipMemcpyAsync(&result->code0, code0_device, sizeof(int32_t), hipMemcpyDeviceToHost, s), "code read-back");
    // (the status word is zero unless the one launch of the frame's steps gave up)
    hip_check(hipMemcpyAsync(&result->status, p.status.raw(), sizeof(uint32_t), hipMemcpyDeviceToHost, s), "status read-back");
    result->talker_status = 0;
    if (talker_status_device)
        hip_check(hipMemcpyAsync(&result->talker_status, talker_status_device, sizeof(uint32_t), hipMemcpyDeviceToHost, s),
                  "talker status read-back");
}

// After the frame has run: a frame kernel that gave up waiting fails the call, and its workspace starts over.
static void predictor_frame_finish(qm_predictor& p, const FrameResult& result) {
    if (result.status == 0) return;
    hipStream_t s = p.stream;
    if (result.status & QM_STATUS_FRAME_TIMEOUT) p.one_launch = false;   // something else holds compute units: operators from now on
    hip_check(hipMemsetAsync(p.status.raw(), 0, sizeof(uint32_t), s), "status reset");
    op_check(qm_predictor_frame_workspace_init(p.frame_workspace.raw(), static_cast<int64_t>(p.frame_workspace.bytes()), s),
             "predictor frame workspace");
    hip_check(hipStreamSynchronize(s), "predictor frame workspace synchronize");
    throw ApiError(QM_ERR_STATUS, "the predictor frame kernel reported status " + std::to_string(result.status));
}

static void predictor_frame(qm_predictor& p, const uint16_t* talker_hidden_device, const int32_t* code0_device,
                            const uint16_t* context_host, bool sampling, int32_t codes_out[16]) {
    if (!codes_out) throw ApiError(QM_ERR_NULL, "predictor frame input is null");
    FrameResult result = {};
    predictor_frame_launch(p, talker_hidden_device, code0_device, context_host, sampling, &result);
    hip_check(hipStreamSynchronize(p.stream), "predictor frame synchronize");
    predictor_frame_finish(p, result);
    std::memcpy(codes_out, result.codes, sizeof result.codes);
}

// Pinned host memory for what the generation loop reads back while more work is queued, and the event it waits for.
struct FrameMailbox {
    FrameResult* result = nullptr;
    hipEvent_t arrived = nullptr;
    FrameMailbox() {
        hip_check(hipHostMalloc(reinterpret_cast<void**>(&result), sizeof(FrameResult), hipHostMallocDefault), "pinned frame result");
        const hipError_t e = hipEventCreateWithFlags(&arrived, hipEventDisableTiming);
        if (e != hipSuccess) {
            (void)hipHostFree(result);
            hip_check(e, "frame event");
        }
    }
    ~FrameMailbox() {
        if (arrived) (void)hipEventDestroy(arrived);
        if (result) (void)hipHostFree(result);
    }
    FrameMailbox(const FrameMailbox&) = delete;
    FrameMailbox& operator=(const FrameMailbox&) = delete;
};

}  // namespace qm_engine

extern "C" int32_t qm_final_head_create(const char* model_dir, int32_t history_capacity, uint64_t seed, void* hip_stream,
                                        qm_final_head** out) {
    if (!model_dir || !out) return QM_ERR_NULL;
    *out = nullptr;
    return guarded([&] { *out = create_final_head(model_dir, history_capacity, seed, static_cast<hipStream_t>(hip_stream)).release(); });
}

extern "C" void qm_final_head_destroy(qm_final_head* head) { delete head; }

extern "C" int32_t qm_final_head_reset(qm_final_head* head, uint64_t seed) {
    if (!head) return QM_ERR_NULL;
    return guarded([&] {
        hip_check(hipMemcpyAsync(head->rng.raw(), &seed, sizeof seed, hipMemcpyHostToDevice, head->stream), "generator seed upload");
        hip_check(hipMemsetAsync(head->history.raw(), 0, head->history.bytes(), head->stream), "history reset");
        hip_check(hipStreamSynchronize(head->stream), "final head reset synchronize");   // `seed` is a stack variable
    });
}

extern "C" int32_t qm_final_head_run(qm_final_head* head, const uint16_t* hidden_device, int32_t frame, int32_t sampling,
                                     int32_t* code_out) {
    if (!head || !hidden_device || !code_out) return QM_ERR_NULL;
    return guarded([&] { *code_out = final_head_run(*head, hidden_device, frame, sampling != 0); });
}

extern "C" uint64_t* qm_final_head_rng_state(qm_final_head* head) { return head ? static_cast<uint64_t*>(head->rng.raw()) : nullptr; }
extern "C" const int32_t* qm_final_head_device_code(qm_final_head* head) { return head ? static_cast<const int32_t*>(head->code.raw()) : nullptr; }

extern "C" int32_t qm_predictor_create(const char* model_dir, uint64_t* rng_state_device, void* hip_stream, qm_predictor** out) {
    if (!model_dir || !out) return QM_ERR_NULL;
    *out = nullptr;
    return guarded([&] { *out = create_predictor(model_dir, rng_state_device, static_cast<hipStream_t>(hip_stream)).release(); });
}

extern "C" void qm_predictor_destroy(qm_predictor* predictor) { delete predictor; }

extern "C" int32_t qm_predictor_run_frame(qm_predictor* predictor, const uint16_t* talker_hidden_device, const int32_t* code0_device,
                                          const uint16_t* context_host, int32_t sampling, int32_t codes_out[16]) {
    if (!predictor) return QM_ERR_NULL;
    return guarded([&] { predictor_frame(*predictor, talker_hidden_device, code0_device, context_host, sampling != 0, codes_out); });
}

extern "C" const uint16_t* qm_predictor_next_input(qm_predictor* predictor) { return predictor ? predictor->next_input.u16() : nullptr; }

extern "C" int32_t qm_generate(qm_talker* talker, qm_final_head* head, qm_predictor* predictor, const uint16_t* prompt_device,
                               int32_t prompt_rows, int32_t maximum_frames, const uint16_t* tts_pad_host,
                               const uint16_t* trailing_text_host, int32_t trailing_rows, int32_t sampling, int32_t* codes_out,
                               int32_t* frames_out, uint64_t* hash_out) {
    if (!talker || !head || !predictor || !prompt_device || !tts_pad_host || !codes_out || !frames_out) return QM_ERR_NULL;
    if (prompt_rows <= 0 || maximum_frames <= 0 || trailing_rows < 0 || (trailing_rows > 0 && !trailing_text_host)) return QM_ERR_ARGUMENT;
    *frames_out = 0;
    if (head->stream != qm_talker_stream(talker) || predictor->stream != qm_talker_stream(talker)) return QM_ERR_ARGUMENT;
    return guarded([&] {
        // prompt pass (generate_codec_sequence, R17:21887-22538, prefill side): RoPE rows of positions 0..rows-1
        std::vector<uint16_t> cosine(static_cast<size_t>(prompt_rows) * kHeadDim), sine(cosine.size());
        op_check(qm_rope_rows(prompt_rows, 0, kHeadDim, 1000000.0, cosine.data(), sine.data()), "prompt rope rows");
        const uint16_t* hidden = nullptr;
        op_check(qm_talker_prefill(talker, prompt_device, cosine.data(), sine.data(), prompt_rows, &hidden), "talker prefill");
        op_check(qm_talker_synchronize(talker), "talker prefill synchronize");     // the rope rows are stack-owned
        // decode rope rows of positions prompt_rows .. (R17:21762)
        const int decode_rows = maximum_frames > 1 ? maximum_frames - 1 : 0;
        std::vector<uint16_t> decode_cos(static_cast<size_t>(decode_rows) * kHeadDim), decode_sin(decode_cos.size());
        if (decode_rows > 0)
            op_check(qm_rope_rows(decode_rows, prompt_rows, kHeadDim, 1000000.0, decode_cos.data(), decode_sin.data()), "decode rope rows");
        // ... uploaded once: a decode step then starts without host-to-device copies in front of it
        DeviceBuffer rope_device(2 * decode_cos.size() * sizeof(uint16_t) + 256);
        uint16_t* const cos_device = rope_device.u16();
        uint16_t* const sin_device = cos_device + decode_cos.size();
        if (decode_rows > 0) {
            hipStream_t stream = static_cast<hipStream_t>(qm_talker_stream(talker));
            hip_check(hipMemcpyAsync(cos_device, decode_cos.data(), decode_cos.size() * 2, hipMemcpyHostToDevice, stream), "decode rope upload");
            hip_check(hipMemcpyAsync(sin_device, decode_sin.data(), decode_sin.size() * 2, hipMemcpyHostToDevice, stream), "decode rope upload");
            hip_check(hipStreamSynchronize(stream), "decode rope upload synchronize");
        }
        // Per frame the host waits ONCE, and not with an idle GPU: the final head's code stays on the device, where the
        // predictor reads it; the frame's codes, that code and the status word come back through pinned memory; and the
        // talker's next step is queued before the host waits for them.  The reference reads the final head's code first
        // and stops before the predictor at the end-of-sequence code (R17:22222-22232); here the frame that follows that
        // code — and the talker step after it — have been queued when it is seen: the frame's codes are dropped and the
        // generator state is put back to where the final head left it, which is what the reference leaves (the extra
        // cache row lies beyond what any later call reads: a generation starts with a prefill).
        FrameMailbox mailbox;
        hipStream_t stream = static_cast<hipStream_t>(qm_talker_stream(talker));
        int frames = 0;
        // (work queued ahead reads the rope rows and writes the mailbox: nothing may unwind past them while it runs)
        try {
            for (int frame = 0; frame < maximum_frames; ++frame) {
                final_head_launch(*head, hidden, frame, sampling != 0);
                hip_check(hipMemcpyAsync(head->rng_after_head.raw(), head->rng.raw(), sizeof(uint64_t), hipMemcpyDeviceToDevice, stream),
                          "generator state snapshot");
                const uint16_t* context = frame < trailing_rows ? trailing_text_host + static_cast<size_t>(frame) * kOuter : tts_pad_host;
                predictor_frame_launch(*predictor, hidden, static_cast<const int32_t*>(head->code.raw()), context, sampling != 0, mailbox.result,
                                       qm_talker_status_device(talker));
                hip_check(hipEventRecord(mailbox.arrived, stream), "frame event record");
                if (frame + 1 < maximum_frames)
                    op_check(qm_talker_decode_device_rope(talker, predictor->next_input.u16(), cos_device + static_cast<size_t>(frame) * kHeadDim,
                                                          sin_device + static_cast<size_t>(frame) * kHeadDim, frame, &hidden), "talker decode");
                hip_check(hipEventSynchronize(mailbox.arrived), "frame boundary synchronize");
                const FrameResult result = *mailbox.result;
                if (result.talker_status != 0) {
                    // a talker kernel flagged this step or an earlier one (a launch that gave up waiting returns at once from
                    // then on, and the frames after it would run on a stale hidden state): stop here; the synchronisation
                    // reports the bits, clears them and sets the hand-off workspace up again
                    (void)hipStreamSynchronize(stream);
                    op_check(qm_talker_synchronize(talker), "talker status during generation");
                    throw ApiError(QM_ERR_STATUS, "talker kernels reported status bits " + std::to_string(result.talker_status));
                }
                predictor_frame_finish(*predictor, result);
                if (result.code0 == kCodecEos && frame >= 2) {
                    hip_check(hipMemcpyAsync(head->rng.raw(), head->rng_after_head.raw(), sizeof(uint64_t), hipMemcpyDeviceToDevice, stream),
                              "generator state restore");
                    break;
                }
                if (result.codes[0] != result.code0) throw ApiError(QM_ERR_ARGUMENT, "native Predictor recurrence output mismatch");
                std::memcpy(codes_out + static_cast<size_t>(frame) * kCodeGroups, result.codes, sizeof result.codes);
                ++frames;
            }
        } catch (...) {
            (void)hipStreamSynchronize(stream);
            throw;
        }
        op_check(qm_talker_synchronize(talker), "generation synchronize");
        *frames_out = frames;
        if (hash_out) *hash_out = qm_fnv1a64(codes_out, static_cast<size_t>(frames) * kCodeGroups * sizeof(int32_t));
    });
}
