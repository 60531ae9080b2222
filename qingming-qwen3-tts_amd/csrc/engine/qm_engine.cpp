// qm_engine.cpp — host-side engine shell: talker weights from safetensors, per-layer KV caches,
// the decode layer loop over the C-ABI operators of libqm_attn, RoPE rows, trajectory hash.
//
// Reference: TalkerWeights (R17:14710-15021), NativeTalkerEngine (buffers R17:16392-16470, request
// reset :16526-16546, decode_device :17097-17262), make_talker_rope (R17:21576-21590), fnv1a64
// (R17:833-842).  The decode step enqueues five launches per layer where the reference enqueues
// eight (the fused operators give the same bits) and nothing else: no allocation, no
// synchronisation, no host read.
#include "../../../include/qm_engine.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "qm_engine_common.hpp"

namespace qm_engine {

struct Layer {
    Param input_norm, q_weight, q_bias, k_weight, k_bias, v_weight, v_bias, q_norm, k_norm, o_weight, o_bias, post_norm,
        gate_weight, up_weight, down_weight;
    DeviceBuffer key_cache, value_cache;
};

}  // namespace qm_engine

struct qm_safefile {
    qm_engine::SafeFile file;
    std::vector<const qm_engine::TensorView*> order;
    explicit qm_safefile(const std::string& path) : file(path) {
        for (const auto& kv : file.tensors()) order.push_back(&kv.second);
    }
};

struct qm_talker {
    std::vector<qm_engine::Layer> layers;
    qm_engine::Param final_norm;
    int q_heads = 0, kv_heads = 0, q_dim = 0, kv_dim = 0, intermediate = 0, max_cache = 0, prefill_length = 0;
    hipStream_t stream = nullptr;
    bool own_stream = false;
    qm_engine::DeviceBuffer hidden_a, hidden_b, q, k, v, q_rotated, context, attention, residual, swiglu, final_hidden,
        cosine, sine, workspace;
    // the prompt pass's row buffers ([rows][...]), allocated by the first prefill for max_cache rows
    qm_engine::DeviceBuffer p_hidden_a, p_hidden_b, p_norm, p_q, p_k, p_v, p_q_rotated, p_k_rotated, p_context, p_residual,
        p_swiglu, p_cosine, p_sine;
    // the prompt pass's key-split workspace (prompts whose attention grid leaves compute units idle), grown on demand
    qm_engine::DeviceBuffer p_split;
    qm_engine::DeviceBuffer p_rows_split;   // partial sums of the prompt pass's linears where they cut their reductions
    // device status word the attention kernels OR their QM_STATUS_* bits into; read at qm_talker_synchronize
    qm_engine::DeviceBuffer status;
    // hand-off words of qm_talker_post_attention_m1 (checkpoints of the geometry it serves)
    qm_engine::DeviceBuffer chain_workspace;
    bool chain_geometry = false;
    // That launch needs every compute unit of the chip at once.  False where the engine's stream cannot give it that
    // (a stream created with a CU mask), and from the first time a launch gave up waiting (something else held compute
    // units): the layers then run operator by operator, which gives the same bits.
    bool chain_usable = false;

    ~qm_talker() {
        if (own_stream && stream) (void)hipStreamDestroy(stream);
    }
};

namespace qm_engine {

static std::string layer_name(int layer, const char* tail) {      // layer_suffix, R17:14633-14638
    return "talker.model.layers." + std::to_string(layer) + "." + tail;
}

static void check_layer(int index, const Layer& w) {               // validate_layer, R17:14968-15008
    const std::vector<int64_t> hidden{kHidden};
    auto rank2 = [](const Param& p) { return p.shape.size() == 2; };
    if (w.input_norm.shape != hidden || w.post_norm.shape != hidden || !rank2(w.q_weight) || !rank2(w.k_weight)
        || !rank2(w.v_weight) || !rank2(w.o_weight) || !rank2(w.gate_weight) || !rank2(w.up_weight) || !rank2(w.down_weight))
        throw TensorError("talker layer geometry/rank mismatch at layer " + std::to_string(index));
    if (w.q_weight.shape[1] != kHidden || w.k_weight.shape[1] != kHidden || w.v_weight.shape[1] != kHidden
        || w.o_weight.shape[0] != kHidden || w.o_weight.shape[1] != w.q_weight.shape[0]
        || w.k_weight.shape[0] != w.v_weight.shape[0] || w.gate_weight.shape[1] != kHidden
        || w.up_weight.shape != w.gate_weight.shape || w.down_weight.shape[0] != kHidden
        || w.down_weight.shape[1] != w.gate_weight.shape[0])
        throw TensorError("talker projection geometry mismatch at layer " + std::to_string(index));
    auto bias_ok = [](const Param& bias, const Param& weight) {
        return !bias.present || (bias.shape.size() == 1 && bias.shape[0] == weight.shape[0]);
    };
    if (!bias_ok(w.q_bias, w.q_weight) || !bias_ok(w.k_bias, w.k_weight) || !bias_ok(w.v_bias, w.v_weight)
        || !bias_ok(w.o_bias, w.o_weight) || w.q_norm.shape != std::vector<int64_t>{kHeadDim}
        || w.k_norm.shape != std::vector<int64_t>{kHeadDim})
        throw TensorError("talker bias/norm geometry mismatch at layer " + std::to_string(index));
}

static std::unique_ptr<qm_talker> create_talker(const std::string& model_dir, int max_cache, hipStream_t stream) {
    if (max_cache <= 0) throw ApiError(QM_ERR_ARGUMENT, "max_cache must be positive");
    ModelDirectory host(model_dir);
    auto engine = std::make_unique<qm_talker>();
    engine->stream = stream;
    if (!stream) {
        hip_check(hipStreamCreateWithFlags(&engine->stream, hipStreamNonBlocking), "generation stream");
        engine->own_stream = true;
    }
    hipStream_t upload = engine->stream;
    StreamDrain drain(upload);             // (uploads read the mapped files: they finish before `host` goes, also on an error)
    auto optional = [&](const std::string& name) {
        const TensorView* t = host.maybe_suffix(name);
        return t ? Param(*t, upload) : Param();
    };
    for (int index = 0;; ++index) {
        const TensorView* input_norm = host.maybe_suffix(layer_name(index, "input_layernorm.weight"));
        if (!input_norm) break;
        Layer w;
        w.input_norm = Param(*input_norm, upload);
        w.q_weight = Param(host.suffix(layer_name(index, "self_attn.q_proj.weight")), upload);
        w.q_bias = optional(layer_name(index, "self_attn.q_proj.bias"));
        w.k_weight = Param(host.suffix(layer_name(index, "self_attn.k_proj.weight")), upload);
        w.k_bias = optional(layer_name(index, "self_attn.k_proj.bias"));
        w.v_weight = Param(host.suffix(layer_name(index, "self_attn.v_proj.weight")), upload);
        w.v_bias = optional(layer_name(index, "self_attn.v_proj.bias"));
        w.q_norm = Param(host.suffix(layer_name(index, "self_attn.q_norm.weight")), upload);
        w.k_norm = Param(host.suffix(layer_name(index, "self_attn.k_norm.weight")), upload);
        w.o_weight = Param(host.suffix(layer_name(index, "self_attn.o_proj.weight")), upload);
        w.o_bias = optional(layer_name(index, "self_attn.o_proj.bias"));
        w.post_norm = Param(host.suffix(layer_name(index, "post_attention_layernorm.weight")), upload);
        w.gate_weight = Param(host.suffix(layer_name(index, "mlp.gate_proj.weight")), upload);
        w.up_weight = Param(host.suffix(layer_name(index, "mlp.up_proj.weight")), upload);
        w.down_weight = Param(host.suffix(layer_name(index, "mlp.down_proj.weight")), upload);
        check_layer(index, w);
        engine->layers.push_back(std::move(w));
    }
    if (engine->layers.empty()) throw TensorError("no talker transformer layers in " + model_dir);
    engine->final_norm = Param(host.suffix("talker.model.norm.weight"), upload);
    if (engine->final_norm.shape != std::vector<int64_t>{kHidden}) throw TensorError("talker final norm geometry mismatch");

    const Layer& first = engine->layers.front();
    engine->q_dim = static_cast<int>(first.q_weight.shape[0]);
    engine->kv_dim = static_cast<int>(first.k_weight.shape[0]);
    engine->intermediate = static_cast<int>(first.gate_weight.shape[0]);
    if (engine->q_dim % kHeadDim || engine->kv_dim % kHeadDim) throw TensorError("invalid talker attention geometry");
    engine->q_heads = engine->q_dim / kHeadDim;
    engine->kv_heads = engine->kv_dim / kHeadDim;
    if (engine->q_heads <= 0 || engine->kv_heads <= 0 || engine->q_heads != 2 * engine->kv_heads)
        throw TensorError("the attention kernels need q_heads == 2 * kv_heads with head_dim 128");
    for (size_t i = 1; i < engine->layers.size(); ++i) {
        const Layer& w = engine->layers[i];
        if (w.q_weight.shape != first.q_weight.shape || w.k_weight.shape != first.k_weight.shape
            || w.gate_weight.shape != first.gate_weight.shape)
            throw TensorError("talker layers differ in geometry at layer " + std::to_string(i));
    }

    engine->max_cache = max_cache;
    const size_t cache_bytes = static_cast<size_t>(engine->kv_heads) * max_cache * kHeadDim * 2;
    for (Layer& w : engine->layers) {
        w.key_cache = DeviceBuffer(cache_bytes);
        w.value_cache = DeviceBuffer(cache_bytes);
    }
    auto vec = [](int n) { return DeviceBuffer(static_cast<size_t>(n) * 2); };
    engine->hidden_a = vec(kHidden); engine->hidden_b = vec(kHidden);
    engine->q = vec(engine->q_dim); engine->k = vec(engine->kv_dim); engine->v = vec(engine->kv_dim);
    engine->q_rotated = vec(engine->q_dim); engine->context = vec(engine->q_dim);
    engine->attention = vec(kHidden); engine->residual = vec(kHidden);
    engine->swiglu = vec(engine->intermediate); engine->final_hidden = vec(kHidden);
    engine->cosine = vec(kHeadDim); engine->sine = vec(kHeadDim);
    engine->workspace = DeviceBuffer(qm_decode_workspace_bytes(1, engine->q_heads, engine->kv_heads, max_cache));
    engine->status = DeviceBuffer(256);
    hip_check(hipMemsetAsync(engine->status.raw(), 0, engine->status.bytes(), engine->stream), "status word reset");
    engine->chain_geometry = engine->q_dim == 2048 && engine->kv_dim == 1024 && engine->intermediate == 6144 && kHidden == 2048;
    if (engine->chain_geometry) {
        int32_t fits = 0;
        op_check(qm_talker_chain_fits(engine->stream, &fits), "talker hand-off launch residency");
        engine->chain_usable = fits != 0;
        engine->chain_workspace = DeviceBuffer(static_cast<size_t>(qm_talker_post_attention_workspace_bytes()));
        op_check(qm_talker_post_attention_workspace_init(engine->chain_workspace.raw(), static_cast<int64_t>(engine->chain_workspace.bytes()),
                                                         engine->stream), "talker hand-off workspace init");
    }
    hip_check(hipStreamSynchronize(upload), "weight upload synchronize");   // the mapped files go away with `host`
    return engine;
}

static void reset_talker(qm_talker& e, int prefill_length) {
    if (prefill_length < 0 || prefill_length > e.max_cache) throw ApiError(QM_ERR_SLOT_RANGE, "prefill length exceeds the cache");
    for (Layer& w : e.layers) {
        hip_check(hipMemsetAsync(w.key_cache.raw(), 0, w.key_cache.bytes(), e.stream), "key cache reset");
        hip_check(hipMemsetAsync(w.value_cache.raw(), 0, w.value_cache.bytes(), e.stream), "value cache reset");
    }
    e.prefill_length = prefill_length;
}

static qm_kv_cache flat_cache_of(const qm_talker& e, const Layer& w) {
    qm_kv_cache cache = {};
    cache.k_pool = w.key_cache.u16();
    cache.v_pool = w.value_cache.u16();
    cache.stride_page = 0;
    cache.stride_head = static_cast<int64_t>(e.max_cache) * kHeadDim;
    cache.stride_token = kHeadDim;
    cache.page_size = e.max_cache;
    cache.n_pages = 1;
    cache.kv_heads = e.kv_heads;
    cache.head_dim = kHeadDim;
    return cache;
}

// `rope_on_device`: cosine and sine are device rows that stay valid until the step has run (a caller that uploaded the
// rows of all its positions once); else host rows, copied into the engine's own.
static const uint16_t* decode(qm_talker& e, const uint16_t* input_device, const uint16_t* cosine, const uint16_t* sine,
                              int decode_index, bool rope_on_device = false) {
    if (!input_device || !cosine || !sine) throw ApiError(QM_ERR_NULL, "talker device decode input is null");
    if (decode_index < 0) throw ApiError(QM_ERR_ARGUMENT, "negative decode index");
    const int position = e.prefill_length + decode_index;
    if (position >= e.max_cache) throw ApiError(QM_ERR_SLOT_RANGE, "talker device decode cache overflow");
    hipStream_t s = e.stream;
    hip_check(hipMemcpyAsync(e.hidden_a.raw(), input_device, kHidden * 2, hipMemcpyDeviceToDevice, s), "decode input copy");
    const uint16_t* cos_row = cosine;
    const uint16_t* sin_row = sine;
    if (!rope_on_device) {
        hip_check(hipMemcpyAsync(e.cosine.raw(), cosine, kHeadDim * 2, hipMemcpyHostToDevice, s), "decode cosine");
        hip_check(hipMemcpyAsync(e.sine.raw(), sine, kHeadDim * 2, hipMemcpyHostToDevice, s), "decode sine");
        cos_row = e.cosine.u16();
        sin_row = e.sine.u16();
    }
    DeviceBuffer* current = &e.hidden_a;
    DeviceBuffer* next = &e.hidden_b;
    // What lies between two attentions — o_proj, residual + post-norm + gate/up/SwiGLU, down_proj + residual and the next
    // layer's RMSNorm + Q/K/V — is one launch where the checkpoint has the geometry that launch serves (same bits).
    int32_t by_operators = 0;
    op_check(qm_get_option(QM_OPT_TALKER_LAYER_OPERATORS, &by_operators), "talker layer option");
    bool chained = e.chain_geometry && e.chain_usable && by_operators != 1;
    bool merge_in_chain = chained && by_operators == 0;   // the attention's split records are combined by the launch that follows it
    bool qkv_ready = false;                               // the layer's Q/K/V were left by the launch of the layer before
    for (size_t index = 0; index < e.layers.size(); ++index) {
        Layer& w = e.layers[index];
        qm_kv_cache cache = flat_cache_of(e, w);
        // launch_rmsnorm + launch_qkv_m1 (R17:17163-17176)
        if (!qkv_ready)
            op_check(qm_rmsnorm_qkv_m1(current->u16(), w.input_norm.data(), kEpsilon, w.q_weight.data(), w.q_bias.data(),
                                       w.k_weight.data(), w.k_bias.data(), w.v_weight.data(), w.v_bias.data(), e.q.u16(),
                                       e.k.u16(), e.v.u16(), kHidden, e.q_dim, e.kv_dim, s),
                     "talker RMSNorm + Q/K/V");
        // launch_qk_norm_rope_cache_m1 + launch_attention (R17:17181-17195)
        if (!merge_in_chain)
            op_check(qm_decode_step_fused(e.q.u16(), e.k.u16(), e.v.u16(), w.q_norm.data(), w.k_norm.data(), cos_row,
                                          sin_row, e.q_rotated.u16(), &cache, nullptr, 1, e.context.u16(), e.q_heads,
                                          position, -1, kScale, kEpsilon, e.workspace.raw(), e.workspace.bytes(),
                                          static_cast<uint32_t*>(e.status.raw()), s),
                     "talker norm/RoPE/append + attention");
        if (chained) {
            qm_talker_post_attention op = {};
            op.context = e.context.u16(); op.hidden = current->u16();
            op.o_weight = w.o_weight.data(); op.o_bias = w.o_bias.data(); op.post_norm = w.post_norm.data();
            op.gate_weight = w.gate_weight.data(); op.up_weight = w.up_weight.data(); op.down_weight = w.down_weight.data();
            op.hidden_out = next->u16();
            if (index + 1 < e.layers.size()) {
                Layer& after = e.layers[index + 1];
                op.next_input_norm = after.input_norm.data();
                op.next_q_weight = after.q_weight.data(); op.next_q_bias = after.q_bias.data();
                op.next_k_weight = after.k_weight.data(); op.next_k_bias = after.k_bias.data();
                op.next_v_weight = after.v_weight.data(); op.next_v_bias = after.v_bias.data();
                op.q_out = e.q.u16(); op.k_out = e.k.u16(); op.v_out = e.v.u16();
            }
            op.hidden_columns = kHidden; op.q_columns = e.q_dim; op.kv_columns = e.kv_dim; op.intermediate_columns = e.intermediate;
            op.epsilon = kEpsilon;
            int32_t rc = QM_OK;
            if (merge_in_chain) {
                qm_talker_layer_step step = {};
                step.q = e.q.u16(); step.k = e.k.u16(); step.v = e.v.u16();
                step.q_norm_w = w.q_norm.data(); step.k_norm_w = w.k_norm.data();
                step.cos_row = cos_row; step.sin_row = sin_row; step.q_rotated_out = e.q_rotated.u16();
                step.cache = &cache; step.page_table = nullptr; step.max_pages = 1;
                step.attention_workspace = e.workspace.raw(); step.attention_workspace_bytes = e.workspace.bytes();
                step.context = e.context.u16();
                step.q_heads = e.q_heads; step.position = position; step.sliding_window = -1;
                step.scale = kScale; step.epsilon = kEpsilon;
                step.post = op;
                rc = qm_talker_layer_step_m1(&step, e.chain_workspace.raw(), static_cast<int64_t>(e.chain_workspace.bytes()),
                                             static_cast<uint32_t*>(e.status.raw()), s);
            } else {
                rc = qm_talker_post_attention_m1(&op, e.chain_workspace.raw(), static_cast<int64_t>(e.chain_workspace.bytes()),
                                                 static_cast<uint32_t*>(e.status.raw()), s);
            }
            if (rc != QM_ERR_NO_DEVICE) {
                op_check(rc, "talker (norm/RoPE/append + attention) o_proj ... next Q/K/V");
                qkv_ready = index + 1 < e.layers.size();
                std::swap(current, next);
                continue;
            }
            // The stream cannot hold that launch (nothing of it has been queued: the call checks before it launches):
            // this layer and the ones after it run operator by operator, and so does every later step.
            e.chain_usable = false;
            chained = false;
            if (merge_in_chain)
                op_check(qm_decode_step_fused(e.q.u16(), e.k.u16(), e.v.u16(), w.q_norm.data(), w.k_norm.data(), cos_row,
                                              sin_row, e.q_rotated.u16(), &cache, nullptr, 1, e.context.u16(), e.q_heads,
                                              position, -1, kScale, kEpsilon, e.workspace.raw(), e.workspace.bytes(),
                                              static_cast<uint32_t*>(e.status.raw()), s),
                         "talker norm/RoPE/append + attention");
            merge_in_chain = false;
        }
        qkv_ready = false;
        // launch_linear_m1: o_proj (R17:17203-17210)
        op_check(qm_linear_m1(e.context.u16(), w.o_weight.data(), w.o_bias.data(), nullptr, e.attention.u16(), kHidden,
                              e.q_dim, s),
                 "talker o_proj");
        // launch_add_postnorm_m1 + launch_gate_up_swiglu_m1 (R17:17215-17229)
        op_check(qm_add_postnorm_gate_up_swiglu_m1(current->u16(), e.attention.u16(), w.post_norm.data(), kEpsilon,
                                                   e.residual.u16(), w.gate_weight.data(), w.up_weight.data(),
                                                   e.swiglu.u16(), kHidden, e.intermediate, s),
                 "talker add + post-norm + gate/up/SwiGLU");
        // launch_linear_m1: down_proj + residual (R17:17236-17244)
        op_check(qm_linear_m1(e.swiglu.u16(), w.down_weight.data(), nullptr, e.residual.u16(), next->u16(), kHidden,
                              e.intermediate, s),
                 "talker down_proj + residual");
        std::swap(current, next);
    }
    op_check(qm_rmsnorm_rows(current->u16(), e.final_norm.data(), e.final_hidden.u16(), 1, kHidden, kEpsilon, s),
             "talker final RMSNorm");
    return e.final_hidden.u16();
}

// NativeTalkerEngine::prefill (R17:16561-16800): the prompt's rows through every layer.  The
// reference's launches per layer and what runs here:
//   rmsnorm                                   -> qm_rmsnorm_rows
//   3 x linear_generic (q, k, v)              -> qm_qkv_rows (every linear through its _split entry: short prompts)
//   2 x rmsnorm + 2 x rope_rows               -> qm_qk_norm_rope_rows (one launch)
//   scatter_prefill_cache + attention         -> qm_prefill_attention_causal_split (writes the cache itself; long
//                                                query tiles of a prompt are shared by two or three blocks)
//   linear_generic (o_proj) + add             -> qm_linear_rows with the residual folded in
//   rmsnorm                                   -> qm_rmsnorm_rows
//   2 x linear_generic + swiglu               -> qm_gate_up_swiglu_rows
//   linear_generic (down) + add               -> qm_linear_rows with the residual folded in
// and the final RMSNorm, of the last row only (the one row the reference reads back).
static const uint16_t* prefill(qm_talker& e, const uint16_t* input_device, const uint16_t* cosine, const uint16_t* sine,
                               int rows) {
    if (!input_device || !cosine || !sine) throw ApiError(QM_ERR_NULL, "talker prefill input is null");
    if (rows <= 0) throw ApiError(QM_ERR_ARGUMENT, "a prompt has at least one row");
    if (rows > e.max_cache) throw ApiError(QM_ERR_SLOT_RANGE, "talker prefill exceeds the cache");
    if (!e.p_hidden_a.raw()) {
        auto rows_of = [&](int width) { return DeviceBuffer(static_cast<size_t>(e.max_cache) * width * 2); };
        e.p_hidden_a = rows_of(kHidden); e.p_hidden_b = rows_of(kHidden); e.p_norm = rows_of(kHidden);
        e.p_q = rows_of(e.q_dim); e.p_k = rows_of(e.kv_dim); e.p_v = rows_of(e.kv_dim);
        e.p_q_rotated = rows_of(e.q_dim); e.p_k_rotated = rows_of(e.kv_dim); e.p_context = rows_of(e.q_dim);
        e.p_residual = rows_of(kHidden); e.p_swiglu = rows_of(e.intermediate);
        e.p_cosine = rows_of(kHeadDim); e.p_sine = rows_of(kHeadDim);
    }
    reset_talker(e, rows);
    hipStream_t s = e.stream;
    const int64_t split_bytes = qm_prefill_split_workspace_bytes(1, rows, e.kv_heads);
    if (split_bytes < 0) op_check(static_cast<int32_t>(split_bytes), "prefill key-split workspace size");
    if (static_cast<size_t>(split_bytes) > e.p_split.bytes()) {
        hip_check(hipStreamSynchronize(s), "prefill workspace growth");   // nothing in flight reads the old one
        e.p_split = DeviceBuffer(static_cast<size_t>(split_bytes));
        op_check(qm_prefill_split_workspace_init(e.p_split.raw(), split_bytes, s), "prefill key-split workspace init");
    }
    // A short prompt leaves most compute units without a block of a linear: with this workspace the linears cut their
    // reductions (qm_linear_rows_split; 0 bytes where a shape is not cut, and then the call is the uncut one).
    int64_t rows_bytes = 0;
    for (const int64_t need : {qm_linear_rows_split_workspace_bytes(rows, e.q_dim, kHidden, 0),
                               qm_linear_rows_split_workspace_bytes(rows, e.kv_dim, kHidden, 0),
                               qm_linear_rows_split_workspace_bytes(rows, kHidden, e.q_dim, 0),
                               qm_linear_rows_split_workspace_bytes(rows, e.intermediate, kHidden, 1),
                               qm_linear_rows_split_workspace_bytes(rows, kHidden, e.intermediate, 0)})
        rows_bytes = std::max(rows_bytes, need);
    if (static_cast<size_t>(rows_bytes) > e.p_rows_split.bytes()) {
        hip_check(hipStreamSynchronize(s), "prefill workspace growth");
        e.p_rows_split = DeviceBuffer(static_cast<size_t>(rows_bytes));
    }
    void* const rows_ws = rows_bytes > 0 ? e.p_rows_split.raw() : nullptr;
    const size_t rope_bytes = static_cast<size_t>(rows) * kHeadDim * 2;
    hip_check(hipMemcpyAsync(e.p_hidden_a.raw(), input_device, static_cast<size_t>(rows) * kHidden * 2,
                             hipMemcpyDeviceToDevice, s), "prefill input copy");
    hip_check(hipMemcpyAsync(e.p_cosine.raw(), cosine, rope_bytes, hipMemcpyHostToDevice, s), "prefill cosine upload");
    hip_check(hipMemcpyAsync(e.p_sine.raw(), sine, rope_bytes, hipMemcpyHostToDevice, s), "prefill sine upload");
    DeviceBuffer* current = &e.p_hidden_a;
    DeviceBuffer* next = &e.p_hidden_b;
    for (Layer& w : e.layers) {
        const qm_kv_cache cache = flat_cache_of(e, w);
        op_check(qm_rmsnorm_rows(current->u16(), w.input_norm.data(), e.p_norm.u16(), rows, kHidden, kEpsilon, s),
                 "prefill input RMSNorm");
        op_check(qm_qkv_rows_split(e.p_norm.u16(), w.q_weight.data(), w.k_weight.data(), w.v_weight.data(), w.q_bias.data(),
                                   w.k_bias.data(), w.v_bias.data(), e.p_q.u16(), e.p_k.u16(), e.p_v.u16(), rows, e.q_dim, e.kv_dim,
                                   kHidden, rows_ws, rows_bytes, s), "prefill q/k/v_proj");
        op_check(qm_qk_norm_rope_rows(e.p_q.u16(), e.p_k.u16(), w.q_norm.data(), w.k_norm.data(), e.p_cosine.u16(), e.p_sine.u16(),
                                      e.p_q_rotated.u16(), e.p_k_rotated.u16(), rows, e.q_heads, e.kv_heads, kEpsilon, s),
                 "prefill q and k norm + RoPE");
        op_check(qm_prefill_attention_causal_split(e.p_q_rotated.u16(), e.p_k_rotated.u16(), e.p_v.u16(), e.p_context.u16(),
                                                   &cache, nullptr, 1, 1, rows, e.q_heads, e.kv_heads, kScale, 0, 0, 0,
                                                   split_bytes > 0 ? e.p_split.raw() : nullptr, split_bytes,
                                                   static_cast<uint32_t*>(e.status.raw()), s),
                 "prefill attention + cache write");
        op_check(qm_linear_rows_split(e.p_context.u16(), w.o_weight.data(), w.o_bias.data(), current->u16(), e.p_residual.u16(),
                                      rows, kHidden, e.q_dim, rows_ws, rows_bytes, s), "prefill o_proj + residual");
        op_check(qm_rmsnorm_rows(e.p_residual.u16(), w.post_norm.data(), e.p_norm.u16(), rows, kHidden, kEpsilon, s),
                 "prefill post-attention RMSNorm");
        op_check(qm_gate_up_swiglu_rows_split(e.p_norm.u16(), w.gate_weight.data(), w.up_weight.data(), e.p_swiglu.u16(), rows,
                                              kHidden, e.intermediate, rows_ws, rows_bytes, s), "prefill gate/up/SwiGLU");
        op_check(qm_linear_rows_split(e.p_swiglu.u16(), w.down_weight.data(), nullptr, e.p_residual.u16(), next->u16(), rows,
                                      kHidden, e.intermediate, rows_ws, rows_bytes, s), "prefill down_proj + residual");
        std::swap(current, next);
    }
    op_check(qm_rmsnorm_rows(current->u16() + static_cast<size_t>(rows - 1) * kHidden, e.final_norm.data(),
                             e.final_hidden.u16(), 1, kHidden, kEpsilon, s), "prefill final RMSNorm");
    return e.final_hidden.u16();
}

}  // namespace qm_engine

using namespace qm_engine;

namespace qm_engine {
std::string& last_error() {
    thread_local std::string text;
    return text;
}
}  // namespace qm_engine

extern "C" const char* qm_engine_last_error(void) { return qm_engine::last_error().c_str(); }

extern "C" uint64_t qm_fnv1a64(const void* data, size_t bytes) {
    const uint8_t* p = static_cast<const uint8_t*>(data);
    uint64_t value = 1469598103934665603ULL;
    for (size_t i = 0; i < bytes; ++i) {
        value ^= p[i];
        value *= 1099511628211ULL;
    }
    return value;
}

static uint16_t to_bf16(float value) {
    uint32_t bits;
    std::memcpy(&bits, &value, sizeof bits);
    if ((bits & 0x7fffffffU) > 0x7f800000U) return static_cast<uint16_t>((bits >> 16) | 0x0040U);
    bits += 0x7fffU + ((bits >> 16) & 1U);
    return static_cast<uint16_t>(bits >> 16);
}

extern "C" int32_t qm_rope_rows(int32_t rows, int32_t start, int32_t head_dim, double theta, uint16_t* cos_out,
                                uint16_t* sin_out) {
    if (!cos_out || !sin_out) return QM_ERR_NULL;
    if (rows < 0 || start < 0 || head_dim <= 0 || (head_dim & 1)) return QM_ERR_GEOMETRY;
    const int half = head_dim / 2;
    for (int row = 0; row < rows; ++row) {
        const double position = static_cast<double>(start + row);
        for (int i = 0; i < half; ++i) {
            const double inverse = std::pow(theta, -2.0 * static_cast<double>(i) / static_cast<double>(head_dim));
            const double angle = position * inverse;
            const uint16_t c = to_bf16(static_cast<float>(std::cos(angle)));
            const uint16_t s = to_bf16(static_cast<float>(std::sin(angle)));
            const size_t base = static_cast<size_t>(row) * head_dim;
            cos_out[base + i] = cos_out[base + i + half] = c;
            sin_out[base + i] = sin_out[base + i + half] = s;
        }
    }
    return QM_OK;
}

extern "C" int32_t qm_safefile_open(const char* path, qm_safefile** out) {
    if (!path || !out) return QM_ERR_NULL;
    *out = nullptr;
    return guarded([&] { *out = new qm_safefile(path); });
}

extern "C" void qm_safefile_close(qm_safefile* file) { delete file; }

extern "C" int32_t qm_safefile_count(const qm_safefile* file) { return file ? static_cast<int32_t>(file->order.size()) : 0; }

extern "C" int32_t qm_safefile_tensor(const qm_safefile* file, int32_t index, const char** name, const char** dtype,
                                      int32_t* rank, int64_t* shape, const void** data, uint64_t* bytes) {
    if (!file) return QM_ERR_NULL;
    if (index < 0 || index >= static_cast<int32_t>(file->order.size())) return QM_ERR_ARGUMENT;
    const TensorView& t = *file->order[static_cast<size_t>(index)];
    if (t.shape.size() > 8) return QM_ERR_GEOMETRY;
    if (name) *name = t.name.c_str();
    if (dtype) *dtype = t.dtype.c_str();
    if (rank) *rank = static_cast<int32_t>(t.shape.size());
    if (shape) for (size_t i = 0; i < t.shape.size(); ++i) shape[i] = t.shape[i];
    if (data) *data = t.data;
    if (bytes) *bytes = t.bytes;
    return QM_OK;
}

extern "C" int32_t qm_talker_create(const char* model_dir, int32_t max_cache, void* hip_stream, qm_talker** out) {
    if (!model_dir || !out) return QM_ERR_NULL;
    *out = nullptr;
    return guarded([&] { *out = create_talker(model_dir, max_cache, static_cast<hipStream_t>(hip_stream)).release(); });
}

extern "C" void qm_talker_destroy(qm_talker* engine) { delete engine; }

extern "C" int32_t qm_talker_info(const qm_talker* e, int32_t info[7]) {
    if (!e || !info) return QM_ERR_NULL;
    info[0] = static_cast<int32_t>(e->layers.size());
    info[1] = e->q_heads; info[2] = e->kv_heads; info[3] = e->q_dim; info[4] = e->kv_dim;
    info[5] = e->intermediate; info[6] = e->max_cache;
    return QM_OK;
}

extern "C" int32_t qm_talker_reset(qm_talker* engine, int32_t prefill_length) {
    if (!engine) return QM_ERR_NULL;
    return guarded([&] { reset_talker(*engine, prefill_length); });
}

extern "C" int32_t qm_talker_cache(qm_talker* engine, int32_t layer, uint16_t** key_cache, uint16_t** value_cache) {
    if (!engine || !key_cache || !value_cache) return QM_ERR_NULL;
    if (layer < 0 || layer >= static_cast<int32_t>(engine->layers.size())) return QM_ERR_ARGUMENT;
    *key_cache = engine->layers[static_cast<size_t>(layer)].key_cache.u16();
    *value_cache = engine->layers[static_cast<size_t>(layer)].value_cache.u16();
    return QM_OK;
}

extern "C" int32_t qm_talker_decode(qm_talker* engine, const uint16_t* input_device, const uint16_t* cosine,
                                    const uint16_t* sine, int32_t decode_index, const uint16_t** final_hidden_device) {
    if (!engine || !final_hidden_device) return QM_ERR_NULL;
    return guarded([&] { *final_hidden_device = decode(*engine, input_device, cosine, sine, decode_index); });
}

extern "C" int32_t qm_talker_decode_device_rope(qm_talker* engine, const uint16_t* input_device, const uint16_t* cosine_device,
                                                const uint16_t* sine_device, int32_t decode_index,
                                                const uint16_t** final_hidden_device) {
    if (!engine || !final_hidden_device) return QM_ERR_NULL;
    return guarded([&] { *final_hidden_device = decode(*engine, input_device, cosine_device, sine_device, decode_index, true); });
}

extern "C" int32_t qm_talker_prefill(qm_talker* engine, const uint16_t* input_device, const uint16_t* cosine,
                                     const uint16_t* sine, int32_t rows, const uint16_t** final_hidden_device) {
    if (!engine || !final_hidden_device) return QM_ERR_NULL;
    return guarded([&] { *final_hidden_device = prefill(*engine, input_device, cosine, sine, rows); });
}

extern "C" void* qm_talker_stream(qm_talker* engine) { return engine ? engine->stream : nullptr; }

extern "C" const uint32_t* qm_talker_status_device(qm_talker* engine) {
    return engine ? static_cast<const uint32_t*>(engine->status.raw()) : nullptr;
}

extern "C" int32_t qm_talker_synchronize(qm_talker* engine) {
    if (!engine) return QM_ERR_NULL;
    return guarded([&] {
        hip_check(hipStreamSynchronize(engine->stream), "generation stream synchronize");
        // What the kernels flagged since the last synchronisation (a page or position out of range, a key-split
        // block that gave up waiting for its partner): the results are not to be used.
        uint32_t bits = 0;
        hip_check(hipMemcpy(&bits, engine->status.raw(), sizeof bits, hipMemcpyDeviceToHost), "status word read");
        if (bits != 0) {
            hip_check(hipMemset(engine->status.raw(), 0, sizeof bits), "status word reset");
            if ((bits & QM_STATUS_SPLIT_TIMEOUT) && engine->p_split.raw())
                op_check(qm_prefill_split_workspace_init(engine->p_split.raw(), static_cast<int64_t>(engine->p_split.bytes()),
                                                         engine->stream), "prefill key-split workspace init");
            if (bits & QM_STATUS_FRAME_TIMEOUT) engine->chain_usable = false;   // something else holds compute units: operators from now on
            if ((bits & QM_STATUS_FRAME_TIMEOUT) && engine->chain_workspace.raw())
                op_check(qm_talker_post_attention_workspace_init(engine->chain_workspace.raw(),
                                                                 static_cast<int64_t>(engine->chain_workspace.bytes()), engine->stream),
                         "talker hand-off workspace init");
            throw ApiError(QM_ERR_STATUS, "talker kernels reported status bits " + std::to_string(bits));
        }
    });
}
