"""ctypes binding of lib/libqm_attn.so.

Arguments are raw device addresses (int) or objects with `.data_ptr()` (torch tensors);
nothing here touches tensor contents on the host.  There is deliberately no fallback: if
the library is absent, `lib()` raises.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(HERE, "lib", "libqm_attn.so")

SCALE_128 = 0.08838834764831845  # 1/sqrt(128), bit pattern 0x3db504f3 (R17:9354-9356)


class QmError(RuntimeError):
    """A C-ABI call returned a negative code (the reference throws std::runtime_error)."""

    def __init__(self, code, what):
        self.code = code
        super().__init__(f"{what}: {error_string(code)} ({code})")


class KvCache(C.Structure):
    """Mirror of qm_kv_cache (include/qm_attn.h)."""
    _fields_ = [
        ("k_pool", C.c_void_p), ("v_pool", C.c_void_p),
        ("stride_page", C.c_int64), ("stride_head", C.c_int64), ("stride_token", C.c_int64),
        ("page_size", C.c_int32), ("n_pages", C.c_int32),
        ("kv_heads", C.c_int32), ("head_dim", C.c_int32),
    ]


class PredictorFrameLayer(C.Structure):
    """Mirror of qm_predictor_frame_layer (include/qm_attn.h)."""
    _fields_ = [(name, C.c_void_p) for name in (
        "input_norm", "q_weight", "k_weight", "v_weight", "q_norm", "k_norm", "o_weight", "post_norm",
        "gate_weight", "up_weight", "down_weight", "key_cache", "value_cache")]


class PredictorFrame(C.Structure):
    """Mirror of qm_predictor_frame (include/qm_attn.h)."""
    _fields_ = [
        ("layers", PredictorFrameLayer * 5),
        ("projection_weight", C.c_void_p), ("projection_bias", C.c_void_p), ("final_norm", C.c_void_p),
        ("heads", C.c_void_p * 15), ("embeddings", C.c_void_p * 15),
        ("cosine", C.c_void_p), ("sine", C.c_void_p),
        ("free_input", C.c_void_p), ("selected", C.c_void_p), ("codes", C.c_void_p), ("rng_state", C.c_void_p),
        ("epsilon", C.c_float),
        ("step0_input", C.c_void_p),
        ("projected", C.c_void_p * 15),
    ]


class TalkerPostAttention(C.Structure):
    """Mirror of qm_talker_post_attention (include/qm_attn.h)."""
    _fields_ = [(name, C.c_void_p) for name in (
        "context", "hidden", "o_weight", "o_bias", "post_norm", "gate_weight", "up_weight", "down_weight", "hidden_out",
        "next_input_norm", "next_q_weight", "next_q_bias", "next_k_weight", "next_k_bias", "next_v_weight", "next_v_bias",
        "q_out", "k_out", "v_out")] + [
        ("hidden_columns", C.c_int32), ("q_columns", C.c_int32), ("kv_columns", C.c_int32),
        ("intermediate_columns", C.c_int32), ("epsilon", C.c_float)]


class TalkerLayerStep(C.Structure):
    """Mirror of qm_talker_layer_step (include/qm_attn.h)."""
    _fields_ = [(name, C.c_void_p) for name in ("q", "k", "v", "q_norm_w", "k_norm_w", "cos_row", "sin_row", "q_rotated_out")] + [
        ("cache", C.POINTER(KvCache)), ("page_table", C.c_void_p), ("attention_workspace", C.c_void_p),
        ("attention_workspace_bytes", C.c_size_t), ("context", C.c_void_p),
        ("max_pages", C.c_int32), ("q_heads", C.c_int32), ("position", C.c_int32), ("sliding_window", C.c_int32),
        ("scale", C.c_float), ("epsilon", C.c_float), ("post", TalkerPostAttention)]


def lib_path():
    return _LIB_PATH


_lib = None

_PTR = C.c_void_p
_I32 = C.c_int32
_F32 = C.c_float

_SIGNATURES = {
    "qm_abi_version": (C.c_int32, []),
    "qm_selftest_bf16_rounding": (C.c_int32, [C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]),
    "qm_error_string": (C.c_char_p, [_I32]),
    "qm_target_arch": (C.c_char_p, []),
    "qm_set_option": (_I32, [_I32, _I32]),
    "qm_get_option": (_I32, [_I32, C.POINTER(_I32)]),
    "qm_qk_norm_rope_kv_append": (_I32, [_PTR] * 8 + [C.POINTER(KvCache), _PTR, _I32, _I32, _I32, _F32, _PTR]),
    "qm_qk_norm_rope_kv_append_ragged": (_I32, [_PTR] * 7 + [_I32, _PTR, C.POINTER(KvCache), _PTR, _I32, _PTR,
                                                 _I32, _I32, _F32, _PTR, _PTR]),
    "qm_decode_workspace_bytes": (C.c_size_t, [_I32, _I32, _I32, _I32]),
    "qm_decode_attention": (_I32, [_PTR, C.POINTER(KvCache), _PTR, _I32, _PTR, _I32, _I32, _I32, _F32,
                                   _PTR, C.c_size_t, _PTR]),
    "qm_decode_step_fused": (_I32, [_PTR] * 8 + [C.POINTER(KvCache), _PTR, _I32, _PTR, _I32, _I32, _I32, _F32, _F32,
                                    _PTR, C.c_size_t, _PTR, _PTR]),
    "qm_decode_attention_ragged": (_I32, [_PTR, C.POINTER(KvCache), _PTR, _I32, _PTR, _I32, _I32, _PTR, _I32,
                                          _F32, _PTR, C.c_size_t, _PTR, _PTR]),
    "qm_decode_attention_ragged_static": (_I32, [_PTR, C.POINTER(KvCache), _PTR, _I32, _PTR, _I32, _I32, _PTR, _I32,
                                                 _F32, _PTR, _PTR]),
    "qm_prefill_chunk_workspace_bytes": (C.c_int64, [_I32, _I32, _I32, _I32]),
    "qm_prefill_attention_chunk": (_I32, [_PTR] * 4 + [_I32, _I32, _I32, _I32, _I32, _F32, C.c_int64, C.c_int64, C.c_int64,
                                          _PTR, C.c_int64, _PTR]),
    "qm_prefill_attention_chunk_paged": (_I32, [_PTR, C.POINTER(KvCache), _PTR, _I32, _PTR, _I32, _I32, _I32, _I32, _I32, _F32,
                                                _PTR, C.c_int64, _PTR, _PTR]),
    "qm_attention_rows_workspace_bytes": (C.c_size_t, [_I32, _I32, _I32, _I32]),
    "qm_attention_rows": (_I32, [_PTR, C.POINTER(KvCache), _PTR, _I32, _PTR, _I32, _I32, _I32, _I32, _F32,
                                 _PTR, C.c_size_t, _PTR, _PTR]),
    "qm_norm_rope_rows": (_I32, [_PTR] * 5 + [_I32, _I32, _F32, _PTR]),
    "qm_qk_norm_rope_rows": (_I32, [_PTR] * 8 + [_I32, _I32, _I32, _F32, _PTR]),
    "qm_scatter_kv": (_I32, [_PTR, _PTR, C.POINTER(KvCache), _PTR, _I32, _I32, _I32, _PTR, _PTR]),
    "qm_prefill_attention_causal": (_I32, [_PTR] * 4 + [C.POINTER(KvCache), _PTR, _I32, _I32, _I32, _I32, _I32,
                                           _F32, C.c_int64, C.c_int64, C.c_int64, _PTR, _PTR]),
    "qm_prefill_split_workspace_bytes": (C.c_int64, [_I32, _I32, _I32]),
    "qm_prefill_split_workspace_init": (_I32, [_PTR, C.c_int64, _PTR]),
    "qm_prefill_attention_causal_split": (_I32, [_PTR] * 4 + [C.POINTER(KvCache), _PTR, _I32, _I32, _I32, _I32, _I32,
                                                 _F32, C.c_int64, C.c_int64, C.c_int64, _PTR, C.c_int64, _PTR, _PTR]),
    "qm_predictor_attention_loop": (_I32, [_PTR] * 10 + [_I32, _I32, _I32, _I32, _F32, _PTR]),
    "qm_predictor_attention_staged": (_I32, [_PTR] * 4 + [_I32, _I32, _I32, _PTR]),
    "qm_predictor_step_attention_m1": (_I32, [_PTR] * 10 + [_I32, _F32, _PTR]),
    "qm_set_thread_option": (_I32, [_I32, _I32]),
    "qm_predictor_frame_workspace_bytes": (C.c_int64, []),
    "qm_predictor_frame_workspace_init": (_I32, [_PTR, C.c_int64, _PTR]),
    "qm_predictor_frame_fits": (_I32, [_PTR, C.POINTER(C.c_int32)]),
    "qm_talker_chain_fits": (_I32, [_PTR, C.POINTER(C.c_int32)]),
    "qm_predictor_frame_steps": (_I32, [C.POINTER(PredictorFrame), _I32, _I32, _I32, _F32, _PTR, C.c_int64, _PTR, _PTR]),
    "qm_talker_post_attention_workspace_bytes": (C.c_int64, []),
    "qm_talker_post_attention_workspace_init": (_I32, [_PTR, C.c_int64, _PTR]),
    "qm_talker_post_attention_m1": (_I32, [C.POINTER(TalkerPostAttention), _PTR, C.c_int64, _PTR, _PTR]),
    "qm_talker_layer_step_m1": (_I32, [C.POINTER(TalkerLayerStep), _PTR, C.c_int64, _PTR, _PTR]),
    "qm_predictor_transpose": (_I32, [_PTR, _PTR, _I32, _I32, _PTR]),
    "qm_predictor_rope_bhsd": (_I32, [_PTR] * 4 + [_I32, _I32, _PTR]),
    "qm_predictor_update_cache": (_I32, [_PTR, _PTR, _I32, _I32, _PTR]),
    "qm_linear_m1": (_I32, [_PTR] * 5 + [_I32, _I32, _PTR]),
    "qm_qkv_m1": (_I32, [_PTR] * 10 + [_I32, _I32, _I32, _PTR]),
    "qm_gate_up_swiglu_m1": (_I32, [_PTR] * 4 + [_I32, _I32, _PTR]),
    "qm_rmsnorm_rows": (_I32, [_PTR] * 3 + [_I32, _I32, _F32, _PTR]),
    "qm_add_postnorm_m1": (_I32, [_PTR] * 5 + [_I32, _F32, _PTR]),
    "qm_rmsnorm_qkv_m1": (_I32, [_PTR, _PTR, _F32] + [_PTR] * 9 + [_I32, _I32, _I32, _PTR]),
    "qm_add_postnorm_gate_up_swiglu_m1": (_I32, [_PTR, _PTR, _PTR, _F32] + [_PTR] * 4 + [_I32, _I32, _PTR]),
    "qm_predictor_linear_m1": (_I32, [_PTR] * 4 + [_I32, _I32, _PTR]),
    "qm_predictor_qkv_m1": (_I32, [_PTR] * 7 + [_I32, _I32, _I32, _PTR]),
    "qm_predictor_gate_up_swiglu_m1": (_I32, [_PTR] * 4 + [_I32, _I32, _PTR]),
    "qm_predictor_rmsnorm_qkv_m1": (_I32, [_PTR, _PTR, _F32] + [_PTR] * 6 + [_I32, _I32, _I32, _PTR]),
    "qm_predictor_add_postnorm_gate_up_swiglu_m1": (_I32, [_PTR, _PTR, _PTR, _F32] + [_PTR] * 4 + [_I32, _I32, _PTR]),
    "qm_sample_topk": (_I32, [_PTR, _I32, _I32, _I32, _I32, _F32, _PTR, _PTR, _PTR]),
    "qm_final_head_process": (_I32, [_PTR, _PTR, _I32, _I32, _I32, _I32, _I32, _F32, _PTR, _PTR]),
    "qm_final_head_sample": (_I32, [_PTR, _PTR, _I32, _I32, _I32, _I32, _F32, _I32, _F32, _PTR, _PTR, _PTR, _PTR]),
    "qm_gather_embedding": (_I32, [_PTR, _I32, _PTR, _I32, _I32, _PTR, _PTR, _PTR]),
    "qm_predictor_prepare_group0": (_I32, [_PTR, _I32, _PTR, _I32, _PTR, _PTR, _PTR, _PTR]),
    "qm_predictor_next_talker_input": (_I32, [_PTR, _I32, _PTR, _I32, _PTR, _PTR, _PTR]),
    "qm_linear_rows": (_I32, [_PTR] * 5 + [_I32, _I32, _I32, _PTR]),
    "qm_gate_up_swiglu_rows": (_I32, [_PTR] * 4 + [_I32, _I32, _I32, _PTR]),
    "qm_linear_rows_split_workspace_bytes": (C.c_int64, [_I32, _I32, _I32, _I32]),
    "qm_linear_rows_split": (_I32, [_PTR] * 5 + [_I32, _I32, _I32, _PTR, C.c_int64, _PTR]),
    "qm_gate_up_swiglu_rows_split": (_I32, [_PTR] * 4 + [_I32, _I32, _I32, _PTR, C.c_int64, _PTR]),
    "qm_qkv_rows": (_I32, [_PTR] * 10 + [_I32, _I32, _I32, _I32, _PTR]),
    "qm_qkv_rows_split": (_I32, [_PTR] * 10 + [_I32, _I32, _I32, _I32, _PTR, C.c_int64, _PTR]),
}

EXPORTS = tuple(_SIGNATURES)


def lib():
    """Loads the shared library (once).  Raises FileNotFoundError if it was not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise FileNotFoundError(
                f"{_LIB_PATH} is missing: build it with `python qingming-qwen3-tts_amd/build.py` "
                "(there is no CPU fallback)")
        handle = C.CDLL(_LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def error_string(code):
    return lib().qm_error_string(code).decode()


def _addr(x):
    if x is None:
        return None
    if isinstance(x, int):
        return x
    return x.data_ptr()


def _check(code, what):
    if code != 0:
        raise QmError(code, what)


OPT_PREFILL_SCORE_ROUNDING = 0
OPT_DECODE_TILES_PER_BLOCK = 1
OPT_PREFILL_KERNEL = 2
OPT_DECODE_STREAMING_LOADS = 3
OPT_PREDICTOR_LOOP_KERNEL = 4
OPT_PREDICTOR_FRAME_OPERATORS = 5
OPT_PREDICTOR_FRAME_SPIN_LIMIT = 6
OPT_LINEAR_ROWS_KERNEL = 7
OPT_TALKER_LAYER_OPERATORS = 8


def set_option(option, value):
    _check(lib().qm_set_option(option, value), "qm_set_option")


def set_thread_option(option, value):
    """The option for calls made by this thread only; -1 removes the thread's own value."""
    _check(lib().qm_set_thread_option(option, value), "qm_set_thread_option")


def get_option(option):
    out = C.c_int32(0)
    _check(lib().qm_get_option(option, C.byref(out)), "qm_get_option")
    return out.value


def paged_cache(k_pool, v_pool, n_pages, kv_heads=8, page_size=16):
    """Descriptor of the native [page][kv_head][page_size][128] layout."""
    return KvCache(_addr(k_pool), _addr(v_pool), kv_heads * page_size * 128, page_size * 128, 128,
                   page_size, n_pages, kv_heads, 128)


def flat_cache(key_cache, value_cache, kv_heads, max_cache):
    """Descriptor of the reference LayerCache [kv_head][max_cache][128] (R17:16371-16390)."""
    return KvCache(_addr(key_cache), _addr(value_cache), 0, max_cache * 128, 128, max_cache, 1,
                   kv_heads, 128)


def qk_norm_rope_kv_append(q, k, v, gq, gk, cos, sin, q_rot, cache, page_table, max_pages, q_heads,
                           position, eps=1e-6, stream=0):
    _check(lib().qm_qk_norm_rope_kv_append(
        _addr(q), _addr(k), _addr(v), _addr(gq), _addr(gk), _addr(cos), _addr(sin), _addr(q_rot),
        C.byref(cache), _addr(page_table), max_pages, q_heads, position, eps, stream),
        "qm_qk_norm_rope_kv_append")


def qk_norm_rope_kv_append_ragged(q, k, v, gq, gk, cos, sin, by_position, q_rot, cache, page_table,
                                  max_pages, positions, n_streams, q_heads, eps=1e-6, status=None,
                                  stream=0):
    _check(lib().qm_qk_norm_rope_kv_append_ragged(
        _addr(q), _addr(k), _addr(v), _addr(gq), _addr(gk), _addr(cos), _addr(sin), int(by_position),
        _addr(q_rot), C.byref(cache), _addr(page_table), max_pages, _addr(positions), n_streams,
        q_heads, eps, _addr(status), stream), "qm_qk_norm_rope_kv_append_ragged")


def decode_workspace_bytes(n_streams, q_heads, kv_heads, max_seq_len):
    return lib().qm_decode_workspace_bytes(n_streams, q_heads, kv_heads, max_seq_len)


def decode_attention(query, cache, page_table, max_pages, out, q_heads, cache_before,
                     sliding_window=-1, scale=SCALE_128, workspace=None, workspace_bytes=0, stream=0):
    _check(lib().qm_decode_attention(
        _addr(query), C.byref(cache), _addr(page_table), max_pages, _addr(out), q_heads, cache_before,
        sliding_window, scale, _addr(workspace), workspace_bytes, stream), "qm_decode_attention")


def decode_step_fused(q, k, v, gq, gk, cos, sin, q_rot, cache, page_table, max_pages, out, q_heads, position,
                      sliding_window, scale, eps, workspace, workspace_bytes, status=None, stream=0):
    _check(lib().qm_decode_step_fused(
        _addr(q), _addr(k), _addr(v), _addr(gq), _addr(gk), _addr(cos), _addr(sin), _addr(q_rot),
        C.byref(cache), _addr(page_table), max_pages, _addr(out), q_heads, position, sliding_window, scale, eps,
        _addr(workspace), workspace_bytes, _addr(status), stream), "qm_decode_step_fused")


def decode_attention_ragged(query, cache, page_table, max_pages, seq_lens, n_streams, max_seq_len, out,
                            q_heads, scale=SCALE_128, workspace=None, workspace_bytes=0, status=None,
                            stream=0):
    _check(lib().qm_decode_attention_ragged(
        _addr(query), C.byref(cache), _addr(page_table), max_pages, _addr(seq_lens), n_streams,
        max_seq_len, _addr(out), q_heads, scale, _addr(workspace), workspace_bytes, _addr(status),
        stream), "qm_decode_attention_ragged")


def prefill_chunk_workspace_bytes(batch, rows, cache_before, kv_heads):
    n = lib().qm_prefill_chunk_workspace_bytes(batch, rows, cache_before, kv_heads)
    if n < 0:
        _check(n, "qm_prefill_chunk_workspace_bytes")
    return n


def prefill_attention_chunk(query, key, value, out, batch, rows, cache_before, q_heads, kv_heads, scale=SCALE_128,
                            stream=0, kv_strides=(0, 0, 0), workspace=None, workspace_bytes=0):
    _check(lib().qm_prefill_attention_chunk(
        _addr(query), _addr(key), _addr(value), _addr(out), batch, rows, cache_before, q_heads, kv_heads, scale,
        kv_strides[0], kv_strides[1], kv_strides[2], _addr(workspace), workspace_bytes, stream), "qm_prefill_attention_chunk")


def prefill_attention_chunk_paged(query, cache, page_table, max_pages, out, batch, rows, cache_before, q_heads, kv_heads,
                                  scale=SCALE_128, workspace=None, workspace_bytes=0, status=None, stream=0):
    _check(lib().qm_prefill_attention_chunk_paged(
        _addr(query), C.byref(cache), _addr(page_table), max_pages, _addr(out), batch, rows, cache_before, q_heads, kv_heads,
        scale, _addr(workspace), workspace_bytes, _addr(status), stream), "qm_prefill_attention_chunk_paged")


def attention_rows_workspace_bytes(query_length, q_heads, kv_heads, key_end):
    return lib().qm_attention_rows_workspace_bytes(query_length, q_heads, kv_heads, key_end)


def attention_rows(query, cache, page_table, max_pages, out, query_length, cache_before, q_heads, sliding_window=-1,
                   scale=SCALE_128, workspace=None, workspace_bytes=0, status=None, stream=0):
    _check(lib().qm_attention_rows(
        _addr(query), C.byref(cache), _addr(page_table), max_pages, _addr(out), query_length, cache_before, q_heads,
        sliding_window, scale, _addr(workspace), workspace_bytes, _addr(status), stream), "qm_attention_rows")


def norm_rope_rows(x, norm_w, cos, sin, out, rows, heads, eps=1e-6, stream=0):
    _check(lib().qm_norm_rope_rows(_addr(x), _addr(norm_w), _addr(cos), _addr(sin), _addr(out), rows,
                                   heads, eps, stream), "qm_norm_rope_rows")


def qk_norm_rope_rows(q, k, q_norm_w, k_norm_w, cos, sin, q_out, k_out, rows, q_heads, kv_heads, eps=1e-6, stream=0):
    _check(lib().qm_qk_norm_rope_rows(_addr(q), _addr(k), _addr(q_norm_w), _addr(k_norm_w), _addr(cos), _addr(sin), _addr(q_out),
                                      _addr(k_out), rows, q_heads, kv_heads, eps, stream), "qm_qk_norm_rope_rows")


def scatter_kv(key, value, cache, page_table, max_pages, rows, first_position, status=None, stream=0):
    _check(lib().qm_scatter_kv(_addr(key), _addr(value), C.byref(cache), _addr(page_table), max_pages,
                               rows, first_position, _addr(status), stream), "qm_scatter_kv")


def prefill_attention_causal(query, key, value, out, cache, page_table, max_pages, batch, seq, q_heads,
                             kv_heads, scale=SCALE_128, status=None, stream=0, kv_strides=(0, 0, 0)):
    _check(lib().qm_prefill_attention_causal(
        _addr(query), _addr(key), _addr(value), _addr(out),
        C.byref(cache) if cache is not None else None, _addr(page_table), max_pages, batch, seq,
        q_heads, kv_heads, scale, kv_strides[0], kv_strides[1], kv_strides[2], _addr(status), stream),
        "qm_prefill_attention_causal")


def prefill_split_workspace_bytes(batch, seq, kv_heads):
    """Bytes of workspace with which prefill_attention_causal_split shares long query tiles between
    two blocks on the current device; 0 when that shape would not split."""
    n = lib().qm_prefill_split_workspace_bytes(batch, seq, kv_heads)
    if n < 0:
        _check(int(n), "qm_prefill_split_workspace_bytes")
    return int(n)


def prefill_split_workspace_init(workspace, workspace_bytes, stream=0):
    _check(lib().qm_prefill_split_workspace_init(_addr(workspace), workspace_bytes, stream),
           "qm_prefill_split_workspace_init")


def prefill_attention_causal_split(query, key, value, out, cache, page_table, max_pages, batch, seq, q_heads,
                                   kv_heads, workspace, workspace_bytes, scale=SCALE_128, status=None, stream=0,
                                   kv_strides=(0, 0, 0)):
    _check(lib().qm_prefill_attention_causal_split(
        _addr(query), _addr(key), _addr(value), _addr(out),
        C.byref(cache) if cache is not None else None, _addr(page_table), max_pages, batch, seq,
        q_heads, kv_heads, scale, kv_strides[0], kv_strides[1], kv_strides[2], _addr(workspace), workspace_bytes,
        _addr(status), stream),
        "qm_prefill_attention_causal_split")


def predictor_attention_loop(q, k, v, gq, gk, cos, sin, out, k_cache_out, v_cache_out, units, n_layers,
                             rows, first_rows=1, eps=1e-6, stream=0):
    _check(lib().qm_predictor_attention_loop(
        _addr(q), _addr(k), _addr(v), _addr(gq), _addr(gk), _addr(cos), _addr(sin), _addr(out),
        _addr(k_cache_out), _addr(v_cache_out), units, n_layers, rows, first_rows, eps, stream),
        "qm_predictor_attention_loop")


def linear_m1(x, weight, bias, residual, out, output_columns, reduction_columns, stream=0):
    _check(lib().qm_linear_m1(_addr(x), _addr(weight), _addr(bias), _addr(residual), _addr(out),
                              output_columns, reduction_columns, stream), "qm_linear_m1")


def qkv_m1(x, q_w, q_b, k_w, k_b, v_w, v_b, q_out, k_out, v_out, hidden, q_dim, kv_dim, stream=0):
    _check(lib().qm_qkv_m1(_addr(x), _addr(q_w), _addr(q_b), _addr(k_w), _addr(k_b), _addr(v_w), _addr(v_b),
                           _addr(q_out), _addr(k_out), _addr(v_out), hidden, q_dim, kv_dim, stream),
           "qm_qkv_m1")


def gate_up_swiglu_m1(x, gate_w, up_w, out, hidden, intermediate, stream=0):
    _check(lib().qm_gate_up_swiglu_m1(_addr(x), _addr(gate_w), _addr(up_w), _addr(out), hidden, intermediate, stream),
           "qm_gate_up_swiglu_m1")


def rmsnorm_rows(x, weight, out, rows, dimension, eps=1e-6, stream=0):
    _check(lib().qm_rmsnorm_rows(_addr(x), _addr(weight), _addr(out), rows, dimension, eps, stream), "qm_rmsnorm_rows")


def add_postnorm_m1(hidden, attention, norm_weight, residual, normalized, dimension, eps=1e-6, stream=0):
    _check(lib().qm_add_postnorm_m1(_addr(hidden), _addr(attention), _addr(norm_weight), _addr(residual),
                                    _addr(normalized), dimension, eps, stream), "qm_add_postnorm_m1")


def rmsnorm_qkv_m1(hidden_state, norm_weight, q_w, q_b, k_w, k_b, v_w, v_b, q_out, k_out, v_out, hidden, q_dim,
                   kv_dim, eps=1e-6, stream=0):
    _check(lib().qm_rmsnorm_qkv_m1(_addr(hidden_state), _addr(norm_weight), eps, _addr(q_w), _addr(q_b), _addr(k_w),
                                   _addr(k_b), _addr(v_w), _addr(v_b), _addr(q_out), _addr(k_out), _addr(v_out),
                                   hidden, q_dim, kv_dim, stream), "qm_rmsnorm_qkv_m1")


def add_postnorm_gate_up_swiglu_m1(hidden_state, attention, norm_weight, residual, gate_w, up_w, out, hidden,
                                   intermediate, eps=1e-6, stream=0):
    _check(lib().qm_add_postnorm_gate_up_swiglu_m1(_addr(hidden_state), _addr(attention), _addr(norm_weight), eps,
                                                   _addr(residual), _addr(gate_w), _addr(up_w), _addr(out), hidden,
                                                   intermediate, stream), "qm_add_postnorm_gate_up_swiglu_m1")


def predictor_linear_m1(x, weight, residual, out, output_columns, reduction_columns, stream=0):
    _check(lib().qm_predictor_linear_m1(_addr(x), _addr(weight), _addr(residual), _addr(out), output_columns,
                                        reduction_columns, stream), "qm_predictor_linear_m1")


def predictor_qkv_m1(x, q_w, k_w, v_w, q_out, k_out, v_out, hidden, q_dim, kv_dim, stream=0):
    _check(lib().qm_predictor_qkv_m1(_addr(x), _addr(q_w), _addr(k_w), _addr(v_w), _addr(q_out), _addr(k_out),
                                     _addr(v_out), hidden, q_dim, kv_dim, stream), "qm_predictor_qkv_m1")


def predictor_gate_up_swiglu_m1(x, gate_w, up_w, out, hidden, intermediate, stream=0):
    _check(lib().qm_predictor_gate_up_swiglu_m1(_addr(x), _addr(gate_w), _addr(up_w), _addr(out), hidden,
                                                intermediate, stream), "qm_predictor_gate_up_swiglu_m1")


def predictor_rmsnorm_qkv_m1(hidden_state, norm_weight, q_w, k_w, v_w, q_out, k_out, v_out, hidden, q_dim, kv_dim,
                             eps=1e-6, stream=0):
    _check(lib().qm_predictor_rmsnorm_qkv_m1(_addr(hidden_state), _addr(norm_weight), eps, _addr(q_w), _addr(k_w),
                                             _addr(v_w), _addr(q_out), _addr(k_out), _addr(v_out), hidden, q_dim,
                                             kv_dim, stream), "qm_predictor_rmsnorm_qkv_m1")


def predictor_add_postnorm_gate_up_swiglu_m1(hidden_state, attention, norm_weight, residual, gate_w, up_w, out,
                                             hidden, intermediate, eps=1e-6, stream=0):
    _check(lib().qm_predictor_add_postnorm_gate_up_swiglu_m1(
        _addr(hidden_state), _addr(attention), _addr(norm_weight), eps, _addr(residual), _addr(gate_w), _addr(up_w),
        _addr(out), hidden, intermediate, stream), "qm_predictor_add_postnorm_gate_up_swiglu_m1")


def sample_topk(logits, logits_are_bf16, offset, vocab, top_k, temperature, rng_state, output_id, stream=0):
    _check(lib().qm_sample_topk(_addr(logits), int(logits_are_bf16), offset, vocab, top_k, temperature,
                                _addr(rng_state), _addr(output_id), stream), "qm_sample_topk")


def final_head_process(logits, history, history_count, generation_index, vocab, eos, suppressed_tail, penalty,
                       scores, stream=0):
    _check(lib().qm_final_head_process(_addr(logits), _addr(history), history_count, generation_index, vocab, eos,
                                       suppressed_tail, penalty, _addr(scores), stream), "qm_final_head_process")


def final_head_sample(logits, history, generation_index, vocab, eos, suppressed_tail, penalty, top_k, temperature,
                      rng_state, code_out, scores_out=None, stream=0):
    _check(lib().qm_final_head_sample(_addr(logits), _addr(history), generation_index, vocab, eos, suppressed_tail,
                                      penalty, top_k, temperature, _addr(rng_state), _addr(code_out),
                                      _addr(scores_out), stream), "qm_final_head_sample")


def linear_rows(x, weight, bias, residual, out, rows, output_columns, reduction_columns, stream=0):
    _check(lib().qm_linear_rows(_addr(x), _addr(weight), _addr(bias), _addr(residual), _addr(out), rows,
                                output_columns, reduction_columns, stream), "qm_linear_rows")


def gate_up_swiglu_rows(x, gate_w, up_w, out, rows, hidden, intermediate, stream=0):
    _check(lib().qm_gate_up_swiglu_rows(_addr(x), _addr(gate_w), _addr(up_w), _addr(out), rows, hidden,
                                        intermediate, stream), "qm_gate_up_swiglu_rows")


def linear_rows_split_workspace_bytes(rows, output_columns, reduction_columns, gate_up_pair=False):
    return lib().qm_linear_rows_split_workspace_bytes(rows, output_columns, reduction_columns, int(gate_up_pair))


def linear_rows_split(x, weight, bias, residual, out, rows, output_columns, reduction_columns, workspace, workspace_bytes, stream=0):
    _check(lib().qm_linear_rows_split(_addr(x), _addr(weight), _addr(bias), _addr(residual), _addr(out), rows, output_columns,
                                      reduction_columns, _addr(workspace), workspace_bytes, stream), "qm_linear_rows_split")


def qkv_rows(x, weights, biases, outs, rows, q_columns, kv_columns, reduction_columns, workspace=None, workspace_bytes=0, stream=0):
    """weights / biases / outs: (q, k, v) triples; a bias may be None."""
    _check(lib().qm_qkv_rows_split(_addr(x), *[_addr(w) for w in weights], *[_addr(b) for b in biases], *[_addr(o) for o in outs],
                                   rows, q_columns, kv_columns, reduction_columns, _addr(workspace), workspace_bytes, stream),
           "qm_qkv_rows_split")


def gate_up_swiglu_rows_split(x, gate_weight, up_weight, out, rows, hidden, intermediate, workspace, workspace_bytes, stream=0):
    _check(lib().qm_gate_up_swiglu_rows_split(_addr(x), _addr(gate_weight), _addr(up_weight), _addr(out), rows, hidden, intermediate,
                                              _addr(workspace), workspace_bytes, stream), "qm_gate_up_swiglu_rows_split")


def gather_embedding(table, table_rows, codes, group, dimension, selected, next_input, stream=0):
    _check(lib().qm_gather_embedding(_addr(table), table_rows, _addr(codes), group, dimension, _addr(selected),
                                     _addr(next_input), stream), "qm_gather_embedding")


def predictor_attention_staged(query_bhsd, key_cache, value_cache, out, rows, key_length, causal, stream=0):
    _check(lib().qm_predictor_attention_staged(_addr(query_bhsd), _addr(key_cache), _addr(value_cache), _addr(out),
                                               rows, key_length, int(causal), stream), "qm_predictor_attention_staged")


def predictor_step_attention_m1(q, k, v, gq, gk, cos_row, sin_row, key_cache, value_cache, out, position,
                                eps=1e-6, stream=0):
    _check(lib().qm_predictor_step_attention_m1(_addr(q), _addr(k), _addr(v), _addr(gq), _addr(gk), _addr(cos_row),
                                                _addr(sin_row), _addr(key_cache), _addr(value_cache), _addr(out),
                                                position, eps, stream), "qm_predictor_step_attention_m1")


STATUS_BAD_PAGE, STATUS_BAD_POSITION, STATUS_SPLIT_TIMEOUT, STATUS_FRAME_TIMEOUT = 1, 2, 4, 8


def predictor_frame(layers, projection_weight, projection_bias, final_norm, heads, embeddings, cosine, sine, free_input,
                    selected, codes, rng_state, epsilon=1e-6, step0_input=None, projected=None):
    """qm_predictor_frame from tensors: `layers` is five dicts with the field names of qm_predictor_frame_layer,
    `heads` / `embeddings` (and `projected`, optional) map a step to its tensor.  The tensors must outlive the descriptor."""
    frame = PredictorFrame()
    for i, layer in enumerate(layers):
        for name, _ in PredictorFrameLayer._fields_:
            setattr(frame.layers[i], name, _addr(layer[name]))
    frame.projection_weight, frame.projection_bias, frame.final_norm = (_addr(projection_weight), _addr(projection_bias),
                                                                        _addr(final_norm))
    for step, tensor in heads.items():
        frame.heads[step] = _addr(tensor)
    for step, tensor in embeddings.items():
        frame.embeddings[step] = _addr(tensor)
    frame.cosine, frame.sine = _addr(cosine), _addr(sine)
    frame.free_input, frame.selected, frame.codes, frame.rng_state = (_addr(free_input), _addr(selected), _addr(codes),
                                                                      _addr(rng_state))
    frame.epsilon = epsilon
    frame.step0_input = _addr(step0_input)
    for step, tensor in (projected or {}).items():
        frame.projected[step] = _addr(tensor)
    return frame


def predictor_frame_workspace_bytes():
    return lib().qm_predictor_frame_workspace_bytes()


def predictor_frame_workspace_init(workspace, workspace_bytes, stream=0):
    _check(lib().qm_predictor_frame_workspace_init(_addr(workspace), workspace_bytes, stream),
           "qm_predictor_frame_workspace_init")


def predictor_frame_fits(stream=0):
    """Whether the one-launch predictor frame can run on `stream` (device and stream CU mask hold its 256 blocks)."""
    fits = C.c_int32(0)
    _check(lib().qm_predictor_frame_fits(stream, C.byref(fits)), "qm_predictor_frame_fits")
    return bool(fits.value)


def talker_chain_fits(stream=0):
    """Whether the talker's one launch between two attentions can run on `stream`."""
    fits = C.c_int32(0)
    _check(lib().qm_talker_chain_fits(stream, C.byref(fits)), "qm_talker_chain_fits")
    return bool(fits.value)


def predictor_frame_steps(frame, first_step, last_step, top_k, temperature, workspace, workspace_bytes, status=None, stream=0):
    _check(lib().qm_predictor_frame_steps(C.byref(frame), first_step, last_step, top_k, temperature, _addr(workspace),
                                          workspace_bytes, _addr(status), stream), "qm_predictor_frame_steps")


def talker_post_attention(hidden_columns=2048, q_columns=2048, kv_columns=1024, intermediate_columns=6144, epsilon=1e-6,
                          **tensors):
    """qm_talker_post_attention from tensors named like its fields (absent ones stay NULL).  The tensors must outlive
    the descriptor."""
    op = TalkerPostAttention()
    for name, tensor in tensors.items():
        setattr(op, name, _addr(tensor))
    op.hidden_columns, op.q_columns, op.kv_columns, op.intermediate_columns = (hidden_columns, q_columns, kv_columns,
                                                                               intermediate_columns)
    op.epsilon = epsilon
    return op


def talker_post_attention_workspace_bytes():
    return lib().qm_talker_post_attention_workspace_bytes()


def talker_post_attention_workspace_init(workspace, workspace_bytes, stream=0):
    _check(lib().qm_talker_post_attention_workspace_init(_addr(workspace), workspace_bytes, stream),
           "qm_talker_post_attention_workspace_init")


def talker_post_attention_m1(op, workspace, workspace_bytes, status=None, stream=0):
    _check(lib().qm_talker_post_attention_m1(C.byref(op), _addr(workspace), workspace_bytes, _addr(status), stream),
           "qm_talker_post_attention_m1")


def talker_layer_step(q, k, v, gq, gk, cos, sin, q_rot, cache, page_table, max_pages, context, q_heads, position, sliding_window,
                      scale, eps, attention_workspace, attention_workspace_bytes, post):
    """qm_talker_layer_step: the arguments of decode_step_fused and a TalkerPostAttention.  Everything named must outlive the
    descriptor (the cache descriptor is kept with it)."""
    step = TalkerLayerStep()
    for name, tensor in (("q", q), ("k", k), ("v", v), ("q_norm_w", gq), ("k_norm_w", gk), ("cos_row", cos), ("sin_row", sin),
                         ("q_rotated_out", q_rot), ("page_table", page_table), ("attention_workspace", attention_workspace),
                         ("context", context)):
        setattr(step, name, _addr(tensor))
    step._cache = cache
    step.cache = C.pointer(cache)
    step.attention_workspace_bytes = attention_workspace_bytes
    step.max_pages, step.q_heads, step.position, step.sliding_window = max_pages, q_heads, position, sliding_window
    step.scale, step.epsilon = scale, eps
    step.post = post
    return step


def talker_layer_step_m1(step, workspace, workspace_bytes, status=None, stream=0):
    _check(lib().qm_talker_layer_step_m1(C.byref(step), _addr(workspace), workspace_bytes, _addr(status), stream),
           "qm_talker_layer_step_m1")


def predictor_transpose(x, out, rows, heads, stream=0):
    _check(lib().qm_predictor_transpose(_addr(x), _addr(out), rows, heads, stream), "qm_predictor_transpose")


def predictor_rope_bhsd(x, cos, sin, out, rows, heads, stream=0):
    _check(lib().qm_predictor_rope_bhsd(_addr(x), _addr(cos), _addr(sin), _addr(out), rows, heads, stream),
           "qm_predictor_rope_bhsd")


def predictor_update_cache(source, cache, rows, start, stream=0):
    _check(lib().qm_predictor_update_cache(_addr(source), _addr(cache), rows, start, stream),
           "qm_predictor_update_cache")


DECODE_STATIC_SCRATCH_BYTES = 8 << 20


def decode_attention_ragged_static(query, cache, page_table, max_pages, seq_lens, n_streams, max_seq_len, out,
                                   q_heads, scale=SCALE_128, status=None, stream=0):
    _check(lib().qm_decode_attention_ragged_static(
        _addr(query), C.byref(cache), _addr(page_table), max_pages, _addr(seq_lens), n_streams,
        max_seq_len, _addr(out), q_heads, scale, _addr(status), stream), "qm_decode_attention_ragged_static")


def predictor_prepare_group0(table, table_rows, code0, dimension, free_input, selected, codes, stream=0):
    _check(lib().qm_predictor_prepare_group0(_addr(table), table_rows, _addr(code0), dimension, _addr(free_input),
                                             _addr(selected), _addr(codes), stream), "qm_predictor_prepare_group0")


def predictor_next_talker_input(selected, groups, context, dimension, embedding_sum, next_input, stream=0):
    _check(lib().qm_predictor_next_talker_input(_addr(selected), groups, _addr(context), dimension, _addr(embedding_sum),
                                                _addr(next_input), stream), "qm_predictor_next_talker_input")
