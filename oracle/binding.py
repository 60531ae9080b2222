"""ctypes binding of the CPU oracle (oracle/libqm_oracle.so).

TEST INFRASTRUCTURE: imported only by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  Arrays are numpy uint16 (bf16 bit patterns) / int32.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libqm_oracle.so")

POLICY_REFERENCE = 0
POLICY_ONLINE = 1
POLICY_FP32 = 2


class KvCache(C.Structure):
    """Mirror of qm_kv_cache (include/qm_attn.h)."""
    _fields_ = [
        ("k_pool", C.c_void_p), ("v_pool", C.c_void_p),
        ("stride_page", C.c_int64), ("stride_head", C.c_int64), ("stride_token", C.c_int64),
        ("page_size", C.c_int32), ("n_pages", C.c_int32),
        ("kv_heads", C.c_int32), ("head_dim", C.c_int32),
    ]


def build(force=False):
    """Compile the oracle with g++ (no GPU toolchain involved)."""
    src = os.path.join(HERE, "qm_oracle.cpp")
    if not force and os.path.exists(LIB_PATH) and os.path.getmtime(LIB_PATH) >= os.path.getmtime(src):
        return LIB_PATH
    cmd = ["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-fPIC", "-shared", "-Wall", "-Wextra",
           "-pthread", "-o", LIB_PATH, src]
    subprocess.run(cmd, check=True, cwd=HERE)
    return LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = C.CDLL(LIB_PATH)
        _lib.qmo_bf16_to_f32.restype = C.c_float
        _lib.qmo_bf16_to_f32.argtypes = [C.c_uint16]
        _lib.qmo_f32_to_bf16.restype = C.c_uint16
        _lib.qmo_f32_to_bf16.argtypes = [C.c_float]
        _lib.qmo_head_sum_squares.restype = C.c_float
    return _lib


def _p(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be contiguous"
    return a.ctypes.data_as(C.c_void_p)


def paged_cache(k_pool, v_pool, kv_heads=8, page_size=16):
    """Descriptor of the native [page][kv_head][page_size][128] layout over numpy pools."""
    n_pages = k_pool.size // (kv_heads * page_size * 128)
    return KvCache(k_pool.ctypes.data, v_pool.ctypes.data, kv_heads * page_size * 128,
                   page_size * 128, 128, page_size, n_pages, kv_heads, 128)


def flat_cache(key_cache, value_cache, kv_heads, max_cache):
    """Descriptor of the reference LayerCache [kv_head][max_cache][128] (one page)."""
    return KvCache(key_cache.ctypes.data, value_cache.ctypes.data, 0, max_cache * 128, 128,
                   max_cache, 1, kv_heads, 128)


# ---- helpers -------------------------------------------------------------------------
def f32_to_bf16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().qmo_f32_to_bf16_array(_p(x), _p(out), C.c_int64(x.size))
    return out


def bf16_to_f32(x):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, dtype=np.float32)
    lib().qmo_bf16_to_f32_array(_p(x), _p(out), C.c_int64(x.size))
    return out


def normal_bf16(shape, seed, mean=0.0, std=1.0, threads=8):
    out = np.empty(shape, dtype=np.uint16)
    lib().qmo_fill_normal_bf16(_p(out), C.c_int64(out.size), C.c_uint64(seed),
                               C.c_float(mean), C.c_float(std), C.c_int(threads))
    return out


def uniform_int(n, seed, lo, hi):
    out = np.empty(n, dtype=np.int32)
    lib().qmo_fill_uniform_int(_p(out), C.c_int64(n), C.c_uint64(seed), C.c_int32(lo), C.c_int32(hi))
    return out


def permutation(n, seed):
    out = np.empty(n, dtype=np.int32)
    lib().qmo_permutation(_p(out), C.c_int64(n), C.c_uint64(seed))
    return out


def rope_table(rows, start=0, head_dim=128, theta=1.0e6):
    cos = np.empty((rows, head_dim), dtype=np.uint16)
    sin = np.empty((rows, head_dim), dtype=np.uint16)
    rc = lib().qmo_rope_table(C.c_int32(rows), C.c_int32(start), C.c_int32(head_dim),
                              C.c_double(theta), _p(cos), _p(sin))
    if rc != 0:
        raise ValueError(f"qmo_rope_table failed: {rc}")
    return cos, sin


# ---- operators (return the C return code; outputs written in place) ----------------------
def qk_norm_rope_kv_append(q, k, v, gq, gk, cos, sin, q_rot, cache, page_table, max_pages,
                           q_heads, position, eps=1e-6):
    return lib().qmo_qk_norm_rope_kv_append(
        _p(q), _p(k), _p(v), _p(gq), _p(gk), _p(cos), _p(sin), _p(q_rot), C.byref(cache),
        _p(page_table), C.c_int32(max_pages), C.c_int32(q_heads), C.c_int32(position),
        C.c_float(eps))


def qk_norm_rope_kv_append_ragged(q, k, v, gq, gk, cos, sin, by_position, q_rot, cache,
                                  page_table, max_pages, positions, q_heads, eps=1e-6,
                                  status=None):
    return lib().qmo_qk_norm_rope_kv_append_ragged(
        _p(q), _p(k), _p(v), _p(gq), _p(gk), _p(cos), _p(sin), C.c_int32(by_position),
        _p(q_rot), C.byref(cache), _p(page_table), C.c_int32(max_pages), _p(positions),
        C.c_int32(len(positions)), C.c_int32(q_heads), C.c_float(eps), _p(status))


def norm_rope_rows(x, norm_w, cos, sin, out, rows, heads, eps=1e-6):
    return lib().qmo_norm_rope_rows(_p(x), _p(norm_w), _p(cos), _p(sin), _p(out),
                                    C.c_int32(rows), C.c_int32(heads), C.c_float(eps))


def scatter_kv(key, value, cache, page_table, max_pages, rows, first_position):
    return lib().qmo_scatter_kv(_p(key), _p(value), C.byref(cache), _p(page_table),
                                C.c_int32(max_pages), C.c_int32(rows), C.c_int32(first_position))


def attention(query, cache, page_table, max_pages, out, query_length, cache_before, q_heads,
              sliding_window=-1, scale=0.08838834764831845, policy=POLICY_REFERENCE, threads=8):
    return lib().qmo_attention(
        _p(query), C.byref(cache), _p(page_table), C.c_int32(max_pages), _p(out),
        C.c_int32(query_length), C.c_int32(cache_before), C.c_int32(q_heads),
        C.c_int32(sliding_window), C.c_float(scale), C.c_int32(policy), C.c_int32(threads))


def decode_attention_ragged(query, cache, page_table, max_pages, seq_lens, out, q_heads,
                            scale=0.08838834764831845, policy=POLICY_REFERENCE, threads=8):
    return lib().qmo_decode_attention_ragged(
        _p(query), C.byref(cache), _p(page_table), C.c_int32(max_pages), _p(seq_lens),
        C.c_int32(len(seq_lens)), _p(out), C.c_int32(q_heads), C.c_float(scale),
        C.c_int32(policy), C.c_int32(threads))


def prefill_attention_causal(query, key, value, out, cache, page_table, max_pages, batch, seq,
                             q_heads, kv_heads, scale=0.08838834764831845,
                             policy=POLICY_REFERENCE, threads=8):
    return lib().qmo_prefill_attention_causal(
        _p(query), _p(key), _p(value), _p(out), C.byref(cache) if cache is not None else None,
        _p(page_table), C.c_int32(max_pages), C.c_int32(batch), C.c_int32(seq),
        C.c_int32(q_heads), C.c_int32(kv_heads), C.c_float(scale), C.c_int32(policy),
        C.c_int32(threads))


def predictor_attention_m1(query, key_cache, value_cache, out, key_length):
    return lib().qmo_predictor_attention_m1(_p(query), _p(key_cache), _p(value_cache), _p(out),
                                            C.c_int32(key_length))


def predictor_attention_staged(query_bhsd, key_cache, value_cache, out_bshd, rows, key_length,
                               causal=True):
    return lib().qmo_predictor_attention_staged(_p(query_bhsd), _p(key_cache), _p(value_cache),
                                                _p(out_bshd), C.c_int32(rows),
                                                C.c_int32(key_length), C.c_int32(int(causal)))


def predictor_transpose(x, out, rows, heads):
    return lib().qmo_predictor_transpose(_p(x), _p(out), C.c_int32(rows), C.c_int32(heads))


def predictor_rope_bhsd(x, cos, sin, out, rows, heads):
    return lib().qmo_predictor_rope_bhsd(_p(x), _p(cos), _p(sin), _p(out), C.c_int32(rows), C.c_int32(heads))


def predictor_update_cache(source, cache, rows, start):
    return lib().qmo_predictor_update_cache(_p(source), _p(cache), C.c_int32(rows), C.c_int32(start))


def predictor_attention_loop(q, k, v, gq, gk, cos, sin, out, k_cache_out, v_cache_out, units,
                             n_layers, rows, first_rows=1, eps=1e-6, threads=8):
    return lib().qmo_predictor_attention_loop(
        _p(q), _p(k), _p(v), _p(gq), _p(gk), _p(cos), _p(sin), _p(out), _p(k_cache_out),
        _p(v_cache_out), C.c_int32(units), C.c_int32(n_layers), C.c_int32(rows),
        C.c_int32(first_rows), C.c_float(eps), C.c_int32(threads))


def linear_m1(x, weight, bias, residual, out, output_columns, reduction_columns, threads=8):
    return lib().qmo_linear_m1(_p(x), _p(weight), _p(bias), _p(residual), _p(out),
                               C.c_int32(output_columns), C.c_int32(reduction_columns), C.c_int32(threads))


def qkv_m1(x, q_w, q_b, k_w, k_b, v_w, v_b, q_out, k_out, v_out, hidden, q_dim, kv_dim, threads=8):
    return lib().qmo_qkv_m1(_p(x), _p(q_w), _p(q_b), _p(k_w), _p(k_b), _p(v_w), _p(v_b), _p(q_out),
                            _p(k_out), _p(v_out), C.c_int32(hidden), C.c_int32(q_dim), C.c_int32(kv_dim),
                            C.c_int32(threads))


def rmsnorm_rows(x, weight, out, rows, dimension, eps=1e-6, threads=8):
    return lib().qmo_rmsnorm_rows(_p(x), _p(weight), _p(out), C.c_int32(rows), C.c_int32(dimension),
                                  C.c_float(eps), C.c_int32(threads))


def add_postnorm_m1(hidden, attention, norm_weight, residual, normalized, dimension, eps=1e-6):
    return lib().qmo_add_postnorm_m1(_p(hidden), _p(attention), _p(norm_weight), _p(residual), _p(normalized),
                                     C.c_int32(dimension), C.c_float(eps))


def gate_up_swiglu_m1(x, gate_w, up_w, out, hidden, intermediate, threads=8):
    return lib().qmo_gate_up_swiglu_m1(_p(x), _p(gate_w), _p(up_w), _p(out), C.c_int32(hidden),
                                       C.c_int32(intermediate), C.c_int32(threads))


def predictor_linear_m1(x, weight, residual, out, output_columns, reduction_columns, threads=8):
    return lib().qmo_predictor_linear_m1(_p(x), _p(weight), _p(residual), _p(out), C.c_int32(output_columns),
                                         C.c_int32(reduction_columns), C.c_int32(threads))


def predictor_qkv_m1(x, q_w, k_w, v_w, q_out, k_out, v_out, hidden, q_dim, kv_dim, threads=8):
    return lib().qmo_predictor_qkv_m1(_p(x), _p(q_w), _p(k_w), _p(v_w), _p(q_out), _p(k_out), _p(v_out),
                                      C.c_int32(hidden), C.c_int32(q_dim), C.c_int32(kv_dim), C.c_int32(threads))


def predictor_gate_up_swiglu_m1(x, gate_w, up_w, out, hidden, intermediate, threads=8):
    return lib().qmo_predictor_gate_up_swiglu_m1(_p(x), _p(gate_w), _p(up_w), _p(out), C.c_int32(hidden),
                                                 C.c_int32(intermediate), C.c_int32(threads))


def splitmix64(state, count):
    """state: numpy uint64 array of one element (advanced in place); returns (raw uint64[count], uniform f64[count])."""
    import numpy as np
    raw = np.zeros(count, dtype=np.uint64)
    uni = np.zeros(count, dtype=np.float64)
    assert lib().qmo_splitmix64(_p(state), C.c_int32(count), _p(raw), _p(uni)) == 0
    return raw, uni


def sample_topk(logits, is_bf16, offset, vocab, top_k, temperature, rng_state, output_id):
    return lib().qmo_sample_topk(_p(logits), C.c_int32(int(is_bf16)), C.c_int32(offset), C.c_int32(vocab),
                                 C.c_int32(top_k), C.c_float(temperature), _p(rng_state), _p(output_id))


def final_head_process(logits, history, history_count, generation_index, vocab, eos, suppressed_tail, penalty, scores):
    return lib().qmo_final_head_process(_p(logits), _p(history), C.c_int32(history_count),
                                        C.c_int32(generation_index), C.c_int32(vocab), C.c_int32(eos),
                                        C.c_int32(suppressed_tail), C.c_float(penalty), _p(scores))


def final_head_sample(logits, history, generation_index, vocab, eos, suppressed_tail, penalty, top_k, temperature,
                      rng_state, code_out, scores_out=None):
    return lib().qmo_final_head_sample(_p(logits), _p(history), C.c_int32(generation_index), C.c_int32(vocab),
                                       C.c_int32(eos), C.c_int32(suppressed_tail), C.c_float(penalty),
                                       C.c_int32(top_k), C.c_float(temperature), _p(rng_state), _p(code_out),
                                       _p(scores_out))


def linear_rows(x, weight, bias, residual, out, rows, output_columns, reduction_columns, threads=8):
    return lib().qmo_linear_rows(_p(x), _p(weight), _p(bias), _p(residual), _p(out), C.c_int32(rows),
                                 C.c_int32(output_columns), C.c_int32(reduction_columns), C.c_int32(threads))


def gate_up_swiglu_rows(x, gate_w, up_w, out, rows, hidden, intermediate, threads=8):
    return lib().qmo_gate_up_swiglu_rows(_p(x), _p(gate_w), _p(up_w), _p(out), C.c_int32(rows), C.c_int32(hidden),
                                         C.c_int32(intermediate), C.c_int32(threads))
