"""ctypes binding of libqm_engine.so: the host-side engine shell (safetensors reader, talker
weights and decode layer loop, RoPE rows, trajectory hash).  Mirrors include/qm_engine.h.
Tensors on the device are torch tensors (or raw addresses); the library itself never sees torch."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(HERE, "lib", "libqm_engine.so")
_lib = None

_P, _I32, _U64 = C.c_void_p, C.c_int32, C.c_uint64
_SIGNATURES = {
    "qm_engine_last_error": (C.c_char_p, []),
    "qm_fnv1a64": (_U64, [_P, C.c_size_t]),
    "qm_rope_rows": (_I32, [_I32, _I32, _I32, C.c_double, _P, _P]),
    "qm_safefile_open": (_I32, [C.c_char_p, C.POINTER(_P)]),
    "qm_safefile_close": (None, [_P]),
    "qm_safefile_count": (_I32, [_P]),
    "qm_safefile_tensor": (_I32, [_P, _I32, C.POINTER(C.c_char_p), C.POINTER(C.c_char_p), C.POINTER(_I32),
                                  C.POINTER(C.c_int64), C.POINTER(_P), C.POINTER(_U64)]),
    "qm_talker_create": (_I32, [C.c_char_p, _I32, _P, C.POINTER(_P)]),
    "qm_talker_destroy": (None, [_P]),
    "qm_talker_info": (_I32, [_P, C.POINTER(_I32)]),
    "qm_talker_reset": (_I32, [_P, _I32]),
    "qm_talker_cache": (_I32, [_P, _I32, C.POINTER(_P), C.POINTER(_P)]),
    "qm_talker_decode": (_I32, [_P, _P, _P, _P, _I32, C.POINTER(_P)]),
    "qm_talker_decode_device_rope": (_I32, [_P, _P, _P, _P, _I32, C.POINTER(_P)]),
    "qm_talker_prefill": (_I32, [_P, _P, _P, _P, _I32, C.POINTER(_P)]),
    "qm_talker_synchronize": (_I32, [_P]),
    "qm_talker_stream": (_P, [_P]),
    "qm_talker_status_device": (_P, [_P]),
    "qm_final_head_create": (_I32, [C.c_char_p, _I32, _U64, _P, C.POINTER(_P)]),
    "qm_final_head_destroy": (None, [_P]),
    "qm_final_head_reset": (_I32, [_P, _U64]),
    "qm_final_head_run": (_I32, [_P, _P, _I32, _I32, C.POINTER(_I32)]),
    "qm_final_head_rng_state": (_P, [_P]),
    "qm_final_head_device_code": (_P, [_P]),
    "qm_predictor_create": (_I32, [C.c_char_p, _P, _P, C.POINTER(_P)]),
    "qm_predictor_destroy": (None, [_P]),
    "qm_predictor_run_frame": (_I32, [_P, _P, _P, _P, _I32, C.POINTER(_I32)]),
    "qm_predictor_next_input": (_P, [_P]),
    "qm_generate": (_I32, [_P, _P, _P, _P, _I32, _I32, _P, _P, _I32, _I32, _P, C.POINTER(_I32), C.POINTER(_U64)]),
}
EXPORTS = tuple(_SIGNATURES)


class EngineError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"{message} (code {code})")
        self.code = code


def lib():
    """Loads the shared library (once).  Raises FileNotFoundError if it was not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise FileNotFoundError(f"{_LIB_PATH} is missing: build it with `python qingming-qwen3-tts_amd/build.py`")
        handle = C.CDLL(_LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = restype, argtypes
        _lib = handle
    return _lib


def _check(code):
    if code != 0:
        raise EngineError(code, lib().qm_engine_last_error().decode("utf-8", "replace"))


def fnv1a64(data: bytes) -> int:
    return int(lib().qm_fnv1a64(data, len(data)))


def rope_rows(rows, start, head_dim=128, theta=1.0e6):
    """(cos, sin) as uint16 arrays [rows][head_dim] of bf16 bit patterns."""
    cos = np.zeros((rows, head_dim), dtype=np.uint16)
    sin = np.zeros((rows, head_dim), dtype=np.uint16)
    _check(lib().qm_rope_rows(rows, start, head_dim, theta, cos.ctypes.data, sin.ctypes.data))
    return cos, sin


def read_safetensors(path):
    """{name: (dtype name, shape tuple, bytes)} as the library's reader sees the file."""
    handle = _P()
    _check(lib().qm_safefile_open(os.fsencode(path), C.byref(handle)))
    try:
        out = {}
        for i in range(lib().qm_safefile_count(handle)):
            name, dtype, rank, data, nbytes = C.c_char_p(), C.c_char_p(), _I32(), _P(), _U64()
            shape = (C.c_int64 * 8)()
            _check(lib().qm_safefile_tensor(handle, i, C.byref(name), C.byref(dtype), C.byref(rank), shape,
                                            C.byref(data), C.byref(nbytes)))
            out[name.value.decode()] = (dtype.value.decode(), tuple(shape[:rank.value]),
                                        C.string_at(data.value, nbytes.value) if nbytes.value else b"")
        return out
    finally:
        lib().qm_safefile_close(handle)


class Talker:
    """qm_talker: weights from a model directory, per-layer KV caches, decode_device."""

    def __init__(self, model_dir, max_cache, stream=0):
        self._handle = _P()
        _check(lib().qm_talker_create(os.fsencode(model_dir), max_cache, stream or None, C.byref(self._handle)))
        info = (_I32 * 7)()
        _check(lib().qm_talker_info(self._handle, info))
        (self.layers, self.q_heads, self.kv_heads, self.q_dim, self.kv_dim, self.intermediate, self.max_cache) = list(info)

    def close(self):
        if self._handle:
            lib().qm_talker_destroy(self._handle)
            self._handle = _P()

    def __del__(self):
        self.close()

    def reset(self, prefill_length):
        _check(lib().qm_talker_reset(self._handle, prefill_length))

    def cache_addresses(self, layer):
        k, v = _P(), _P()
        _check(lib().qm_talker_cache(self._handle, layer, C.byref(k), C.byref(v)))
        return k.value, v.value

    def decode(self, input_device, cosine_host, sine_host, decode_index):
        """input_device: torch bf16/int16 tensor [2048] (or an address); cosine/sine: numpy uint16 [128] on
        the host.  Returns the device address of the final hidden vector [2048] (engine-owned)."""
        address = input_device if isinstance(input_device, int) else input_device.data_ptr()
        cosine_host = np.ascontiguousarray(cosine_host, dtype=np.uint16)
        sine_host = np.ascontiguousarray(sine_host, dtype=np.uint16)
        out = _P()
        _check(lib().qm_talker_decode(self._handle, address, cosine_host.ctypes.data, sine_host.ctypes.data,
                                      decode_index, C.byref(out)))
        return out.value

    def prefill(self, input_device, cosine_host, sine_host, rows):
        """input_device: torch tensor [rows][2048] (or an address); cosine/sine: numpy uint16 [rows][128] on the
        host.  Returns the device address of the last row's final hidden vector."""
        address = input_device if isinstance(input_device, int) else input_device.data_ptr()
        cosine_host = np.ascontiguousarray(cosine_host, dtype=np.uint16)
        sine_host = np.ascontiguousarray(sine_host, dtype=np.uint16)
        out = _P()
        _check(lib().qm_talker_prefill(self._handle, address, cosine_host.ctypes.data, sine_host.ctypes.data, rows,
                                       C.byref(out)))
        return out.value

    def synchronize(self):
        _check(lib().qm_talker_synchronize(self._handle))

    @property
    def stream(self):
        return lib().qm_talker_stream(self._handle)


class FinalHead:
    """qm_final_head: codec_head, score processing, sampler, history and the generator state."""

    def __init__(self, model_dir, history_capacity, seed, stream):
        self._handle = _P()
        _check(lib().qm_final_head_create(os.fsencode(model_dir), history_capacity, seed, stream, C.byref(self._handle)))

    def close(self):
        if self._handle:
            lib().qm_final_head_destroy(self._handle)
            self._handle = _P()

    def __del__(self):
        self.close()

    def reset(self, seed):
        _check(lib().qm_final_head_reset(self._handle, seed))

    def run(self, hidden_device, frame, sampling=True):
        address = hidden_device if isinstance(hidden_device, int) else hidden_device.data_ptr()
        code = _I32()
        _check(lib().qm_final_head_run(self._handle, address, frame, int(sampling), C.byref(code)))
        return code.value

    @property
    def rng_state(self):
        return lib().qm_final_head_rng_state(self._handle)

    @property
    def device_code(self):
        return lib().qm_final_head_device_code(self._handle)


class Predictor:
    """qm_predictor: the code predictor's weights and its fifteen-step frame."""

    def __init__(self, model_dir, rng_state_device, stream):
        self._handle = _P()
        _check(lib().qm_predictor_create(os.fsencode(model_dir), rng_state_device, stream, C.byref(self._handle)))

    def close(self):
        if self._handle:
            lib().qm_predictor_destroy(self._handle)
            self._handle = _P()

    def __del__(self):
        self.close()

    def run_frame(self, talker_hidden_device, code0_device, context_host, sampling=True):
        hidden = talker_hidden_device if isinstance(talker_hidden_device, int) else talker_hidden_device.data_ptr()
        code0 = code0_device if isinstance(code0_device, int) else code0_device.data_ptr()
        context_host = np.ascontiguousarray(context_host, dtype=np.uint16)
        codes = (_I32 * 16)()
        _check(lib().qm_predictor_run_frame(self._handle, hidden, code0, context_host.ctypes.data, int(sampling), codes))
        return list(codes)

    @property
    def next_input(self):
        return lib().qm_predictor_next_input(self._handle)


def generate(talker, head, predictor, prompt_device, prompt_rows, maximum_frames, tts_pad_host, trailing_text_host=None,
             sampling=True):
    """qm_generate: (codes [frames][16] int32, trajectory hash)."""
    prompt = prompt_device if isinstance(prompt_device, int) else prompt_device.data_ptr()
    tts_pad_host = np.ascontiguousarray(tts_pad_host, dtype=np.uint16)
    trailing_rows = 0 if trailing_text_host is None else int(trailing_text_host.shape[0])
    trailing = None if trailing_text_host is None else np.ascontiguousarray(trailing_text_host, dtype=np.uint16)
    codes = np.zeros((maximum_frames, 16), dtype=np.int32)
    frames, digest = _I32(), _U64()
    _check(lib().qm_generate(talker._handle, head._handle, predictor._handle, prompt, prompt_rows, maximum_frames,
                             tts_pad_host.ctypes.data, trailing.ctypes.data if trailing is not None else None, trailing_rows,
                             int(sampling), codes.ctypes.data, C.byref(frames), C.byref(digest)))
    return codes[:frames.value].copy(), int(digest.value)
