"""CPU-only checks of the engine shell (libqm_engine.so): exported symbols, the trajectory hash
against FNV-1a's published vectors, RoPE rows against the oracle's table and closed forms, and
the safetensors reader against files written by the `safetensors` package (an independent
writer) plus malformed files."""
import json
import os
import re
import struct

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_symbols_are_exported(engine):
    text = open(os.path.join(ROOT, "include", "qm_engine.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(qm_[a-z0-9_]+)\s*\(", text)))
    assert len(names) >= 12
    lib = engine.lib()
    for name in names:
        assert hasattr(lib, name), f"{name} declared in qm_engine.h but not exported"
    assert sorted(engine.EXPORTS) == names


def test_fnv1a64_is_the_references_variant(engine):
    """The reference's trajectory hash (R17:833-842) is FNV-1a's recurrence with the 64-bit FNV prime,
    but its offset basis is 1469598103934665603 — the published basis 14695981039346656037 without
    its last digit.  Trajectory hashes are compared with the reference's, so that constant is kept;
    the published FNV-1a test vectors (Fowler / Noll / Vo: "" -> cbf29ce484222325, "a" ->
    af63dc4c8601ec8c) therefore do NOT hold, and the recurrence is pinned on its own."""
    prime, basis = 0x100000001b3, 1469598103934665603
    assert engine.fnv1a64(b"") == basis
    assert engine.fnv1a64(b"") != 0xcbf29ce484222325
    assert engine.fnv1a64(b"a") == ((basis ^ 0x61) * prime) % 2 ** 64
    # xor-then-multiply, byte by byte, in order: undo the last step of a longer message
    h2 = engine.fnv1a64(b"ab")
    assert h2 == ((engine.fnv1a64(b"a") ^ 0x62) * prime) % 2 ** 64
    assert engine.fnv1a64(b"ba") != h2
    # with the published basis the same recurrence gives the published vector for "a": the
    # difference to standard FNV-1a is the basis alone
    assert ((0xcbf29ce484222325 ^ 0x61) * prime) % 2 ** 64 == 0xaf63dc4c8601ec8c


def test_rope_rows_equal_the_oracle_table_and_closed_forms(engine, oracle):
    cos, sin = engine.rope_rows(40, 5)
    want_cos, want_sin = oracle.rope_table(40, 5)
    assert np.array_equal(cos, want_cos) and np.array_equal(sin, want_sin)
    c0, s0 = engine.rope_rows(1, 0)
    assert np.all(c0 == 0x3f80) and np.all(s0 == 0)                     # position 0: cos 1, sin 0
    assert np.array_equal(cos[:, :64], cos[:, 64:]) and np.array_equal(sin[:, :64], sin[:, 64:])
    c1, s1 = engine.rope_rows(1, 1)                                     # pair 0 turns by one radian per position
    assert c1[0, 0] == oracle.f32_to_bf16(np.array([np.cos(1.0)], dtype=np.float32))[0]
    assert s1[0, 0] == oracle.f32_to_bf16(np.array([np.sin(1.0)], dtype=np.float32))[0]
    assert engine.lib().qm_rope_rows(1, 0, 127, 1.0e6, c0.ctypes.data, s0.ctypes.data) == -2
    assert engine.lib().qm_rope_rows(1, -1, 128, 1.0e6, c0.ctypes.data, s0.ctypes.data) == -2


def _torch_file(tmp_path, tensors, name="model.safetensors", metadata=None):
    from safetensors.torch import save_file
    path = os.path.join(tmp_path, name)
    save_file(tensors, path, metadata=metadata)
    return path


def test_reader_agrees_with_the_safetensors_package(engine, tmp_path):
    import torch
    g = torch.Generator().manual_seed(3)
    tensors = {
        "talker.model.layers.0.self_attn.q_proj.weight": torch.randn(24, 16, generator=g).to(torch.bfloat16),
        "a.scalar": torch.tensor(3.5),
        "b.empty": torch.zeros((0, 4), dtype=torch.float16),
        "c.int64": torch.arange(10, dtype=torch.int64).reshape(2, 5),
        "d.u8 é\"quoted\"": torch.arange(7, dtype=torch.uint8),
        "e.bool": torch.tensor([True, False, True]),
    }
    path = _torch_file(str(tmp_path), tensors, metadata={"format": "pt", "note": "nested {braces} [and] \\ slashes"})
    got = engine.read_safetensors(path)
    assert sorted(got) == sorted(tensors)
    names = {torch.bfloat16: "BF16", torch.float32: "F32", torch.float16: "F16", torch.int64: "I64", torch.uint8: "U8",
             torch.bool: "BOOL"}
    for name, t in tensors.items():
        dtype, shape, data = got[name]
        assert dtype == names[t.dtype] and shape == tuple(t.shape)
        raw = t.contiguous().reshape(-1).view(torch.uint8).numpy().tobytes() if t.numel() else b""
        assert data == raw, name
    # and with the package's own reader
    from safetensors import safe_open
    with safe_open(path, framework="pt") as f:
        assert sorted(f.keys()) == sorted(got)


def _raw_file(tmp_path, header, payload=b"", name="x.safetensors", header_len=None):
    text = header if isinstance(header, bytes) else json.dumps(header).encode()
    path = os.path.join(tmp_path, name)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text) if header_len is None else header_len) + text + payload)
    return path


def test_reader_rejects_malformed_files(engine, tmp_path):
    tmp = str(tmp_path)
    good = {"t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}
    assert engine.read_safetensors(_raw_file(tmp, good, b"\0" * 8))["t"][1] == (2,)
    cases = {
        "short file": lambda: open(os.path.join(tmp, "s.safetensors"), "wb").write(b"\1\2\3") and os.path.join(tmp, "s.safetensors"),
        "header longer than the file": lambda: _raw_file(tmp, good, b"\0" * 8, header_len=10 ** 6),
        "zero header": lambda: _raw_file(tmp, b"", b"", header_len=0),
        "tensor beyond the data": lambda: _raw_file(tmp, good, b"\0" * 4),
        "bytes do not match the shape": lambda: _raw_file(tmp, {"t": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}, b"\0" * 8),
        "unknown dtype": lambda: _raw_file(tmp, {"t": {"dtype": "Q4", "shape": [8], "data_offsets": [0, 8]}}, b"\0" * 8),
        "reversed offsets": lambda: _raw_file(tmp, {"t": {"dtype": "U8", "shape": [0], "data_offsets": [4, 2]}}, b"\0" * 8),
        "negative extent": lambda: _raw_file(tmp, {"t": {"dtype": "U8", "shape": [-1], "data_offsets": [0, 0]}}, b""),
        # 2^32 x 2^32 x 2 wraps to 0 elements in 64 bits and would match the empty byte range
        "element count that wraps": lambda: _raw_file(tmp, {"t": {"dtype": "U8", "shape": [4294967296, 4294967296, 2],
                                                                  "data_offsets": [0, 0]}}, b""),
        "extent beyond an int": lambda: _raw_file(tmp, {"t": {"dtype": "U8", "shape": [2147483648, 0], "data_offsets": [0, 0]}}, b""),
        "not JSON": lambda: _raw_file(tmp, b"{\"t\": [1, 2,}", b""),
        "entry without offsets": lambda: _raw_file(tmp, {"t": {"dtype": "U8", "shape": [1]}}, b"\0"),
        "trailing text": lambda: _raw_file(tmp, b"{} x", b""),
    }
    for what, make in cases.items():
        with pytest.raises(engine.EngineError) as err:
            engine.read_safetensors(make())
        assert err.value.code in (-7, -8), what
    with pytest.raises(engine.EngineError) as err:
        engine.read_safetensors(os.path.join(tmp, "does-not-exist.safetensors"))
    assert err.value.code == -7


def test_talker_create_fails_cleanly_without_files(engine, tmp_path):
    import ctypes as C
    handle = C.c_void_p()
    assert engine.lib().qm_talker_create(os.fsencode(str(tmp_path)), 64, None, C.byref(handle)) == -7
    assert not handle.value
    assert b"safetensors" in engine.lib().qm_engine_last_error()
    assert engine.lib().qm_talker_create(None, 64, None, C.byref(handle)) == -1
