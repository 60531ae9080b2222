"""CPU-only checks of the C-ABI library: it loads without a GPU, exports every symbol declared in
include/qm_attn.h, and its host-side validation (forceable without a device) matches the
reference's guards (cache overflow R17:16844-16847, geometry R17:14881-14892)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "qm_attn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(qm_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(qm):
    lib = qm.lib()
    names = _declared()
    assert len(names) >= 12
    for name in names:
        assert hasattr(lib, name), f"{name} declared in qm_attn.h but not exported"
    assert sorted(qm.EXPORTS) == names, "binding.py and qm_attn.h disagree on the entry points"
    assert lib.qm_abi_version() == 2
    assert lib.qm_target_arch() == b"gfx950"


def test_error_strings(qm):
    for code in (0, -1, -2, -3, -4, -5, -6):
        assert qm.error_string(code) not in ("", "unknown error")
    assert qm.error_string(-77) == "unknown error"


def _cache(qm, page_size=16, n_pages=4, kv_heads=8, head_dim=128, k=0x1000, v=0x2000):
    c = qm.KvCache(k, v, kv_heads * page_size * 128, page_size * 128, 128, page_size, n_pages, kv_heads, head_dim)
    return c


def test_host_validation_without_device(qm):
    """Every call below must be rejected before any HIP call (there is no GPU here)."""
    lib = qm.lib()
    fake = 0x10000   # never dereferenced
    c = _cache(qm)
    # NULL pointers
    assert lib.qm_qk_norm_rope_kv_append(None, fake, fake, fake, fake, fake, fake, fake, C.byref(c), fake, 4, 16, 0, 1e-6, None) == -1
    assert lib.qm_decode_attention(None, C.byref(c), fake, 4, fake, 16, 0, -1, 0.1, None, 0, None) == -1
    # geometry: head_dim, group, page size that cuts 16-token tiles, misaligned pool
    bad = _cache(qm, head_dim=64)
    assert lib.qm_qk_norm_rope_kv_append(fake, fake, fake, fake, fake, fake, fake, fake, C.byref(bad), fake, 4, 16, 0, 1e-6, None) == -2
    assert lib.qm_decode_attention(fake, C.byref(c), fake, 4, fake, 12, 0, -1, 0.1, None, 0, None) == -2
    odd = _cache(qm, page_size=24)
    assert lib.qm_decode_attention(fake, C.byref(odd), fake, 4, fake, 16, 0, -1, 0.1, None, 0, None) == -2
    mis = _cache(qm, k=0x1008)
    assert lib.qm_decode_attention(fake, C.byref(mis), fake, 4, fake, 16, 0, -1, 0.1, None, 0, None) == -2
    # slot range: the reference's "cache overflow"
    assert lib.qm_qk_norm_rope_kv_append(fake, fake, fake, fake, fake, fake, fake, fake, C.byref(c), fake, 4, 16, 64, 1e-6, None) == -3
    assert lib.qm_qk_norm_rope_kv_append(fake, fake, fake, fake, fake, fake, fake, fake, C.byref(c), fake, 4, 16, -1, 1e-6, None) == -3
    assert lib.qm_decode_attention(fake, C.byref(c), fake, 4, fake, 16, 64, -1, 0.1, None, 0, None) == -3
    assert lib.qm_scatter_kv(fake, fake, C.byref(c), fake, 4, 10, 60, None, None) == -3
    # workspace: long contexts need one
    big = _cache(qm, n_pages=1024)
    need = lib.qm_decode_workspace_bytes(1, 16, 8, 8192)
    assert need > 0
    assert lib.qm_decode_attention(fake, C.byref(big), fake, 1024, fake, 16, 8191, -1, 0.1, None, 0, None) == -4
    assert lib.qm_decode_attention(fake, C.byref(big), fake, 1024, fake, 16, 8191, -1, 0.1, fake, need - 4, None) == -4
    # arguments
    assert lib.qm_decode_attention(fake, C.byref(c), fake, 4, fake, 16, -2, -1, 0.1, None, 0, None) == -5
    assert lib.qm_norm_rope_rows(fake, fake, fake, fake, fake, -1, 16, 1e-6, None) == -5
    assert lib.qm_prefill_attention_causal(fake, fake, fake, fake, None, None, 0, 1, 64, 16, 4, 0.1, 0, 0, 0, None, None) == -2
    # the key-split prefill entry checks its workspace arguments before anything else
    split = lib.qm_prefill_attention_causal_split
    assert split(fake, fake, fake, fake, None, None, 0, 1, 64, 16, 8, 0.1, 0, 0, 0, None, -1, None, None) == -5
    assert split(fake, fake, fake, fake, None, None, 0, 1, 64, 16, 8, 0.1, 0, 0, 0, None, 256, None, None) == -5
    assert split(fake, fake, fake, fake, None, None, 0, 1, 64, 16, 8, 0.1, 0, 0, 0, C.c_void_p(4096 + 16), 256, None, None) == -2
    assert split(fake, fake, fake, fake, None, None, 0, 1, 64, 16, 4, 0.1, 0, 0, 0, None, 0, None, None) == -2
    assert split(fake, fake, fake, fake, None, None, 0, 0, 64, 16, 8, 0.1, 0, 0, 0, None, 0, None, None) == 0
    assert lib.qm_prefill_split_workspace_init(None, 0, None) == 0
    assert lib.qm_prefill_split_workspace_init(None, 256, None) == -1
    assert lib.qm_prefill_split_workspace_init(fake, -1, None) == -5
    assert lib.qm_prefill_split_workspace_bytes(0, 1024, 8) == 0
    assert lib.qm_predictor_attention_loop(fake, fake, fake, fake, fake, fake, fake, fake, None, None, 1, 1, 17, 1, 1e-6, None) == -5
    assert lib.qm_predictor_attention_loop(fake, fake, fake, fake, fake, fake, fake, fake, None, None, 1, 1, 16, 3, 1e-6, None) == -5
    # empty work is a successful no-op
    assert lib.qm_norm_rope_rows(fake, fake, fake, fake, fake, 0, 16, 1e-6, None) == 0
    assert lib.qm_prefill_attention_causal(fake, fake, fake, fake, None, None, 0, 0, 64, 16, 8, 0.1, 0, 0, 0, None, None) == 0
    assert lib.qm_predictor_attention_loop(fake, fake, fake, fake, fake, fake, fake, fake, None, None, 0, 1, 16, 1, 1e-6, None) == 0


def test_options_round_trip_and_validation(qm):
    assert qm.get_option(qm.OPT_PREFILL_SCORE_ROUNDING) == 1      # reference roundings by default
    assert qm.get_option(qm.OPT_DECODE_TILES_PER_BLOCK) == 0
    assert qm.get_option(qm.OPT_PREFILL_KERNEL) == 0 and qm.get_option(qm.OPT_DECODE_STREAMING_LOADS) == 0
    lib = qm.lib()
    assert lib.qm_set_option(99, 1) == -5 and lib.qm_set_option(-1, 1) == -5
    assert lib.qm_set_option(qm.OPT_TALKER_LAYER_OPERATORS + 1, 1) == -5      # one past the last option
    assert qm.get_option(qm.OPT_PREDICTOR_FRAME_OPERATORS) == 0 and qm.get_option(qm.OPT_PREDICTOR_FRAME_SPIN_LIMIT) == 0
    assert lib.qm_set_option(qm.OPT_DECODE_TILES_PER_BLOCK, -3) == -5
    assert lib.qm_get_option(qm.OPT_DECODE_TILES_PER_BLOCK, None) == -1
    base = qm.decode_workspace_bytes(64, 16, 8, 4096)
    qm.set_option(qm.OPT_DECODE_TILES_PER_BLOCK, 4)
    try:
        assert qm.get_option(qm.OPT_DECODE_TILES_PER_BLOCK) == 4
        assert qm.decode_workspace_bytes(64, 16, 8, 4096) > base     # more splits, more partial records
    finally:
        qm.set_option(qm.OPT_DECODE_TILES_PER_BLOCK, 0)
    assert qm.decode_workspace_bytes(64, 16, 8, 4096) == base


def test_a_threads_own_option_value_is_seen_by_that_thread_only(qm):
    import threading
    lib = qm.lib()
    assert lib.qm_set_thread_option(99, 1) == -5 and lib.qm_set_thread_option(qm.OPT_PREFILL_KERNEL, -2) == -5
    assert lib.qm_set_thread_option(qm.OPT_DECODE_TILES_PER_BLOCK, 5000) == -5
    base = qm.decode_workspace_bytes(64, 16, 8, 4096)
    seen = {}

    def other():
        # this thread forces 4-tile blocks for its own calls
        qm.set_thread_option(qm.OPT_DECODE_TILES_PER_BLOCK, 4)
        seen["value"] = qm.get_option(qm.OPT_DECODE_TILES_PER_BLOCK)
        seen["bytes"] = qm.decode_workspace_bytes(64, 16, 8, 4096)
        qm.set_thread_option(qm.OPT_DECODE_TILES_PER_BLOCK, -1)
        seen["after"] = qm.get_option(qm.OPT_DECODE_TILES_PER_BLOCK)

    worker = threading.Thread(target=other)
    worker.start()
    worker.join()
    assert seen["value"] == 4 and seen["bytes"] > base and seen["after"] == 0
    assert qm.get_option(qm.OPT_DECODE_TILES_PER_BLOCK) == 0 and qm.decode_workspace_bytes(64, 16, 8, 4096) == base
    # a thread's own value wins over the process-wide one, and goes away with -1
    qm.set_option(qm.OPT_PREFILL_KERNEL, 1)
    try:
        qm.set_thread_option(qm.OPT_PREFILL_KERNEL, 0)
        assert qm.get_option(qm.OPT_PREFILL_KERNEL) == 0
        qm.set_thread_option(qm.OPT_PREFILL_KERNEL, -1)
        assert qm.get_option(qm.OPT_PREFILL_KERNEL) == 1
    finally:
        qm.set_thread_option(qm.OPT_PREFILL_KERNEL, -1)
        qm.set_option(qm.OPT_PREFILL_KERNEL, 0)


def test_workspace_size_is_monotone_and_pure(qm):
    lib = qm.lib()
    prev = 0
    for L in (1, 16, 63, 64, 512, 2048, 8192, 65536):
        n = lib.qm_decode_workspace_bytes(1, 16, 8, L)
        assert n == lib.qm_decode_workspace_bytes(1, 16, 8, L)
        assert n >= prev
        prev = n
    # a workspace sized for the longest context serves every shorter one, whatever block length the plan picks
    for streams in (1, 3, 64, 1000):
        prev = 0
        for L in range(1, 70000, 29):
            n = lib.qm_decode_workspace_bytes(streams, 16, 8, L)
            assert n >= prev, (streams, L)
            prev = n
    assert lib.qm_decode_workspace_bytes(64, 16, 8, 4096) >= 64 * 8 * 2 * (2 * 128 + 4) * 4
    assert lib.qm_decode_workspace_bytes(0, 16, 8, 10) == 0
    assert lib.qm_decode_workspace_bytes(1, 16, 5, 10) == 0


def test_missing_library_fails_loudly(qm, monkeypatch, tmp_path):
    import importlib
    mod = importlib.import_module("qingming-qwen3-tts_amd.binding")
    monkeypatch.setattr(mod, "_lib", None)
    monkeypatch.setattr(mod, "_LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(FileNotFoundError):
        mod.lib()


def test_cpp_host_adapters_throw_like_the_reference(qm, tmp_path):
    """Compiles tests/host_adapter_check.cpp against include/qm_attn.hpp and the built library."""
    import subprocess
    exe = tmp_path / "host_adapter_check"
    lib_dir = os.path.dirname(qm.lib_path())
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-o", str(exe),
                    os.path.join(ROOT, "tests", "host_adapter_check.cpp"), "-L" + lib_dir, "-lqm_attn",
                    "-Wl,-rpath," + lib_dir, "-Wl,-rpath,/opt/rocm/lib"], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "0 failure(s)" in out.stdout
