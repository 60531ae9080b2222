"""MI355X (gfx950) attention / KV-cache operators behind a C ABI.

The product is lib/libqm_attn.so (HIP kernels + the entry points declared in
include/qm_attn.h).  `binding` is a thin ctypes layer used by the tests and the benchmark;
it has no CPU fallback and raises if the library is missing.
"""
from . import binding  # noqa: F401
from .binding import QmError, KvCache, lib, lib_path  # noqa: F401
