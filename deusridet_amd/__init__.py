"""MI355X-native paged KV cache hot path (DeusRidet Memoria/Machina drop-in).

The product is the C-ABI library ``lib/libdrk_kv.so`` (hand-written HIP kernels
for gfx950, declared in ``include/drk_kv.h``) and the C++ host classes built on
it (``lib/libdeusridet_memoria.so``).  The Python modules here are thin ctypes
bindings used by the tests and the benchmark; they load the built libraries and
raise if those are missing -- there is no fallback path.
"""
from . import cabi  # noqa: F401

__all__ = ["cabi"]
