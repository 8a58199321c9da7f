"""Helpers shared by the tests: seeded inputs, 16-bit float bit patterns,
device buffers (torch is plumbing for memory only)."""
import ctypes as C

import numpy as np

from deusridet_amd import cabi
from oracle import binding as orc


def f32_to_bf16_bits(x):
    """round-to-nearest-even, numpy restatement (independent of the oracle's C)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return r


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_f16_bits(x):
    return np.ascontiguousarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def f16_bits_to_f32(b):
    return np.ascontiguousarray(b, dtype=np.uint16).view(np.float16).astype(np.float32)


def to_bits(x, dtype):
    return f32_to_bf16_bits(x) if dtype == cabi.BF16 else f32_to_f16_bits(x)


def from_bits(b, dtype):
    return bf16_bits_to_f32(b) if dtype == cabi.BF16 else f16_bits_to_f32(b)


def normal_bits(rng, shape, dtype, mul=1.0):
    return to_bits(rng.standard_normal(shape).astype(np.float32) * np.float32(mul), dtype)


def both_layouts(L, KVH, QH, D, bs, NB, dtype):
    """(product layout, oracle layout) for the same geometry."""
    return cabi.layout(L, KVH, QH, D, bs, NB, dtype), orc.layout(L, KVH, QH, D, bs, NB, dtype)


def shuffled_table(rng, NB, n_logical, max_logical=None):
    perm = rng.permutation(NB).astype(np.int32)
    t = np.full(max_logical or n_logical, -1, dtype=np.int32)
    t[:n_logical] = perm[:n_logical]
    return t


# ---- device plumbing ------------------------------------------------------
def dev_bytes(arr):
    """numpy array -> torch uint8 tensor on the GPU holding the same bytes."""
    import torch
    a = np.ascontiguousarray(arr)
    return torch.from_numpy(a.view(np.uint8).reshape(-1).copy()).cuda()


def dev_zeros(nbytes):
    import torch
    return torch.zeros(int(nbytes), dtype=torch.uint8, device="cuda")


def dev_i32(arr):
    import torch
    return torch.from_numpy(np.ascontiguousarray(arr, dtype=np.int32)).cuda()


def host(t, dtype, shape=None):
    a = t.cpu().numpy().view(dtype)
    return a.reshape(shape) if shape is not None else a


def p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def stream_ptr():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def sync():
    import torch
    torch.cuda.synchronize()


def rel_abs_ok(got, want, rel=1e-2, abs_=2e-2):
    """|got-want| <= abs_ + rel*|want| elementwise (the stated attention tolerance)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    err = np.abs(got - want)
    lim = abs_ + rel * np.abs(want)
    return bool(np.all(err <= lim)), float(err.max()), float((err / np.maximum(np.abs(want), 1e-30)).max())


def ulp_distance(a_bits, b_bits):
    """Distance in units in the last place between two arrays of 16-bit float bit
    patterns (fp16 or bf16: both are sign-magnitude, so the patterns order like
    the values once negative ones are mirrored)."""
    def key(b):
        b = np.ascontiguousarray(b, dtype=np.uint16).astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))
