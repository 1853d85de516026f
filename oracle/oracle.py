"""ctypes loader for the CPU oracle (oracle/matmul_oracle.c). TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module; the
product package never does.
"""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "build", "liboracle.so")

DT_F16, DT_BF16, DT_F32, DT_I32 = 0, 1, 2, 3


def build(force=False):
    src = os.path.join(HERE, "matmul_oracle.c")
    if force or not os.path.exists(LIB) or os.path.getmtime(LIB) < os.path.getmtime(src):
        subprocess.run(["make", "-C", HERE, "-B"], check=True, capture_output=True)
    return LIB


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        L = ctypes.CDLL(LIB)
        c_int, c_float, c_void_p, c_int64 = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_int64
        L.oracle_half_to_float.restype = c_float
        L.oracle_half_to_float.argtypes = [ctypes.c_uint16]
        L.oracle_bf16_to_float.restype = c_float
        L.oracle_bf16_to_float.argtypes = [ctypes.c_uint16]
        L.oracle_num_threads.restype = c_int
        for name in ("oracle_gemm_rows", "oracle_gemm_blocked"):
            f = getattr(L, name)
            f.restype = c_int
            f.argtypes = [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_float, c_int, c_int, c_int, c_int,
                          c_int, c_int]
        L.oracle_matmul.restype = c_int
        L.oracle_matmul.argtypes = [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                    c_int]
        L.oracle_count_incorrect.restype = c_int64
        L.oracle_count_incorrect.argtypes = [c_void_p, c_void_p, c_int64, c_float]
        L.oracle_count_outside_rel.restype = c_int64
        L.oracle_count_outside_rel.argtypes = [c_void_p, c_void_p, c_int64, c_float, ctypes.POINTER(c_float)]
        L.oracle_get_num_acc.restype = c_int
        L.oracle_get_num_acc.argtypes = [c_int, c_int]
        L.oracle_get_warp_tile_rows.restype = c_int
        L.oracle_get_warp_tile_rows.argtypes = [c_int, c_int]
        L.oracle_get_tile_offset_cd.restype = c_int
        L.oracle_get_tile_offset_cd.argtypes = [c_int] * 5
        L.oracle_get_shmem_req.restype = c_int
        L.oracle_get_shmem_req.argtypes = [c_int] * 10
        _lib = L
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _as_u16(x):
    """fp16 numpy arrays or raw uint16 bit patterns (bf16) -> contiguous uint16 view."""
    x = np.ascontiguousarray(x)
    if x.dtype == np.float16:
        return x.view(np.uint16)
    assert x.dtype == np.uint16, x.dtype
    return x


def gemm(dtype, a, bt, c=None, alpha=1.0, beta=0.0, rows=None, blocked=True, threads=0):
    """alpha * A @ Bt.T + beta * C, fp32, sequential-k accumulation. a: (M,K), bt: (N,K) as fp16 arrays
    or uint16 bit patterns; rows=(begin,end) restricts the output rows."""
    a16, b16 = _as_u16(a), _as_u16(bt)
    M, K = a16.shape
    N, K2 = b16.shape
    assert K == K2
    r0, r1 = (0, M) if rows is None else rows
    out = np.empty((r1 - r0, N), dtype=np.float32)
    cc = None if c is None else np.ascontiguousarray(c, dtype=np.float32)
    fn = lib().oracle_gemm_blocked if blocked else lib().oracle_gemm_rows
    rc = fn(dtype, _ptr(a16), _ptr(b16), _ptr(cc), _ptr(out), alpha, beta, M, N, K, r0, r1, threads)
    assert rc == 0, rc
    return out


def matmul(dtype, a, b, b_transposed=False, fused=False, rows=None, threads=0):
    """matmul_shmem check. Returns float32 (F32/F16 inputs, not yet rounded to the element type) or int32."""
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    M, K = a.shape
    N = b.shape[0] if b_transposed else b.shape[1]
    r0, r1 = (0, M) if rows is None else rows
    out = np.empty((r1 - r0, N), dtype=np.int32 if dtype == DT_I32 else np.float32)
    av = a.view(np.uint16) if a.dtype == np.float16 else a
    bv = b.view(np.uint16) if b.dtype == np.float16 else b
    rc = lib().oracle_matmul(dtype, _ptr(av), _ptr(bv), _ptr(out), M, N, K, int(b_transposed), int(fused), r0, r1, threads)
    assert rc == 0, rc
    return out


def count_incorrect(expected, res, atol):
    e = np.ascontiguousarray(expected, dtype=np.float32)
    r = np.ascontiguousarray(res, dtype=np.float32)
    return int(lib().oracle_count_incorrect(_ptr(e), _ptr(r), e.size, atol))


def count_outside_rel(ref, res, rtol):
    """(#elements with |res-ref| > rtol*(|ref|+1), worst ratio)"""
    e = np.ascontiguousarray(ref, dtype=np.float32)
    r = np.ascontiguousarray(res, dtype=np.float32)
    worst = ctypes.c_float(0)
    n = int(lib().oracle_count_outside_rel(_ptr(e), _ptr(r), e.size, rtol, ctypes.byref(worst)))
    return n, float(worst.value)


# ---- numpy restatement of the input generator (checks the product's C generator) ------------------
_GOLD = np.uint64(0x9E3779B97F4A7C15)


def splitmix64_at(base, idx):
    """Outputs idx (array, 0-based) of SplitMix64 started at state `base` (published algorithm, S. Vigna)."""
    with np.errstate(over="ignore"):
        z = np.uint64(base) + (idx.astype(np.uint64) + np.uint64(1)) * _GOLD
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def stream_base(seed, stream_id):
    return (int(seed) + int(stream_id) * 0xD1342543DE82EF95) & 0xFFFFFFFFFFFFFFFF


def uniform_f32(n, seed, stream_id, lo, hi):
    z = splitmix64_at(stream_base(seed, stream_id), np.arange(n, dtype=np.uint64))
    u = (z >> np.uint64(40)).astype(np.float32) * np.float32(1.0 / 16777216.0)
    return np.float32(lo) + u * (np.float32(hi) - np.float32(lo))
