"""CPU oracle for the tiled GEMM path -- TEST INFRASTRUCTURE ONLY.

ctypes front end of oracle/frisk_oracle.c.  Only tests, the smoke check and the
CPU-baseline leg of bench.py may import this package; nothing under frisk_amd/
does.  See the header of frisk_oracle.c for what each routine restates and how
it is pinned.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libfrisk_oracle.so")

F32, F16, BF16, I8, E4M3, I32 = 0, 1, 2, 3, 4, 5
NP_STORAGE = {F32: np.float32, F16: np.uint16, BF16: np.uint16, I8: np.int8, E4M3: np.uint8, I32: np.int32}


def build():
    subprocess.run(["make", "-C", _HERE, "-B"], check=True, capture_output=True)
    return _LIB_PATH


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    i64, u64, c_int, vp, f32 = ctypes.c_int64, ctypes.c_uint64, ctypes.c_int, ctypes.c_void_p, ctypes.c_float
    lib.oracle_hash.restype = u64
    lib.oracle_hash.argtypes = [u64, u64, u64]
    lib.oracle_fill_uniform_f32.argtypes = [vp, i64, u64, u64, f32, f32]
    lib.oracle_fill_normal_f32.argtypes = [vp, i64, u64, u64, f32]
    lib.oracle_fill_int8.argtypes = [vp, i64, u64, u64, c_int, c_int]
    lib.oracle_encode.argtypes = [c_int, vp, vp, i64]
    lib.oracle_decode.argtypes = [c_int, vp, vp, i64]
    for name in ("oracle_f32_to_f16", "oracle_f32_to_bf16"):
        getattr(lib, name).restype = ctypes.c_uint16
        getattr(lib, name).argtypes = [f32]
    lib.oracle_f32_to_e4m3.restype = ctypes.c_uint8
    lib.oracle_f32_to_e4m3.argtypes = [f32]
    lib.oracle_gemm_naive.argtypes = [c_int, c_int, c_int, i64, i64, i64, vp, i64, vp, i64, vp]
    lib.oracle_gemm_f64.argtypes = [c_int, c_int, c_int, i64, i64, i64, vp, i64, vp, i64, i64, i64, vp]
    lib.oracle_gemm_f32.argtypes = [c_int, c_int, c_int, i64, i64, i64, vp, i64, vp, i64, i64, i64, vp]
    lib.oracle_gemm_i32.argtypes = [c_int, c_int, i64, i64, i64, vp, i64, vp, i64, i64, i64, vp]
    lib.oracle_epilogue_rowcol_f16.argtypes = [vp, i64, i64, vp, vp, vp]
    lib.oracle_epilogue_rowcol_f32.argtypes = [vp, i64, i64, vp, vp, vp]
    lib.oracle_epilogue_tensor_f64.argtypes = [vp, i64, f32, f32]
    lib.oracle_compare.argtypes = [c_int, vp, vp, i64, vp]
    lib.oracle_num_threads.restype = c_int
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


# ---------------------------------------------------------------- inputs
def uniform(n, seed, tensor, lo, hi):
    out = np.empty(n, dtype=np.float32)
    lib().oracle_fill_uniform_f32(_p(out), out.size, seed, tensor, lo, hi)
    return out


def normal(n, seed, tensor, scale=1.0):
    out = np.empty(n, dtype=np.float32)
    lib().oracle_fill_normal_f32(_p(out), out.size, seed, tensor, scale)
    return out


def int8_uniform(n, seed, tensor, lo=-127, hi=127):
    out = np.empty(n, dtype=np.int8)
    lib().oracle_fill_int8(_p(out), out.size, seed, tensor, lo, hi)
    return out


def encode(dtype, x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=NP_STORAGE[dtype])
    lib().oracle_encode(dtype, _p(x), _p(out), x.size)
    return out


def decode(dtype, x):
    x = np.ascontiguousarray(x)
    out = np.empty(x.shape, dtype=np.float32)
    lib().oracle_decode(dtype, _p(x), _p(out), x.size)
    return out


# ---------------------------------------------------------------- GEMM
def _dims(A, B, transA, transB):
    M, K = (A.shape[1], A.shape[0]) if transA else A.shape
    N = B.shape[0] if transB else B.shape[1]
    Kb = B.shape[1] if transB else B.shape[0]
    assert K == Kb, "inner dimensions differ"
    return M, N, K


def gemm_naive(dtype, A, B, transA=False, transB=False):
    A, B = np.ascontiguousarray(A), np.ascontiguousarray(B)
    M, N, K = _dims(A, B, transA, transB)
    C = np.empty((M, N), dtype=np.float64)
    rc = lib().oracle_gemm_naive(dtype, int(transA), int(transB), M, N, K, _p(A), A.shape[1], _p(B), B.shape[1], _p(C))
    assert rc == 0
    return C


def gemm_f64(dtype, A, B, transA=False, transB=False, row0=0, nrows=None):
    """rows [row0, row0+nrows) of op(A).op(B), double accumulation"""
    A, B = np.ascontiguousarray(A), np.ascontiguousarray(B)
    M, N, K = _dims(A, B, transA, transB)
    nrows = M - row0 if nrows is None else nrows
    C = np.empty((nrows, N), dtype=np.float64)
    rc = lib().oracle_gemm_f64(dtype, int(transA), int(transB), M, N, K, _p(A), A.shape[1], _p(B), B.shape[1], row0, nrows, _p(C))
    assert rc == 0
    return C


def gemm_f32(dtype, A, B, transA=False, transB=False, row0=0, nrows=None):
    """same in fp32 arithmetic (the timed CPU baseline)"""
    A, B = np.ascontiguousarray(A), np.ascontiguousarray(B)
    M, N, K = _dims(A, B, transA, transB)
    nrows = M - row0 if nrows is None else nrows
    C = np.empty((nrows, N), dtype=np.float32)
    rc = lib().oracle_gemm_f32(dtype, int(transA), int(transB), M, N, K, _p(A), A.shape[1], _p(B), B.shape[1], row0, nrows, _p(C))
    assert rc == 0
    return C


def gemm_i32(A, B, transA=False, transB=False, row0=0, nrows=None):
    """exact int8 x int8 -> int32"""
    A, B = np.ascontiguousarray(A, dtype=np.int8), np.ascontiguousarray(B, dtype=np.int8)
    M, N, K = _dims(A, B, transA, transB)
    nrows = M - row0 if nrows is None else nrows
    C = np.empty((nrows, N), dtype=np.int32)
    rc = lib().oracle_gemm_i32(int(transA), int(transB), M, N, K, _p(A), A.shape[1], _p(B), B.shape[1], row0, nrows, _p(C))
    assert rc == 0
    return C


def epilogue_rowcol_f16(acc, sA, sB):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    sA, sB = np.ascontiguousarray(sA, dtype=np.float32), np.ascontiguousarray(sB, dtype=np.float32)
    out = np.empty(acc.shape, dtype=np.uint16)
    lib().oracle_epilogue_rowcol_f16(_p(acc), acc.shape[0], acc.shape[1], _p(sA), _p(sB), _p(out))
    return out


def epilogue_rowcol_f32(acc, sA, sB):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    sA, sB = np.ascontiguousarray(sA, dtype=np.float32), np.ascontiguousarray(sB, dtype=np.float32)
    out = np.empty(acc.shape, dtype=np.float32)
    lib().oracle_epilogue_rowcol_f32(_p(acc), acc.shape[0], acc.shape[1], _p(sA), _p(sB), _p(out))
    return out


def epilogue_tensor(acc64, sA, sB):
    out = np.array(acc64, dtype=np.float64, copy=True)
    lib().oracle_epilogue_tensor_f64(_p(out), out.size, float(sA), float(sB))
    return out


def compare(dtype_out, got, ref64):
    """returns dict(max_rel, fro_rel, rms, nonfinite); max_rel = max |d-r| / max(|r|, rms(R))"""
    got = np.ascontiguousarray(got)
    ref64 = np.ascontiguousarray(ref64, dtype=np.float64)
    assert got.size == ref64.size
    res = np.zeros(4, dtype=np.float64)
    lib().oracle_compare(dtype_out, _p(got), _p(ref64), got.size, _p(res))
    return {"max_rel": float(res[0]), "fro_rel": float(res[1]), "rms": float(res[2]), "nonfinite": int(res[3])}


def num_threads():
    return int(lib().oracle_num_threads())
