"""ctypes loader for the CPU oracle (oracle/liboracle.so, built from tuna_oracle.c).

TEST INFRASTRUCTURE ONLY.  Importers: tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  Nothing under tuna_amd/ may import this module.

All fp16 data crosses this boundary as numpy uint16 bit patterns (use
``.view(np.float16)`` to look at values); layouts follow the reference's
tensors (extension.cpp:26-49):
    q       uint8  [m/8, k/8, 32]   packed codes
    x       fp16   [n, k]
    code    fp32   [16]
    absmax  fp32   [m]
    out     fp16   [n, m]           (dequant: [m, k])
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

D1 = 1  # GEMM in-register decode (kernel.cu:2178-2192): fp16(code) * fp16(absmax) in fp16
D2 = 2  # dequant op decode (kernel.cu:3222-3228): fp32 multiply, then round to fp16


def build(force: bool = False) -> str:
    """Compile liboracle.so with gcc (make -C oracle)."""
    if force or not os.path.exists(_LIB_PATH):
        if force and os.path.exists(_LIB_PATH):
            os.remove(_LIB_PATH)
        subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i32, f32, f64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_double
        L.orc_f16_to_f32.restype = f32
        L.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_f32_to_f16.restype = ctypes.c_uint16
        L.orc_f32_to_f16.argtypes = [f32]
        L.orc_f64_to_f16.restype = ctypes.c_uint16
        L.orc_f64_to_f16.argtypes = [f64]
        L.orc_decode_d1.restype = ctypes.c_uint16
        L.orc_decode_d1.argtypes = [f32, f32]
        L.orc_decode_d2.restype = ctypes.c_uint16
        L.orc_decode_d2.argtypes = [f32, f32]
        L.orc_nf4_codebook.restype = None
        L.orc_nf4_codebook.argtypes = [vp]
        L.orc_pack.restype = i32
        L.orc_pack.argtypes = [vp, vp, i32, i32]
        L.orc_unpack.restype = i32
        L.orc_unpack.argtypes = [vp, vp, i32, i32]
        L.orc_dequant.restype = i32
        L.orc_dequant.argtypes = [vp, vp, vp, vp, i32, i32, i32]
        L.orc_quantize.restype = i32
        L.orc_quantize.argtypes = [vp, vp, vp, vp, i32, i32]
        L.orc_quantize_blk.restype = i32
        L.orc_quantize_blk.argtypes = [vp, vp, vp, vp, i32, i32, i32]
        L.orc_dequant_blk.restype = i32
        L.orc_dequant_blk.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32]
        L.orc_gemm_rows_f64_blk.restype = i32
        L.orc_gemm_rows_f64_blk.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, vp, i32]
        L.orc_gemm.restype = i32
        L.orc_gemm.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32]
        L.orc_gemm_rows.restype = i32
        L.orc_gemm_rows.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, vp, i32]
        L.orc_gemm_rows_f64.restype = i32
        L.orc_gemm_rows_f64.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, vp, i32]
        L.orc_max_threads.restype = i32
        L.orc_max_threads.argtypes = []
        L.orc_cpu_baseline.restype = i32
        L.orc_cpu_baseline.argtypes = [vp, vp, vp, vp, vp, vp, i32, i32, i32, i32,
                                       ctypes.POINTER(f64), ctypes.POINTER(f64)]
        L.orc_f32_to_f16_many.restype = None
        L.orc_f32_to_f16_many.argtypes = [vp, vp, ctypes.c_size_t]
        L.orc_f64_to_f16_many.restype = None
        L.orc_f64_to_f16_many.argtypes = [vp, vp, ctypes.c_size_t]
        L.orc_f16_to_f32_many.restype = None
        L.orc_f16_to_f32_many.argtypes = [vp, vp, ctypes.c_size_t]
        L.orc_decode_many.restype = None
        L.orc_decode_many.argtypes = [vp, vp, vp, ctypes.c_size_t, i32]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16 and dtype == np.uint16:
        a = a.view(np.uint16)
    assert a.dtype == dtype, (a.dtype, dtype)
    return a


def nf4_codebook() -> np.ndarray:
    out = np.empty(16, np.float32)
    lib().orc_nf4_codebook(_p(out))
    return out


def f32_to_f16(v) -> np.ndarray:
    """float32 array -> fp16 bit patterns (uint16), RN-even."""
    v = np.ascontiguousarray(v, np.float32).ravel()
    out = np.empty(v.size, np.uint16)
    lib().orc_f32_to_f16_many(_p(v), _p(out), v.size)
    return out


def f64_to_f16(v) -> np.ndarray:
    v = np.ascontiguousarray(v, np.float64).ravel()
    out = np.empty(v.size, np.uint16)
    lib().orc_f64_to_f16_many(_p(v), _p(out), v.size)
    return out


def f16_to_f32(h) -> np.ndarray:
    h = np.ascontiguousarray(h, np.uint16).ravel()
    out = np.empty(h.size, np.float32)
    lib().orc_f16_to_f32_many(_p(h), _p(out), h.size)
    return out


def decode(code, absmax, mode) -> np.ndarray:
    """Elementwise decode of (code[i], absmax[i]) pairs -> fp16 bit patterns."""
    code = np.ascontiguousarray(code, np.float32).ravel()
    absmax = np.ascontiguousarray(absmax, np.float32).ravel()
    assert code.size == absmax.size
    out = np.empty(code.size, np.uint16)
    lib().orc_decode_many(_p(code), _p(absmax), _p(out), code.size, mode)
    return out


def pack(codes: np.ndarray) -> np.ndarray:
    """codes uint8 [m, k] (values 0..15) -> q uint8 [m/8, k/8, 32] (test.py:58-65)."""
    codes = _c(codes, np.uint8)
    m, k = codes.shape
    q = np.empty((m // 8, k // 8, 32), np.uint8)
    rc = lib().orc_pack(_p(codes), _p(q), m, k)
    if rc:
        raise ValueError(f"orc_pack rc={rc}")
    return q


def unpack(q: np.ndarray, m: int, k: int) -> np.ndarray:
    q = _c(q, np.uint8)
    codes = np.empty((m, k), np.uint8)
    rc = lib().orc_unpack(_p(q), _p(codes), m, k)
    if rc:
        raise ValueError(f"orc_unpack rc={rc}")
    return codes


def dequant(q, absmax, code, m, k, mode=D2, block_size=None) -> np.ndarray:
    """-> fp16 bit patterns uint16 [m, k].  block_size: weights per scale along a row (absmax is then
    [m, k/block_size]); None = one scale per row."""
    q, absmax, code = _c(q, np.uint8), _c(absmax, np.float32), _c(code, np.float32)
    bs = k if block_size is None else int(block_size)
    assert absmax.size == m * (k // bs)
    out = np.empty((m, k), np.uint16)
    rc = lib().orc_dequant_blk(_p(q), _p(absmax), _p(code), _p(out), m, k, mode, bs)
    if rc:
        raise ValueError(f"orc_dequant rc={rc}")
    return out


def quantize(w_bits, code, m, k, block_size=None):
    """fp16 bit patterns [m, k] -> (packed uint8 [m/8, k/8, 32], absmax float32 [m] or [m, k/block_size])."""
    w_bits, code = _c(w_bits, np.uint16), _c(code, np.float32)
    bs = k if block_size is None else int(block_size)
    q = np.empty((m // 8, k // 8, 32), np.uint8)
    absmax = np.empty(m * (k // bs), np.float32)
    rc = lib().orc_quantize_blk(_p(w_bits), _p(code), _p(q), _p(absmax), m, k, bs)
    if rc:
        raise ValueError(f"orc_quantize rc={rc}")
    return q, (absmax if block_size is None else absmax.reshape(m, k // bs))


def gemm(q, x, code, absmax, m, n, k, mode=D1, acc64=True, rows=None) -> np.ndarray:
    """-> fp16 bit patterns uint16 [n, m] (or [n, len(rows)])."""
    q, absmax, code = _c(q, np.uint8), _c(absmax, np.float32), _c(code, np.float32)
    x = _c(x, np.uint16)
    assert x.shape == (n, k)
    if rows is None:
        out = np.empty((n, m), np.uint16)
        rc = lib().orc_gemm(_p(q), _p(x), _p(code), _p(absmax), _p(out), m, n, k, mode, int(acc64))
    else:
        rows = np.ascontiguousarray(rows, np.int32)
        out = np.empty((n, len(rows)), np.uint16)
        rc = lib().orc_gemm_rows(_p(q), _p(x), _p(code), _p(absmax), _p(out), m, n, k, mode,
                                 int(acc64), _p(rows), len(rows))
    if rc:
        raise ValueError(f"orc_gemm rc={rc}")
    return out


def gemm_f64(q, x, code, absmax, m, n, k, mode=D1, rows=None, block_size=None) -> np.ndarray:
    """Un-rounded float64 sums, [n, m] (or [n, len(rows)]).  block_size as in dequant."""
    q, absmax, code = _c(q, np.uint8), _c(absmax, np.float32), _c(code, np.float32)
    x = _c(x, np.uint16)
    bs = k if block_size is None else int(block_size)
    assert absmax.size == m * (k // bs)
    if rows is None:
        rows_a, nr, rp = None, m, None
    else:
        rows_a = np.ascontiguousarray(rows, np.int32)
        nr, rp = len(rows_a), _p(rows_a)
    out = np.empty((n, nr), np.float64)
    rc = lib().orc_gemm_rows_f64_blk(_p(q), _p(x), _p(code), _p(absmax), _p(out), m, n, k, mode, bs, rp, nr)
    if rc:
        raise ValueError(f"orc_gemm_rows_f64 rc={rc}")
    return out


def max_threads() -> int:
    return lib().orc_max_threads()


def cpu_baseline(q, x, code, absmax, m, n, k, threads=None):
    """Dequantize (D2) then matmul (fp32 accumulate) on the host.

    Returns (out uint16 [n, m], seconds_decode, seconds_matmul, threads_used)."""
    q, absmax, code = _c(q, np.uint8), _c(absmax, np.float32), _c(code, np.float32)
    x = _c(x, np.uint16)
    if threads is None:
        threads = max_threads()
    out = np.empty((n, m), np.uint16)
    wbuf = np.empty((m, k), np.uint16)
    td, tm = ctypes.c_double(0), ctypes.c_double(0)
    rc = lib().orc_cpu_baseline(_p(q), _p(x), _p(code), _p(absmax), _p(out), _p(wbuf), m, n, k,
                                int(threads), ctypes.byref(td), ctypes.byref(tm))
    if rc:
        raise ValueError(f"orc_cpu_baseline rc={rc}")
    return out, td.value, tm.value, int(threads)
