"""ctypes front-end of the CPU oracle (oracle/kx_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py, never by the package that ships.  All arrays are numpy;
16-bit floats travel as uint16 bit patterns so that no library cast sits between the
caller and the oracle.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

ORDER = (0, 2, 4, 6, 1, 3, 5, 7)


def build(force=False):
    """Compile oracle/kx_oracle.c with the Makefile beside it."""
    cmd = ["make", "-C", _HERE] + (["-B"] if force else [])
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


_P = ctypes.c_void_p
_I = ctypes.c_int64


def _declare(L):
    L.kxo_f32_to_bf16_n.argtypes = [_P, _P, ctypes.c_size_t]
    L.kxo_bf16_to_f32_n.argtypes = [_P, _P, ctypes.c_size_t]
    L.kxo_f32_to_f16_n.argtypes = [_P, _P, ctypes.c_size_t]
    L.kxo_f16_to_f32_n.argtypes = [_P, _P, ctypes.c_size_t]
    for f in (L.kxo_f32_to_bf16_n, L.kxo_bf16_to_f32_n, L.kxo_f32_to_f16_n, L.kxo_f16_to_f32_n):
        f.restype = None
    L.kxo_awq_pack.argtypes = [_P, _I, _I, _P]
    L.kxo_awq_unpack.argtypes = [_P, _I, _I, _P]
    L.kxo_awq_dequant_bf16.argtypes = [_P, _P, _P, _I, _I, _I, _P]
    L.kxo_awq_dequant_one.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint16]
    L.kxo_awq_dequant_one.restype = ctypes.c_uint16
    L.kxo_gemv_awq_f64.argtypes = [_P, _P, _P, _P, _I, _I, _I, _I, _P]
    L.kxo_gemv_awq_f32.argtypes = [_P, _P, _P, _P, _I, _I, _I, _I, _P]
    L.kxo_gemv_awq_f32_range.argtypes = [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P]
    L.kxo_gemv_awq_f32_range.restype = ctypes.c_int
    L.kxo_gemv_bf16_f64.argtypes = [_P, _P, _I, _I, _I, _P]
    L.kxo_gemv_bf16_f32.argtypes = [_P, _P, _I, _I, _I, _P]
    for f in (L.kxo_awq_pack, L.kxo_awq_unpack, L.kxo_awq_dequant_bf16, L.kxo_gemv_awq_f64,
              L.kxo_gemv_awq_f32, L.kxo_gemv_bf16_f64, L.kxo_gemv_bf16_f32):
        f.restype = ctypes.c_int


def _c(a, dtype):
    a = np.ascontiguousarray(a)
    if a.dtype != np.dtype(dtype):
        raise TypeError(f"expected {np.dtype(dtype)}, got {a.dtype}")
    return a


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _check(rc, what):
    if rc != 0:
        raise ValueError(f"oracle {what} rejected its arguments (code {rc})")


# ---------------------------------------------------------------- conversions
def f32_to_bf16(a):
    a = _c(a, np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().kxo_f32_to_bf16_n(_ptr(a), _ptr(out), a.size)
    return out


def bf16_to_f32(a):
    a = _c(a, np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().kxo_bf16_to_f32_n(_ptr(a), _ptr(out), a.size)
    return out


def f32_to_f16(a):
    a = _c(a, np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().kxo_f32_to_f16_n(_ptr(a), _ptr(out), a.size)
    return out


def f16_to_f32(a):
    a = _c(a, np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().kxo_f16_to_f32_n(_ptr(a), _ptr(out), a.size)
    return out


# ---------------------------------------------------------------- nibble stream
def awq_pack(codes):
    codes = _c(codes, np.uint8)
    rows, cols = codes.shape
    out = np.empty((rows, cols // 8), np.int32)
    _check(lib().kxo_awq_pack(_ptr(codes), rows, cols, _ptr(out)), "awq_pack")
    return out


def awq_unpack(words):
    words = _c(words, np.int32)
    rows, wcols = words.shape
    out = np.empty((rows, wcols * 8), np.uint8)
    _check(lib().kxo_awq_unpack(_ptr(words), rows, wcols * 8, _ptr(out)), "awq_unpack")
    return out


# ---------------------------------------------------------------- dequant
def awq_dequant_bf16(qweight, scales_f16, qzeros, group):
    qweight = _c(qweight, np.int32)
    scales_f16 = _c(scales_f16, np.uint16)
    qzeros = _c(qzeros, np.int32)
    K, wcols = qweight.shape
    N = wcols * 8
    out = np.empty((K, N), np.uint16)
    _check(lib().kxo_awq_dequant_bf16(_ptr(qweight), _ptr(scales_f16), _ptr(qzeros), K, N, group,
                                      _ptr(out)), "awq_dequant_bf16")
    return out


def awq_dequant_one(q, z, scale_bits):
    return int(lib().kxo_awq_dequant_one(int(q), int(z), int(scale_bits)))


# ---------------------------------------------------------------- GEMV
def _awq_args(x_bf16, qweight, scales_f16, qzeros, group):
    x_bf16 = _c(x_bf16, np.uint16)
    qweight = _c(qweight, np.int32)
    scales_f16 = _c(scales_f16, np.uint16)
    qzeros = _c(qzeros, np.int32)
    if x_bf16.ndim == 1:
        x_bf16 = x_bf16[None, :]
    M, K = x_bf16.shape
    N = qweight.shape[1] * 8
    if qweight.shape[0] != K or scales_f16.shape != (K // group, N) or \
            qzeros.shape != (K // group, N // 8):
        raise ValueError("inconsistent AWQ tensor shapes")
    return x_bf16, qweight, scales_f16, qzeros, M, K, N


def gemv_awq_f64(x_bf16, qweight, scales_f16, qzeros, group):
    x_bf16, qweight, scales_f16, qzeros, M, K, N = _awq_args(x_bf16, qweight, scales_f16, qzeros,
                                                             group)
    y = np.empty((M, N), np.float64)
    _check(lib().kxo_gemv_awq_f64(_ptr(x_bf16), _ptr(qweight), _ptr(scales_f16), _ptr(qzeros),
                                  M, K, N, group, _ptr(y)), "gemv_awq_f64")
    return y


def gemv_awq_f32(x_bf16, qweight, scales_f16, qzeros, group):
    x_bf16, qweight, scales_f16, qzeros, M, K, N = _awq_args(x_bf16, qweight, scales_f16, qzeros,
                                                             group)
    y = np.empty((M, N), np.uint16)
    _check(lib().kxo_gemv_awq_f32(_ptr(x_bf16), _ptr(qweight), _ptr(scales_f16), _ptr(qzeros),
                                  M, K, N, group, _ptr(y)), "gemv_awq_f32")
    return y


def gemv_awq_f32_threads(x_bf16, qweight, scales_f16, qzeros, group, threads):
    """The fp32 evaluation spread over `threads` host threads, each a contiguous range of word columns
    (the C call releases the interpreter lock).  Same bits as gemv_awq_f32 for any thread count."""
    from concurrent.futures import ThreadPoolExecutor
    x_bf16, qweight, scales_f16, qzeros, M, K, N = _awq_args(x_bf16, qweight, scales_f16, qzeros,
                                                             group)
    y = np.empty((M, N), np.uint16)
    wcols = N // 8
    threads = max(1, min(threads, wcols))
    bounds = [wcols * t // threads for t in range(threads + 1)]

    def work(t):
        return lib().kxo_gemv_awq_f32_range(_ptr(x_bf16), _ptr(qweight), _ptr(scales_f16), _ptr(qzeros),
                                            M, K, N, group, bounds[t], bounds[t + 1], _ptr(y))

    with ThreadPoolExecutor(max_workers=threads) as pool:
        for rc in pool.map(work, range(threads)):
            _check(rc, "gemv_awq_f32_range")
    return y


def gemv_bf16_f64(x_bf16, w_bf16):
    x_bf16 = _c(x_bf16, np.uint16)
    w_bf16 = _c(w_bf16, np.uint16)
    if x_bf16.ndim == 1:
        x_bf16 = x_bf16[None, :]
    M, K = x_bf16.shape
    N = w_bf16.shape[0]
    if w_bf16.shape[1] != K:
        raise ValueError("inconsistent BF16 GEMV shapes")
    y = np.empty((M, N), np.float64)
    _check(lib().kxo_gemv_bf16_f64(_ptr(x_bf16), _ptr(w_bf16), M, K, N, _ptr(y)), "gemv_bf16_f64")
    return y


def gemv_bf16_f32(x_bf16, w_bf16):
    x_bf16 = _c(x_bf16, np.uint16)
    w_bf16 = _c(w_bf16, np.uint16)
    if x_bf16.ndim == 1:
        x_bf16 = x_bf16[None, :]
    M, K = x_bf16.shape
    N = w_bf16.shape[0]
    if w_bf16.shape[1] != K:
        raise ValueError("inconsistent BF16 GEMV shapes")
    y = np.empty((M, N), np.uint16)
    _check(lib().kxo_gemv_bf16_f32(_ptr(x_bf16), _ptr(w_bf16), M, K, N, _ptr(y)), "gemv_bf16_f32")
    return y
