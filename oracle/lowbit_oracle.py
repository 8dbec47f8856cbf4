"""ctypes front end of the CPU oracle (TEST INFRASTRUCTURE - not product code).

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module.  It loads ``liblowbit_oracle.so`` (built
from ``lowbit_oracle.c`` by ``oracle/Makefile``) and exposes numpy-in /
numpy-out helpers named after the reference calls they stand for
(python/llm/src/ipex_llm/ggml/model/llama/llama_cpp.py:945-1185).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liblowbit_oracle.so")

QTYPES = {"sym_int4": 2, "asym_int4": 3, "sym_int8": 8, "nf4": 10, "fp8_e4m3": 15}


def build(force=False):
    """Compile the C restatement (gcc only; no GPU toolchain involved)."""
    if force or not os.path.exists(_SO) or \
            os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "lowbit_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liblowbit_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def use_fast_build():
    """Switches to the -O3 AVX2 build of the same source (for timing only: bench.py's cpu_baseline).  Has to be
    called before the first use; returns the ISA string of the build that will be loaded."""
    global _SO
    fast = os.path.join(_HERE, "liblowbit_oracle_avx2.so")
    try:
        flags = open("/proc/cpuinfo").read().split("flags", 1)[1].split("\n", 1)[0].split()
    except Exception:  # noqa: BLE001
        flags = []
    if _lib is None and os.path.exists(fast) and all(f in flags for f in ("avx2", "fma", "f16c")):
        _SO = fast
        return "gcc -O3 -mavx2 -mfma -mf16c (auto-vectorized C)"
    return "gcc -O2 (portable x86-64 C)"


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        L.oracle_qk_size.argtypes = [ctypes.c_int]
        L.oracle_qk_size.restype = ctypes.c_int
        L.oracle_type_size.argtypes = [ctypes.c_int]
        L.oracle_type_size.restype = ctypes.c_size_t
        L.oracle_quantize_tensor.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                             ctypes.c_size_t, ctypes.c_int]
        L.oracle_quantize_tensor.restype = ctypes.c_size_t
        L.oracle_dequantize.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                                        ctypes.c_int]
        L.oracle_dequantize.restype = None
        for name in ("oracle_mul_mat_q_fp32", "oracle_mul_mat_exact"):
            f = getattr(L, name)
            f.argtypes = [ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p, ctypes.c_int,
                          ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p, ctypes.c_void_p]
            f.restype = None
        L.oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.oracle_f32_to_f16.restype = ctypes.c_uint16
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f16_to_f32.restype = ctypes.c_float
        L.oracle_f32_to_e4m3fn.argtypes = [ctypes.c_float]
        L.oracle_f32_to_e4m3fn.restype = ctypes.c_uint8
        L.oracle_e4m3fn_to_f32.argtypes = [ctypes.c_uint8]
        L.oracle_e4m3fn_to_f32.restype = ctypes.c_float
        L.oracle_nf4_codebook.argtypes = []
        L.oracle_nf4_codebook.restype = ctypes.POINTER(ctypes.c_float)
        L.oracle_max_threads.argtypes = []
        L.oracle_max_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def qk_size(qtype):
    return lib().oracle_qk_size(qtype)


def type_size(qtype):
    return lib().oracle_type_size(qtype)


def blob_bytes(qtype, n_weights):
    return (n_weights // qk_size(qtype)) * type_size(qtype)


def quantize(w, qtype):
    """fp32 array [..., K] -> 1-D uint8 ggml blob (low_bit_linear.py:104-175)."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    k = w.shape[-1]
    qk = qk_size(qtype)
    if qk == 0:
        raise ValueError(f"unsupported qtype {qtype}")
    if k % qk:
        raise ValueError(f"last dim must be a multiple of {qk}")
    out = np.empty(blob_bytes(qtype, w.size), dtype=np.uint8)
    if w.size:
        written = lib().oracle_quantize_tensor(w.ctypes.data, out.ctypes.data, qtype, w.size, k)
        assert written == out.size
    return out


def dequantize(blob, qtype, shape):
    """1-D uint8 ggml blob -> fp32 array of `shape` (low_bit_linear.py:249-259)."""
    blob = np.ascontiguousarray(blob, dtype=np.uint8)
    n = int(np.prod(shape))
    assert blob.size == blob_bytes(qtype, n)
    out = np.empty(n, dtype=np.float32)
    if n:
        lib().oracle_dequantize(blob.ctypes.data, out.ctypes.data, n, qtype)
    return out.reshape(shape)


def _mm(fn, blob, x, shape, qtype):
    n_rows, k = shape
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.ndim == 2 and x.shape[1] == k
    blob = np.ascontiguousarray(blob, dtype=np.uint8)
    out = np.empty((x.shape[0], n_rows), dtype=np.float32)
    ne0 = (ctypes.c_int64 * 2)(k, n_rows)
    ne1 = (ctypes.c_int64 * 2)(k, x.shape[0])
    fn(ne0, blob.ctypes.data, qtype, ne1, x.ctypes.data, out.ctypes.data)
    return out


def mul_mat_q(blob, x, shape, qtype):
    """ggml-style low-bit matmul (low_bit_linear.py:462-497): x [M,K] fp32 -> [M,N] fp32."""
    return _mm(lib().oracle_mul_mat_q_fp32, blob, x, shape, qtype)


def mul_mat_exact(blob, x, shape, qtype):
    """x @ dequant(W).T with fp64 accumulation."""
    return _mm(lib().oracle_mul_mat_exact, blob, x, shape, qtype)


def nf4_codebook():
    p = lib().oracle_nf4_codebook()
    return np.array([p[i] for i in range(16)], dtype=np.float32)


def max_threads():
    return lib().oracle_max_threads()
