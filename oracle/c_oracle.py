"""ctypes access to oracle/libmfq_oracle.so (the C restatement of the reference CPU path).
Test infrastructure: used by tests/ and by bench.py's cpu_baseline leg only."""
import ctypes as C
from pathlib import Path

import numpy as np

LIB = Path(__file__).resolve().parent / "libmfq_oracle.so"
_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(str(LIB))
        _lib.oracle_threads.restype = C.c_int
        _lib.oracle_nint_dequant.argtypes = [C.c_void_p] + [C.c_int] * 5 + [C.c_void_p]
        _lib.oracle_matmul_nt.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]
    return _lib


def threads() -> int:
    return int(lib().oracle_threads())


def nint_dequant(body: bytes, bits, sub_bits, gs, out, K) -> np.ndarray:
    W = np.empty((out, K), dtype=np.float32)
    buf = np.frombuffer(body, dtype=np.uint8)
    lib().oracle_nint_dequant(buf.ctypes.data, bits, sub_bits, gs, out, K, W.ctypes.data)
    return W


def matmul_nt(x: np.ndarray, W: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    W = np.ascontiguousarray(W, dtype=np.float32)
    y = np.empty((x.shape[0], W.shape[0]), dtype=np.float32)
    lib().oracle_matmul_nt(x.ctypes.data, W.ctypes.data, x.shape[0], W.shape[0], W.shape[1], y.ctypes.data)
    return y
