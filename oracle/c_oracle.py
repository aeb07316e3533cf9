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
        vp, ci = C.c_void_p, C.c_int
        _lib.oracle_nint_dequant_rows.argtypes = [vp] + [ci] * 7 + [vp]
        _lib.oracle_nvq_jsc_dequant.argtypes = [vp, vp, vp, vp, vp, ci, vp, ci, vp, ci, ci, ci, ci, vp]
        _lib.oracle_nepq1s_dequant.argtypes = [vp, vp, vp, vp, vp, ci, vp, ci, ci, vp]
        _lib.oracle_moe_ffn.argtypes = [vp, vp, vp, ci, ci, ci, vp, vp, ci, ci, vp, vp]
    return _lib


def threads() -> int:
    return int(lib().oracle_threads())


def nint_dequant(body: bytes, bits, sub_bits, gs, out, K) -> np.ndarray:
    W = np.empty((out, K), dtype=np.float32)
    buf = np.frombuffer(body, dtype=np.uint8)
    lib().oracle_nint_dequant(buf.ctypes.data, bits, sub_bits, gs, out, K, W.ctypes.data)
    return W


def nint_dequant_rows(body, bits, sub_bits, gs, out, K, row0, nrows) -> np.ndarray:
    """Rows [row0, row0 + nrows) of the tensor whose packed body (all `out` rows) is given."""
    W = np.empty((nrows, K), dtype=np.float32)
    buf = np.frombuffer(body, dtype=np.uint8)
    lib().oracle_nint_dequant_rows(buf.ctypes.data, bits, sub_bits, gs, out, K, row0, nrows, W.ctypes.data)
    return W


def matmul_nt(x: np.ndarray, W: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    W = np.ascontiguousarray(W, dtype=np.float32)
    y = np.empty((x.shape[0], W.shape[0]), dtype=np.float32)
    lib().oracle_matmul_nt(x.ctypes.data, W.ctypes.data, x.shape[0], W.shape[0], W.shape[1], y.ctypes.data)
    return y


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def nvq_jsc_dequant(t) -> np.ndarray:
    """dequantize_nvq_jsc of an oracle NvqJscTensor (unpacked fields) in C."""
    out, K = t.shape
    anchor, lut = _c(t.neuron_scale, np.float32), _c(t.scale_lut, np.float32)
    bfs, state = _c(t.bank_for_state, np.uint8), _c(t.state, np.uint8)
    idx, signs, cb = _c(t.indices, np.uint16), _c(t.signs, np.uint8), _c(t.codebooks, np.int8)
    W = np.empty((out, K), dtype=np.float32)
    lib().oracle_nvq_jsc_dequant(anchor.ctypes.data, lut.ctypes.data, bfs.ctypes.data, state.ctypes.data, idx.ctypes.data,
                                 idx.shape[1], signs.ctypes.data, signs.shape[1], cb.ctypes.data, cb.shape[1], cb.shape[2],
                                 out, K, W.ctypes.data)
    return W


def nepq1s_dequant(t, tables) -> np.ndarray:
    """dequantize_nepq of an oracle NepqTensor with label NEPQ1-S in C; tables = int8 [banks, 2, 512, 8] (the ternary
    tables unpacked once, as at load time)."""
    E, out, K = t.shape
    rows = E * out
    anchor = _c(t.neuron_scale.reshape(rows), np.float32)
    state, aux = _c(t.state.reshape(rows, -1), np.uint8), _c(t.aux.reshape(rows, -1), np.uint8)
    idx, banks, tb = _c(t.indices.reshape(rows, -1), np.uint16), _c(t.bank_ids.reshape(rows, -1), np.uint8), _c(tables, np.int8)
    W = np.empty((rows, K), dtype=np.float32)
    lib().oracle_nepq1s_dequant(anchor.ctypes.data, state.ctypes.data, idx.ctypes.data, aux.ctypes.data, banks.ctypes.data,
                                banks.shape[1], tb.ctypes.data, rows, K, W.ctypes.data)
    return W.reshape(E, out, K)


def moe_ffn(x, ids, w, gu_dense: dict, dn_dense: dict, E: int) -> np.ndarray:
    """The routed part of the oracle's moe_ffn (grouped matmul, SwiGLU, grouped matmul, weighted reduce) in C.
    gu_dense / dn_dense map expert id -> dense fp32 matrix for the experts the ids name."""
    x, ids, w = _c(x, np.float32), _c(ids, np.int32), _c(w, np.float32)
    T, k = ids.shape
    H = x.shape[1]
    W = next(iter(dn_dense.values())).shape[1]
    keep = [_c(v, np.float32) for v in list(gu_dense.values()) + list(dn_dense.values())]
    gu_ptr, dn_ptr = (C.c_void_p * E)(), (C.c_void_p * E)()
    for (e, _), a in zip(list(gu_dense.items()), keep[:len(gu_dense)]):
        gu_ptr[e] = a.ctypes.data
    for (e, _), a in zip(list(dn_dense.items()), keep[len(gu_dense):]):
        dn_ptr[e] = a.ctypes.data
    scratch = np.empty(T * k * (3 * W + H), dtype=np.float32)
    out = np.empty((T, H), dtype=np.float32)
    lib().oracle_moe_ffn(x.ctypes.data, ids.ctypes.data, w.ctypes.data, T, k, E, gu_ptr, dn_ptr, H, W, scratch.ctypes.data,
                         out.ctypes.data)
    return out
