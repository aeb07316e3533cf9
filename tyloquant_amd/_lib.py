"""ctypes binding of libmfq_hip.so (the C ABI declared in include/mfq_hip.h).

The library is built in-tree by `make -C tyloquant_amd/csrc` (see __graft_entry__.build).
Loading fails loudly when it is missing: there is no CPU fallback for any kernel.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

_HERE = Path(__file__).resolve().parent
LIB_PATH = _HERE / "lib" / "libmfq_hip.so"

X_BF16, X_F16, X_F32 = 0, 1, 2
TOPK_SOFTMAX, TOPK_SIGMOID, TOPK_SQRT_SOFTPLUS, TOPK_DELAYED_SOFTMAX = 0, 1, 2, 3
GLU_SILU, GLU_GELU = 0, 1
NVQS_NVQ1_L, NVQS_NVQ1_S, NVQS_NPQ0_L, NVQS_NPQ0_S = 1, 2, 3, 4
OK, ERR_INVALID, ERR_UNSUPPORTED, ERR_LAUNCH, ERR_WORKSPACE = 0, 1, 2, 3, 4

i32, i64, vp, sz = C.c_int32, C.c_int64, C.c_void_p, C.c_size_t


class NintDesc(C.Structure):
    _fields_ = [(n, i32) for n in ("bits", "sub_bits", "gs", "out", "neuron_len", "ng", "kind", "dwords",
                                   "tail_bytes", "ngp", "nsteps", "n_rowblocks")] + \
               [(n, i64) for n in ("step_bytes", "rowblock_bytes", "anchors_off", "total_bytes", "payload_bytes")]


class NvqDesc(C.Structure):
    _fields_ = [(n, i32) for n in ("index_bits", "entries", "banks", "out", "neuron_len", "ng", "nvec", "nsign",
                                   "ngp", "nsteps", "n_rowblocks")] + \
               [(n, i64) for n in ("step_bytes", "rowblock_bytes", "tables_off", "anchors_off", "total_bytes",
                                   "payload_bytes")]


class NvqsDesc(C.Structure):
    _fields_ = [(n, i32) for n in ("vector_size", "index_bits", "entries", "banks", "index_parity", "out", "neuron_len",
                                   "ng", "nvec", "nsign")] + \
               [(n, i64) for n in ("tables_off", "anchors_off", "state_off", "index_off", "sign_off", "total_bytes",
                                   "payload_bytes")] + \
               [("kind", i32), ("state_bits", i32), ("cb_bytes", i32), ("delta", C.c_float), ("nbank", i32), ("nsuper", i32)]


class NepqDesc(C.Structure):
    _fields_ = [(n, i32) for n in ("profile", "state_bits", "index_bits", "banks", "rows", "neuron_len", "ng", "nvec",
                                   "nsuper", "ngp", "nsteps", "n_rowblocks", "table_entries")] + \
               [(n, i64) for n in ("step_bytes", "rowblock_bytes", "tables_off", "anchors_off", "total_bytes",
                                   "payload_bytes")]


class Nint8zDesc(C.Structure):
    _fields_ = [(n, i32) for n in ("out", "neuron_len", "ng", "reserved")] + \
               [(n, i64) for n in ("scales_off", "codes_off", "total_bytes", "payload_bytes")]


class MoePool(C.Structure):
    _fields_ = [("desc", NintDesc), ("weight", vp)]


class MfqError(RuntimeError):
    pass


_SIGS = {
    "mfq_hip_version": (C.c_int, []),
    "mfq_hip_config": (C.c_char_p, []),
    "mfq_hip_set_cu_count": (None, [C.c_int]),
    "mfq_hip_read_probe": (C.c_int, [vp, sz, vp, vp]),
    "mfq_hip_fill_zero": (C.c_int, [vp, sz, vp]),
    "mfq_hip_moe_decode_capable": (C.c_int, [C.POINTER(MoePool), C.c_int, C.c_int, C.c_int, C.POINTER(NintDesc), C.c_int,
                                             C.c_int, C.c_int]),
    "mfq_hip_nint_plan": (C.c_int, [C.c_int] * 5 + [C.POINTER(NintDesc)]),
    "mfq_hip_nint_repack": (C.c_int, [C.POINTER(NintDesc), vp, i64, C.c_int, vp, vp]),
    "mfq_hip_nint_dequant_f32": (C.c_int, [C.POINTER(NintDesc), vp, vp, i64, vp]),
    "mfq_hip_nint_gemv": (C.c_int, [C.POINTER(NintDesc), vp, vp, C.c_int, i64, C.c_int, vp, i64, vp]),
    "mfq_hip_nint_gemv_swiglu": (C.c_int, [C.POINTER(NintDesc), vp, vp, C.c_int, i64, C.c_int, vp, C.c_int, i64, vp]),
    "mfq_hip_input_gate": (C.c_int, [vp, vp, C.c_int, i64, i64, C.c_int, C.c_int, C.c_int, vp, i64, vp]),
    "mfq_hip_nint_gemv_gate": (C.c_int, [C.POINTER(NintDesc), vp, vp, vp, C.c_int, i64, i64, C.c_int, C.c_int, vp, i64,
                                         vp]),
    "mfq_hip_nint_gemv_glu": (C.c_int, [C.POINTER(NintDesc), vp, vp, C.c_int, i64, C.c_int, vp, C.c_int, i64, C.c_int, vp]),
    "mfq_hip_nint_gemm_glu": (C.c_int, [C.POINTER(NintDesc), vp, vp, C.c_int, i64, C.c_int, C.c_int, vp, C.c_int, i64, vp,
                                        sz, vp]),
    "mfq_hip_nint_ffn_decode_workspace_bytes": (sz, [C.POINTER(NintDesc), C.POINTER(NintDesc)]),
    "mfq_hip_nint_ffn_decode_workspace_init": (C.c_int, [vp, vp]),
    "mfq_hip_nint_ffn_decode_status": (C.c_int, [vp, vp]),
    "mfq_hip_nint_ffn_decode": (C.c_int, [C.POINTER(NintDesc), vp, C.POINTER(NintDesc), vp, vp, C.c_int, C.c_int, vp, vp, sz,
                                          vp]),
    "mfq_hip_nint_embedding": (C.c_int, [C.POINTER(NintDesc), vp, vp, C.c_int, vp, C.c_int, i64, vp]),
    "mfq_hip_nint_gemv_argmax_workspace_bytes": (sz, [C.POINTER(NintDesc), C.c_int]),
    "mfq_hip_nint_gemv_argmax": (C.c_int, [C.POINTER(NintDesc), vp, vp, C.c_int, i64, C.c_int, vp, i64, vp, vp, sz, vp]),
    "mfq_hip_nint_gemv_argmax_static_init": (C.c_int, []),
    "mfq_hip_nint_gemv_argmax_static": (C.c_int, [C.POINTER(NintDesc), vp, vp, C.c_int, i64, C.c_int, vp, i64, vp, vp]),
    "mfq_hip_nint_gemm_workspace_bytes": (sz, [C.POINTER(NintDesc), C.c_int]),
    "mfq_hip_nint_gemm": (C.c_int, [C.POINTER(NintDesc), vp, vp, C.c_int, i64, C.c_int, vp, i64, vp, sz, vp]),
    "mfq_hip_nint8z_plan": (C.c_int, [C.c_int, C.c_int, C.POINTER(Nint8zDesc)]),
    "mfq_hip_nint8z_repack": (C.c_int, [C.POINTER(Nint8zDesc), vp, i64, vp, vp]),
    "mfq_hip_nint8z_dequant_f32": (C.c_int, [C.POINTER(Nint8zDesc), vp, vp, i64, vp]),
    "mfq_hip_nint8z_embedding": (C.c_int, [C.POINTER(Nint8zDesc), vp, vp, C.c_int, vp, C.c_int, i64, vp]),
    "mfq_hip_nint8z_gemv_pairs": (C.c_int, [C.POINTER(Nint8zDesc), vp, vp, C.c_int, vp, C.c_int, i64, C.c_int, vp, C.c_int, C.c_int,
                                  vp, i64, vp]),
    "mfq_hip_nint8z_gemv": (C.c_int, [C.POINTER(Nint8zDesc), vp, vp, C.c_int, i64, C.c_int, vp, i64, vp]),
    "mfq_hip_nint8z_gemm_workspace_bytes": (sz, [C.POINTER(Nint8zDesc), C.c_int]),
    "mfq_hip_nint8z_gemm": (C.c_int, [C.POINTER(Nint8zDesc), vp, vp, C.c_int, i64, C.c_int, vp, i64, vp, sz, vp]),
    "mfq_hip_nvq_plan": (C.c_int, [C.c_int] * 4 + [C.POINTER(NvqDesc)]),
    "mfq_hip_nvq_repack": (C.c_int, [C.POINTER(NvqDesc), vp, i64, vp, vp]),
    "mfq_hip_nvq_repack_plain": (C.c_int, [C.POINTER(NvqDesc), vp, i64, vp, vp, vp]),
    "mfq_hip_nvq_dequant_f32": (C.c_int, [C.POINTER(NvqDesc), vp, vp, i64, vp]),
    "mfq_hip_nvq_embedding": (C.c_int, [C.POINTER(NvqDesc), vp, vp, C.c_int, vp, C.c_int, i64, vp]),
    "mfq_hip_nvq_gemv_pairs": (C.c_int, [C.POINTER(NvqDesc), vp, vp, C.c_int, vp, C.c_int, i64, C.c_int, vp, C.c_int, C.c_int, vp,
                               i64, vp]),
    "mfq_hip_nvq_gemv": (C.c_int, [C.POINTER(NvqDesc), vp, vp, C.c_int, i64, C.c_int, vp, i64, vp]),
    "mfq_hip_nvq_gemv_multi2": (C.c_int, [C.POINTER(NvqDesc), vp, C.POINTER(NvqDesc), vp, vp, C.c_int, i64, C.c_int, vp, i64, vp]),
    "mfq_hip_nvq_gemm_workspace_bytes": (sz, [C.POINTER(NvqDesc), C.c_int]),
    "mfq_hip_nvq_gemm": (C.c_int, [C.POINTER(NvqDesc), vp, vp, C.c_int, i64, C.c_int, vp, i64, vp, sz, vp]),
    "mfq_hip_nvqs_plan": (C.c_int, [C.c_int] * 6 + [C.POINTER(NvqsDesc)]),
    "mfq_hip_nvqs_repack": (C.c_int, [C.POINTER(NvqsDesc), vp, i64, C.c_int, vp, vp, vp]),
    "mfq_hip_nvqs_plan_nepq0": (C.c_int, [C.c_int] * 4 + [C.POINTER(NvqsDesc)]),
    "mfq_hip_nvqs_repack_nepq0": (C.c_int, [C.POINTER(NvqsDesc), vp, i64, vp, vp]),
    "mfq_hip_nvqs_dequant_rows_f32": (C.c_int, [C.POINTER(NvqsDesc), vp, C.c_int, C.c_int, vp, i64, vp]),
    "mfq_hip_nvqs_embedding": (C.c_int, [C.POINTER(NvqsDesc), vp, vp, C.c_int, vp, C.c_int, i64, vp]),
    "mfq_hip_nvqs_gemv_pairs": (C.c_int, [C.POINTER(NvqsDesc), vp, vp, C.c_int, vp, C.c_int, vp, C.c_int, i64, C.c_int, vp, C.c_int,
                                C.c_int, vp, i64, vp]),
    "mfq_hip_nvqs_gemv_rows": (C.c_int, [C.POINTER(NvqsDesc), vp, C.c_int, C.c_int, vp, C.c_int, i64, C.c_int, vp, i64, vp]),
    "mfq_hip_nvqs_gemm_rows_workspace_bytes": (sz, [C.POINTER(NvqsDesc), C.c_int, C.c_int]),
    "mfq_hip_nvqs_gemm_rows": (C.c_int, [C.POINTER(NvqsDesc), vp, C.c_int, C.c_int, vp, C.c_int, i64, C.c_int, vp, i64, vp, sz,
                                         vp]),
    "mfq_hip_moe_move_rows": (C.c_int, [vp, i64, vp, C.c_int, C.c_int, C.c_int, vp, i64, vp]),
    "mfq_hip_nvqs_plan_lowbit": (C.c_int, [C.c_int] * 4 + [C.POINTER(NvqsDesc)]),
    "mfq_hip_nvqs_repack_lowbit": (C.c_int, [C.POINTER(NvqsDesc), vp, i64, vp, vp, vp]),
    "mfq_hip_nvqs_dequant_f32": (C.c_int, [C.POINTER(NvqsDesc), vp, vp, i64, vp]),
    "mfq_hip_nvqs_gemv": (C.c_int, [C.POINTER(NvqsDesc), vp, vp, C.c_int, i64, C.c_int, vp, i64, vp]),
    "mfq_hip_nvqs_gemm_workspace_bytes": (sz, [C.POINTER(NvqsDesc), C.c_int]),
    "mfq_hip_nvqs_gemm": (C.c_int, [C.POINTER(NvqsDesc), vp, vp, C.c_int, i64, C.c_int, vp, i64, vp, sz, vp]),
    "mfq_hip_mx_dequant_rows": (C.c_int, [C.c_int, vp, vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, vp, i64, vp]),
    "mfq_hip_mx_gemm_rows_workspace_bytes": (sz, [C.c_int, C.c_int, C.c_int]),
    "mfq_hip_mx_gemv_pairs": (C.c_int, [C.c_int, vp, vp, C.c_int, C.c_int, C.c_int, vp, C.c_int, vp, C.c_int, i64, C.c_int, vp, C.c_int,
                              C.c_int, vp, i64, vp]),
    "mfq_hip_mx_gemm_rows": (C.c_int, [C.c_int, vp, vp, C.c_int, C.c_int, C.c_int, C.c_int, vp, C.c_int, i64, C.c_int, vp, i64,
                                       vp, sz, vp]),
    "mfq_hip_nepq_plan": (C.c_int, [C.c_int] * 4 + [C.POINTER(NepqDesc)]),
    "mfq_hip_nepq_repack": (C.c_int, [C.POINTER(NepqDesc), vp, i64, vp, vp]),
    "mfq_hip_nepq_dequant_f32": (C.c_int, [C.POINTER(NepqDesc), vp, vp, i64, vp]),
    "mfq_hip_nepq_gemv": (C.c_int, [C.POINTER(NepqDesc), vp, C.c_int, C.c_int, vp, C.c_int, i64, C.c_int, vp, i64, vp]),
    "mfq_hip_nepq_gemv_pairs": (C.c_int, [C.POINTER(NepqDesc), vp, C.c_int, vp, C.c_int, vp, C.c_int, i64, C.c_int, vp, C.c_int,
                                C.c_int, vp, i64, vp]),
    "mfq_hip_nepq_gemm_workspace_bytes": (sz, [C.POINTER(NepqDesc), C.c_int, C.c_int]),
    "mfq_hip_nepq_gemm": (C.c_int, [C.POINTER(NepqDesc), vp, C.c_int, C.c_int, vp, C.c_int, i64, C.c_int, vp, i64,
                                    vp, sz, vp]),
    "mfq_hip_nepq_hadamard": (C.c_int, [vp, C.c_int, i64, C.c_int, C.c_int, C.c_int, vp, vp, i64, vp]),
    "mfq_hip_moe_topk": (C.c_int, [vp, vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, vp, vp,
                                   vp]),
    "mfq_hip_moe_route_map": (C.c_int, [vp, C.c_int, C.c_int, C.c_int, vp, vp, vp, vp, C.c_int, vp, vp]),
    "mfq_hip_moe_tile_m": (C.c_int, []),
    "mfq_hip_moe_grouped_matmul": (C.c_int, [C.POINTER(MoePool), C.c_int, vp, vp, C.c_int, C.c_int, C.c_int, vp,
                                             C.c_int, i64, C.c_int, vp, C.c_int, C.c_int, vp, vp, vp, vp, vp, i64,
                                             vp]),
    "mfq_hip_moe_grouped_workspace_bytes": (sz, [C.POINTER(MoePool), C.c_int, C.c_int, C.c_int]),
    "mfq_hip_moe_grouped_glu_ws": (C.c_int, [C.POINTER(MoePool), C.c_int, vp, vp, C.c_int, C.c_int, C.c_int, vp,
                                             C.c_int, i64, C.c_int, vp, C.c_int, C.c_int, vp, vp, C.c_int, vp, C.c_int,
                                             i64, vp, sz, vp]),
    "mfq_hip_moe_grouped_matmul_ws": (C.c_int, [C.POINTER(MoePool), C.c_int, vp, vp, C.c_int, C.c_int, C.c_int, vp,
                                                C.c_int, i64, C.c_int, vp, C.c_int, C.c_int, vp, vp, vp, vp, vp, i64,
                                                vp, sz, vp]),
    "mfq_hip_moe_decode_matmul": (C.c_int, [C.POINTER(MoePool), C.c_int, vp, vp, C.c_int, C.c_int, C.c_int, vp, C.c_int,
                                            i64, C.c_int, vp, C.c_int, C.c_int, vp, vp, C.c_int, vp, C.c_int, i64, vp]),
    "mfq_hip_moe_swiglu": (C.c_int, [vp, i64, C.c_int, C.c_int, vp, C.c_int, i64, vp]),
    "mfq_hip_moe_glu": (C.c_int, [vp, i64, C.c_int, C.c_int, vp, C.c_int, i64, C.c_int, vp]),
    "mfq_hip_moe_weighted_reduce": (C.c_int, [vp, vp, C.c_int, C.c_int, C.c_int, vp, vp, vp, vp]),
    "mfq_hip_cache_scatter": (C.c_int, [vp, i64, C.c_int, i64, vp]),
    "mfq_hip_gemm_f16_nt": (C.c_int, [vp, i64, vp, i64, C.c_int, C.c_int, C.c_int, vp, i64, vp]),
}

_lib = None


def exported_symbols() -> list[str]:
    """Every entry point include/mfq_hip.h declares (kept in step with the header by a test)."""
    return sorted(list(_SIGS) + ["mfq_hip_last_error"])


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise MfqError(f"{LIB_PATH} is missing: build it with `make -C tyloquant_amd/csrc` "
                           "(or python -c 'import __graft_entry__ as g; g.build()'); there is no CPU fallback")
        _lib = C.CDLL(str(LIB_PATH))
        _lib.mfq_hip_last_error.restype = C.c_char_p
        _lib.mfq_hip_last_error.argtypes = []
        for name, (res, args) in _SIGS.items():
            fn = getattr(_lib, name, None)
            if fn is None:
                raise MfqError(f"{LIB_PATH} does not export {name}: rebuild it (make -C tyloquant_amd/csrc)")
            fn.restype, fn.argtypes = res, args
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise MfqError(f"mfq_hip status {rc}: {lib().mfq_hip_last_error().decode(errors='replace')}")
