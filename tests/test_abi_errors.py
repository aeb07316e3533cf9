"""Argument checks of the C ABI (include/mfq_hip.h): every entry point validates before it touches the GPU, so these run
without one.  A rejected call returns its status code, launches nothing and leaves a message for mfq_hip_last_error();
the reference raises std::runtime_error / TORCH_CHECK failures from the same places (cpp_runtime/mfq_decode.cpp:8130-8260,
mfq/kernels/cuda/mfq_cuda.cpp argument checks)."""
import ctypes as C

import pytest

from tyloquant_amd import _lib as L

FAKE = C.c_void_p(0x1000)      # a non-null address that a rejected call never dereferences


@pytest.fixture(scope="module")
def lib():
    return L.lib()


def _nint(lib, bits=4, sb=6, gs=32, out=64, K=256):
    d = L.NintDesc()
    assert lib.mfq_hip_nint_plan(bits, sb, gs, out, K, C.byref(d)) == L.OK
    return d


def _msg(lib):
    return lib.mfq_hip_last_error().decode()


def test_plans_reject_impossible_profiles(lib):
    d = L.NintDesc()
    assert lib.mfq_hip_nint_plan(0, 6, 32, 64, 256, C.byref(d)) == L.ERR_UNSUPPORTED and "bits=0" in _msg(lib)
    assert lib.mfq_hip_nint_plan(4, 6, 31, 64, 256, C.byref(d)) == L.ERR_UNSUPPORTED and "groupsize" in _msg(lib)
    assert lib.mfq_hip_nint_plan(4, 6, 32, 0, 256, C.byref(d)) == L.ERR_INVALID
    assert lib.mfq_hip_nint_plan(4, 6, 32, 64, 256, None) == L.ERR_INVALID
    v = L.NvqsDesc()
    assert lib.mfq_hip_nvqs_plan(5, 8, 1, 0, 16, 64, C.byref(v)) == L.ERR_INVALID          # vector size
    assert lib.mfq_hip_nvqs_plan(8, 8, 3, 0, 16, 64, C.byref(v)) == L.ERR_INVALID          # banks
    assert lib.mfq_hip_nvqs_plan(4, 8, 1, 1, 16, 64, C.byref(v)) == L.ERR_INVALID          # index parity is E8-256 only
    assert lib.mfq_hip_nvqs_plan_lowbit(9, 3, 16, 64, C.byref(v)) == L.ERR_INVALID
    assert lib.mfq_hip_nvqs_plan_lowbit(L.NVQS_NVQ1_L, 5, 16, 64, C.byref(v)) == L.ERR_UNSUPPORTED
    assert lib.mfq_hip_nvqs_plan_lowbit(L.NVQS_NPQ0_S, 2, 16, 100, C.byref(v)) == L.ERR_INVALID and "divisible by 8" in _msg(lib)
    assert lib.mfq_hip_nvqs_plan_nepq0(2, 3, 16, 64, C.byref(v)) == L.ERR_INVALID
    assert lib.mfq_hip_nvqs_plan_nepq0(0, 0, 16, 64, C.byref(v)) == L.ERR_INVALID
    assert lib.mfq_hip_nvqs_plan_nepq0(1, 4, 16, 64, C.byref(v)) == L.OK and v.kind == 3 and v.nbank == 4


def test_matmul_entry_points_check_their_arguments(lib):
    d = _nint(lib)
    assert lib.mfq_hip_nint_gemv(C.byref(d), None, FAKE, L.X_BF16, 256, 1, FAKE, 64, None) == L.ERR_INVALID
    assert lib.mfq_hip_nint_gemv(C.byref(d), FAKE, FAKE, L.X_BF16, 256, 0, FAKE, 64, None) == L.ERR_INVALID
    assert lib.mfq_hip_nint_gemv(C.byref(d), FAKE, FAKE, 7, 256, 1, FAKE, 64, None) == L.ERR_INVALID and "x_dtype" in _msg(lib)
    assert lib.mfq_hip_nint_gemv(C.byref(d), FAKE, FAKE, L.X_BF16, 100, 1, FAKE, 64, None) == L.ERR_INVALID   # ldx < K
    assert lib.mfq_hip_nint_gemv(C.byref(d), FAKE, FAKE, L.X_BF16, 256, 1, FAKE, 10, None) == L.ERR_INVALID   # ldy < out
    big = _nint(lib, out=4096, K=4096)
    need = lib.mfq_hip_nint_gemm_workspace_bytes(C.byref(big), 2048)
    assert need > 0
    rc = lib.mfq_hip_nint_gemm(C.byref(big), FAKE, FAKE, L.X_BF16, 4096, 2048, FAKE, 4096, FAKE, need - 1, None)
    assert rc == L.ERR_WORKSPACE and "workspace" in _msg(lib)
    rc = lib.mfq_hip_nint_gemm(C.byref(big), FAKE, FAKE, L.X_BF16, 4096, 2048, FAKE, 4096, None, 0, None)
    assert rc == L.ERR_WORKSPACE
    # fused epilogues
    assert lib.mfq_hip_nint_gemv_glu(C.byref(d), FAKE, FAKE, L.X_BF16, 256, 1, FAKE, L.X_F16, 32, 5, None) == L.ERR_INVALID
    rc = lib.mfq_hip_nint_gemv_glu(C.byref(d), FAKE, FAKE, L.X_BF16, 256, 3, FAKE, L.X_F16, 32, L.GLU_SILU, None)
    assert rc == L.ERR_UNSUPPORTED
    rc = lib.mfq_hip_nint_gemm_glu(C.byref(big), FAKE, FAKE, L.X_BF16, 4096, 4, L.GLU_SILU, FAKE, L.X_F16, 2048, FAKE, 1 << 30, None)
    assert rc == L.ERR_UNSUPPORTED and "one-pass" in _msg(lib)
    rc = lib.mfq_hip_nint_gemm_glu(C.byref(big), FAKE, FAKE, L.X_BF16, 4096, 2048, 9, FAKE, L.X_F16, 2048, FAKE, 1 << 30, None)
    assert rc == L.ERR_INVALID and "activation" in _msg(lib)
    rc = lib.mfq_hip_nint_gemv_gate(C.byref(d), FAKE, FAKE, FAKE, L.X_BF16, 256, 256, 3, 0, FAKE, 64, None)
    assert rc == L.ERR_UNSUPPORTED


def test_repack_checks_the_payload_length(lib):
    d = _nint(lib)
    rc = lib.mfq_hip_nint_repack(C.byref(d), FAKE, int(d.payload_bytes) - 1, 0, FAKE, None)
    assert rc == L.ERR_INVALID and "invalid NINT blob tail" in _msg(lib)
    v = L.NvqsDesc()
    assert lib.mfq_hip_nvqs_plan_lowbit(L.NVQS_NVQ1_L, 3, 16, 96, C.byref(v)) == L.OK
    rc = lib.mfq_hip_nvqs_repack_lowbit(C.byref(v), FAKE, int(v.payload_bytes) + 7, None, FAKE, None)
    assert rc == L.ERR_INVALID
    rc = lib.mfq_hip_nvqs_repack_lowbit(C.byref(v), FAKE, int(v.payload_bytes), None, FAKE, None)      # no table, no grid
    assert rc == L.ERR_INVALID and "built-in grid" in _msg(lib)
    k = L.NvqsDesc()
    assert lib.mfq_hip_nvqs_plan(8, 8, 2, 0, 16, 96, C.byref(k)) == L.OK
    assert lib.mfq_hip_nvqs_repack_lowbit(C.byref(k), FAKE, 100, None, FAKE, None) == L.ERR_INVALID    # wrong descriptor kind


def test_row_ranges_must_lie_inside_the_tensor(lib):
    v = L.NvqsDesc()
    assert lib.mfq_hip_nvqs_plan_nepq0(0, 2, 64, 96, C.byref(v)) == L.OK
    for row0, nrows in ((-1, 4), (60, 8), (0, 0), (64, 1)):
        rc = lib.mfq_hip_nvqs_gemv_rows(C.byref(v), FAKE, row0, nrows, FAKE, L.X_BF16, 96, 1, FAKE, 64, None)
        assert rc == L.ERR_INVALID and "outside the tensor" in _msg(lib)
        assert lib.mfq_hip_nvqs_dequant_rows_f32(C.byref(v), FAKE, row0, nrows, FAKE, 96, None) == L.ERR_INVALID
    assert lib.mfq_hip_nvqs_gemm_rows(C.byref(v), FAKE, 0, 32, FAKE, L.X_BF16, 96, 200, FAKE, 32, None, 0, None) == L.ERR_WORKSPACE


def test_moe_helpers_check_their_arguments(lib):
    assert lib.mfq_hip_moe_weighted_reduce(None, FAKE, 4, 2, 64, None, None, FAKE, None) == L.ERR_INVALID
    assert lib.mfq_hip_moe_weighted_reduce(FAKE, FAKE, 0, 2, 64, None, None, FAKE, None) == L.ERR_INVALID
    assert lib.mfq_hip_moe_move_rows(FAKE, 64, FAKE, 4, 30, 0, FAKE, 64, None) == L.ERR_INVALID and "32-bit" in _msg(lib)
    assert lib.mfq_hip_moe_move_rows(FAKE, 64, None, 4, 32, 0, FAKE, 64, None) == L.ERR_INVALID
    assert lib.mfq_hip_moe_glu(FAKE, 10, 4, 8, FAKE, L.X_F16, 8, L.GLU_SILU, None) == L.ERR_INVALID      # ld < 2 W
    assert lib.mfq_hip_moe_glu(FAKE, 16, 4, 8, FAKE, L.X_F16, 8, 3, None) == L.ERR_INVALID
    d = _nint(lib, out=8 * 48, K=256)
    pools = (L.MoePool * 1)()
    pools[0].desc = d
    pools[0].weight = 0x1000
    rc = lib.mfq_hip_moe_grouped_glu_ws(pools, 1, FAKE, FAKE, 8, 48, 256, FAKE, L.X_BF16, 256, 0, FAKE, 16, 2, FAKE, FAKE,
                                        L.GLU_SILU, FAKE, L.X_F16, 24, FAKE, 1 << 20, None)
    assert rc == L.ERR_UNSUPPORTED and "row-blocks" in _msg(lib)             # 48 is not two halves of whole row-blocks


def test_mx_entry_points_check_geometry_rows_and_workspace(lib):
    rc = lib.mfq_hip_mx_dequant_rows(5, FAKE, FAKE, 4, 96, 0, 4, L.X_F32, FAKE, 96, None)
    assert rc == L.ERR_INVALID and "neither MXFP4 (4) nor MXFP8 (8)" in _msg(lib)
    rc = lib.mfq_hip_mx_dequant_rows(4, FAKE, FAKE, 4, 48, 0, 4, L.X_F32, FAKE, 48, None)
    assert rc == L.ERR_INVALID and "MXFP4 columns must be divisible by 32" in _msg(lib)
    rc = lib.mfq_hip_mx_dequant_rows(8, FAKE, FAKE, 4, 96, 0, 4, L.X_F32, FAKE, 96, None)
    assert rc == L.ERR_INVALID and "MXFP8 columns must be divisible by 128" in _msg(lib)
    assert lib.mfq_hip_mx_dequant_rows(4, FAKE, FAKE, 4, 96, 0, 4, L.X_BF16, FAKE, 96, None) == L.ERR_INVALID   # fp32 / fp16 only
    assert lib.mfq_hip_mx_dequant_rows(4, FAKE, None, 4, 96, 0, 4, L.X_F32, FAKE, 96, None) == L.ERR_INVALID
    for row0, nrows in ((-1, 2), (3, 2), (0, 0), (4, 1)):
        rc = lib.mfq_hip_mx_gemm_rows(4, FAKE, FAKE, 4, 96, row0, nrows, FAKE, L.X_BF16, 96, 1, FAKE, 4, None, 0, None)
        assert rc == L.ERR_INVALID and "outside the tensor" in _msg(lib)
    assert lib.mfq_hip_mx_gemm_rows(4, FAKE, FAKE, 4, 96, 0, 4, FAKE, L.X_F32, 96, 1, FAKE, 4, None, 0, None) == L.ERR_INVALID
    assert lib.mfq_hip_mx_gemm_rows(4, FAKE, FAKE, 4, 96, 0, 4, FAKE, L.X_BF16, 64, 1, FAKE, 4, None, 0, None) == L.ERR_INVALID
    # up to 256 rows run on the tile kernels without a workspace, the fp16 copy + GEMM above needs one
    assert lib.mfq_hip_mx_gemm_rows_workspace_bytes(96, 4, 256) == 0 and lib.mfq_hip_mx_gemm_rows_workspace_bytes(96, 4, 257) > 0
    assert lib.mfq_hip_mx_gemm_rows(4, FAKE, FAKE, 4, 96, 0, 4, FAKE, L.X_BF16, 96, 257, FAKE, 4, None, 0, None) == L.ERR_WORKSPACE



def test_embedding_and_decode_pair_entry_points_check_their_arguments(lib):
    """The embedding-row entry points of the NVQ / NINT8-0 tables and the per-cohort launches of a MoE decode step
    (mfq_hip_*_gemv_pairs): null pointers, output types, strides, pair counts and expert row counts are refused before
    anything is launched."""
    v = L.NvqDesc()
    assert lib.mfq_hip_nvq_plan(9, 2, 64, 96, C.byref(v)) == L.OK
    assert lib.mfq_hip_nvq_embedding(C.byref(v), None, FAKE, 2, FAKE, L.X_F16, 96, None) == L.ERR_INVALID
    assert lib.mfq_hip_nvq_embedding(C.byref(v), FAKE, FAKE, 2, FAKE, 9, 96, None) == L.ERR_INVALID and "out_dtype" in _msg(lib)
    assert lib.mfq_hip_nvq_embedding(C.byref(v), FAKE, FAKE, 2, FAKE, L.X_F16, 95, None) == L.ERR_INVALID and "ldo" in _msg(lib)
    assert lib.mfq_hip_nvq_embedding(C.byref(v), FAKE, None, 2, FAKE, L.X_F16, 96, None) == L.ERR_INVALID
    assert lib.mfq_hip_nvq_embedding(C.byref(v), FAKE, None, 0, None, L.X_F16, 96, None) == L.OK          # no ids: nothing to do
    z = L.Nint8zDesc()
    assert lib.mfq_hip_nint8z_plan(64, 96, C.byref(z)) == L.OK
    assert lib.mfq_hip_nint8z_embedding(C.byref(z), FAKE, FAKE, -1, FAKE, L.X_F16, 96, None) == L.ERR_INVALID
    assert lib.mfq_hip_nvq_gemv_pairs(C.byref(v), None, FAKE, 8, FAKE, L.X_BF16, 96, 0, FAKE, 1, 2, FAKE, 64, None) == L.ERR_INVALID
    assert lib.mfq_hip_nvq_gemv_pairs(C.byref(v), FAKE, FAKE, 8, FAKE, 5, 96, 0, FAKE, 1, 2, FAKE, 64, None) == L.ERR_INVALID
    assert lib.mfq_hip_nvq_gemv_pairs(C.byref(v), FAKE, FAKE, 8, FAKE, L.X_BF16, 96, 0, FAKE, 40000, 2, FAKE, 64,
                                      None) == L.ERR_UNSUPPORTED and "65535" in _msg(lib)
    assert lib.mfq_hip_nvq_gemv_pairs(C.byref(v), FAKE, FAKE, 8, FAKE, L.X_BF16, 96, 0, FAKE, 1, 2, FAKE, 63, None) == L.ERR_INVALID
    assert lib.mfq_hip_nvq_gemv_pairs(C.byref(v), FAKE, FAKE, 8, FAKE, L.X_BF16, 96, 0, FAKE, 0, 2, FAKE, 64, None) == L.OK
    assert lib.mfq_hip_nint8z_gemv_pairs(C.byref(z), FAKE, None, 8, FAKE, L.X_BF16, 96, 0, FAKE, 1, 2, FAKE, 64, None) == L.ERR_INVALID
    assert lib.mfq_hip_mx_gemv_pairs(4, FAKE, FAKE, 64, 96, 24, FAKE, 8, FAKE, L.X_BF16, 96, 0, FAKE, 1, 2, FAKE, 24,
                                     None) == L.ERR_INVALID and "do not divide" in _msg(lib)
    assert lib.mfq_hip_mx_gemv_pairs(8, FAKE, FAKE, 256, 128, 64, FAKE, 8, FAKE, L.X_BF16, 128, 0, FAKE, 1, 2, FAKE, 64,
                                     None) == L.ERR_UNSUPPORTED and "128-row" in _msg(lib)
    s = L.NvqsDesc()
    assert lib.mfq_hip_nvqs_plan(8, 8, 2, 0, 64, 96, C.byref(s)) == L.OK
    assert lib.mfq_hip_nvqs_gemv_pairs(C.byref(s), None, None, 64, FAKE, 8, FAKE, L.X_BF16, 96, 0, FAKE, 1, 2, FAKE, 64,
                                       None) == L.ERR_INVALID
    assert lib.mfq_hip_nvqs_gemv_pairs(C.byref(s), None, FAKE, 24, FAKE, 8, FAKE, L.X_BF16, 96, 0, FAKE, 1, 2, FAKE, 64,
                                       None) == L.ERR_INVALID and "rows per expert" in _msg(lib)
