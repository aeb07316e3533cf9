"""GPU parity of the NINT path against the oracle (through the C ABI)."""
import ctypes as C

import re

import numpy as np
import pytest

import synth
from conftest import ABS_TOL, REL_TOL, rel_l2
from oracle import mfq_oracle as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

# (bits, gs, sub_bits): the production profiles plus odd ones that take the generic unit
SPECS = [(4, 32, 6), (4, 24, 6), (3, 24, 5), (2, 16, 5), (5, 28, 7), (6, 24, 6), (8, 24, 8), (4, 16, 6), (4, 48, 6),
         (6, 26, 6), (2, 32, 5), (5, 16, 5), (6, 24, 7), (8, 48, 7)]   # the last two: the production NINT6 / NINT8 profiles


_rand_tensor = synth.nint_random


def _load(t):
    from tyloquant_amd import runtime as R
    return R.load_quant_linear(f"NINT{t.bits}", O.pack_nint(t))


def _x(rng, M, K, dtype=None):
    dtype = dtype or torch.bfloat16
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(dtype)
    return x.cuda(), x.float().numpy()


@pytest.mark.parametrize("bits,gs,sb", SPECS)
@pytest.mark.parametrize("out,K", [(48, 88), (37, 96), (64, 200), (257, 224), (73, 1537)])
def test_dequant_bit_exact(bits, gs, sb, out, K):
    rng = np.random.default_rng(1000 + bits * 100 + gs + out)
    t = _rand_tensor(rng, out, K, bits, gs, sb)
    lin = _load(t)
    got = lin.dequantize().cpu().numpy()
    want = O.dequantize_nint(t)
    assert got.shape == want.shape
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("bits,gs,sb", SPECS)
@pytest.mark.parametrize("M", [1, 2, 3, 8])
def test_gemv_matches_oracle(bits, gs, sb, M):
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(70 + bits + M)
    out, K = 48, 88
    t = O.quantize_nint((rng.standard_normal((out, K)) * 0.02).astype(np.float32), bits, gs, sb)
    lin = _load(t)
    for dtype in (torch.bfloat16, torch.float16):
        x, xf = _x(rng, M, K, dtype)
        y = R.nint_matmul(lin.weight, x, force="gemv").cpu().numpy()
        ref = O.linear_forward(O.dequantize_nint(t), xf)
        assert rel_l2(y, ref) < REL_TOL, (dtype, rel_l2(y, ref))
        assert np.abs(y - ref).max() < ABS_TOL


@pytest.mark.parametrize("bits,gs,sb", [(4, 32, 6), (4, 24, 6), (3, 24, 5), (2, 16, 5), (5, 28, 7), (4, 16, 6), (4, 48, 6),
                                        (2, 32, 5), (4, 32, 8), (6, 24, 7), (8, 48, 7)])
@pytest.mark.parametrize("out,K,M", [(128, 1024, 2), (200, 2056, 16), (80, 4096, 5), (96, 1544, 17), (64, 12288, 40)])
def test_small_batch_matrix_core_path(bits, gs, sb, out, K, M):
    """Batches of 2..64 rows stream the packed weights once per 16 rows through the MFMA kernel (K % 8 == 0,
    16-byte aligned rows); ragged K, a row stride above K and more rows than one 16-row tile."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(900 + bits * 10 + gs + M)
    t = O.quantize_nint((rng.standard_normal((out, K)) * 0.02).astype(np.float32), bits, gs, sb)
    lin = _load(t)
    deq = O.dequantize_nint(t)
    for dtype in (torch.bfloat16, torch.float16):
        xw = torch.from_numpy(rng.standard_normal((M, K + 8)).astype(np.float32)).to(dtype).cuda()
        x = xw[:, :K]                       # row stride K + 8
        y = R.nint_matmul(lin.weight, x, force="gemv").cpu().numpy()
        ref = O.linear_forward_f64(deq, x.float().cpu().numpy())
        assert rel_l2(y, ref) < REL_TOL, (dtype, rel_l2(y, ref))
        assert np.abs(y - ref).max() < ABS_TOL


@pytest.mark.parametrize("bits,gs,sb", [(4, 32, 6), (3, 24, 5), (2, 16, 5), (5, 28, 7), (4, 24, 6), (6, 24, 7), (8, 48, 7)])
@pytest.mark.parametrize("out,K,M", [(128, 280, 16), (257, 224, 23), (73, 1537, 65), (512, 1024, 257)])
def test_gemm_matches_oracle(bits, gs, sb, out, K, M):
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(170 + bits + M)
    t = O.quantize_nint((rng.standard_normal((out, K)) * 0.02).astype(np.float32), bits, gs, sb)
    lin = _load(t)
    x, xf = _x(rng, M, K)
    y = lin(x).cpu().numpy()
    ref = O.linear_forward_f64(O.dequantize_nint(t), xf)
    assert rel_l2(y, ref) < REL_TOL, rel_l2(y, ref)
    assert np.abs(y - ref).max() < ABS_TOL


@pytest.mark.parametrize("bits,gs,sb", [(4, 32, 6), (3, 24, 5), (2, 16, 5), (5, 28, 7), (4, 48, 6)])
@pytest.mark.parametrize("out,M", [(1040, 3329), (256, 16500)])
def test_gemm_many_rows_takes_the_large_tiles(bits, gs, sb, out, M):
    """More than one block per CU with 64 x 256 tiles: the prefill kernel switches to 64 x 384 tiles (65 row-blocks x
    53 token tiles: one round of 159 blocks instead of 135 larger ones; the profiles with wide units keep 128 x 256) or
    to 128 x 256 tiles (16 row-blocks x 16500 tokens: 129 blocks instead of 258).  Ragged everywhere: row-blocks, K not
    a multiple of the groupsize, a last token tile with one or 116 rows."""
    rng = np.random.default_rng(270 + bits + out)
    K = 280
    t = O.quantize_nint((rng.standard_normal((out, K)) * 0.02).astype(np.float32), bits, gs, sb)
    lin = _load(t)
    x, xf = _x(rng, M, K)
    y = lin(x).cpu().numpy()
    ref = O.linear_forward_f64(O.dequantize_nint(t), xf)
    assert rel_l2(y, ref) < REL_TOL, rel_l2(y, ref)
    assert np.abs(y - ref).max() < ABS_TOL


@pytest.mark.parametrize("bits,gs,sb", [(4, 32, 6), (4, 24, 6), (4, 16, 6), (4, 48, 6), (3, 24, 5), (2, 16, 5), (2, 32, 5)])
@pytest.mark.parametrize("out,M", [(1040, 3329), (256, 16500), (512, 300)])
def test_gemm_tiles_copied_straight_into_lds(bits, gs, sb, out, M):
    """Profiles whose groups are whole 16-byte chunks copy the activation tiles from global memory straight into a ring
    of LDS buffers, three sub-steps ahead of the multiply, on all three tile shapes (64 x 384, 128 x 256 -- not for
    groups of 48, whose four buffers would not fit -- and 64 x 256).  K spans several steps and ends inside one; the
    result is the same on every run."""
    rng = np.random.default_rng(570 + bits + gs + out)
    K = 2056
    t = O.quantize_nint((rng.standard_normal((out, K)) * 0.02).astype(np.float32), bits, gs, sb)
    lin = _load(t)
    x, xf = _x(rng, M, K)
    y = lin(x).cpu().numpy()
    ref = O.linear_forward_f64(O.dequantize_nint(t), xf)
    assert rel_l2(y, ref) < REL_TOL, rel_l2(y, ref)
    assert np.abs(y - ref).max() < ABS_TOL
    for _ in range(3):
        assert np.array_equal(y, lin(x).cpu().numpy())


@pytest.mark.parametrize("bits,gs,sb", [(4, 32, 6), (3, 24, 5), (5, 28, 7)])
def test_gemm_long_k_few_neurons_is_split_over_k(bits, gs, sb):
    """A grid of nine 64-token tiles on 256 neurons leaves most CUs idle: the prefill launch is cut along K (four
    splits of five steps, the last one shorter and ragged) and the partial results are added afterwards."""
    rng = np.random.default_rng(370 + bits)
    out, K, M = 256, 8200, 520
    t = O.quantize_nint((rng.standard_normal((out, K)) * 0.02).astype(np.float32), bits, gs, sb)
    lin = _load(t)
    x, xf = _x(rng, M, K)
    y = lin(x).cpu().numpy()
    ref = O.linear_forward_f64(O.dequantize_nint(t), xf)
    assert rel_l2(y, ref) < REL_TOL, rel_l2(y, ref)
    assert np.abs(y - ref).max() < ABS_TOL
    assert np.array_equal(y, lin(x).cpu().numpy())   # partial sums are added in a fixed order


@pytest.mark.parametrize("bits,gs,sb", [(4, 32, 6), (3, 24, 5), (2, 16, 5), (5, 28, 7), (4, 24, 6)])
@pytest.mark.parametrize("W,K", [(48, 280), (64, 9000)])
def test_gate_up_gemv_with_fused_swiglu(bits, gs, sb, W, K):
    """silu(gate) * up in the GEMV's epilogue for one and two rows (K = 9000: more than three steps per wave for the
    16-wide groups, the variant with a prefetch ring); three rows fall back to matmul + SwiGLU."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(470 + bits + W)
    t = O.quantize_nint((rng.standard_normal((2 * W, K)) * 0.02).astype(np.float32), bits, gs, sb)
    lin = _load(t)
    deq = O.dequantize_nint(t)
    for M in (1, 2, 3):
        for dtype in (torch.bfloat16, torch.float16):
            x, xf = _x(rng, M, K, dtype)
            h = R.nint_matmul_swiglu(lin.weight, x).float().cpu().numpy()
            y = O.linear_forward_f64(deq, xf)
            g, u = y[:, :W], y[:, W:]
            ref = g / (1.0 + np.exp(-g)) * u
            assert h.shape == (M, W)
            assert rel_l2(h, ref) < 2e-3, rel_l2(h, ref)   # fp16 output: half an ulp is 5e-4


@pytest.mark.parametrize("bits,gs,sb", [(4, 32, 6), (3, 24, 5), (5, 28, 7)])
def test_gate_up_gemv_with_fused_geglu(bits, gs, sb):
    """gelu_tanh(gate) * up in the same epilogue (one and two rows) and through matmul + the elementwise kernel (three
    rows); the weights are scaled up so that the gate values cover the curved part of the GELU."""
    from tyloquant_amd import runtime as R
    W, K = 64, 1000
    rng = np.random.default_rng(480 + bits)
    t = O.quantize_nint((rng.standard_normal((2 * W, K)) * 0.06).astype(np.float32), bits, gs, sb)
    lin = _load(t)
    deq = O.dequantize_nint(t)
    for M in (1, 2, 3):
        for dtype in (torch.bfloat16, torch.float16):
            x, xf = _x(rng, M, K, dtype)
            h = R.nint_matmul_geglu(lin.weight, x).float().cpu().numpy()
            y = O.linear_forward_f64(deq, xf)
            ref = O.moe_geglu(y)
            assert h.shape == (M, W) and np.abs(y[:, :W]).max() > 2.0
            assert rel_l2(h, ref) < 2e-3, rel_l2(h, ref)   # fp16 output: half an ulp is 5e-4
            sw = R.nint_matmul_swiglu(lin.weight, x).float().cpu().numpy()
            assert rel_l2(sw, O.moe_swiglu(y)) < 2e-3 and rel_l2(sw, h) > 1e-2   # the two activations differ


@pytest.mark.parametrize("bits,gs,sb,W,K,M", [
    (4, 32, 6, 1024, 200, 1100),   # 64-token tiles, ragged last tile, K short of a whole step
    (4, 32, 6, 1040, 256, 2200),   # 128-token tiles; 65 gate row-blocks: the last block holds one
    (3, 24, 5, 1024, 240, 1100),
    (2, 16, 4, 1024, 256, 1100),
    (5, 28, 7, 1024, 224, 1100),   # the natural-order unit
    (4, 48, 6, 1024, 384, 2200),   # activation tiles through registers
])
def test_gate_up_prefill_with_fused_glu(bits, gs, sb, W, K, M):
    """act(gate) * up in the epilogue of the block-tiled prefill kernel: the C entry point takes the call, its values
    are those of matmul + the element-wise GLU kernel (same fp32 sums; the fused kernel contracts the last multiply,
    so a product on a 16-bit rounding midpoint may land one unit apart) and match the float64 oracle."""
    from tyloquant_amd import _lib as L
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_moe import moe_glu
    rng = np.random.default_rng(4700 + bits + W + M)
    t = O.quantize_nint((rng.standard_normal((2 * W, K)) * 0.08).astype(np.float32), bits, gs, sb)
    lin = _load(t)
    w = lin.weight
    deq = O.dequantize_nint(t)
    lib = L.lib()
    for dtype, act in ((torch.bfloat16, L.GLU_SILU), (torch.float16, L.GLU_GELU)):
        x, xf = _x(rng, M, K, dtype)
        need = lib.mfq_hip_nint_gemm_workspace_bytes(C.byref(w.desc), M)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        h = torch.full((M, W + 8), 7.0, dtype=dtype, device="cuda")   # padded rows: the padding must stay untouched
        rc = lib.mfq_hip_nint_gemm_glu(C.byref(w.desc), w.data.data_ptr(), x.data_ptr(), R._x_dtype(x), x.stride(0), M, act,
                                       h.data_ptr(), R._x_dtype(h), h.stride(0), ws.data_ptr(), need, None)
        assert rc == L.OK, L.lib().mfq_hip_last_error()
        assert (h[:, W:] == 7.0).all()
        two = moe_glu(R.nint_matmul(w, x), dtype, act)
        def ordinal(v):                       # 16-bit patterns on a line: neighbours differ by 1, -0 and +0 coincide
            i = v.contiguous().view(torch.int16).int()
            return torch.where(i < 0, -(i & 0x7FFF), i)
        diff = (ordinal(h[:, :W]) - ordinal(two)).abs()
        assert diff.max().item() <= 1 and (diff != 0).float().mean().item() < 1e-3
        y = O.linear_forward_f64(deq, xf)
        ref = O.moe_swiglu(y) if act == L.GLU_SILU else O.moe_geglu(y)
        assert np.abs(y[:, :W]).max() > 2.0
        tol = 6e-3 if dtype == torch.bfloat16 else 2e-3                # one 16-bit rounding of the result
        assert rel_l2(h[:, :W].float().cpu().numpy(), ref) < tol
        host = (R.nint_matmul_swiglu if act == L.GLU_SILU else R.nint_matmul_geglu)(w, x, out_dtype=dtype)
        assert torch.equal(host, h[:, :W])                             # the host wrapper takes the same path


def test_gate_up_prefill_glu_declines_what_the_kernel_does_not_take():
    """Few rows (the streaming kernels' range), grids that are split over K and an odd neuron count: nothing is launched,
    the error names the reason, and the host wrapper runs matmul + GLU instead."""
    from tyloquant_amd import _lib as L
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(4790)
    t = O.quantize_nint((rng.standard_normal((2 * 64, 2048)) * 0.05).astype(np.float32), 4, 32, 6)
    lin = _load(t)
    w = lin.weight
    lib = L.lib()
    for M in (4, 700):
        x, xf = _x(rng, M, 2048, torch.bfloat16)
        need = lib.mfq_hip_nint_gemm_workspace_bytes(C.byref(w.desc), M)
        ws = torch.empty(max(need, 256), dtype=torch.uint8, device="cuda")
        h = torch.zeros((M, 64), dtype=torch.bfloat16, device="cuda")
        rc = lib.mfq_hip_nint_gemm_glu(C.byref(w.desc), w.data.data_ptr(), x.data_ptr(), L.X_BF16, x.stride(0), M,
                                       L.GLU_SILU, h.data_ptr(), L.X_BF16, 64, ws.data_ptr(), need, None)
        assert rc == L.ERR_UNSUPPORTED and b"one-pass" in lib.mfq_hip_last_error()
        assert not h.any()
        got = R.nint_matmul_swiglu(w, x, out_dtype=torch.bfloat16).float().cpu().numpy()
        ref = O.moe_swiglu(O.linear_forward_f64(O.dequantize_nint(t), xf))
        assert rel_l2(got, ref) < 6e-3


@pytest.mark.parametrize("K", [1000, 77])
@pytest.mark.parametrize("mode", [0, 1])
def test_input_gate_then_matmul(mode, K):
    """x * silu(gate) or x * sigmoid(gate) ahead of the projection: the gated rows against the float64 product (one
    16-bit rounding), the matmul against the oracle on those rows; K = 77 takes the element-wise kernel."""
    from tyloquant_amd import _lib as L
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(490 + mode + K)
    t = O.quantize_nint((rng.standard_normal((48, K)) * 0.02).astype(np.float32), 4, 24, 6)
    lin = _load(t)
    deq = O.dequantize_nint(t)
    for M in (1, 5):
        for dtype in (torch.bfloat16, torch.float16):
            x, xf = _x(rng, M, K, dtype)
            g, gf = _x(rng, M, K, dtype)
            gated = torch.empty_like(x)
            L.check(L.lib().mfq_hip_input_gate(x.data_ptr(), g.data_ptr(), R._x_dtype(x), x.stride(0), g.stride(0), M, K,
                                               mode, gated.data_ptr(), gated.stride(0), None))
            want = O.input_mul(xf, gf, mode)
            eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
            got = gated.float().cpu().numpy().astype(np.float64)
            assert np.all(np.abs(got - want) <= eps * np.abs(want) + 1e-7)      # one rounding of the exact product
            assert np.array_equal(got[want == 0], want[want == 0])
            y = R.nint_matmul_input_mul(lin.weight, x, g, mode).cpu().numpy()
            ref = O.linear_forward_f64(deq, got.astype(np.float32))
            assert rel_l2(y, ref) < REL_TOL and np.abs(y - ref).max() < ABS_TOL


@pytest.mark.parametrize("bits,gs,sb", [(4, 32, 6), (4, 24, 6), (3, 24, 5), (2, 16, 5), (5, 28, 7), (6, 20, 6), (6, 24, 7),
                                        (8, 48, 7)])
@pytest.mark.parametrize("mode", [0, 1])
def test_input_gate_inside_the_gemv(bits, gs, sb, mode):
    """One or two rows: the gate is applied by the GEMV's own activation staging (mfq_hip_nint_gemv_gate).  Against the
    oracle on the once-rounded gated rows, and against the two-launch form (same rounding of the gated rows: the results
    differ by fp32 summation order at most); three rows and misaligned rows take the two launches."""
    from tyloquant_amd import _lib as L
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(4900 + 16 * bits + gs + mode)
    for out, K in ((80, 2048), (48, 4096), (33, 840)):
        t = O.quantize_nint((rng.standard_normal((out, K)) * 0.02).astype(np.float32), bits, gs, sb)
        lin = _load(t)
        deq = O.dequantize_nint(t)
        for M in (1, 2):
            for dtype in (torch.bfloat16, torch.float16):
                x, xf = _x(rng, M, K, dtype)
                g, gf = _x(rng, M, K, dtype)
                y = torch.empty((M, out), dtype=torch.float32, device="cuda")
                rc = L.lib().mfq_hip_nint_gemv_gate(C.byref(lin.weight.desc), lin.weight.data.data_ptr(), x.data_ptr(),
                                                    g.data_ptr(), R._x_dtype(x), x.stride(0), g.stride(0), M, mode,
                                                    y.data_ptr(), y.stride(0), None)
                assert rc == 0, L.lib().mfq_hip_last_error()
                two = R.nint_matmul_input_mul(lin.weight, x, g, mode, fused=False)
                # (NINT8-48 takes its plain matmul on the matrix cores, where 8-bit code x 7-bit sub-scale is rounded to
                # fp16's eleven bits: the two forms then agree to that rounding, not to the summation order)
                assert torch.allclose(y, two, rtol=1e-3, atol=1e-4 if bits < 8 else 2e-3)
                one = R.nint_matmul_input_mul(lin.weight, x, g, mode)
                assert torch.equal(one, y)
                gated = torch.from_numpy(O.input_mul(xf, gf, mode).astype(np.float32)).to(dtype).float().numpy()
                ref = O.linear_forward_f64(deq, gated)
                yn = y.cpu().numpy()
                assert rel_l2(yn, ref) < REL_TOL and np.abs(yn - ref).max() < ABS_TOL
    # declined: three rows, a misaligned row
    x, _ = _x(rng, 3, K, torch.bfloat16)
    y = torch.empty((3, out), dtype=torch.float32, device="cuda")
    args = (C.byref(lin.weight.desc), lin.weight.data.data_ptr())
    assert L.lib().mfq_hip_nint_gemv_gate(*args, x.data_ptr(), x.data_ptr(), L.X_BF16, K, K, 3, 0, y.data_ptr(), out,
                                          None) == L.ERR_UNSUPPORTED
    assert L.lib().mfq_hip_nint_gemv_gate(*args, x.data_ptr() + 2, x.data_ptr(), L.X_BF16, K, K, 1, 0, y.data_ptr(), out,
                                          None) == L.ERR_UNSUPPORTED


@pytest.mark.parametrize("out,K", [(37, 96), (130, 1056), (64, 4096), (9000, 64)])
def test_nint8_zero_dequant_bit_exact_and_matmul(out, K):
    """NINT8-0 (GGML Q8_0 blocks): the device dequantizer against the oracle bit for bit; the streaming kernel for 1..33
    rows (8 per pass, more than 8192 rows: several rows per wave) and the dequantize + fp16 GEMM path above it."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(600 + out + K)
    w = (rng.standard_normal((out, K)) * 0.02).astype(np.float32)
    w[0, :32] = 0.0                                   # an all-zero block: scale 0
    t = O.quantize_nint8_zero(w)
    dtype, blob = O.pack_tensor(t)
    assert dtype == "NINT8-0"
    lin = R.load_quant_linear(dtype, blob)
    deq = O.dequantize_nint8_zero(O.unpack_nint8_zero(blob))
    got = lin.dequantize().cpu().numpy()
    assert np.array_equal(got.view(np.uint32), deq.view(np.uint32))
    for M in (1, 2, 3, 8, 11, 33, 300):
        if out * K * M > 3e8:
            continue
        for xd in (torch.bfloat16, torch.float16):
            x, xf = _x(rng, M, K, xd)
            y = lin(x).cpu().numpy()
            ref = O.linear_forward_f64(deq, xf)
            assert rel_l2(y, ref) < REL_TOL, (M, rel_l2(y, ref))
            assert np.abs(y - ref).max() < ABS_TOL
    x, xf = _x(rng, 40, K)                            # the streaming kernel beyond its default range
    y = R.nint8_zero_matmul(lin.weight, x, force="gemv").cpu().numpy()
    assert rel_l2(y, O.linear_forward_f64(deq, xf)) < REL_TOL
    # bf16 rows far outside fp16's range on the streaming kernel (every row scaled by its own power of two): one row at a
    # time, and three rows of different magnitudes in one misaligned batch (aligned batches run on the matrix cores)
    x, xf = _x(rng, 3, K)
    sc = torch.tensor([[1e-6], [1.0], [3e6]])
    xs = (x.float().cpu() * sc).to(torch.bfloat16)
    ref = O.linear_forward_f64(deq, xs.float().numpy())
    ys = [R.nint8_zero_matmul(lin.weight, xs[m:m + 1].cuda(), force="gemv").cpu().numpy()[0] for m in range(3)]
    ys3 = R.nint8_zero_matmul(lin.weight, torch.zeros((3, K + 3), dtype=torch.bfloat16, device="cuda")[:, 1:K + 1].copy_(xs),
                              force="gemv").cpu().numpy()
    for m in range(3):
        assert rel_l2(ys[m], ref[m]) < REL_TOL, (m, rel_l2(ys[m], ref[m]))
        assert rel_l2(ys3[m], ref[m]) < REL_TOL, (m, rel_l2(ys3[m], ref[m]))


@pytest.mark.parametrize("cus,out,K", [(4, 200, 1056), (3, 96, 4096), (2, 40, 96), (64, 33, 2048)])
def test_nint8_zero_tile_kernel_row_blocks_per_block(cu_count, cus, out, K):
    """2 .. 32 rows on the matrix cores: a block owns ceil(row-blocks / CUs) row-blocks, up to four (4, 2, 2 and 1 here),
    the last block fewer; one and two 16-row tiles; K with a partial last chunk of eight blocks (1056 = 33 blocks, 96 = 3);
    a row stride above K; rows that are not 16-byte aligned fall back to the vector-ALU kernel."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(640 + out + K)
    t = O.quantize_nint8_zero((rng.standard_normal((out, K)) * 0.02).astype(np.float32))
    lin = R.load_quant_linear("NINT8-0", O.pack_nint8_zero(t))
    deq = O.dequantize_nint8_zero(t)
    cu_count(cus)
    for M in (2, 9, 16, 21, 32):
        for xd in (torch.bfloat16, torch.float16):
            xw = torch.from_numpy(rng.standard_normal((M, K + 8)).astype(np.float32)).to(xd).cuda()
            x = xw[:, :K]
            y = lin(x).cpu().numpy()
            ref = O.linear_forward_f64(deq, x.float().cpu().numpy())
            assert rel_l2(y, ref) < REL_TOL and np.abs(y - ref).max() < ABS_TOL, (M, xd)
    xo = torch.from_numpy(rng.standard_normal((5, K + 9)).astype(np.float32)).to(torch.bfloat16).cuda()[:, 1:K + 1]
    y = lin(xo).cpu().numpy()
    assert rel_l2(y, O.linear_forward_f64(deq, xo.float().cpu().numpy())) < REL_TOL


def test_nint8_zero_loader_errors():
    from tyloquant_amd import runtime as R
    t = O.quantize_nint8_zero(np.ones((4, 64), np.float32))
    blob = O.pack_nint8_zero(t)
    with pytest.raises(ValueError, match="invalid NINT8-0 block bytes"):
        R.load_quant_linear("NINT8-0", blob[:-2])
    with pytest.raises(ValueError, match="invalid NINT8-0 magic"):
        R.load_quant_linear("NINT8-0", b"NI81" + blob[4:])
    t1 = O.quantize_nint8_zero(np.ones((64, 4), np.float32), axis=1)
    with pytest.raises(ValueError, match="axis 0"):
        R.load_quant_linear("NINT8-0", O.pack_nint8_zero(t1))


def test_config1_shape_nint3():
    """BASELINE config 1: 4096x4096 N(0, 0.02) NINT3 (3,24,5), bf16 x at batch 1."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(1)
    out = K = 4096
    W = (rng.standard_normal((out, K)) * 0.02).astype(np.float32)
    t = O.quantize_nint(W, 3, 24, 5)
    blob = O.pack_nint(t)
    assert len(blob) - 0 >= O.nint_payload_nbytes(out, K, 3, 24, 5) == 7195648
    lin = R.load_quant_linear("NINT3", blob)
    deq = O.dequantize_nint(t)
    assert np.array_equal(lin.dequantize().cpu().numpy().view(np.uint32), deq.view(np.uint32))
    x, xf = _x(rng, 1, K)
    y = lin(x).cpu().numpy()
    ref = O.linear_forward(deq, xf)
    assert rel_l2(y, ref) < REL_TOL
    assert np.abs(y - ref).max() < ABS_TOL


def test_legacy_byte_tail_and_errors():
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(5)
    t = _rand_tensor(rng, 8, 96, 4, 24, 6)
    blob = O.pack_nint(t)
    hdr = blob[: len(blob) - (O.nint_payload_nbytes(8, 96, 4, 24, 6) - 32)]
    legacy = hdr + t.sub_scale.tobytes() + t.sub_min.tobytes() + t.q.tobytes()
    lin = R.load_quant_linear("NINT4", legacy)
    assert np.array_equal(lin.dequantize().cpu().numpy(), O.dequantize_nint(t))
    with pytest.raises(ValueError, match="invalid NINT blob tail"):
        R.load_quant_linear("NINT4", blob[:-1])
    with pytest.raises(ValueError, match="dtype/blob mismatch"):
        R.load_quant_linear("NINT5", blob)
    with pytest.raises(ValueError):
        R.load_quant_linear("NOPE", blob)


@pytest.mark.parametrize("K", [32768, 81920])
def test_gemv_long_neurons(K):
    """Neurons whose staged activation slice exceeds 64 KB of LDS: up to 160 KB the GEMV block opts in to the larger
    LDS (K = 32768: 74 KB), beyond that the matrix-core streaming kernel takes over (K = 81920).  One and two rows,
    and the fused gate/up SwiGLU on the first shape."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(K)
    t = synth.nint_random(rng, 64, K, 4, 32, 6)
    t.neuron_scale = O._f16_round(t.neuron_scale * 0.02)
    t.neuron_min = O._f16_round(t.neuron_min * 0.02)
    lin = _load(t)
    deq = O.dequantize_nint(t)
    for M in (1, 2):
        x, xf = _x(rng, M, K)
        y = R.nint_matmul(lin.weight, x, force="gemv").cpu().numpy()
        ref = O.linear_forward_f64(deq, xf)
        assert rel_l2(y, ref) < REL_TOL, (M, rel_l2(y, ref))
    if K == 32768:
        x, xf = _x(rng, 1, K)
        h = R.nint_matmul_swiglu(lin.weight, x).float().cpu().numpy()
        want = O.moe_swiglu(O.linear_forward_f64(deq, xf).astype(np.float32))
        assert rel_l2(h, want) < 2e-3


@pytest.mark.parametrize("bits,gs,sb", [(4, 32, 6), (4, 24, 6), (3, 24, 5), (2, 16, 5)])
@pytest.mark.parametrize("H,W,N,cus", [(256, 384, 256, 8), (4096, 112, 128, 8), (520, 368, 48, 8), (512, 8448, 64, 0),
                                       (1024, 160, 4096, 0)])
def test_ffn_decode_one_launch(cu_count, bits, gs, sb, H, W, N, cus):
    """The one-launch decode FFN (gate/up + GLU, grid barrier, down) against the oracle's fp64 FFN and the two-launch
    path.  With the grid sized for 8 compute units the blocks own three row-block pairs and two down row-blocks;
    W = 8448 gives the down phase two K steps per wave on the full grid; H = 520 ends inside a group; N = 4096 has
    more down row-blocks than gate/up pairs.  Called twice per activation type: every block's barrier flag advances by one per call."""
    from tyloquant_amd import _lib as L
    from tyloquant_amd import runtime as R
    if cus:
        cu_count(cus)
    if W == 8448 and gs == 16:
        W = 8192                      # 32 steps: two per wave, as 8448 gives the wider groups
    rng = np.random.default_rng(bits * 1000 + H + W)
    tg = O.quantize_nint((rng.standard_normal((2 * W, H)) * 0.02).astype(np.float32), bits, gs, sb)
    td = O.quantize_nint((rng.standard_normal((N, W)) * 0.02).astype(np.float32), bits, gs, sb)
    gu, dn = _load(tg).weight, _load(td).weight
    assert L.lib().mfq_hip_nint_ffn_decode_workspace_bytes(gu.desc, dn.desc) > 0
    dg, dd = O.dequantize_nint(tg), O.dequantize_nint(td)
    for dtype, act, glu in ((torch.bfloat16, L.GLU_SILU, O.moe_swiglu), (torch.float16, L.GLU_GELU, O.moe_geglu)):
        x, xf = _x(rng, 1, H, dtype)
        y1 = R.nint_ffn_decode(gu, dn, x, act, one_launch=True)
        y2 = R.nint_ffn_decode(gu, dn, x, act, one_launch=True)
        assert torch.equal(y1, y2) and bool(torch.isfinite(y1).all())
        hidden = glu(O.linear_forward_f64(dg, xf).astype(np.float32)).astype(np.float64)
        ref = hidden @ dd.astype(np.float64).T
        y = y1.cpu().numpy()
        assert rel_l2(y, ref) < REL_TOL, (dtype, rel_l2(y, ref))
        assert np.abs(y - ref).max() < ABS_TOL
        two = R.nint_matmul(dn, R._nint_matmul_glu(gu, x, torch.float16, act)).cpu().numpy()
        assert rel_l2(y, two) < 1e-4                     # same hidden rounding, another order of the sums over K
    G = int(re.search(r"cu_count=(\d+)", L.lib().mfq_hip_config().decode()).group(1))   # the grid the library launched
    assert G == cus or not cus
    words = gu._ffn_ws[:4096].view(torch.int32).cpu().numpy()
    assert np.all(words[:G] == 4) and words[G] == 0       # every block crossed four barriers; the error word is clear
    assert L.lib().mfq_hip_nint_ffn_decode_status(gu._ffn_ws.data_ptr(), None) == 0


def test_ffn_decode_refuses_a_grid_the_device_cannot_hold(cu_count):
    """More blocks than the device has compute units could never all reach the grid barrier: the call refuses
    (no launch), the workspace query still answers for the forced grid, and the host path runs the two launches."""
    import ctypes as C
    from tyloquant_amd import _lib as L
    from tyloquant_amd import runtime as R
    lib = L.lib()
    real = int(re.search(r"cu_count=(\d+)", lib.mfq_hip_config().decode()).group(1))
    rng = np.random.default_rng(9)
    H, W, N = 256, 16 * (real + 8), 64
    tg = O.quantize_nint((rng.standard_normal((2 * W, H)) * 0.02).astype(np.float32), 4, 32, 6)
    td = O.quantize_nint((rng.standard_normal((N, W)) * 0.02).astype(np.float32), 4, 32, 6)
    gu, dn = _load(tg).weight, _load(td).weight
    x, xf = _x(rng, 1, H, torch.bfloat16)
    cu_count(real + 8)
    need = lib.mfq_hip_nint_ffn_decode_workspace_bytes(C.byref(gu.desc), C.byref(dn.desc))
    if need:
        ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
        y = torch.empty((1, N), dtype=torch.float32, device="cuda")
        rc = lib.mfq_hip_nint_ffn_decode(C.byref(gu.desc), gu.data.data_ptr(), C.byref(dn.desc), dn.data.data_ptr(), x.data_ptr(),
                                         L.X_BF16, L.GLU_SILU, y.data_ptr(), ws.data_ptr(), need, None)
        assert rc == L.ERR_UNSUPPORTED and b"cannot all run at once" in lib.mfq_hip_last_error()


def test_ffn_decode_shapes_outside_the_kernel_take_two_launches():
    """Different profiles for gate/up and down, or more work per wave than the kernel keeps in registers: the
    workspace query says 0, the C entry point refuses with a message, and the host path runs the two launches."""
    import ctypes as C
    from tyloquant_amd import _lib as L
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(3)
    H, W, N = 256, 128, 64
    tg = O.quantize_nint((rng.standard_normal((2 * W, H)) * 0.02).astype(np.float32), 4, 32, 6)
    td = O.quantize_nint((rng.standard_normal((N, W)) * 0.02).astype(np.float32), 3, 24, 5)
    gu, dn = _load(tg).weight, _load(td).weight
    lib = L.lib()
    assert lib.mfq_hip_nint_ffn_decode_workspace_bytes(gu.desc, dn.desc) == 0
    x, xf = _x(rng, 1, H)
    y = torch.empty((1, N), dtype=torch.float32, device="cuda")
    ws = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    p = lambda t: C.c_void_p(t.data_ptr())
    rc = lib.mfq_hip_nint_ffn_decode(C.byref(gu.desc), p(gu.data), C.byref(dn.desc), p(dn.data), p(x), L.X_BF16, L.GLU_SILU,
                                     p(y), p(ws), 4096, None)
    assert rc == 2 and b"outside the one-launch kernel" in lib.mfq_hip_last_error()
    out = R.nint_ffn_decode(gu, dn, x, one_launch=True).cpu().numpy()
    hidden = O.moe_swiglu(O.linear_forward_f64(O.dequantize_nint(tg), xf).astype(np.float32)).astype(np.float64)
    assert rel_l2(out, hidden @ O.dequantize_nint(td).astype(np.float64).T) < REL_TOL
    # three rows: the batch path
    x3, x3f = _x(rng, 3, H)
    assert R.nint_ffn_decode(gu, dn, x3).shape == (3, N)


@pytest.mark.parametrize("bits,gs,sb", [(4, 32, 6), (3, 24, 5), (2, 16, 5), (5, 28, 7), (6, 24, 6)])
@pytest.mark.parametrize("scale", [1e-6, 1e-4, 1e4, 3e6])
def test_gemv_bf16_rows_of_any_magnitude(bits, gs, sb, scale):
    """The stated range contract: a bf16 row far outside fp16's comfortable range (all of it scaled by 1e-6 ... 3e6,
    i.e. beyond 65504 and deep inside fp16's subnormals) gives the accuracy of an ordinary row on the batch-1 / batch-2
    NINT kernels and the fused GLU, and on the prefill kernel; config 2's outlier channels (x 20) on top."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd import synth as P
    rng = np.random.default_rng(int(scale * 1e6) % 1000 + bits)
    out, K = 64, 2048
    t = O.quantize_nint((rng.standard_normal((out, K)) * 0.02).astype(np.float32), bits, gs, sb)
    lin = _load(t)
    deq = O.dequantize_nint(t)
    for M in (1, 2, 300):
        x = torch.from_numpy(P.activations(rng, M, K, outlier_frac=0.001) * np.float32(scale)).to(torch.bfloat16)
        ref = O.linear_forward_f64(deq, x.float().numpy())
        y = (lin(x.cuda()) if M > 2 else R.nint_matmul(lin.weight, x.cuda(), force="gemv")).cpu().numpy()
        assert np.isfinite(y).all()
        assert rel_l2(y, ref) < REL_TOL, (M, scale, rel_l2(y, ref))
    if bits != 6:
        x = torch.from_numpy(P.activations(rng, 1, K) * np.float32(scale)).to(torch.bfloat16)
        g = R.nint_matmul(lin.weight, x.cuda(), force="gemv").cpu().numpy()
        want = O.moe_swiglu(O.linear_forward_f64(deq, x.float().numpy()).astype(np.float32))
        if scale <= 1e4:                                   # beyond that silu(gate) * up leaves fp16's range by itself
            h = R.nint_matmul_swiglu(lin.weight, x.cuda(), torch.bfloat16).float().cpu().numpy()
            assert rel_l2(h, want) < 6e-3                  # bf16 output: half an ulp is 4e-3


@pytest.mark.parametrize("bits,gs,sb,K", [(4, 32, 6, 2048), (4, 32, 6, 4040), (2, 16, 5, 1536), (2, 32, 5, 4096)])
def test_small_batches_take_bf16_rows_of_any_magnitude(bits, gs, sb, K):
    """3 to 16 rows on the kernel that keeps the activations in LDS (one K step per wave, groups of 32 or 16): every row
    of the tile has its own magnitude, from 1e-6 to 3e6 times an ordinary row, in one batch -- each comes out with the
    accuracy of an ordinary row, as on the one-row kernels.  K = 4040 ends inside a step (the rest of the step reads zeros)."""
    from tyloquant_amd import synth as P
    rng = np.random.default_rng(bits * 100 + gs + K)
    out = 80
    t = O.quantize_nint((rng.standard_normal((out, K)) * 0.02).astype(np.float32), bits, gs, sb)
    lin = _load(t)
    deq = O.dequantize_nint(t)
    for M in (3, 5, 16):
        scales = np.float32(10.0) ** rng.uniform(-6, 6.4, size=(M, 1)).astype(np.float32)
        scales[0], scales[-1] = np.float32(1e-6), np.float32(3e6)
        x = torch.from_numpy(P.activations(rng, M, K, outlier_frac=0.001) * scales).to(torch.bfloat16)
        ref = O.linear_forward_f64(deq, x.float().numpy())
        y = lin(x.cuda()).cpu().numpy()
        assert np.isfinite(y).all()
        for m in range(M):
            assert rel_l2(y[m], ref[m]) < REL_TOL, (M, m, float(scales[m, 0]), rel_l2(y[m], ref[m]))
    # groups whose 32 activations all sit at the row's largest magnitude, with one sign: the group sums of the minimum term
    x = torch.full((4, K), 3.0, dtype=torch.bfloat16) * torch.tensor([[1.0], [-1.0], [1e-5], [2e5]], dtype=torch.bfloat16)
    ref = O.linear_forward_f64(deq, x.float().numpy())
    y = lin(x.cuda()).cpu().numpy()
    for m in range(4):
        assert rel_l2(y[m], ref[m]) < REL_TOL, (m, rel_l2(y[m], ref[m]))


def test_reserved_workspace_lets_forward_run_under_graph_capture():
    """QuantLinear.reserve(max_rows) sizes the weight's workspace once; forward() of any smaller batch then allocates
    nothing of its own and can be captured into a HIP graph (batch-1 GEMV, streaming kernel and prefill kernel with its
    activation prep).  Every replay, with eager work in between, equals the eager result."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(77)
    t = O.quantize_nint((rng.standard_normal((96, 1024)) * 0.02).astype(np.float32), 4, 32, 6)
    lin = _load(t)
    lin.reserve(300)
    buf = lin.weight._ws.buf
    for M in (1, 16, 300):
        x, _ = _x(rng, M, 1024)
        eager = lin(x).clone()
        assert lin.weight._ws.buf is buf                     # no regrowth after reserve()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            lin(x)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            y = lin(x)
        for rep in range(3):
            y.fill_(float("nan"))
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, eager), (M, rep)
            other, _ = _x(rng, 7, 1024)                      # eager work between the replays
            lin(other)
            torch.cuda.synchronize()
