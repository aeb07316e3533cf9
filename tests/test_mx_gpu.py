"""MXFP4 / MXFP8 on the GPU against the oracle: bit-exact dequantizer (fp32 and the fp16 copy), matmul on the GEMV and
GEMM routes, expert slices of a pool, the reference-written payload, loader errors."""
from pathlib import Path

import numpy as np
import pytest
import torch

import synth
from conftest import check_close
from oracle import mfq_oracle as O

pytestmark = pytest.mark.gpu
G = np.load(Path(__file__).resolve().parent / "golden" / "reference_mx.npz")


def same_bits(got, want, zero_sign=True):
    """bit-equal, a NaN matching any NaN; zero_sign=False: a zero of either sign matches a zero"""
    got, want = np.asarray(got), np.asarray(want)
    if got.shape != want.shape or got.dtype != want.dtype or not np.array_equal(np.isnan(got), np.isnan(want)):
        return False
    drop = (lambda a: np.isnan(a)) if zero_sign else (lambda a: np.isnan(a) | (a == 0))
    bits = np.uint32 if got.dtype == np.float32 else np.uint16
    return np.array_equal(np.where(drop(got), 0, got).view(bits), np.where(drop(want), 0, want).view(bits))


@pytest.mark.parametrize("key,dtype", [("fp4", "MXFP4"), ("fp8", "MXFP8")])
def test_reference_payload_dequantizes_bit_exactly(key, dtype):
    """The reference-written blob (every nibble / byte code, scales 0, 1, 254 and the NaN 255, a partial block row)."""
    from tyloquant_amd import runtime as R
    blob = G[f"{key}_blob"].tobytes()
    lin = R.load_quant_linear(dtype, blob)
    want = O.dequantize_mx(O.unpack_mx(dtype, blob))
    assert same_bits(lin.dequantize().cpu().numpy(), want)              # -0 for the E2M1 code 8, as the runtime has it
    with np.errstate(over="ignore"):
        # the fp16 copy: one more rounding; the hardware conversion drops the sign of a product that was an fp32 subnormal
        assert same_bits(lin.weight.dequantize(dtype=torch.float16).cpu().numpy(), want.astype(np.float16), zero_sign=False)
    ref = G[f"{key}_dequant"]                                            # the reference's own values (it writes +0)
    got = lin.dequantize().cpu().numpy()
    assert np.array_equal(np.isnan(got), np.isnan(ref)) and np.array_equal(np.nan_to_num(got), np.nan_to_num(ref))


@pytest.mark.parametrize("dtype,rows,cols", [("MXFP4", 70, 96), ("MXFP4", 257, 4096), ("MXFP8", 130, 256), ("MXFP8", 512, 2048)])
def test_mx_matmul_all_routes(dtype, rows, cols):
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(rows + cols)
    t = synth.mx_random(rng, dtype, rows, cols)
    lin = R.load_quant_linear(dtype, O.pack_mx(t))
    want = O.dequantize_mx(t)
    assert lin.out == rows and lin.neuron_len == cols
    assert same_bits(lin.dequantize().cpu().numpy(), want)
    for M, xdt in ((1, torch.bfloat16), (2, torch.float16), (3, torch.bfloat16), (16, torch.bfloat16), (17, torch.float16),
                   (70, torch.bfloat16), (300, torch.bfloat16), (257, torch.float16)):   # above 256 rows: fp16 copy + GEMM
        x = torch.from_numpy(rng.standard_normal((M, cols)).astype(np.float32)).to(xdt).cuda()
        check_close(lin(x).cpu().numpy(), O.linear_forward_f64(want, x.float().cpu().numpy()))
    assert lin(torch.empty((0, cols), dtype=torch.bfloat16, device="cuda")).shape == (0, rows)
    xw = torch.from_numpy(rng.standard_normal((5, cols + 8)).astype(np.float32)).to(torch.bfloat16).cuda()[:, :cols]
    check_close(lin(xw).cpu().numpy(), O.linear_forward_f64(want, xw.float().cpu().numpy()))    # a row stride above K


@pytest.mark.parametrize("dtype,rows,cols", [("MXFP4", 200, 2880), ("MXFP4", 48, 4096), ("MXFP8", 256, 384), ("MXFP8", 384, 2944)])
def test_mx_matrix_core_tiles(dtype, rows, cols):
    """The tile kernel's corners: K that ends inside a unit (2880 = 22.5 units of four scale blocks, scale rows off
    4-byte boundaries), row counts off the 16-neuron row-blocks, tiles of 1 .. 32 rows and passes of them, both
    activation types, rows of bf16 magnitudes fp16 cannot hold, and activations the kernel cannot take in 16-byte pieces."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(rows * 7 + cols)
    t = synth.mx_random(rng, dtype, rows, cols)
    lin = R.load_quant_linear(dtype, O.pack_mx(t))
    want = O.dequantize_mx(t)
    for M, xdt in ((1, torch.bfloat16), (1, torch.float16), (5, torch.bfloat16), (16, torch.float16), (31, torch.bfloat16),
                   (32, torch.bfloat16), (33, torch.float16), (100, torch.bfloat16), (256, torch.bfloat16)):
        x = torch.from_numpy(rng.standard_normal((M, cols)).astype(np.float32)).to(xdt).cuda()
        check_close(lin(x).cpu().numpy(), O.linear_forward_f64(want, x.float().cpu().numpy()))
    big = torch.from_numpy((rng.standard_normal((3, cols)) * 3.0e5).astype(np.float32)).to(torch.bfloat16).cuda()
    check_close(lin(big).cpu().numpy() / 3.0e5, O.linear_forward_f64(want, big.float().cpu().numpy()) / 3.0e5)
    odd = torch.from_numpy(rng.standard_normal((6, cols + 4)).astype(np.float32)).to(torch.bfloat16).cuda()[:, 4:]
    check_close(lin(odd).cpu().numpy(), O.linear_forward_f64(want, odd.float().cpu().numpy()))


@pytest.mark.parametrize("cus", [1, 2, 3, 5])
@pytest.mark.parametrize("dtype,rows,cols", [("MXFP4", 200, 2880), ("MXFP4", 272, 512), ("MXFP8", 384, 640)])
def test_mx_tiles_with_several_row_blocks_per_block(cu_count, cus, dtype, rows, cols):
    """Blocks of two to four row-blocks (the shapes a large tensor gets) on small tensors: the grid is sized for a few
    compute units, which makes the launcher share the staged rows between row-blocks -- whole and partial last blocks,
    one tile, several staged tiles and the 32-row tiles."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(rows + cols + cus)
    t = synth.mx_random(rng, dtype, rows, cols)
    lin = R.load_quant_linear(dtype, O.pack_mx(t))
    want = O.dequantize_mx(t)
    cu_count(cus)
    for M, xdt in ((1, torch.bfloat16), (6, torch.bfloat16), (16, torch.float16), (40, torch.bfloat16), (90, torch.bfloat16)):
        x = torch.from_numpy(rng.standard_normal((M, cols)).astype(np.float32)).to(xdt).cuda()
        check_close(lin(x).cpu().numpy(), O.linear_forward_f64(want, x.float().cpu().numpy()))


@pytest.mark.parametrize("dtype", ["MXFP4", "MXFP8"])
def test_mx_scale_bytes_0_and_255_in_the_matmul(dtype):
    """E8M0 0 is 2^-127 and 255 a NaN (mx_matmul.cu:17-28): a neuron whose row holds a NaN scale comes out NaN, the
    others are untouched; blocks under the smallest scale add nothing visible."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(77)
    rows, cols = 256, 512
    t = synth.mx_random(rng, dtype, rows, cols)
    t.scales[0, 0] = 255
    t.scales[-1, -1] = 0
    lin = R.load_quant_linear(dtype, O.pack_mx(t))
    want = O.dequantize_mx(t)
    nan_rows = np.isnan(want).any(axis=1)
    assert 0 < nan_rows.sum() < rows
    for M, xdt in ((1, torch.bfloat16), (4, torch.float16), (20, torch.bfloat16)):
        x = torch.from_numpy(rng.standard_normal((M, cols)).astype(np.float32)).to(xdt).cuda()
        got = lin(x).cpu().numpy()
        assert np.isnan(got[:, nan_rows]).all() and not np.isnan(got[:, ~nan_rows]).any()
        check_close(got[:, ~nan_rows], O.linear_forward_f64(want[~nan_rows], x.float().cpu().numpy()))


def test_mx_wide_scale_range_survives_the_fp16_copy():
    """Block scales 2^-40 .. 2^+40 in one tensor: the products leave fp16's range (the reference's fp16 copy saturates
    there); rows relative to their own largest scale keep the GEMM route within tolerance of the fp64 product."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(8)
    t = synth.mx_random(rng, "MXFP8", 256, 512)
    t.scales[:] = np.array([[87, 100, 127, 140], [167, 150, 127, 90]], np.uint8)
    lin = R.load_quant_linear("MXFP8", O.pack_mx(t))
    want = O.dequantize_mx(t)
    for M in (4, 40, 260):
        x = torch.from_numpy(rng.standard_normal((M, 512)).astype(np.float32)).to(torch.bfloat16).cuda()
        check_close(lin(x).cpu().numpy(), O.linear_forward_f64(want, x.float().cpu().numpy()))


@pytest.mark.parametrize("dtype,out", [("MXFP4", 48), ("MXFP8", 128)])
def test_mx_expert_slices_of_a_pool(dtype, out):
    from tyloquant_amd.runtime_mx import MxWeight, mx_matmul
    rng = np.random.default_rng(out)
    E, cols = 3, 384
    t = synth.mx_random(rng, dtype, E * out, cols)
    w = MxWeight.from_blob(dtype, O.pack_mx(t), out=out)
    want = O.dequantize_mx(t).reshape(E, out, cols)
    assert w.n_experts == E
    for e in range(E):
        assert same_bits(w.dequantize(e).cpu().numpy(), want[e])
        for M in (1, 5, 33):
            x = torch.from_numpy(rng.standard_normal((M, cols)).astype(np.float32)).to(torch.bfloat16).cuda()
            check_close(mx_matmul(w, x, e).cpu().numpy(), O.linear_forward_f64(want[e], x.float().cpu().numpy()))
    with pytest.raises(IndexError):
        mx_matmul(w, x, E)
    if dtype == "MXFP8":
        with pytest.raises(ValueError, match="128-row blocks"):
            MxWeight.from_blob(dtype, O.pack_mx(t), out=64)


def test_mx_loader_errors():
    from tyloquant_amd import runtime as R
    blob = G["fp4_blob"].tobytes()
    with pytest.raises(ValueError, match="invalid MXFP8 payload header"):
        R.load_quant_linear("MXFP8", blob)
    with pytest.raises(ValueError, match="truncated MFQ MX tensor header"):
        R.load_quant_linear("MXFP4", blob[:10])
    with pytest.raises(ValueError, match="payload size"):
        R.load_quant_linear("MXFP4", blob[:-1])
