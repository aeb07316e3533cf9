"""GPU parity of the NVQ (D4 family) and NEPQ1 paths against the oracle (through the C ABI)."""
import numpy as np
import pytest

import synth
from conftest import REL_TOL, check_close, rel_l2
from oracle import mfq_oracle as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _x(rng, M, K, dtype=None):
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(dtype or torch.bfloat16)
    return x.cuda(), x.float().numpy()


_check = check_close



@pytest.mark.parametrize("codebook,banks", [("d4_512", 2), ("d4_512", 4), ("d4_512", 1), ("d4_256", 2)])
@pytest.mark.parametrize("out,K", [(37, 96), (24, 80), (64, 200), (73, 1537), (33, 100)])
def test_nvq_jsc_dequant_bit_exact_and_gemv(codebook, banks, out, K):
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_vq import nvq_matmul
    rng = np.random.default_rng(7 + out + K + banks)
    t = synth.nvq_jsc_random(rng, out, K, codebook, banks)
    dtype, blob = O.pack_tensor(t)
    lin = R.load_quant_linear(dtype, blob)
    want = O.dequantize_nvq_jsc(O.unpack_nvq(blob))
    got = lin.dequantize().cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    for M in (1, 4, 8):
        for xd in (torch.bfloat16, torch.float16):
            x, xf = _x(rng, M, K, xd)
            _check(nvq_matmul(lin.weight, x, force="gemv").cpu().numpy(), O.linear_forward(want, xf))
    x, xf = _x(rng, 65, K)
    _check(lin(x).cpu().numpy(), O.linear_forward_f64(want, xf))


@pytest.mark.parametrize("out,K,M", [(48, 2048, 1), (40, 4104, 16), (130, 1024, 33), (64, 5120, 8)])
def test_nvq_matrix_core_path_multi_step(out, K, M):
    """K % 8 == 0 rows take the MFMA streaming kernel: several steps per neuron, K split over waves, ragged last
    group, more rows than one 16-row tile, a row stride above K."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_vq import nvq_matmul
    rng = np.random.default_rng(70 + out + M)
    t = synth.nvq_jsc_random(rng, out, K, "d4_512", 2)
    dtype, blob = O.pack_tensor(t)
    lin = R.load_quant_linear(dtype, blob)
    want = O.dequantize_nvq_jsc(O.unpack_nvq(blob))
    xw = torch.from_numpy(rng.standard_normal((M, K + 16)).astype(np.float32)).to(torch.bfloat16).cuda()
    x = xw[:, :K]
    _check(nvq_matmul(lin.weight, x, force="gemv").cpu().numpy(), O.linear_forward_f64(want, x.float().cpu().numpy()))


@pytest.mark.parametrize("K", [1560, 6160])
@pytest.mark.parametrize("rpb", [1, 2, 3, 4, 5, 6])
def test_nvq_signed_table_kernel_row_blocks_per_block(cu_count, rpb, K):
    """Up to 32 rows (16 per tile) with the (entry, sign nibble) table in LDS: one block per CU and tile owning rpb row-blocks.  With the CU
    count the grid is sized for set to 8, 128 * rpb - 5 neurons give every rpb variant (ragged last row-block, last
    block with fewer row-blocks); K = 1560 is one step per wave (5 waves), K = 6160 two steps per wave with a ragged
    last group.  One- and two-bank 512-entry codebooks and the 256-entry one."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_vq import nvq_matmul
    cu_count(8)
    out = 128 * rpb - 5
    rng = np.random.default_rng(900 + rpb + K)
    for codebook, banks in (("d4_512", 2), ("d4_512", 1), ("d4_256", 2)):
        t = synth.nvq_jsc_random(rng, out, K, codebook, banks)
        dtype, blob = O.pack_tensor(t)
        lin = R.load_quant_linear(dtype, blob)
        want = O.dequantize_nvq_jsc(O.unpack_nvq(blob))
        for M, xd in ((1, torch.bfloat16), (7, torch.float16), (16, torch.bfloat16), (17, torch.bfloat16),
                      (32, torch.float16)):                      # 17 and 32 rows: two 16-row tiles
            x, xf = _x(rng, M, K, xd)
            _check(nvq_matmul(lin.weight, x, force="gemv").cpu().numpy(), O.linear_forward_f64(want, xf))


@pytest.mark.parametrize("cu", ["8", "256"])
def test_nvq_two_projections_in_one_launch(cu_count, cu):
    """Two tensors that share their input: the joint launch gives exactly what the two separate calls give (bit for
    bit: same kernel, same order of sums), for one- and two-bank codebooks, different heights, 1 to 32 rows; with the
    grid sized for 8 CUs the blocks hold several row-blocks.  A four-bank tensor takes the two-call path."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_vq import nvq_matmul, nvq_matmul_multi2
    cu_count(int(cu))
    rng = np.random.default_rng(950 + int(cu))
    K = 1560
    specs = [(("d4_512", 2), 250), (("d4_512", 1), 123), (("d4_256", 2), 64), (("d4_512", 4), 80)]
    lins = []
    for (cb, banks), out in specs:
        dtype, blob = O.pack_tensor(synth.nvq_jsc_random(rng, out, K, cb, banks))
        lins.append(R.load_quant_linear(dtype, blob))
    for a, b in ((0, 1), (1, 2), (2, 0), (0, 3)):
        for M, xd in ((1, torch.bfloat16), (8, torch.float16), (17, torch.bfloat16), (32, torch.bfloat16), (40, torch.bfloat16)):
            x, xf = _x(rng, M, K, xd)
            got = nvq_matmul_multi2(lins[a].weight, lins[b].weight, x)
            force = "gemv" if M <= 32 else None
            want = torch.cat([nvq_matmul(lins[a].weight, x, force=force), nvq_matmul(lins[b].weight, x, force=force)], dim=-1)
            assert got.shape == (M, lins[a].out + lins[b].out)
            assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    from tyloquant_amd.runtime_vq import nvq_matmul_swiglu
    g, u = lins[0].weight, R.load_quant_linear(*O.pack_tensor(synth.nvq_jsc_random(rng, 250, K, "d4_512", 1))).weight
    x, xf = _x(rng, 3, K)
    h = nvq_matmul_swiglu(g, u, x).float().cpu().numpy()
    yg, yu = nvq_matmul(g, x).cpu().numpy(), nvq_matmul(u, x).cpu().numpy()
    assert rel_l2(h, O.moe_swiglu(np.concatenate([yg, yu], axis=-1))) < 1e-3      # fp16 output
    with pytest.raises(ValueError, match="equal-width"):
        nvq_matmul_swiglu(lins[0].weight, lins[1].weight, x)
    with pytest.raises(ValueError, match="compatible formats"):
        other = R.load_quant_linear(*O.pack_tensor(synth.nvq_jsc_random(rng, 32, 96, "d4_512", 2)))
        nvq_matmul_multi2(lins[0].weight, other.weight, torch.zeros((1, K), dtype=torch.bfloat16, device="cuda"))


@pytest.mark.parametrize("out,K,M,banks", [(130, 1024, 520, 2), (96, 4104, 600, 4), (272, 1024, 8300, 2),
                                          (1040, 1024, 3329, 2)])
def test_nvq_prefill_kernel(out, K, M, banks):
    """Above the streaming range (at most 512 rows) the block-tiled kernel takes over: 64-token tiles, and 128-token
    tiles once the grid exceeds one block per CU (130 token tiles x 2 neuron blocks) or 64 x 384 tiles where they take
    fewer rounds (65 row-blocks x 53 token tiles); ragged row-blocks, K not a multiple of 96, a last token tile with one
    row."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(170 + out + M)
    t = synth.nvq_jsc_random(rng, out, K, "d4_512", banks)
    dtype, blob = O.pack_tensor(t)
    lin = R.load_quant_linear(dtype, blob)
    want = O.dequantize_nvq_jsc(O.unpack_nvq(blob))
    for xd in (torch.bfloat16, torch.float16):
        x, xf = _x(rng, M, K, xd)
        _check(lin(x).cpu().numpy(), O.linear_forward_f64(want, xf))


def test_nvq_payload_sizes_match_reference_identities():
    """tests/test_formats/test_nvq.py:44-50 and tests/test_nvq_kernels_cuda.py:410-449 (host side)."""
    from tyloquant_amd import _lib as L
    import ctypes as C
    d = L.NvqDesc()
    L.check(L.lib().mfq_hip_nvq_plan(9, 2, 4096, 5120, C.byref(d)))
    streams = d.payload_bytes - 64 - 2 * 512 * 4
    assert 8.0 * streams / (4096 * 5120) == 3.2953125
    L.check(L.lib().mfq_hip_nvq_plan(9, 2, 17408, 5120, C.byref(d)))
    assert d.payload_bytes - 64 - 4096 == 36713472


def test_nvq_plain_d4_256():
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(11)
    t = synth.nvq_plain_random(rng, 40, 104)
    dtype, blob = O.pack_tensor(t)
    assert dtype == "NVQ3"
    lin = R.load_quant_linear("NIQ3", blob)   # legacy alias
    want = O.dequantize_nvq(O.unpack_nvq(blob))
    assert np.array_equal(lin.dequantize().cpu().numpy().view(np.uint32), want.view(np.uint32))
    x, xf = _x(rng, 3, 104)
    _check(lin(x).cpu().numpy(), O.linear_forward(want, xf))


@pytest.mark.parametrize("label", ["NEPQ1-S", "NEPQ1-L"])
@pytest.mark.parametrize("E,out,K,banks", [(1, 48, 96, 3), (3, 32, 200, 5), (2, 16, 1544, 40), (1, 33, 88, 1)])
def test_nepq_dequant_bit_exact_and_matmul(label, E, out, K, banks):
    from tyloquant_amd.runtime_vq import NepqWeight, nepq_matmul
    rng = np.random.default_rng(23 + E + out + K)
    t = synth.nepq_random(rng, label, E, out, K, banks)
    blob = O.pack_nepq(t)
    w = NepqWeight.from_blob(blob)
    want = O.dequantize_nepq(O.unpack_nepq(blob))
    got = w.dequantize().cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    for e in range(E):
        for M in (1, 5, 16):
            x, xf = _x(rng, M, K)
            _check(nepq_matmul(w, x, e).cpu().numpy(), O.linear_forward(want[e], xf))
        x, xf = _x(rng, 40, K)
        _check(nepq_matmul(w, x, e).cpu().numpy(), O.linear_forward_f64(want[e], xf))


@pytest.mark.parametrize("label,out,K,M,banks", [("NEPQ1-S", 64, 2048, 1, 16), ("NEPQ1-L", 48, 4104, 16, 16),
                                                  ("NEPQ1-S", 130 - 2, 1024, 33, 4), ("NEPQ1-L", 32, 6144, 7, 3)])
def test_nepq_matrix_core_path_multi_step(label, out, K, M, banks):
    """K % 8 == 0 rows take the MFMA streaming kernel: several steps, K split over waves, ragged last group,
    tables in LDS (S) or read from global memory (L, 16 banks), a second expert, a row stride above K."""
    from tyloquant_amd.runtime_vq import NepqWeight, nepq_matmul
    rng = np.random.default_rng(300 + out + M)
    t = synth.nepq_random(rng, label, 2, out, K, banks)
    w = NepqWeight.from_blob(O.pack_nepq(t))
    want = O.dequantize_nepq(t)
    xw = torch.from_numpy(rng.standard_normal((M, K + 8)).astype(np.float32)).to(torch.bfloat16).cuda()
    x = xw[:, :K]
    for e in (0, 1):
        _check(nepq_matmul(w, x, e, force="gemv").cpu().numpy(), O.linear_forward_f64(want[e], x.float().cpu().numpy()))


@pytest.mark.parametrize("label,banks", [("NEPQ1-S", 5), ("NEPQ1-L", 16)])
@pytest.mark.parametrize("E,cus,out", [(2, 4, 128), (2, 2, 96), (2, 3, 208), (1, 2, 88), (1, 3, 200), (2, 2, 16)])
def test_nepq_one_row_gemv_row_blocks_per_block(cu_count, label, banks, E, cus, out):
    """One activation row: a block owns ceil(row-blocks / CUs) row-blocks, up to four (2, 3, 4, 3, 4 and 1 here), the
    last block fewer than the others; a second expert at its own row offset; a ragged last row-block."""
    from tyloquant_amd.runtime_vq import NepqWeight, nepq_matmul
    rng = np.random.default_rng(910 + cus + out)
    K = 1160
    t = synth.nepq_random(rng, label, E, out, K, banks)
    w = NepqWeight.from_blob(O.pack_nepq(t))
    want = O.dequantize_nepq(t)
    cu_count(cus)
    for e in range(E):
        x, xf = _x(rng, 1, K)
        _check(nepq_matmul(w, x, e).cpu().numpy(), O.linear_forward(want[e], xf))
    # 2 .. 32 rows: the 16-row tile kernel with the same ownership (up to three row-blocks per block; four fall back
    # to the streaming kernel), one and two tiles
    for M in (2, 16, 21):
        x, xf = _x(rng, M, K)
        for e in range(E):
            _check(nepq_matmul(w, x, e, force="gemv").cpu().numpy(), O.linear_forward_f64(want[e], xf))


@pytest.mark.parametrize("label,out,K,M,banks", [("NEPQ1-S", 130 - 2, 1024, 70, 4), ("NEPQ1-L", 48, 4104, 300, 16),
                                                  ("NEPQ1-L", 272, 1544, 100, 40), ("NEPQ1-S", 272, 1024, 8300, 3),
                                                  ("NEPQ1-S", 1040, 1024, 3329, 5)])
def test_nepq_prefill_kernel(label, out, K, M, banks):
    """From 64 rows on the block-tiled kernel takes over: 64 x 256 tiles (split over K for the long-K case), 128 x 256
    and 64 x 384 tiles for the large grids, tables in LDS or read from global memory (40 banks of the L profile), a
    second expert's row slice, ragged row-blocks, K not a multiple of 96, a last token tile with one row."""
    from tyloquant_amd.runtime_vq import NepqWeight, nepq_matmul
    rng = np.random.default_rng(500 + out + M)
    t = synth.nepq_random(rng, label, 2, out, K, banks)
    w = NepqWeight.from_blob(O.pack_nepq(t))
    want = O.dequantize_nepq(t)
    for e, xd in ((0, torch.bfloat16), (1, torch.float16)):
        x, xf = _x(rng, M, K, xd)
        _check(nepq_matmul(w, x, e).cpu().numpy(), O.linear_forward_f64(want[e], xf))


def test_nepq_hadamard_matches_fwht():
    from tyloquant_amd.runtime_vq import nepq_hadamard
    rng = np.random.default_rng(3)
    K, block = 512, 128
    x = rng.standard_normal((5, K)).astype(np.float32)
    xb = torch.from_numpy(x).to(torch.bfloat16)
    signs = np.where(rng.integers(0, 2, K), 1, -1).astype(np.int8)
    got = nepq_hadamard(xb.cuda(), torch.from_numpy(signs).cuda(), block).float().cpu().numpy()
    v = (xb.float().numpy() * signs).reshape(5, K // block, block)
    H = np.array([[1.0]])
    while H.shape[0] < block:
        H = np.block([[H, H], [H, -H]])
    ref = (v @ H.T / np.sqrt(block)).reshape(5, K)
    assert np.abs(got - ref).max() < 0.05 and rel_l2(got, ref) < 4e-3   # output is rounded to bf16


def test_vq_loader_errors():
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(9)
    t = synth.nvq_jsc_random(rng, 8, 96)
    dtype, blob = O.pack_tensor(t)
    with pytest.raises(ValueError, match="invalid NVQ"):
        R.load_quant_linear(dtype, blob[:-3])
    with pytest.raises(ValueError, match="invalid NVQ magic"):
        R.load_quant_linear(dtype, b"XXXX" + blob[4:])
    with pytest.raises(ValueError, match="dtype/blob mismatch"):
        R.load_quant_linear("NVQ3J", blob)
    n = synth.nepq_random(rng, "NEPQ1-S", 1, 16, 96, 2)
    nb = O.pack_nepq(n)
    with pytest.raises(ValueError, match="invalid NEPQ tail"):
        R.load_quant_linear("NEPQ1-S", nb + b"\0")
    with pytest.raises(ValueError, match="dtype/blob mismatch"):
        R.load_quant_linear("NEPQ1-L", nb)


def test_nvq_ffn_swiglu_down():
    """Feed-forward block of three NVQ tensors against the oracle's float64 evaluation of the dequantized weights
    (the comparison the reference's tests/test_nvq_kernels_cuda.py:655-675 makes with its unfused path); the hidden
    rows are rounded to fp16 between the two stages, hence the looser bound.  Mismatched widths raise."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_vq import nvq_ffn_swiglu_down
    rng = np.random.default_rng(8032)
    K, W, out = 1560, 240, 72
    blobs = [O.pack_tensor(synth.nvq_jsc_random(rng, W, K, "d4_512", 2)),
             O.pack_tensor(synth.nvq_jsc_random(rng, W, K, "d4_512", 1)),
             O.pack_tensor(synth.nvq_jsc_random(rng, out, W, "d4_512", 2))]
    gate, up, down = (R.load_quant_linear(d, b).weight for d, b in blobs)
    wg, wu, wd = (O.dequantize_nvq_jsc(O.unpack_nvq(b)) for _, b in blobs)
    for M in (1, 5, 40):
        x, xf = _x(rng, M, K)
        got = nvq_ffn_swiglu_down(gate, up, down, x).cpu().numpy()
        g, u = O.linear_forward_f64(wg, xf), O.linear_forward_f64(wu, xf)
        want = O.linear_forward_f64(wd, g / (1.0 + np.exp(-g)) * u)
        assert got.shape == (M, out)
        assert rel_l2(got, want) < 2e-3
    with pytest.raises(ValueError, match="fused FFN weight layouts"):
        nvq_ffn_swiglu_down(gate, up, gate, x)


def test_empty_batch_returns_empty_outputs():
    """A batch with no rows gives an empty output of the right shape and dtype from every host matmul (nothing is
    launched; the C entry points themselves reject M < 1)."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_moe import moe_swiglu
    from tyloquant_amd.runtime_vq import NepqWeight, nepq_matmul, nvq_ffn_swiglu_down, nvq_matmul, nvq_matmul_multi2
    rng = np.random.default_rng(0)
    nint = R.load_quant_linear("NINT4", O.pack_nint(O.quantize_nint(
        (rng.standard_normal((64, 96)) * 0.02).astype(np.float32), 4, 32, 6)))
    q8 = R.load_quant_linear("NINT8-0", O.pack_nint8_zero(O.quantize_nint8_zero(
        (rng.standard_normal((24, 64)) * 0.02).astype(np.float32))))
    vq = [R.load_quant_linear(*O.pack_tensor(synth.nvq_jsc_random(rng, o, k, "d4_512", 2))).weight
          for o, k in ((48, 96), (48, 96), (24, 48))]
    e = lambda *s: torch.zeros(s, dtype=torch.bfloat16, device="cuda")
    y = nint.forward(e(0, 96))
    assert y.shape == (0, 64) and y.dtype == torch.float32
    assert nint.forward(e(2, 0, 96)).shape == (2, 0, 64)
    assert R.nint_matmul_swiglu(nint.weight, e(0, 96)).shape == (0, 32)
    assert R.nint_matmul_input_mul(nint.weight, e(0, 96), e(0, 96)).shape == (0, 64)
    assert q8.forward(e(0, 64)).shape == (0, 24)
    assert nvq_matmul(vq[0], e(0, 96)).shape == (0, 48)
    assert nvq_matmul_multi2(vq[0], vq[1], e(0, 96)).shape == (0, 96)
    assert nvq_ffn_swiglu_down(vq[0], vq[1], vq[2], e(0, 96)).shape == (0, 24)
    assert moe_swiglu(torch.zeros((0, 64), device="cuda")).shape == (0, 32)
    t = synth.nepq_random(rng, "NEPQ1-S", 2, 32, 256, 1)
    w = NepqWeight.from_blob(O.pack_nepq(t))
    assert nepq_matmul(w, e(0, 256), 1).shape == (0, 32)
    with pytest.raises(ValueError, match="activation width"):
        nint.forward(e(0, 95))


def test_multi_expert_nepq_blob_is_not_a_linear():
    """The reference has no linear dtype for NEPQ tensors of several experts (they are NINTM cohorts): both
    load_quant_linear implementations refuse one instead of sizing outputs for a single expert."""
    import ctypes
    from pathlib import Path
    from tyloquant_amd import runtime as R
    blob = O.pack_nepq(synth.nepq_random(np.random.default_rng(3), "NEPQ1-S", 2, 16, 96, 2))
    with pytest.raises(ValueError, match="must hold one expert"):
        R.load_quant_linear("NEPQ1-S", blob)
    lib = ctypes.CDLL(str(Path(R.__file__).resolve().parent / "lib" / "libmfq_runtime.so"))
    lib.mfq_rt_last_error.restype = ctypes.c_char_p
    handle = ctypes.c_void_p()
    assert lib.mfq_rt_load_quant_linear(b"NEPQ1-S", blob, ctypes.c_size_t(len(blob)), ctypes.byref(handle)) != 0
    assert "must hold one expert" in lib.mfq_rt_last_error().decode()


@pytest.mark.parametrize("cus", [1, 2])
@pytest.mark.parametrize("codebook,banks,out,K", [("e8_256", 2, 150, 120), ("e8_1024", 2, 70, 1544), ("e8_4096", 1, 97, 96),
                                                  ("d4_1024", 2, 90, 100)])
def test_e8_kernel_with_several_neurons_per_wave(cu_count, cus, codebook, banks, out, K):
    """A wave of the E8 kernel walks up to four consecutive neurons of a large tensor; sized for one or two compute
    units, small tensors take the same shape: neurons whose stream ranges start inside a byte, waves with fewer neurons
    than the others and waves with none, one and two rows per pass and both activation types (the larger batches of the
    loop take the tile kernel on the same tensors)."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_vq import nvq_matmul
    rng = np.random.default_rng(70 + out + K + cus)
    t = synth.nvq_jsc_random(rng, out, K, codebook, banks)
    _, blob = O.pack_tensor(t)
    lin = R.load_quant_linear(_, blob)
    want = O.dequantize_nvq_jsc(O.unpack_nvq(blob))
    cu_count(cus)
    for M, xd in ((1, torch.bfloat16), (2, torch.float16), (5, torch.bfloat16), (8, torch.float16), (13, torch.bfloat16)):
        x, xf = _x(rng, M, K, xd)
        _check(nvq_matmul(lin.weight, x).cpu().numpy(), O.linear_forward_f64(want, xf))
    big = torch.from_numpy((rng.standard_normal((2, K)) * 2.0e6).astype(np.float32)).to(torch.bfloat16).cuda()
    _check(nvq_matmul(lin.weight, big).cpu().numpy() / 2.0e6, O.linear_forward_f64(want, big.float().cpu().numpy()) / 2.0e6)


@pytest.mark.parametrize("codebook,banks,dtype", [("e8_256", 2, "NVQ2J"), ("e8_256", 4, "NVQ2J"), ("e8_1024", 2, "NVQ2J-L"),
                                                  ("e8_4096", 1, "NVQ2J-XL"), ("e8_4096", 4, "NVQ2J-XL"),
                                                  ("d4_1024", 2, "NVQ3J-L")])
@pytest.mark.parametrize("out,K", [(37, 96), (24, 80), (70, 1544), (33, 100)])
def test_nvq_stream_formats_dequant_bit_exact_and_matmul(codebook, banks, dtype, out, K):
    """The E8 family and the 1024-entry D4 codebook, read in place from their bit streams (mfq_hip_nvqs_*): dequantized
    weights bit for bit against the oracle (ragged K: partial last vector, sign block and group), the wave-per-neuron
    kernel for 1 / 4 / 8 / 13 rows of both activation types, and the fp16 GEMM path above 16 rows."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_vq import NvqsWeight, nvq_matmul
    rng = np.random.default_rng(900 + out + K + banks)
    t = synth.nvq_jsc_random(rng, out, K, codebook, banks)
    got_dtype, blob = O.pack_tensor(t)
    assert got_dtype == dtype
    lin = R.load_quant_linear(dtype, blob)
    assert isinstance(lin.weight, NvqsWeight) and lin.weight.payload_bytes == O.nvq_payload_nbytes(codebook, out, K)
    want = O.dequantize_nvq_jsc(O.unpack_nvq(blob))
    got = lin.dequantize().cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    for M in (1, 4, 8, 13):
        for xd in (torch.bfloat16, torch.float16):
            x, xf = _x(rng, M, K, xd)
            _check(nvq_matmul(lin.weight, x).cpu().numpy(), O.linear_forward_f64(want, xf))
    for M in (17, 70, 200):                      # tiles of the matrix-core kernel; above 192 rows the fp16 GEMM
        x, xf = _x(rng, M, K)
        _check(lin(x).cpu().numpy(), O.linear_forward_f64(want, xf))
    xs = torch.zeros((1, K + 3), dtype=torch.bfloat16, device="cuda")[:, 1:K + 1]       # a misaligned row
    xs.copy_(torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)))
    _check(nvq_matmul(lin.weight, xs).cpu().numpy(), O.linear_forward_f64(want, xs.float().cpu().numpy()))


@pytest.mark.parametrize("sign_mode", ["even", "index_parity"])
def test_nvq2_plain_e8_with_both_sign_rules(sign_mode):
    """Plain NVQ2 (built-in E8 grid, the state is the integer relative scale): parity signs and the index-parity rule
    (bit 7 of a block flips with bit 7 of its vector's index); and the reference-packed index-parity blob of the golden
    fixture against the values the reference dequantized it to."""
    from pathlib import Path

    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(31)
    t = synth.nvq_plain_e8_random(rng, 40, 200, sign_mode)
    dtype, blob = O.pack_tensor(t)
    assert dtype == "NVQ2"
    lin = R.load_quant_linear("NIQ2", blob)           # the legacy alias
    want = O.dequantize_nvq(O.unpack_nvq(blob))
    assert np.array_equal(lin.dequantize().cpu().numpy().view(np.uint32), want.view(np.uint32))
    for M in (1, 5, 40):
        x, xf = _x(rng, M, 200)
        _check(lin(x).cpu().numpy(), O.linear_forward_f64(want, xf))
    gold = np.load(Path(__file__).resolve().parent / "golden" / "reference_blobs.npz")
    ref_blob, ref_w = gold["nvq2ip_blob"].tobytes(), gold["nvq2ip_deq"]
    lin = R.load_quant_linear("NVQ2", ref_blob)
    assert np.array_equal(lin.dequantize().cpu().numpy().view(np.uint32), ref_w.astype(np.float32).view(np.uint32))
    with pytest.raises(ValueError, match="dtype/blob mismatch"):
        R.load_quant_linear("NVQ2J", ref_blob)


LOWBIT_CASES = [("NVQ1-L", dict(state_bits=3)), ("NVQ1-L", dict(state_bits=4, custom=True)), ("NVQ1-S", dict()),
                ("NVQ1-S", dict(custom=True)), ("NPQ0-L", dict()), ("NPQ0-S", dict())]


@pytest.mark.parametrize("dtype,kw", LOWBIT_CASES)
@pytest.mark.parametrize("out,K", [(37, 96), (24, 80), (70, 1544), (33, 104)])
def test_one_bit_families_dequant_bit_exact_and_matmul(dtype, kw, out, K):
    """NVQ1-L / NVQ1-S / NPQ0-L / NPQ0-S through the in-place stream kernels: dequantized weights bit for bit against the
    oracle, the wave-per-neuron kernel for 1 / 4 / 13 rows, the fp16 GEMM path above 16 rows.  K = 100 (NVQ1-L only:
    the other three need whole vectors) leaves a partial last vector and group."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_vq import NvqsWeight, nvq_matmul
    if dtype == "NVQ1-L" and K == 104:
        K = 100
    rng = np.random.default_rng(950 + out + K)
    t = synth.nvq1_random(rng, dtype, out, K, **kw) if dtype.startswith("NVQ1") else synth.npq0_random(rng, dtype, out, K)
    got_dtype, blob = O.pack_tensor(t)
    assert got_dtype == dtype
    lin = R.load_quant_linear(dtype, blob)
    assert isinstance(lin.weight, NvqsWeight)
    want = O.dequantize_tensor(O.unpack_tensor(dtype, blob))
    got = lin.dequantize().cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    for M in (1, 4, 13):
        for xd in (torch.bfloat16, torch.float16):
            x, xf = _x(rng, M, K, xd)
            _check(nvq_matmul(lin.weight, x).cpu().numpy(), O.linear_forward_f64(want, xf))
    for M in (17, 70, 200):                      # tiles of the matrix-core kernel; above 192 rows the fp16 GEMM
        x, xf = _x(rng, M, K)
        _check(lin(x).cpu().numpy(), O.linear_forward_f64(want, xf))


@pytest.mark.parametrize("cus", [1, 2])
@pytest.mark.parametrize("dtype,kw,out,K", [("NVQ1-L", dict(state_bits=3), 150, 100), ("NVQ1-L", dict(state_bits=4), 70, 1544),
                                            ("NVQ1-S", dict(), 97, 1544), ("NPQ0-L", dict(), 150, 120),
                                            ("NPQ0-S", dict(), 70, 1544)])
def test_one_bit_families_with_several_neurons_per_wave(cu_count, cus, dtype, kw, out, K):
    """The decoders of the 1-bit families in the kernel that stages a wave's bit ranges in LDS, sized for one or two
    compute units so that a wave walks several neurons: state fields of 2 to 4 bits and delta signs that start inside a
    byte, waves with fewer neurons than the others and with none, one and two rows per pass, both activation types
    and bf16 rows far outside fp16's range (the larger batches of the loop take the tile kernel)."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_vq import nvq_matmul
    rng = np.random.default_rng(170 + out + K + cus)
    t = synth.nvq1_random(rng, dtype, out, K, **kw) if dtype.startswith("NVQ1") else synth.npq0_random(rng, dtype, out, K)
    _, blob = O.pack_tensor(t)
    lin = R.load_quant_linear(dtype, blob)
    want = O.dequantize_tensor(O.unpack_tensor(dtype, blob))
    cu_count(cus)
    for M, xd in ((1, torch.bfloat16), (2, torch.float16), (5, torch.bfloat16), (8, torch.float16), (16, torch.bfloat16)):
        x, xf = _x(rng, M, K, xd)
        _check(nvq_matmul(lin.weight, x).cpu().numpy(), O.linear_forward_f64(want, xf))
    big = torch.from_numpy((rng.standard_normal((2, K)) * 2.0e6).astype(np.float32)).to(torch.bfloat16).cuda()
    _check(nvq_matmul(lin.weight, big).cpu().numpy() / 2.0e6, O.linear_forward_f64(want, big.float().cpu().numpy()) / 2.0e6)


def test_one_bit_families_reference_blobs_and_loader_errors():
    """The reference-packed blobs of the golden fixture dequantize on the device to the values the reference computed;
    malformed blobs are refused with the reference's messages before anything is uploaded."""
    from pathlib import Path

    from tyloquant_amd import runtime as R
    gold = np.load(Path(__file__).resolve().parent / "golden" / "reference_lowbit.npz")
    keys = {"nvq1l_grid": "NVQ1-L", "nvq1l_custom": "NVQ1-L", "nvq1s_default": "NVQ1-S", "nvq1s_custom": "NVQ1-S",
            "npq0l": "NPQ0-L", "npq0s": "NPQ0-S"}
    for key, dtype in keys.items():
        blob = bytes(gold[f"{key}_blob"])
        lin = R.load_quant_linear(dtype, blob)
        got = lin.dequantize().cpu().numpy()
        assert np.array_equal(got.view(np.uint32), gold[f"{key}_deq"].astype(np.float32).view(np.uint32)), key
        with pytest.raises(ValueError, match="blob tail"):
            R.load_quant_linear(dtype, blob + b"\0")
        with pytest.raises(ValueError, match="magic"):
            R.load_quant_linear(dtype, b"ZZZZ" + blob[4:])
    bad = bytearray(gold["npq0s_blob"].tobytes())
    bad[20 + 16 + 4 + 0] = 9                                   # the table header's version byte
    with pytest.raises(ValueError, match="unsupported NPQ0-S table profile"):
        R.load_quant_linear("NPQ0-S", bytes(bad))
    bad = bytearray(gold["nvq1s_custom_blob"].tobytes())
    bad[20 + 16 + 4] = 0xFF                                    # digit 3 in a ternary entry
    with pytest.raises(ValueError, match="non-ternary"):
        R.load_quant_linear("NVQ1-S", bytes(bad))


@pytest.mark.parametrize("label", ["NEPQ0-S", "NEPQ0-L"])
@pytest.mark.parametrize("E,out,K,banks", [(1, 48, 96, 3), (3, 32, 200, 5), (2, 16, 1544, 40), (1, 33, 88, 1)])
def test_nepq0_dequant_bit_exact_and_matmul(label, E, out, K, banks):
    """The expert form of the product codebooks (NPQ0 tables in the NEPQ container's pool): dequantized experts bit for
    bit, every expert's matmul through the row-range calls for GEMV and GEMM batch sizes, the dense-linear registry for a
    one-expert tensor, the reference-packed blobs of the golden fixture."""
    from pathlib import Path

    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_vq import NepqWeight, nepq_matmul
    rng = np.random.default_rng(123 + E + out + K)
    t = synth.nepq_random(rng, label, E, out, K, banks)
    blob = O.pack_nepq(t)
    w = NepqWeight.from_blob(blob)
    assert w.streams and w.label == label
    want = O.dequantize_nepq(O.unpack_nepq(blob))
    got = w.dequantize().cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    for e in range(E):
        for M in (1, 5, 16):
            x, xf = _x(rng, M, K)
            _check(nepq_matmul(w, x, e).cpu().numpy(), O.linear_forward_f64(want[e], xf))
        for M in (40, 200):
            x, xf = _x(rng, M, K)
            _check(nepq_matmul(w, x, e).cpu().numpy(), O.linear_forward_f64(want[e], xf))
    if E == 1:
        lin = R.load_quant_linear(label, blob)
        x, xf = _x(rng, 3, K)
        _check(lin(x).cpu().numpy(), O.linear_forward_f64(want[0], xf))
    else:
        with pytest.raises(ValueError, match="must hold one expert"):
            R.load_quant_linear(label, blob)
    gold = np.load(Path(__file__).resolve().parent / "golden" / "reference_lowbit.npz")
    key = "nepq0s" if label == "NEPQ0-S" else "nepq0l"
    g = NepqWeight.from_blob(bytes(gold[f"{key}_blob"]))
    assert np.array_equal(g.dequantize().cpu().numpy().view(np.uint32), gold[f"{key}_deq"].astype(np.float32).view(np.uint32))
    bad = bytearray(blob)
    bad[36 + 2] = 9                                    # first index width in the first table's header
    with pytest.raises(ValueError, match="table profile"):
        NepqWeight.from_blob(bytes(bad))


@pytest.mark.parametrize("cus", [1, 2])
@pytest.mark.parametrize("label,E,out,K,banks", [("NEPQ0-S", 2, 75, 1544, 40), ("NEPQ0-L", 3, 50, 200, 5), ("NEPQ0-L", 1, 150, 96, 1)])
def test_nepq0_with_several_neurons_per_wave(cu_count, cus, label, E, out, K, banks):
    """The table-pool decoder in the kernel that stages a wave's bit ranges in LDS, sized for one or two compute units:
    experts whose first neuron starts inside a byte of the streams, waves with several neurons, with fewer and with
    none, one and two rows per pass, both activation types and bf16 rows far outside fp16's range (the larger batches of
    the loop take the tile kernel)."""
    from tyloquant_amd.runtime_vq import NepqWeight, nepq_matmul
    rng = np.random.default_rng(223 + E + out + K + cus)
    blob = O.pack_nepq(synth.nepq_random(rng, label, E, out, K, banks))
    w = NepqWeight.from_blob(blob)
    want = O.dequantize_nepq(O.unpack_nepq(blob))
    cu_count(cus)
    for e in range(E):
        for M, xd in ((1, torch.bfloat16), (2, torch.float16), (5, torch.bfloat16), (8, torch.float16), (16, torch.bfloat16)):
            x, xf = _x(rng, M, K, xd)
            _check(nepq_matmul(w, x, e).cpu().numpy(), O.linear_forward_f64(want[e], xf))
    big = torch.from_numpy((rng.standard_normal((2, K)) * 2.0e6).astype(np.float32)).to(torch.bfloat16).cuda()
    _check(nepq_matmul(w, big, E - 1).cpu().numpy() / 2.0e6, O.linear_forward_f64(want[E - 1], big.float().cpu().numpy()) / 2.0e6)


TILE_CASES = [("jsc", "e8_256", 4, 37, 1544), ("jsc", "e8_1024", 2, 70, 100), ("jsc", "e8_4096", 1, 33, 96),
              ("jsc", "e8_4096", 4, 37, 1544), ("jsc", "e8_4096", 2, 50, 100),   # tables kept as bytes in LDS
             
              ("jsc", "d4_1024", 2, 50, 1540), ("plain_e8", "index_parity", 0, 41, 200), ("NVQ1-L", dict(state_bits=3), 0, 37, 1540),
              ("NVQ1-S", dict(), 0, 33, 1544), ("NPQ0-L", dict(), 0, 70, 104), ("NPQ0-S", dict(), 0, 18, 1544)]


@pytest.mark.parametrize("kind,a,b,out,K", TILE_CASES)
def test_stream_formats_on_the_matrix_core_tile_kernel(kind, a, b, out, K):
    """Three to 192 rows of the formats read in place from their bit streams run as 16-neuron tiles on the matrix
    cores: a last tile with fewer neurons, K that ends inside a group, a block and a vector, every row count of the
    range in both activation types, rows at a stride that is no multiple of 16 bytes (element-wise loads), and bf16 rows
    far outside fp16's range."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_vq import nvq_matmul
    rng = np.random.default_rng(310 + out + K)
    if kind == "jsc":
        t = synth.nvq_jsc_random(rng, out, K, a, b)
    elif kind == "plain_e8":
        t = synth.nvq_plain_e8_random(rng, out, K, a)
    elif kind.startswith("NVQ1"):
        t = synth.nvq1_random(rng, kind, out, K, **a)
    else:
        t = synth.npq0_random(rng, kind, out, K)
    dtype, blob = O.pack_tensor(t)
    lin = R.load_quant_linear(dtype, blob)
    want = O.dequantize_tensor(O.unpack_tensor(dtype, blob))
    for M in list(range(1 if kind == "jsc" and a == "e8_4096" and b > 1 else 3, 17)) + [17, 32, 33, 64, 100, 129, 192, 193]:   # one, two or four tiles per block, several sets of rows; 193: the fp16 GEMM
        xd = torch.bfloat16 if M % 2 else torch.float16
        x, xf = _x(rng, M, K, xd)
        _check(nvq_matmul(lin.weight, x).cpu().numpy(), O.linear_forward_f64(want, xf))
    wide = torch.zeros((9, K + 3), dtype=torch.bfloat16, device="cuda")
    x, xf = _x(rng, 9, K, torch.bfloat16)
    wide[:, 1:K + 1] = x
    view = wide[:, 1:K + 1]
    assert view.stride(0) == K + 3 and view.data_ptr() % 16 != 0
    _check(nvq_matmul(lin.weight, view).cpu().numpy(), O.linear_forward_f64(want, xf))
    big = torch.from_numpy((rng.standard_normal((7, K)) * 2.0e6).astype(np.float32)).to(torch.bfloat16).cuda()
    _check(nvq_matmul(lin.weight, big).cpu().numpy() / 2.0e6, O.linear_forward_f64(want, big.float().cpu().numpy()) / 2.0e6)


@pytest.mark.parametrize("family", ["NVQ3J-512", "NEPQ0-L", "NEPQ1-S", "MXFP8"])
def test_reserve_sizes_the_workspace_of_every_family(family):
    """QuantLinear.reserve(max_rows) on an NVQ, an NEPQ0 (bit streams in place), an NEPQ1 and an MX linear: forward() of
    any smaller batch afterwards leaves the workspace buffer as it is (no regrowth, so nothing to allocate under a HIP
    graph) and still matches the oracle."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(515)
    if family == "NVQ3J-512":
        K = 192
        dtype, blob = O.pack_tensor(synth.nvq_jsc_random(rng, 48, K, "d4_512", 2))
        want = O.dequantize_nvq_jsc(O.unpack_nvq(blob))
    elif family == "MXFP8":
        K = 256
        t = synth.mx_random(rng, "MXFP8", 128, K)
        dtype, blob, want = "MXFP8", O.pack_mx(t), O.dequantize_mx(t)
    else:
        K = 192
        t = synth.nepq_random(rng, family, 1, 48, K, 3)
        dtype, blob = family, O.pack_nepq(t)
        want = O.dequantize_nepq(O.unpack_nepq(blob))[0]
    lin = R.load_quant_linear(dtype, blob)
    lin.reserve(70)
    buf = lin.weight._ws.buf
    for M in (1, 5, 17, 40, 70):
        x, xf = _x(rng, M, K)
        _check(lin(x).cpu().numpy(), O.linear_forward_f64(want, xf))
        assert lin.weight._ws.buf is buf, (family, M)


@pytest.mark.parametrize("scale", [1e-6, 3e6])
def test_nepq_one_row_kernel_takes_bf16_rows_of_any_magnitude(scale):
    """NEPQ1-S for one bf16 row far outside fp16's comfortable range (two rows already run on the matrix-core kernel,
    which converts without scaling): every K-slice is scaled by a power of two before the conversion, so the relative
    accuracy is that of an ordinary row.  (The generic NVQ kernel does the same; it runs behind a MoE decode step, where
    tests/test_moe_gpu.py covers it.)"""
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_vq import nepq_matmul
    rng = np.random.default_rng(4242)
    out, K = 48, 200
    dt, blob = O.pack_tensor(synth.nepq_random(rng, "NEPQ1-S", 1, out, K, 3))
    lin = R.load_quant_linear(dt, blob)
    wq = lin.dequantize().cpu().numpy().reshape(out, K)
    for M in (1,):
        x = torch.from_numpy((rng.standard_normal((M, K)) * scale).astype(np.float32)).to(torch.bfloat16)
        y = nepq_matmul(lin.weight, x.cuda(), force="gemv").cpu().numpy()
        ref = O.linear_forward_f64(wq, x.float().numpy())
        assert rel_l2(y, ref) < REL_TOL, (M, rel_l2(y, ref))
