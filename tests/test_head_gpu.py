"""GPU parity of the two ends of the layer stack on NINT tensors: embedding rows decoded from the packed table
(bit-exact against the oracle's dequantizer) and the LM-head GEMV with the arg-max taken on the device."""
import numpy as np
import pytest

import synth
from conftest import ABS_TOL, REL_TOL, check_close, rel_l2
from oracle import mfq_oracle as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

SPECS = [(4, 32, 6), (4, 24, 6), (3, 24, 5), (2, 16, 5), (5, 28, 7), (6, 24, 6), (8, 24, 8), (6, 26, 6), (8, 48, 7)]
FUSED = [(4, 32, 6), (4, 24, 6), (3, 24, 5), (5, 28, 7), (6, 24, 7)]   # one GEMV launch that also emits the blocks' winners
UNFUSED = [(6, 26, 6), (2, 16, 5), (8, 48, 7)]                          # GEMV into the logits, then two reduction passes


def _load(t):
    from tyloquant_amd import runtime as R
    return R.load_quant_linear(f"NINT{t.bits}", O.pack_nint(t))


def _x(rng, M, K, dtype=torch.bfloat16):
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(dtype)
    return x.cuda(), x.float().numpy()


@pytest.mark.parametrize("bits,gs,sb", SPECS)
@pytest.mark.parametrize("out,K", [(300, 88), (75, 1537)])
def test_embedding_rows_bit_exact(bits, gs, sb, out, K):
    """Rows picked by token id equal the CPU dequantizer's rows bit for bit in fp32, and its rows rounded to nearest
    even in fp16 / bf16; ids outside the table (negative, == out, far beyond) give zeros; repeated ids and an id
    tensor of rank 2."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(900 + bits * 10 + gs + out)
    t = synth.nint_random(rng, out, K, bits, gs, sb)
    lin = _load(t)
    want = O.dequantize_nint(t)
    ids = rng.integers(0, out, (3, 7))
    ids[0, 0], ids[1, 2], ids[2, 6], ids[0, 3], ids[0, 4] = -1, out, 2 ** 40, out - 1, 0
    ids[1, 5] = ids[1, 4]
    rows = np.zeros((3, 7, K), np.float32)
    ok = (ids >= 0) & (ids < out)
    rows[ok] = want[ids[ok]]
    tid = torch.from_numpy(ids).cuda()
    got = R.nint_embedding(lin.weight, tid, torch.float32).cpu().numpy()
    assert got.shape == rows.shape
    assert np.array_equal(got.view(np.uint32), rows.view(np.uint32))
    got16 = R.nint_embedding(lin.weight, tid, torch.float16).cpu().numpy()
    assert np.array_equal(got16.view(np.uint16), rows.astype(np.float16).view(np.uint16))
    gotb = R.nint_embedding(lin.weight, tid, torch.bfloat16).cpu()
    assert torch.equal(gotb.view(torch.int16), torch.from_numpy(rows).to(torch.bfloat16).view(torch.int16))


def _table(kind, rng, out, K):
    """(dtype, blob, the oracle's dequantized rows) of an embedding table of the given format."""
    if kind == "NINT8-0":
        t = O.quantize_nint8_zero((rng.standard_normal((out, K)) * 0.02).astype(np.float32))
        return "NINT8-0", O.pack_nint8_zero(t), O.dequantize_nint8_zero(t)
    if isinstance(kind, str):
        t = synth.nvq1_random(rng, kind, out, K) if kind.startswith("NVQ1") else synth.npq0_random(rng, kind, out, K)
        dtype, blob = O.pack_tensor(t)
        return dtype, blob, O.dequantize_tensor(O.unpack_tensor(dtype, blob))
    codebook, banks = kind
    dtype, blob = O.pack_tensor(synth.nvq_jsc_random(rng, out, K, codebook, banks))
    return dtype, blob, O.dequantize_nvq_jsc(O.unpack_nvq(blob))


@pytest.mark.parametrize("kind", ["NINT8-0", ("d4_512", 2), ("d4_512", 1), ("d4_256", 2), ("e8_256", 2), ("e8_4096", 4),
                                  ("d4_1024", 2), "NVQ1-L", "NVQ1-S", "NPQ0-L", "NPQ0-S"], ids=str)
@pytest.mark.parametrize("out,K", [(300, 96), (75, 1544), (33, 104)])
def test_embedding_rows_of_the_other_table_formats(kind, out, K):
    """embed_forward's other table formats (NINT8-0 and every NVQ family: the lane-major D4 layout and the families read
    in place from their streams): rows picked by token id equal the oracle's dequantized rows bit for bit in fp32 and
    rounded to nearest even in fp16 / bf16; ids outside the table give zeros; K = 104 and 1544 leave partial groups."""
    from tyloquant_amd import runtime as R
    if kind == "NINT8-0":
        K = (K + 31) // 32 * 32                       # the format's rule: whole blocks of 32
    rng = np.random.default_rng(1200 + out + K)
    dtype, blob, want = _table(kind, rng, out, K)
    lin = R.load_quant_linear(dtype, blob)
    ids = rng.integers(0, out, (3, 7))
    ids[0, 0], ids[1, 2], ids[2, 6], ids[0, 3], ids[0, 4] = -1, out, 2 ** 40, out - 1, 0
    ids[1, 5] = ids[1, 4]
    rows = np.zeros((3, 7, K), np.float32)
    ok = (ids >= 0) & (ids < out)
    rows[ok] = want[ids[ok]]
    tid = torch.from_numpy(ids).cuda()
    got = lin.embedding(tid, torch.float32).cpu().numpy()
    assert got.shape == rows.shape
    assert np.array_equal(got.view(np.uint32), rows.view(np.uint32))
    got16 = R.embedding(lin.weight, tid, torch.float16).cpu().numpy()
    assert np.array_equal(got16.view(np.uint16), rows.astype(np.float16).view(np.uint16))
    gotb = R.embedding(lin, tid).to(torch.float32)   # default: fp16, the reference's output type
    assert np.array_equal(gotb.cpu().numpy(), rows.astype(np.float16).astype(np.float32))
    gotb = lin.embedding(tid, torch.bfloat16).cpu()
    assert torch.equal(gotb.view(torch.int16), torch.from_numpy(rows).to(torch.bfloat16).view(torch.int16))
    assert lin.embedding(tid[:0], torch.float16).shape == (0, 7, K)


def test_embedding_refuses_tables_the_reference_refuses():
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(5)
    dtype, blob = O.pack_tensor(synth.nepq_random(rng, "NEPQ1-S", 1, 32, 96, 3))
    lin = R.load_quant_linear(dtype, blob)
    with pytest.raises(TypeError):
        lin.embedding(torch.zeros((2,), dtype=torch.int64, device="cuda"))


def test_embedding_of_no_ids_and_bad_arguments():
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(3)
    lin = _load(synth.nint_random(rng, 40, 96, 4, 24, 6))
    empty = R.nint_embedding(lin.weight, torch.zeros((0,), dtype=torch.int64, device="cuda"))
    assert empty.shape == (0, 96)
    with pytest.raises(TypeError):
        R.nint_embedding(lin.weight, torch.zeros((2,), dtype=torch.int64, device="cuda"), torch.float64)


@pytest.mark.parametrize("bits,gs,sb", FUSED + UNFUSED)
@pytest.mark.parametrize("out,K", [(1000, 1024), (50003, 256), (64, 24584)])
def test_lm_head_argmax(bits, gs, sb, out, K):
    """The token is the arg-max of the logits of the same call; the logits are the plain GEMV's floats and within
    tolerance of the oracle; the chosen neuron's oracle logit is the oracle's maximum up to that tolerance.  Shapes:
    a vocabulary that is not a multiple of 16, one with more blocks than the final pass has threads, and a K long
    enough for the kernel variant with a prefetch ring."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(640 + bits + gs + out)
    t = synth.nint_random(rng, out, K, bits, gs, sb)
    lin = _load(t)
    deq = O.dequantize_nint(t)
    for dtype in (torch.bfloat16, torch.float16):
        x, xf = _x(rng, 1, K, dtype)
        token, logits = R.nint_matmul_argmax(lin.weight, x, return_logits=True)
        only = R.nint_matmul_argmax(lin.weight, x)
        plain = R.nint_matmul(lin.weight, x, force="gemv")
        assert token.dtype == torch.int64 and token.shape == (1,)
        assert torch.equal(logits, plain)
        assert int(token[0]) == int(logits[0].argmax()) == int(only[0])
        ref = O.linear_forward_f64(deq, xf)[0]
        got = logits[0].cpu().numpy()
        assert rel_l2(got, ref) < REL_TOL
        assert ref[int(token[0])] >= ref.max() - 2 * np.abs(got - ref).max()


@pytest.mark.parametrize("bits,gs,sb", [(4, 32, 6), (5, 28, 7), (6, 26, 6)])
def test_lm_head_argmax_ties_go_to_the_lower_index(bits, gs, sb):
    """Two neurons with the same payload give the same logit; the lower index wins whichever of the two comes first,
    inside one block and across blocks."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(77 + bits)
    out, K = 2000, 512
    t = synth.nint_random(rng, out, K, bits, gs, sb)
    x, xf = _x(rng, 1, K)
    a = int(np.argmax(O.linear_forward_f64(O.dequantize_nint(t), xf)[0]))
    for b in (a + 1 if a % 16 < 15 else a - 1, (a + 1000) % out, (a + 37) % out):
        t2 = O.NintTensor(t.bits, t.groupsize, t.sub_bits, t.shape, t.axis, t.neuron_len, t.q.copy(),
                          t.neuron_scale.copy(), t.neuron_min.copy(), t.sub_scale.copy(), t.sub_min.copy())
        for f in (t2.q, t2.neuron_scale, t2.neuron_min, t2.sub_scale, t2.sub_min):
            f[b] = f[a]
        lin = _load(t2)
        token, logits = R.nint_matmul_argmax(lin.weight, x, return_logits=True)
        assert float(logits[0, a]) == float(logits[0, b])
        assert int(token[0]) == min(a, b)


@pytest.mark.parametrize("bits,gs,sb", [(4, 24, 6), (6, 24, 6)])
def test_lm_head_argmax_of_several_rows_and_nan(bits, gs, sb):
    """More than one row reduces the logits of the any-M GEMV row by row; a row of NaN activations has no winner."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(31 + bits)
    out, K = 5000, 512
    t = synth.nint_random(rng, out, K, bits, gs, sb)
    lin = _load(t)
    x, xf = _x(rng, 5, K)
    token, logits = R.nint_matmul_argmax(lin.weight, x.reshape(1, 5, K), return_logits=True)
    assert token.shape == (1, 5) and logits.shape == (1, 5, out)
    assert torch.equal(token[0], logits[0].argmax(-1))
    ref = O.linear_forward_f64(O.dequantize_nint(t), xf)
    check_close(logits[0].cpu().numpy(), ref)   # (packed-domain fixture: logits of order 50, the bound scales with their RMS)
    bad = torch.full((1, K), float("nan"), dtype=torch.bfloat16, device="cuda")
    assert int(R.nint_matmul_argmax(lin.weight, bad)[0]) == -1
    bad3 = torch.full((3, K), float("nan"), dtype=torch.bfloat16, device="cuda")
    assert R.nint_matmul_argmax(lin.weight, bad3).tolist() == [-1, -1, -1]
