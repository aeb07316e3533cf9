"""The C++ host runtime (libmfq_runtime.so) and the mfq-check-linear tool on the GPU, in the style of the
reference's C++-runtime subprocess tests (tests/test_nvq3j512_cpp_runtime.py:111-143): write a tiny .mfq
with Python, run the tool, parse its key=value report."""
import ctypes as C
import re
import subprocess
from pathlib import Path

import numpy as np
import pytest

import synth
from conftest import check_close
from oracle import mfq_oracle as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

LIBDIR = Path(__file__).resolve().parents[1] / "tyloquant_amd" / "lib"


@pytest.fixture(scope="module")
def rt():
    lib = C.CDLL(str(LIBDIR / "libmfq_runtime.so"))
    lib.mfq_rt_last_error.restype = C.c_char_p
    lib.mfq_rt_linear_out.restype = C.c_int64
    lib.mfq_rt_linear_neuron_len.restype = C.c_int64
    lib.mfq_rt_linear_out.argtypes = lib.mfq_rt_linear_neuron_len.argtypes = [C.c_void_p]
    lib.mfq_rt_load_quant_linear.argtypes = [C.c_char_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_void_p)]
    lib.mfq_rt_free_quant_linear.argtypes = [C.c_void_p]
    lib.mfq_rt_linear_forward.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_int, C.c_void_p, C.c_void_p]
    lib.mfq_rt_linear_dequantize.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
    lib.mfq_rt_linear_forward_glu.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_int, C.c_int, C.c_void_p,
                                              C.c_void_p, C.c_void_p]
    lib.mfq_rt_linear_embedding.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_void_p]
    lib.mfq_rt_linear_argmax.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_int, C.c_void_p, C.c_void_p,
                                         C.c_void_p]
    lib.mfq_rt_load_nint_moe.argtypes = [C.c_char_p, C.c_size_t, C.POINTER(C.c_void_p)]
    lib.mfq_rt_free_nint_moe.argtypes = [C.c_void_p]
    lib.mfq_rt_moe_ffn_forward.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_int, C.c_void_p,
                                           C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                           C.c_void_p, C.c_void_p]
    lib.mfq_rt_moe_scratch_create.argtypes = [C.POINTER(C.c_void_p)]
    lib.mfq_rt_moe_scratch_free.argtypes = [C.c_void_p]
    lib.mfq_rt_moe_scratch_reserve.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    lib.mfq_rt_moe_scratch_topk.argtypes = [C.c_void_p, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p)]
    lib.mfq_rt_moe_ffn_forward_scratch.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_int,
                                                   C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                                   C.c_void_p]
    lib.mfq_rt_nvq_ffn_swiglu_down.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_int,
                                               C.c_void_p, C.c_void_p]
    return lib


def _load(rt, dtype, blob):
    h = C.c_void_p()
    rc = rt.mfq_rt_load_quant_linear(dtype.encode(), blob, len(blob), C.byref(h))
    if rc:
        raise RuntimeError(rt.mfq_rt_last_error().decode())
    return h


def test_check_linear_tool_reports_small_error(tmp_path):
    rng = np.random.default_rng(3)
    tensors = {
        "blk.0.q.nint3": synth.nint_random(rng, 37, 96, 3, 24, 5),
        "blk.0.ffn.nint4": O.quantize_nint((rng.standard_normal((64, 200)) * 0.02).astype(np.float32), 4, 32, 6),
        "blk.0.k.nvq3j512": synth.nvq_jsc_random(rng, 37, 96),
        "blk.0.u.nvq2j": synth.nvq_jsc_random(rng, 37, 96, "e8_256", 2),           # E8: read from its bit streams in place
        "blk.0.g.nvq3jl": synth.nvq_jsc_random(rng, 24, 104, "d4_1024", 4),
        "blk.0.v.nepq1s": synth.nepq_random(rng, "NEPQ1-S", 1, 48, 96, 3),
        "blk.0.o.nint8_0": O.quantize_nint8_zero((rng.standard_normal((40, 96)) * 0.02).astype(np.float32)),
        "blk.1.q.nvq1l": synth.nvq1_random(rng, "NVQ1-L", 37, 100, 3, custom=True),   # the 1-bit families
        "blk.1.k.nvq1s": synth.nvq1_random(rng, "NVQ1-S", 24, 104),
        "blk.1.v.npq0l": synth.npq0_random(rng, "NPQ0-L", 40, 96),
        "blk.1.o.npq0s": synth.npq0_random(rng, "NPQ0-S", 33, 200),
        "blk.2.q.nepq0s": synth.nepq_random(rng, "NEPQ0-S", 1, 48, 96, 3),            # NPQ0 tables in the NEPQ container
        "blk.2.k.nepq0l": synth.nepq_random(rng, "NEPQ0-L", 1, 40, 200, 5),
        "blk.3.q.mxfp8": synth.mx_random(rng, "MXFP8", 130, 256),                     # OCP MX payloads
        "blk.3.k.mxfp4": synth.mx_random(rng, "MXFP4", 37, 96),
    }
    path = tmp_path / "tiny.mfq"
    O.mfq_file_write(path, tensors, version=2)
    for name in tensors:
        for M in (1, 16, 65):
            r = subprocess.run([str(LIBDIR / "mfq-check-linear"), str(path), name, str(M), "20"], capture_output=True,
                               text=True, timeout=120)
            assert r.returncode == 0, r.stderr
            rel = float(re.search(r"production_rel=([0-9.eE+-]+)", r.stdout).group(1))
            assert rel < 1e-3, (name, M, r.stdout)
            assert "production_weight_gbps=" in r.stdout and "payload_gbps=" in r.stdout
    r = subprocess.run([str(LIBDIR / "mfq-check-linear"), str(path), "missing"], capture_output=True, text=True)
    assert r.returncode == 1 and "missing tensor" in r.stderr


def test_cpp_load_quant_linear_and_forward(rt):
    rng = np.random.default_rng(4)
    t = O.quantize_nint((rng.standard_normal((48, 88)) * 0.02).astype(np.float32), 3, 24, 5)
    h = _load(rt, "NINT3", O.pack_nint(t))
    assert rt.mfq_rt_linear_out(h) == 48 and rt.mfq_rt_linear_neuron_len(h) == 88
    W = torch.empty((48, 88), dtype=torch.float32, device="cuda")
    assert rt.mfq_rt_linear_dequantize(h, W.data_ptr(), None) == 0
    torch.cuda.synchronize()
    deq = O.dequantize_nint(t)
    assert np.array_equal(W.cpu().numpy().view(np.uint32), deq.view(np.uint32))
    for M in (1, 9, 40):
        x = torch.from_numpy(rng.standard_normal((M, 88)).astype(np.float32)).to(torch.bfloat16).cuda()
        y = torch.empty((M, 48), dtype=torch.float32, device="cuda")
        assert rt.mfq_rt_linear_forward(h, x.data_ptr(), 0, 88, M, y.data_ptr(), None) == 0
        torch.cuda.synchronize()
        check_close(y.cpu().numpy(), O.linear_forward_f64(deq, x.float().cpu().numpy()))
    assert rt.mfq_rt_linear_forward(h, None, 0, 88, 0, None, None) == 0       # an empty batch launches nothing
    assert rt.mfq_rt_linear_forward(h, x.data_ptr(), 0, 88, -1, y.data_ptr(), None) == 1
    rt.mfq_rt_free_quant_linear(h)
    with pytest.raises(RuntimeError, match="invalid NINT blob tail"):
        _load(rt, "NINT3", O.pack_nint(t)[:-1])
    with pytest.raises(RuntimeError, match="dtype/blob mismatch"):
        _load(rt, "NINT4", O.pack_nint(t))
    with pytest.raises(RuntimeError, match="unsupported quantized linear dtype"):
        _load(rt, "TPQ4", b"\0" * 64)
    with pytest.raises(RuntimeError, match="invalid MXFP4 payload header"):
        _load(rt, "MXFP4", b"\0" * 64)
    # MXFP8 / MXFP4 through the same registry: bit-exact dequantizer, GEMV and GEMM routes
    for dtype, rows, cols in (("MXFP8", 130, 256), ("MXFP4", 70, 160)):
        tm = synth.mx_random(rng, dtype, rows, cols)
        hm = _load(rt, dtype, O.pack_mx(tm))
        assert rt.mfq_rt_linear_out(hm) == rows and rt.mfq_rt_linear_neuron_len(hm) == cols
        Wm = torch.empty((rows, cols), dtype=torch.float32, device="cuda")
        assert rt.mfq_rt_linear_dequantize(hm, Wm.data_ptr(), None) == 0
        torch.cuda.synchronize()
        deqm = O.dequantize_mx(tm)
        assert np.array_equal(Wm.cpu().numpy().view(np.uint32), deqm.view(np.uint32))
        for M in (1, 9, 40):
            x = torch.from_numpy(rng.standard_normal((M, cols)).astype(np.float32)).to(torch.bfloat16).cuda()
            y = torch.empty((M, rows), dtype=torch.float32, device="cuda")
            assert rt.mfq_rt_linear_forward(hm, x.data_ptr(), 0, cols, M, y.data_ptr(), None) == 0
            torch.cuda.synchronize()
            check_close(y.cpu().numpy(), O.linear_forward_f64(deqm, x.float().cpu().numpy()))
        rt.mfq_rt_free_quant_linear(hm)
        with pytest.raises(RuntimeError, match="payload size"):
            _load(rt, dtype, O.pack_mx(tm)[:-1])
    # NINT8-0 through the same registry
    t8 = O.quantize_nint8_zero((rng.standard_normal((24, 64)) * 0.02).astype(np.float32))
    h8 = _load(rt, "NINT8-0", O.pack_nint8_zero(t8))
    assert rt.mfq_rt_linear_out(h8) == 24 and rt.mfq_rt_linear_neuron_len(h8) == 64
    W8 = torch.empty((24, 64), dtype=torch.float32, device="cuda")
    assert rt.mfq_rt_linear_dequantize(h8, W8.data_ptr(), None) == 0
    torch.cuda.synchronize()
    deq8 = O.dequantize_nint8_zero(t8)
    assert np.array_equal(W8.cpu().numpy().view(np.uint32), deq8.view(np.uint32))
    for M in (1, 9, 40):
        x = torch.from_numpy(rng.standard_normal((M, 64)).astype(np.float32)).to(torch.bfloat16).cuda()
        y = torch.empty((M, 24), dtype=torch.float32, device="cuda")
        assert rt.mfq_rt_linear_forward(h8, x.data_ptr(), 0, 64, M, y.data_ptr(), None) == 0
        torch.cuda.synchronize()
        check_close(y.cpu().numpy(), O.linear_forward_f64(deq8, x.float().cpu().numpy()))
    rt.mfq_rt_free_quant_linear(h8)
    with pytest.raises(RuntimeError, match="invalid NINT8-0 block payload length"):
        _load(rt, "NINT8-0", O.pack_nint8_zero(t8)[:-1])


def test_cpp_gate_up_glu_across_batch_sizes(rt):
    """nint_matmul_swiglu / nint_matmul_geglu of the C++ runtime: the fused GEMV (1, 2 rows), matmul + GLU kernel through
    the scratch buffer (5 rows), the prefill kernel with the GLU in its epilogue (1100 rows, no scratch needed) --
    against the oracle's float64 product; a batch that needs the scratch buffer without one is an error."""
    rng = np.random.default_rng(41)
    W, K = 1024, 256
    t = O.quantize_nint((rng.standard_normal((2 * W, K)) * 0.08).astype(np.float32), 4, 32, 6)
    h = _load(rt, "NINT4", O.pack_nint(t))
    deq = O.dequantize_nint(t)
    for M, with_scratch in ((1, False), (2, False), (5, True), (1100, False)):
        x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16).cuda()
        scratch = torch.empty((M, 2 * W), dtype=torch.float32, device="cuda") if with_scratch else None
        y = O.linear_forward_f64(deq, x.float().cpu().numpy())
        for gelu, ref in ((0, O.moe_swiglu(y)), (1, O.moe_geglu(y))):
            hid = torch.zeros((M, W), dtype=torch.float16, device="cuda")
            rc = rt.mfq_rt_linear_forward_glu(h, x.data_ptr(), 0, K, M, gelu, hid.data_ptr(),
                                              scratch.data_ptr() if with_scratch else None, None)
            assert rc == 0, rt.mfq_rt_last_error()
            torch.cuda.synchronize()
            got = hid.float().cpu().numpy()
            assert np.linalg.norm(got - ref) / np.linalg.norm(ref) < 2e-3
    x = torch.zeros((5, K), dtype=torch.bfloat16, device="cuda")
    hid = torch.zeros((5, W), dtype=torch.float16, device="cuda")
    assert rt.mfq_rt_linear_forward_glu(h, x.data_ptr(), 0, K, 5, 0, hid.data_ptr(), None, None) == 1
    assert b"scratch" in rt.mfq_rt_last_error()
    rt.mfq_rt_free_quant_linear(h)


def test_cpp_embedding_rows_and_argmax_head(rt):
    """The host library's embed_forward / next_token_from_hidden twins on a NINT5-28 table: rows bit-exact against the
    oracle's dequantizer, the token equal to the arg-max of the logits the call returns; NVQ and NINT8-0 tables give their rows, NEPQ refuses."""
    rng = np.random.default_rng(14)
    out, K = 700, 448
    t = synth.nint_random(rng, out, K, 5, 28, 7)
    h = _load(rt, "NINT5", O.pack_nint(t))
    deq = O.dequantize_nint(t)
    ids = np.array([3, 699, 0, 3, 700, -5], dtype=np.int64)
    rows = torch.empty((len(ids), K), dtype=torch.float32, device="cuda")
    assert rt.mfq_rt_linear_embedding(h, torch.from_numpy(ids).cuda().data_ptr(), len(ids), rows.data_ptr(), 2, None) == 0
    torch.cuda.synchronize()
    want = np.zeros((len(ids), K), np.float32)
    want[:4] = deq[ids[:4]]
    assert np.array_equal(rows.cpu().numpy().view(np.uint32), want.view(np.uint32))
    for M in (1, 4):
        x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16).cuda()
        token = torch.empty((M,), dtype=torch.int64, device="cuda")
        logits = torch.empty((M, out), dtype=torch.float32, device="cuda")
        assert rt.mfq_rt_linear_argmax(h, x.data_ptr(), 0, K, M, token.data_ptr(), logits.data_ptr(), None) == 0
        torch.cuda.synchronize()
        assert torch.equal(token, logits.argmax(-1))
        check_close(logits.cpu().numpy(), O.linear_forward_f64(deq, x.float().cpu().numpy()))
        alone = torch.empty((M,), dtype=torch.int64, device="cuda")
        assert rt.mfq_rt_linear_argmax(h, x.data_ptr(), 0, K, M, alone.data_ptr(), None, None) == 0
        torch.cuda.synchronize()
        assert torch.equal(alone, token)
    rt.mfq_rt_free_quant_linear(h)
    # the other table formats embed_forward takes: an NVQ table in the lane-major layout, one read from its streams, NINT8-0
    tv = synth.nvq_jsc_random(rng, 32, 96)
    te = synth.nvq_jsc_random(rng, 40, 104, "e8_256", 2)
    t8 = O.quantize_nint8_zero((rng.standard_normal((24, 64)) * 0.02).astype(np.float32))
    for dtype, blob, deq in (("NVQ3J-512", O.pack_nvq_jsc(tv), O.dequantize_nvq_jsc(tv)),
                             (O.pack_tensor(te)[0], O.pack_tensor(te)[1], O.dequantize_nvq_jsc(te)),
                             ("NINT8-0", O.pack_nint8_zero(t8), O.dequantize_nint8_zero(t8))):
        hv = _load(rt, dtype, blob)
        n, kk = deq.shape
        ids = np.array([n - 1, 0, 5, n, -1], dtype=np.int64)
        rows = torch.empty((len(ids), kk), dtype=torch.float16, device="cuda")
        assert rt.mfq_rt_linear_embedding(hv, torch.from_numpy(ids).cuda().data_ptr(), len(ids), rows.data_ptr(), 1, None) == 0
        torch.cuda.synchronize()
        want = np.zeros((len(ids), kk), np.float32)
        want[:3] = deq[ids[:3]]
        assert np.array_equal(rows.cpu().numpy().view(np.uint16), want.astype(np.float16).view(np.uint16))
        rt.mfq_rt_free_quant_linear(hv)
    hp = _load(rt, "NEPQ1-S", O.pack_tensor(synth.nepq_random(rng, "NEPQ1-S", 1, 32, 96, 3))[1])
    assert rt.mfq_rt_linear_embedding(hp, None, 0, None, 2, None) != 0
    assert b"NINT, NINT8-0 or NVQ" in rt.mfq_rt_last_error()
    rt.mfq_rt_free_quant_linear(hp)


@pytest.mark.parametrize("T", [1, 20])
def test_cpp_moe_ffn_forward(rt, T):
    rng = np.random.default_rng(40 + T)
    E, H, W, k = 16, 128, 64, 4
    bits = rng.choice([2, 3, 4, 5], size=E, p=[0.1, 0.4, 0.4, 0.1])
    tg, td = synth.moe_random(rng, E, 2 * W, H, bits, True), synth.moe_random(rng, E, H, W, bits, True)
    bg, bd = O.pack_nint_moe(tg), O.pack_nint_moe(td)
    hg, hd = C.c_void_p(), C.c_void_p()
    assert rt.mfq_rt_load_nint_moe(bg, len(bg), C.byref(hg)) == 0, rt.mfq_rt_last_error()
    assert rt.mfq_rt_load_nint_moe(bd, len(bd), C.byref(hd)) == 0, rt.mfq_rt_last_error()
    x = torch.from_numpy(rng.standard_normal((T, H)).astype(np.float32)).to(torch.bfloat16).cuda()
    logits = rng.standard_normal((T, E)).astype(np.float32)
    lg = torch.from_numpy(logits).cuda()
    out = torch.empty((T, H), dtype=torch.float32, device="cuda")
    ids = torch.empty((T, k), dtype=torch.int32, device="cuda")
    wts = torch.empty((T, k), dtype=torch.float32, device="cuda")
    rc = rt.mfq_rt_moe_ffn_forward(hg, hd, x.data_ptr(), 0, H, T, lg.data_ptr(), k, 3, 0, None, None, out.data_ptr(),
                                   ids.data_ptr(), wts.data_ptr(), None)
    assert rc == 0, rt.mfq_rt_last_error()
    torch.cuda.synchronize()
    ref, rids, rw = O.moe_ffn(O.dequantize_expertwise(tg), O.dequantize_expertwise(td), x.float().cpu().numpy(), logits, k,
                              delayed_softmax=True)
    assert np.array_equal(ids.cpu().numpy(), rids)
    check_close(out.cpu().numpy(), ref)
    rt.mfq_rt_free_nint_moe(hg)
    rt.mfq_rt_free_nint_moe(hd)


@pytest.mark.parametrize("T", [1, 64])
def test_cpp_moe_ffn_forward_replays_from_a_graph(rt, T):
    """nint_moe_ffn_forward of the C++ runtime with a reserved scratch is recorded into a HIP graph (it must neither
    allocate nor wait for the device: either would fail the capture) and replayed several times with new activations and
    router logits in the same buffers and eager work in between; every replay equals the eager call bit for bit, and the
    eager call matches the oracle.  T = 1 takes the decode form (no route map), T = 64 the mapped prefill kernels with a
    shared expert next to the routed ones."""
    rng = np.random.default_rng(400 + T)
    E, H, W, k = 16, 256, 128, 4
    bits = rng.choice([2, 3, 4, 5], size=E, p=[0.1, 0.4, 0.4, 0.1])
    tg, td = synth.moe_random(rng, E, 2 * W, H, bits, True), synth.moe_random(rng, E, H, W, bits, True)
    sg_t, sd_t = synth.nint_random(rng, 2 * W, H, 4, 24, 6), synth.nint_random(rng, H, W, 4, 24, 6)
    bg, bd = O.pack_nint_moe(tg), O.pack_nint_moe(td)
    hg, hd = C.c_void_p(), C.c_void_p()
    assert rt.mfq_rt_load_nint_moe(bg, len(bg), C.byref(hg)) == 0, rt.mfq_rt_last_error()
    assert rt.mfq_rt_load_nint_moe(bd, len(bd), C.byref(hd)) == 0, rt.mfq_rt_last_error()
    sg, sd = _load(rt, "NINT4", O.pack_nint(sg_t)), _load(rt, "NINT4", O.pack_nint(sd_t))
    scratch = C.c_void_p()
    assert rt.mfq_rt_moe_scratch_create(C.byref(scratch)) == 0
    assert rt.mfq_rt_moe_scratch_reserve(scratch, hg, hd, T, k, sg, sd) == 0, rt.mfq_rt_last_error()
    x = torch.empty((T, H), dtype=torch.bfloat16, device="cuda")
    lg = torch.empty((T, E), dtype=torch.float32, device="cuda")
    out = torch.empty((T, H), dtype=torch.float32, device="cuda")

    def fill(seed):
        r = np.random.default_rng(seed)
        xs = r.standard_normal((T, H)).astype(np.float32)
        ls = r.standard_normal((T, E)).astype(np.float32)
        x.copy_(torch.from_numpy(xs).to(torch.bfloat16))
        lg.copy_(torch.from_numpy(ls))
        return ls

    def call(stream):
        rc = rt.mfq_rt_moe_ffn_forward_scratch(scratch, hg, hd, x.data_ptr(), 0, H, T, lg.data_ptr(), k, 3, 0, sg, sd,
                                               out.data_ptr(), stream)
        assert rc == 0, rt.mfq_rt_last_error()

    logits = fill(1)
    call(None)  # eager: default stream
    torch.cuda.synchronize()
    eager1 = out.clone()
    Wg, Wd = O.dequantize_expertwise(tg), O.dequantize_expertwise(td)
    ref, rids, _ = O.moe_ffn(Wg, Wd, x.float().cpu().numpy(), logits, k, delayed_softmax=True,
                             shared=(O.dequantize_nint(sg_t), O.dequantize_nint(sd_t)))
    ids_p, w_p = C.c_void_p(), C.c_void_p()
    assert rt.mfq_rt_moe_scratch_topk(scratch, C.byref(ids_p), C.byref(w_p)) == 0
    check_close(eager1.cpu().numpy(), ref)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(C.c_void_p(side.cuda_stream))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call(C.c_void_p(torch.cuda.current_stream().cuda_stream))
    for seed in (1, 2, 3, 1):
        fill(seed)
        call(None)
        torch.cuda.synchronize()
        want = out.clone()
        out.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int32), want.view(torch.int32)), f"replay differs from the eager call (seed {seed})"
    assert torch.equal(want.view(torch.int32), eager1.view(torch.int32))
    rt.mfq_rt_moe_scratch_free(scratch)
    for h in (sg, sd):
        rt.mfq_rt_free_quant_linear(h)
    rt.mfq_rt_free_nint_moe(hg)
    rt.mfq_rt_free_nint_moe(hd)


def _mixed_moe(rng, E_out, K):
    """Eight experts in seven cohorts of different families (NINT4, NINT8-0, NVQ3J-512, MXFP4, NVQ1-S, NEPQ1-S, NEPQ0-L)."""
    def pool(ids, dtype, t):
        return O.MoePool(np.asarray(ids, dtype=np.int32), dtype, t)
    return O.NintMoeTensor((8, E_out, K), [
        pool([0, 7], "NINT4", synth.nint_random(rng, 2 * E_out, K, 4, 32, 6)),
        pool([5], "NINT8-0", O.quantize_nint8_zero((rng.standard_normal((E_out, K)) * 0.02).astype(np.float32))),
        pool([1], "NVQ3J-512", synth.nvq_jsc_random(rng, E_out, K, "d4_512", 2)),
        pool([4], "MXFP4", synth.mx_random(rng, "MXFP4", E_out, K, 112, 116)),
        pool([2], "NVQ1-S", synth.nvq1_random(rng, "NVQ1-S", E_out, K)),
        pool([6], "NEPQ1-S", synth.nepq_random(rng, "NEPQ1-S", 1, E_out, K, 3)),
        pool([3], "NEPQ0-L", synth.nepq_random(rng, "NEPQ0-L", 1, E_out, K, 2))])


@pytest.mark.parametrize("T", [3, 40])
def test_cpp_moe_ffn_with_cohorts_of_other_families(rt, T):
    """Gate/up and down tensors whose cohorts mix NINT with NVQ, MXFP4, a 1-bit family and NEPQ: the C++ runtime splits the
    foreign cohorts into per-expert tensors and walks the routed experts on the host; the layer against the oracle."""
    rng = np.random.default_rng(140 + T)
    E, H, W, k = 8, 192, 96, 3
    tg, td = _mixed_moe(rng, 2 * W, H), _mixed_moe(rng, H, W)
    bg, bd = O.pack_nint_moe(tg), O.pack_nint_moe(td)
    hg, hd = C.c_void_p(), C.c_void_p()
    assert rt.mfq_rt_load_nint_moe(bg, len(bg), C.byref(hg)) == 0, rt.mfq_rt_last_error()
    assert rt.mfq_rt_load_nint_moe(bd, len(bd), C.byref(hd)) == 0, rt.mfq_rt_last_error()
    x = torch.from_numpy((rng.standard_normal((T, H)) * 3).astype(np.float32)).to(torch.bfloat16).cuda()
    logits = rng.standard_normal((T, E)).astype(np.float32)
    lg = torch.from_numpy(logits).cuda()
    out = torch.empty((T, H), dtype=torch.float32, device="cuda")
    ids = torch.empty((T, k), dtype=torch.int32, device="cuda")
    wts = torch.empty((T, k), dtype=torch.float32, device="cuda")
    rc = rt.mfq_rt_moe_ffn_forward(hg, hd, x.data_ptr(), 0, H, T, lg.data_ptr(), k, 3, 0, None, None, out.data_ptr(),
                                   ids.data_ptr(), wts.data_ptr(), None)
    assert rc == 0, rt.mfq_rt_last_error()
    torch.cuda.synchronize()
    ref, rids, rw = O.moe_ffn(O.dequantize_expertwise(tg), O.dequantize_expertwise(td), x.float().cpu().numpy(), logits, k,
                              delayed_softmax=True)
    assert np.array_equal(ids.cpu().numpy(), rids)
    check_close(out.cpu().numpy(), ref)
    rt.mfq_rt_free_nint_moe(hg)
    rt.mfq_rt_free_nint_moe(hd)


def test_cpp_moe_ffn_with_an_expert_overlay(rt):
    """An NINTMD expert overlay on the gate/up tensor (a NINT3 cohort for an expert of the NINT4 cohort and for the NVQ
    expert, an NEPQ1-S cohort for the 1-bit expert): the layer against the oracle on the overlaid tensor, at a decode
    step and on a mapped batch; the delta alone does not load."""
    rng = np.random.default_rng(150)
    E, H, W, k = 8, 192, 96, 3
    tg, td = _mixed_moe(rng, 2 * W, H), _mixed_moe(rng, H, W)
    delta = O.NintMoeTensor((E, 2 * W, H), [
        O.MoePool(np.array([7, 1], dtype=np.int32), "NINT3", synth.nint_random(rng, 2 * 2 * W, H, 3, 24, 5)),
        O.MoePool(np.array([2], dtype=np.int32), "NEPQ1-S", synth.nepq_random(rng, "NEPQ1-S", 1, 2 * W, H, 3))])
    bg, bd, bo = O.pack_nint_moe(tg), O.pack_nint_moe(td), O.pack_nint_moe(delta, delta=True)
    rt.mfq_rt_load_nint_moe_overlay.argtypes = [C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t, C.POINTER(C.c_void_p)]
    hg, hd, hbad = C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert rt.mfq_rt_load_nint_moe(bo, len(bo), C.byref(hbad)) != 0 and b"delta cannot be loaded" in rt.mfq_rt_last_error()
    assert rt.mfq_rt_load_nint_moe_overlay(bg, len(bg), bo, len(bo), C.byref(hg)) == 0, rt.mfq_rt_last_error()
    assert rt.mfq_rt_load_nint_moe(bd, len(bd), C.byref(hd)) == 0, rt.mfq_rt_last_error()
    dg, dd = O.dequantize_expertwise(O.apply_expert_overlay(tg, delta)), O.dequantize_expertwise(td)
    for T in (3, 40):
        x = torch.from_numpy((rng.standard_normal((T, H)) * 3).astype(np.float32)).to(torch.bfloat16).cuda()
        logits = rng.standard_normal((T, E)).astype(np.float32)
        logits[0, [7, 1, 2]] += 8.0                      # the first token routes to the experts that changed hands
        lg = torch.from_numpy(logits).cuda()
        out = torch.empty((T, H), dtype=torch.float32, device="cuda")
        ids = torch.empty((T, k), dtype=torch.int32, device="cuda")
        wts = torch.empty((T, k), dtype=torch.float32, device="cuda")
        rc = rt.mfq_rt_moe_ffn_forward(hg, hd, x.data_ptr(), 0, H, T, lg.data_ptr(), k, 3, 0, None, None, out.data_ptr(),
                                       ids.data_ptr(), wts.data_ptr(), None)
        assert rc == 0, rt.mfq_rt_last_error()
        torch.cuda.synchronize()
        ref, rids, rw = O.moe_ffn(dg, dd, x.float().cpu().numpy(), logits, k, delayed_softmax=True)
        assert np.array_equal(ids.cpu().numpy(), rids) and set(rids[0].tolist()) == {7, 1, 2}
        check_close(out.cpu().numpy(), ref)
    rt.mfq_rt_free_nint_moe(hg)
    rt.mfq_rt_free_nint_moe(hd)


def test_cpp_nvq_ffn_swiglu_down(rt):
    """nvq_ffn_swiglu_down of the C++ runtime (joint gate/up launch, SwiGLU kernel, down projection) against the
    oracle's float64 evaluation of the dequantized weights; the hidden rows pass through fp16."""
    from conftest import rel_l2
    rng = np.random.default_rng(8071)
    K, W, out = 1560, 240, 72
    blobs = [O.pack_tensor(synth.nvq_jsc_random(rng, W, K, "d4_512", 2)),
             O.pack_tensor(synth.nvq_jsc_random(rng, W, K, "d4_512", 1)),
             O.pack_tensor(synth.nvq_jsc_random(rng, out, W, "d4_512", 2))]
    hs = [_load(rt, d, b) for d, b in blobs]
    wg, wu, wd = (O.dequantize_nvq_jsc(O.unpack_nvq(b)) for _, b in blobs)
    for M in (1, 6, 40):
        x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16).cuda()
        y = torch.empty((M, out), dtype=torch.float32, device="cuda")
        assert rt.mfq_rt_nvq_ffn_swiglu_down(hs[0], hs[1], hs[2], x.data_ptr(), 0, K, M, y.data_ptr(), None) == 0
        torch.cuda.synchronize()
        xf = x.float().cpu().numpy()
        g, u = O.linear_forward_f64(wg, xf), O.linear_forward_f64(wu, xf)
        assert rel_l2(y.cpu().numpy(), O.linear_forward_f64(wd, g / (1.0 + np.exp(-g)) * u)) < 2e-3
    assert rt.mfq_rt_nvq_ffn_swiglu_down(hs[0], hs[1], hs[0], x.data_ptr(), 0, K, 1, y.data_ptr(), None) == 1
    assert "fused FFN weight layouts" in rt.mfq_rt_last_error().decode()
    for h in hs:
        rt.mfq_rt_free_quant_linear(h)


def test_cpp_expert_cache_matches_the_resident_tensor():
    """The C++ MoeExpertCache through its C view: three slots per cohort, routes over twelve experts, outputs bit for
    bit those of the fully resident NintMoeWeight (Python twin over the same C ABI), hits / misses / evictions counted."""
    import ctypes as C
    from pathlib import Path
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_moe import MoeExpertCache, NintMoeWeight, build_moe_route_plan
    lib = C.CDLL(str(Path(R.__file__).resolve().parent / "lib" / "libmfq_runtime.so"))
    lib.mfq_rt_last_error.restype = C.c_char_p
    rng = np.random.default_rng(31)
    E, out, K = 12, 32, 96
    t = synth.moe_random(rng, E, out, K, [4, 3] * 6, quantize=True)
    blob = O.pack_nint_moe(t)
    full = NintMoeWeight.from_blob(blob)
    per_slot = sum(c.slot_bytes for c in MoeExpertCache(1 << 30).register_source(blob).cohorts)
    cache, src = C.c_void_p(), C.c_void_p()
    assert lib.mfq_rt_moe_cache_create(C.c_int64(3 * per_slot + 64), C.byref(cache)) == 0
    assert lib.mfq_rt_moe_cache_register(cache, blob, C.c_size_t(len(blob)), 2, C.byref(src)) == 0, lib.mfq_rt_last_error()
    assert lib.mfq_rt_moe_cache_finalize(cache) == 0, lib.mfq_rt_last_error()
    for T in (1, 20, 2, 20, 1):
        even = rng.choice(np.arange(0, E, 2), size=3, replace=False)
        odd = rng.choice(np.arange(1, E, 2), size=3, replace=False)
        ids = np.stack([np.array([rng.choice(even), rng.choice(odd)]) for _ in range(T)]).astype(np.int32)
        ids_d = torch.from_numpy(ids).cuda()
        x = torch.from_numpy((rng.standard_normal((T, K)) * 0.1).astype(np.float32)).to(torch.bfloat16).cuda()
        got = torch.empty((T, 2, out), dtype=torch.float32, device="cuda")
        rc = lib.mfq_rt_moe_cache_forward(cache, src, C.c_void_p(x.data_ptr()), 0, C.c_int64(K), 0, C.c_void_p(ids_d.data_ptr()),
                                          T, 2, C.c_void_p(got.data_ptr()), None)
        assert rc == 0, lib.mfq_rt_last_error()
        want = full(x, build_moe_route_plan(ids_d, E))
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), T
    stats = (C.c_int64 * 5)()
    assert lib.mfq_rt_moe_cache_stats(cache, stats) == 0
    hits, misses, evictions, nbytes, launches = list(stats)
    assert misses >= 6 and evictions > 0 and hits > 0 and nbytes > 0 and launches <= 5
    lib.mfq_rt_moe_cache_free(cache)


def test_linears_load_from_a_mapped_shard_set(rt, tmp_path):
    """A four-format model written as a shard set: both runtimes load every linear straight from the file mappings (any
    shard names the set), dequantize bit-exactly, and mfq-check-linear takes a shard path; a tensor overlay swaps one
    projection for another precision."""
    from tyloquant_amd import formats as F
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(8)
    tensors, want = {}, {}
    for name, t in (("q", synth.nint_random(rng, 32, 96, 4, 24, 6)), ("k", synth.nint_random(rng, 16, 96, 3, 24, 5)),
                    ("gate", synth.nvq_jsc_random(rng, 32, 96)), ("down", synth.nepq_random(rng, "NEPQ1-S", 1, 32, 192, 3))):
        dtype, blob = O.pack_tensor(t)
        tensors[name] = (dtype, blob)
        want[name] = O.dequantize_tensor(t)
    tensors[F.ASSET_PREFIX + "config.json"] = ("BLOB", b'{"hidden":96}')
    paths = F.write_mfq_shards(tmp_path / "tiny.mfq", tensors, "tiny", extra={"general.name": "tiny"}, split_max_tensors=2)
    assert len(paths) == 2
    with F.MfqStore(paths[1], "", "") as st:
        for name in want:
            lin = R.load_quant_linear(st.record(name).dtype, st.blob(name))
            got = lin.dequantize().cpu().numpy().reshape(want[name].shape)
            assert np.array_equal(got.view(np.uint32), want[name].view(np.uint32)), name
    rt.mfq_rt_file_open.argtypes = [C.c_char_p, C.c_char_p, C.c_char_p, C.POINTER(C.c_void_p)]
    rt.mfq_rt_file_load_quant_linear.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p)]
    rt.mfq_rt_file_close.argtypes = [C.c_void_p]
    # an overlay that stores "k" at four bits instead of three
    k4 = synth.nint_random(rng, 16, 96, 4, 24, 6)
    over = tmp_path / "k4.mfq"
    F.write_mfq(over, {"k": O.pack_tensor(k4)}, "tiny", 2)
    for overlay, k_want in ((b"-", want["k"]), (str(over).encode(), O.dequantize_tensor(k4))):
        f = C.c_void_p()
        assert rt.mfq_rt_file_open(str(paths[0]).encode(), overlay, b"-", C.byref(f)) == 0, rt.mfq_rt_last_error()
        for name in ("q", "k"):
            h = C.c_void_p()
            assert rt.mfq_rt_file_load_quant_linear(f, name.encode(), C.byref(h)) == 0, rt.mfq_rt_last_error()
            ref = k_want if name == "k" else want[name]
            out = torch.empty(ref.shape, dtype=torch.float32, device="cuda")
            assert rt.mfq_rt_linear_dequantize(h, out.data_ptr(), None) == 0
            torch.cuda.synchronize()
            assert np.array_equal(out.cpu().numpy().view(np.uint32), ref.view(np.uint32)), name
            rt.mfq_rt_free_quant_linear(h)
        rt.mfq_rt_file_close(f)
    r = subprocess.run([str(LIBDIR / "mfq-check-linear"), str(paths[1]), "q", "1", "20"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    assert float(re.search(r"production_rel=([0-9.e+-]+)", r.stdout).group(1)) < 1e-3
