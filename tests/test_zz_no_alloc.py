"""The allocation-free LM-head entry point (built-in scratch) against the workspace one, through the C ABI."""
import ctypes as C

import numpy as np
import pytest

import synth
from oracle import mfq_oracle as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _both(lin, x, with_logits):
    from tyloquant_amd import _lib as L
    lib = L.lib()
    w = lin.weight
    M = x.shape[0]
    p = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    res = []
    for static in (False, True):
        token = torch.full((M,), -7, dtype=torch.int64, device="cuda")
        logits = torch.zeros((M, w.out), dtype=torch.float32, device="cuda") if with_logits else None
        if static:
            L.check(lib.mfq_hip_nint_gemv_argmax_static(C.byref(w.desc), p(w.data), p(x), L.X_BF16, x.stride(0), M,
                                                        p(logits), w.out, p(token), st))
        else:
            need = lib.mfq_hip_nint_gemv_argmax_workspace_bytes(C.byref(w.desc), M)
            ws = torch.empty(need, dtype=torch.uint8, device="cuda")
            L.check(lib.mfq_hip_nint_gemv_argmax(C.byref(w.desc), p(w.data), p(x), L.X_BF16, x.stride(0), M, p(logits),
                                                 w.out, p(token), p(ws), need, st))
        torch.cuda.synchronize()
        res.append((token.cpu().numpy(), None if logits is None else logits.cpu().numpy()))
    return res


def test_static_scratch_argmax_matches_the_workspace_entry_point():
    """Two calls in a row, the second on a smaller tensor and batch: same tokens (and bit-identical logits) as the
    entry point with a caller workspace, and the oracle's arg-max of the fp64 product.  Then the size limit."""
    from tyloquant_amd import _lib as L
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(77)
    for out, K, bits, gs, sb, M, with_logits in ((4112, 1024, 4, 32, 6, 1, False), (304, 264, 3, 24, 5, 3, True)):
        t = O.quantize_nint((rng.standard_normal((out, K)) * 0.02).astype(np.float32), bits, gs, sb)
        lin = R.load_quant_linear(f"NINT{bits}", O.pack_nint(t))
        x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16).cuda()
        (tok_ws, lg_ws), (tok_st, lg_st) = _both(lin, x, with_logits)
        assert np.array_equal(tok_ws, tok_st)
        ref = O.linear_forward_f64(O.dequantize_nint(t), x.float().cpu().numpy())
        assert np.array_equal(tok_st, ref.argmax(axis=1))
        if with_logits:
            assert np.array_equal(lg_ws.view(np.uint32), lg_st.view(np.uint32))
            assert np.abs(lg_st - ref).max() < 1e-2
    # beyond the built-in buffer: a clear error, nothing launched
    big = L.NintDesc()
    L.check(L.lib().mfq_hip_nint_plan(4, 6, 32, 600000, 64, C.byref(big)))
    token = torch.zeros(4, dtype=torch.int64, device="cuda")
    rc = L.lib().mfq_hip_nint_gemv_argmax_static(C.byref(big), C.c_void_p(token.data_ptr()), C.c_void_p(token.data_ptr()),
                                                 L.X_BF16, 64, 4, None, 0, C.c_void_p(token.data_ptr()), None)
    assert rc == 4 and b"built-in buffer holds" in L.lib().mfq_hip_last_error()


def test_static_scratch_argmax_replays_from_a_graph():
    """After the per-device set-up call the entry point is captured into a HIP graph (nothing in it allocates or looks
    anything up) and replayed three times with eager work and synchronizations in between: every replay gives the
    eager call's tokens and logits."""
    from tyloquant_amd import _lib as L
    from tyloquant_amd import runtime as R
    lib = L.lib()
    rng = np.random.default_rng(78)
    out, K, M = 2064, 512, 2
    t = O.quantize_nint((rng.standard_normal((out, K)) * 0.02).astype(np.float32), 4, 32, 6)
    w = R.load_quant_linear("NINT4", O.pack_nint(t)).weight
    xs = [torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16).cuda() for _ in range(3)]
    x = xs[0].clone()
    token = torch.full((M,), -7, dtype=torch.int64, device="cuda")
    logits = torch.zeros((M, out), dtype=torch.float32, device="cuda")
    p = lambda a: C.c_void_p(a.data_ptr())
    L.check(lib.mfq_hip_nint_gemv_argmax_static_init())

    def call():
        st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        L.check(lib.mfq_hip_nint_gemv_argmax_static(C.byref(w.desc), p(w.data), p(x), L.X_BF16, x.stride(0), M, p(logits), out,
                                                    p(token), st))

    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call()
    for xi in xs:
        x.copy_(xi)
        call()
        torch.cuda.synchronize()
        want_tok, want_lg = token.clone(), logits.clone()
        token.fill_(-7)
        logits.zero_()
        (logits.sum() + 1).item()                       # eager work and a synchronization between the replays
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(token, want_tok) and torch.equal(logits, want_lg)
        ref = O.linear_forward_f64(O.dequantize_nint(t), xi.float().cpu().numpy())
        assert np.array_equal(token.cpu().numpy(), ref.argmax(axis=1))
