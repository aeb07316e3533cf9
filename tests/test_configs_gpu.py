"""The five BASELINE configurations at their stated shapes, HIP path against the oracle (through the C ABI).

Weights that the numpy quantizer handles in seconds go through it (config 1, config 2); the others are drawn in the
packed domain, as the reference's own fixtures are (tests/test_nvq3j512_cpp_runtime.py:58-75,
tests/mixed_family_fixtures.py:55-153).  The oracle decodes the same bytes; the reference output is the fp64 product
with the oracle-dequantized weights, in the style of tests/test_kernels_cuda.py:91-119.  Tolerance: rel-L2 <= 1e-3,
max-abs <= 1e-2 (outputs are of order one by construction); dequantized weights bit for bit.
"""
import numpy as np
import pytest

import synth
from conftest import ABS_TOL, REL_TOL, rel_l2
from oracle import mfq_oracle as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _bf16(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16)


def _close(y, ref, what):
    y = np.asarray(y, dtype=np.float64)
    rel = rel_l2(y, ref)
    err = float(np.abs(y - ref).max())
    assert rel < REL_TOL and err < ABS_TOL, f"{what}: rel-L2 {rel:.3e}, max-abs {err:.3e}"


def _bit_equal(got, want):
    got, want = np.asarray(got), np.asarray(want)
    return got.size == want.size and np.array_equal(got.reshape(-1).view(np.uint32), want.reshape(-1).view(np.uint32))


def test_config1_nint3_4096x4096_batch1():
    from tyloquant_amd import runtime as R
    from tyloquant_amd import synth as P
    dtype, blob = P.nint_linear_blob(1, 4096, 4096, 3, 24, 5)
    lin = R.load_quant_linear(dtype, blob)
    deq = O.dequantize_nint(O.unpack_nint(blob))
    assert _bit_equal(lin.dequantize().cpu().numpy(), deq)
    x = _bf16(P.activations(np.random.default_rng(11), 1, 4096))
    _close(lin(x.cuda()).cpu().numpy(), O.linear_forward_f64(deq, x.float().numpy()), "C1 M=1")


@pytest.mark.parametrize("name,out,K", [("gate_up", 12288, 4096), ("down", 4096, 12288)])
def test_config2_nint4_ffn_shapes_with_outlier_channels(name, out, K):
    """NINT4 (4,32,6), N(0, 0.02) weights through the quantizer (a 1024-row slab tiled over the rows), activations
    N(0,1) with 0.1 % of the channels scaled by 20, M in {1, 16, 512, 2048}: the batch-1 GEMV, the streaming
    matrix-core kernel and the prefill kernel, each on the rows of one fp64 reference product."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd import synth as P
    dtype, blob = P.nint_linear_blob(100 + out, out, K, 4, 32, 6, slab_rows=1024)
    lin = R.load_quant_linear(dtype, blob)
    deq = O.dequantize_nint(O.unpack_nint(blob))
    assert _bit_equal(lin.dequantize().cpu().numpy(), deq)
    x = _bf16(P.activations(np.random.default_rng(12), 2048, K, outlier_frac=0.001))
    assert float(x.float().abs().max()) > 40.0            # the outlier channels are there
    ref = O.linear_forward_f64(deq, x.float().numpy())
    xd = x.cuda()
    for M in (1, 16, 512, 2048):
        _close(lin(xd[:M]).cpu().numpy(), ref[:M], f"C2 {name} M={M}")
    _close(R.nint_matmul(lin.weight, xd[:16], force="gemv").cpu().numpy(), ref[:16], f"C2 {name} M=16 streaming")


@pytest.mark.parametrize("out,K", [(17408, 5120), (5120, 17408)])
def test_config3_nvq3j512_27b_shapes(out, K):
    """NVQ3J-512 (d4_512, two banks, 16-entry scale LUT) at the 27B FFN shapes, batch {1, 4, 8}."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(30 + out % 7)
    t = synth.nvq_jsc_random(rng, out, K, "d4_512", 2)
    t.neuron_scale = O._f16_round(t.neuron_scale * 0.02)            # outputs of order one
    dtype, blob = O.pack_tensor(t)
    lin = R.load_quant_linear(dtype, blob)
    deq = O.dequantize_nvq_jsc(O.unpack_nvq(blob))
    assert _bit_equal(lin.dequantize().cpu().numpy(), deq)
    x = _bf16(rng.standard_normal((8, K)))
    ref = O.linear_forward_f64(deq, x.float().numpy())
    xd = x.cuda()
    for M in (1, 4, 8):
        _close(lin(xd[:M]).cpu().numpy(), ref[:M], f"C3 {out}x{K} M={M}")


def _expert_dense(pools, owner, local, out, e):
    """Oracle-dequantized [out, K] weights of expert e of a packed-domain NINTM tensor."""
    return O.dequantize_nint(synth.nint_blob_rows(pools[owner[e]][1], int(local[e]) * out, out))


def test_config4_moe_256_experts_mixed_bits():
    """256 routed experts (bit widths 2/3/4/5 with p = .1/.4/.4/.1, N(0, 0.02) weights through the expert-wise
    quantizer) + one shared NINT4 expert, hidden 4096, intermediate 2048, top-8 delayed softmax, T in {1, 64, 2048}.  Two layers of checking: (a) the tokens of a fixed
    sample against the oracle alone (its own top-k, its own dequantizer on the experts they hit, the fp32 loop of
    tests/test_moe_kernels_cuda.py:58-68); (b) every token against an fp64 reference that multiplies with the
    GPU-dequantized weights, which (a) shows to be bit-identical to the oracle's on every sampled expert."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd import synth as psynth
    from tyloquant_amd.runtime_moe import NintMoeWeight, nint_moe_ffn_forward
    E, H, W, k = 256, 4096, 2048, 8
    rng = np.random.default_rng(4)
    bits = rng.choice([2, 3, 4, 5], size=E, p=[0.1, 0.4, 0.4, 0.1])
    # N(0, 0.02) weights through the expert-wise quantizer (one 1024-row slab per precision, tiled over the cohort)
    gu_blob, gu_pools = psynth.nintm_quantized_blob(40, E, 2 * W, H, bits)
    dn_blob, dn_pools = psynth.nintm_quantized_blob(41, E, H, W, bits)
    gu, dn = NintMoeWeight.from_blob(gu_blob), NintMoeWeight.from_blob(dn_blob)
    del gu_blob, dn_blob
    sg_blob = synth.nint_packed_blob(rng, 2 * W, H, 4, 24, 6)
    sd_blob = synth.nint_packed_blob(rng, H, W, 4, 24, 6)
    shared = (R.load_quant_linear("NINT4", sg_blob).weight, R.load_quant_linear("NINT4", sd_blob).weight)
    sg, sd = O.dequantize_nint(O.unpack_nint(sg_blob)), O.dequantize_nint(O.unpack_nint(sd_blob))
    assert _bit_equal(shared[0].dequantize().cpu().numpy(), sg) and _bit_equal(shared[1].dequantize().cpu().numpy(), sd)
    owner = np.zeros(E, dtype=np.int64)
    local = np.zeros(E, dtype=np.int64)
    for pi, (ids, _) in enumerate(gu_pools):
        owner[ids], local[ids] = pi, np.arange(len(ids))
    dense_gu = gu.dequantize()                             # [E, 2W, H] fp32 on the device, checked expert by expert below
    dense_dn = dn.dequantize()
    checked = {}

    def oracle_expert(e):
        if e not in checked:
            a, b = _expert_dense(gu_pools, owner, local, 2 * W, e), _expert_dense(dn_pools, owner, local, H, e)
            assert _bit_equal(dense_gu[e].cpu().numpy(), a) and _bit_equal(dense_dn[e].cpu().numpy(), b), f"expert {e}"
            checked[e] = (a, b)
        return checked[e]

    def silu_mul(g):                                       # fp64 SwiGLU on the device
        gate, up = g[..., :W], g[..., W:]
        return gate / (1.0 + torch.exp(-gate)) * up

    sgd, sdd = torch.from_numpy(sg).cuda().double(), torch.from_numpy(sd).cuda().double()
    x_all = _bf16(rng.standard_normal((2048, H)))
    logit_all = rng.standard_normal((2048, E)).astype(np.float32)
    for T, sample in ((1, [0]), (64, [5, 40]), (2048, [1234])):
        x, logits = x_all[:T], logit_all[:T]
        out, ids, wts = nint_moe_ffn_forward(gu, dn, x.cuda(), torch.from_numpy(logits).cuda(), k, delayed_softmax=True,
                                             shared=shared)
        got = out.cpu().numpy()
        rids, rw = O.moe_topk(logits, k, delayed_softmax=True)
        assert np.array_equal(ids.cpu().numpy(), rids)
        np.testing.assert_allclose(wts.cpu().numpy(), rw, rtol=2e-6, atol=2e-7)
        # (a) sampled tokens, oracle only
        xf = x.float().numpy()
        for t in sample:
            acc = np.zeros(H, dtype=np.float32)
            for r in range(k):
                a, b = oracle_expert(int(rids[t, r]))
                acc += rw[t, r] * O.linear_forward(b, O.moe_swiglu(O.linear_forward(a, xf[t:t + 1])))[0]
            acc += O.linear_forward(sd, O.moe_swiglu(O.linear_forward(sg, xf[t:t + 1])))[0]
            _close(got[t], acc.astype(np.float64), f"C4 T={T} token {t} (oracle)")
        # (b) all tokens, fp64 over the dequantized weights, expert by expert
        xd = x.cuda().double()
        ref = silu_mul(xd @ sgd.T) @ sdd.T
        idt, wt = torch.from_numpy(rids.astype(np.int64)).cuda(), torch.from_numpy(rw).cuda().double()
        for e in np.unique(rids):
            tok, slot = torch.nonzero(idt == int(e), as_tuple=True)
            h = silu_mul(xd[tok] @ dense_gu[e].double().T)
            ref.index_add_(0, tok, (h @ dense_dn[e].double().T) * wt[tok, slot][:, None])
        _close(got, ref.cpu().numpy(), f"C4 T={T} all tokens")
    assert len(checked) >= 24


def test_config5_one_decoder_layer_in_the_four_formats():
    """QKV 6144x4096, O 4096x4096, gate and up 12288x4096, down 4096x12288 of one layer, one tensor per format
    (NEPQ1-S, NINT3, NVQ3J-512, NINT5-28) plus NEPQ1-S and NINT5-28 on the K = 12288 down shape, batch {1, 16}."""
    from tyloquant_amd import runtime as R
    rng = np.random.default_rng(5)

    def nint(out, K, b, gs, sb):
        blob = synth.nint_packed_blob(rng, out, K, b, gs, sb)
        return f"NINT{b}", blob, lambda: O.dequantize_nint(O.unpack_nint(blob))

    def nvq(out, K):
        t = synth.nvq_jsc_random(rng, out, K, "d4_512", 2)
        t.neuron_scale = O._f16_round(t.neuron_scale * 0.02)
        dtype, blob = O.pack_tensor(t)
        return dtype, blob, lambda: O.dequantize_nvq_jsc(O.unpack_nvq(blob))

    def nepq(out, K):
        t = synth.nepq_random(rng, "NEPQ1-S", 1, out, K, 16)
        dtype, blob = O.pack_tensor(t)
        return dtype, blob, lambda: O.dequantize_nepq(O.unpack_nepq(blob)).reshape(out, K)

    layer = [("qkv", nepq(6144, 4096)), ("o", nint(4096, 4096, 3, 24, 5)), ("gate", nvq(12288, 4096)),
             ("up", nint(12288, 4096, 5, 28, 7)), ("down", nint(4096, 12288, 3, 24, 5)),
             ("down/NEPQ1-S", nepq(4096, 12288)), ("down/NINT5", nint(4096, 12288, 5, 28, 7)),
             ("down/NVQ3J-512", nvq(4096, 12288))]
    xs = {K: _bf16(rng.standard_normal((16, K))) for K in (4096, 12288)}
    for name, (dtype, blob, dequant) in layer:
        lin = R.load_quant_linear(dtype, blob)
        deq = dequant()
        assert _bit_equal(lin.dequantize().cpu().numpy(), deq), name
        x = xs[lin.neuron_len]
        ref = O.linear_forward_f64(deq, x.float().numpy())
        assert 0.05 < float(np.sqrt(np.mean(ref * ref))) < 20.0, name   # of order one: the absolute bound means something
        for M in (1, 16):
            _close(lin(x[:M].cuda()).cpu().numpy(), ref[:M], f"C5 {name} {dtype} M={M}")
