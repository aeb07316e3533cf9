"""GPU parity of the MoE path (top-k, expert map, grouped matmul, FFN) against the oracle."""
import numpy as np
import pytest

import synth
from conftest import ABS_TOL, REL_TOL, rel_l2
from oracle import mfq_oracle as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _topk(logits, k, **kw):
    from tyloquant_amd.runtime_moe import moe_topk
    ids, w = moe_topk(torch.from_numpy(logits).cuda(), k, **kw)
    return ids.cpu().numpy(), w.cpu().numpy()


@pytest.mark.parametrize("T,E,k", [(9, 64, 6), (1, 256, 8), (5, 128, 8), (33, 300, 16), (3, 8, 8), (4, 701, 9), (2, 1024, 8),
                                   (3, 1500, 8)])
def test_topk_modes_match_oracle(T, E, k):
    rng = np.random.default_rng(71 + T)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    bias = (rng.standard_normal(E) * 0.1).astype(np.float32)
    for kw in ({}, {"delayed_softmax": True}, {"normalize": True}, {"use_sigmoid": True, "normalize": True},
               {"use_sqrt_softplus": True, "normalize": True, "scale": 2.5}):
        ids, w = _topk(logits, k, **kw)
        rids, rw = O.moe_topk(logits, k, **kw)
        assert np.array_equal(ids, rids), kw
        np.testing.assert_allclose(w, rw, rtol=2e-6, atol=2e-7)
    from tyloquant_amd.runtime_moe import moe_topk
    ids, w = moe_topk(torch.from_numpy(logits).cuda(), k, use_sigmoid=True, bias=torch.from_numpy(bias).cuda())
    rids, rw = O.moe_topk(logits, k, use_sigmoid=True, bias=bias)
    assert np.array_equal(ids.cpu().numpy(), rids)
    np.testing.assert_allclose(w.cpu().numpy(), rw, rtol=2e-6, atol=2e-7)


def test_topk_ties_and_nan():
    logits = np.zeros((2, 16), dtype=np.float32)
    logits[1, 3] = np.nan
    logits[1, 7] = 1.0
    ids, w = _topk(logits, 4, delayed_softmax=True)
    assert ids[0].tolist() == [0, 1, 2, 3]            # ties -> lower expert id
    assert ids[1].tolist() == [7, 0, 1, 2]            # NaN sinks to -FLT_MAX
    rids, rw = O.moe_topk(logits, 4, delayed_softmax=True)
    assert np.array_equal(ids, rids)
    np.testing.assert_allclose(w, rw, rtol=2e-6, atol=2e-7)


@pytest.mark.parametrize("T,R,E,tile_m", [(17, 2, 5, 8), (64, 8, 256, 4), (300, 3, 40, 4), (9, 1, 2000, 8)])
def test_expert_map_invariants(T, R, E, tile_m):
    from tyloquant_amd.runtime_moe import build_expert_map
    rng = np.random.default_rng(991 + T)
    ids = rng.integers(0, E, (T, R)).astype(np.int32)
    ids[0, 0] = E + 5 if T > 9 else ids[0, 0]         # one out-of-range id is dropped
    dst, eb, tb, te, counts = [a.cpu().numpy() for a in build_expert_map(torch.from_numpy(ids).cuda(), E, tile_m)]
    rdst, reb, rtb, rte, rcounts = O.build_expert_map(ids, E, tile_m)
    assert np.array_equal(counts, rcounts) and np.array_equal(eb, reb) and np.array_equal(tb, rtb)
    assert np.array_equal(te[: rtb[-1]], rte)
    assert np.array_equal(dst[: reb[-1]], rdst)       # deterministic: ascending pair index inside an expert


def _moe(rng, E, out, K, bits, quantize=True):
    from tyloquant_amd.runtime_moe import NintMoeWeight
    t = synth.moe_random(rng, E, out, K, bits, quantize)
    blob = O.pack_nint_moe(t)
    return O.unpack_nint_moe(blob), NintMoeWeight.from_blob(blob)


@pytest.mark.parametrize("tokens", [1, 4, 13, 70])
def test_grouped_matmul_matches_reference_loop(tokens):
    from tyloquant_amd.runtime_moe import build_moe_route_plan
    rng = np.random.default_rng(10 + tokens)
    E, out, K, R = 10, 48, 88, 3
    bits = [(2, 4, 6, 8, 5, 3)[i % 6] for i in range(E)]
    t, w = _moe(rng, E, out, K, bits)
    dense = O.dequantize_expertwise(t)
    assert np.array_equal(w.dequantize().cpu().numpy().view(np.uint32), dense.view(np.uint32))
    scores = rng.standard_normal((tokens, E))
    ids = np.argsort(-scores, axis=1)[:, :R].astype(np.int32)
    x = torch.from_numpy((rng.standard_normal((tokens, K)) * 0.1).astype(np.float32)).to(torch.bfloat16)
    route = build_moe_route_plan(torch.from_numpy(ids).cuda(), E)
    got = w(x.cuda(), route).cpu().numpy()
    ref = O.moe_grouped_matmul(dense, x.float().numpy(), ids)
    assert rel_l2(got, ref) < REL_TOL and np.abs(got - ref).max() < ABS_TOL


@pytest.mark.parametrize("routed", [False, True])
def test_grouped_matmul_prefill_path_many_pairs_per_expert(routed):
    """At 24+ pairs per expert the paired cohorts run the prefill kernel (64 pairs of an expert per block), the
    NINT5-28 cohort stays on the streaming kernel; experts with 0, 1 and > 64 pairs, an invalid id, ragged K."""
    from tyloquant_amd.runtime_moe import build_moe_route_plan
    rng = np.random.default_rng(77)
    E, out, K, T, R = 6, 80, 776, 150, 2
    t, w = _moe(rng, E, out, K, [4, 3, 2, 5, 4, 3])
    dense = O.dequantize_expertwise(t)
    ids = rng.choice(5, size=(T, R), p=[0.5, 0.2, 0.15, 0.1, 0.05]).astype(np.int32)   # expert 5 unused
    ids[0, 0] = 5
    ids[7, 1] = 99
    shape = (T, R, K) if routed else (T, K)
    x = torch.from_numpy((rng.standard_normal(shape) * 0.1).astype(np.float32)).to(torch.bfloat16)
    route = build_moe_route_plan(torch.from_numpy(ids).cuda(), E)
    got = w(x.cuda(), route).cpu().numpy()
    ref = O.moe_grouped_matmul(dense, x.float().numpy(), ids)
    assert rel_l2(got, ref) < REL_TOL and np.abs(got - ref).max() < ABS_TOL
    assert np.all(got[7, 1] == 0)


def test_grouped_matmul_without_workspace_keeps_the_streaming_kernels():
    """The plain entry point (no workspace) runs mapped calls on the streaming kernels; same result as the prefill path."""
    import ctypes as C
    from tyloquant_amd import _lib as L
    from tyloquant_amd.runtime_moe import build_moe_route_plan
    rng = np.random.default_rng(78)
    E, out, K, T, R = 6, 48, 512, 40, 2
    t, w = _moe(rng, E, out, K, [4, 3, 2, 5, 4, 3])
    ids = rng.integers(0, E, (T, R)).astype(np.int32)
    x = torch.from_numpy((rng.standard_normal((T, K)) * 0.1).astype(np.float32)).to(torch.bfloat16).cuda()
    route = build_moe_route_plan(torch.from_numpy(ids).cuda(), E)
    with_ws = w(x, route)
    plain = torch.empty_like(with_ws)
    p = lambda t_: C.c_void_p(t_.data_ptr())
    L.check(L.lib().mfq_hip_moe_grouped_matmul(
        w._pool_array, len(w.pools), p(w.expert_pool), p(w.expert_local), E, out, K, p(x), L.X_BF16, K, 0, p(route.ids), T, R,
        p(route.ids_dst), p(route.expert_bounds), p(route.tile_bounds), p(route.tile_experts), p(plain), out, None))
    torch.cuda.synchronize()
    ref = O.moe_grouped_matmul(O.dequantize_expertwise(t), x.float().cpu().numpy(), ids)
    for got in (with_ws.cpu().numpy(), plain.cpu().numpy()):
        assert rel_l2(got, ref) < REL_TOL and np.abs(got - ref).max() < ABS_TOL


def test_grouped_matmul_routed_input_and_invalid_expert():
    from tyloquant_amd.runtime_moe import build_moe_route_plan
    rng = np.random.default_rng(44)
    E, out, K, T, R = 6, 16, 64, 17, 2
    t, w = _moe(rng, E, out, K, [4, 3, 4, 2, 3, 5])
    dense = O.dequantize_expertwise(t)
    ids = rng.integers(0, E, (T, R)).astype(np.int32)
    ids[3, 1] = 99                                     # invalid id -> zero row, not garbage
    x = torch.from_numpy((rng.standard_normal((T, R, K)) * 0.1).astype(np.float32)).to(torch.float16)
    for sub in (slice(0, T), slice(0, 4)):             # mapped (T > 8) and unmapped paths
        route = build_moe_route_plan(torch.from_numpy(ids[sub]).cuda(), E)
        got = w(x[sub].cuda(), route).cpu().numpy()
        ref = O.moe_grouped_matmul(dense, x[sub].float().numpy(), ids[sub])
        assert rel_l2(got, ref) < REL_TOL and np.abs(got - ref).max() < ABS_TOL
        assert np.all(got[3, 1] == 0)


@pytest.mark.parametrize("T", [1, 5, 64])
def test_moe_ffn_forward_matches_oracle(T):
    """Scaled-down BASELINE config 4: mixed 2/3/4/5-bit experts, top-8 delayed softmax, ungated shared expert."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_moe import nint_moe_ffn_forward
    rng = np.random.default_rng(400 + T)
    E, H, W, k = 32, 256, 128, 8
    bits = rng.choice([2, 3, 4, 5], size=E, p=[0.1, 0.4, 0.4, 0.1])
    tg, gu = _moe(rng, E, 2 * W, H, bits)
    td, dn = _moe(rng, E, H, W, bits)
    sg = O.quantize_nint((rng.standard_normal((2 * W, H)) * 0.02).astype(np.float32), 4, 24, 6)
    sd = O.quantize_nint((rng.standard_normal((H, W)) * 0.02).astype(np.float32), 4, 24, 6)
    shared = (R.load_quant_linear("NINT4", O.pack_nint(sg)).weight, R.load_quant_linear("NINT4", O.pack_nint(sd)).weight)
    x = torch.from_numpy(rng.standard_normal((T, H)).astype(np.float32)).to(torch.bfloat16)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    out, ids, wts = nint_moe_ffn_forward(gu, dn, x.cuda(), torch.from_numpy(logits).cuda(), k, delayed_softmax=True,
                                         shared=shared)
    ref, rids, rw = O.moe_ffn(O.dequantize_expertwise(tg), O.dequantize_expertwise(td), x.float().numpy(), logits, k,
                              shared=(O.dequantize_nint(sg), O.dequantize_nint(sd)), delayed_softmax=True)
    assert np.array_equal(ids.cpu().numpy(), rids)
    got = out.cpu().numpy()
    assert rel_l2(got, ref) < REL_TOL, rel_l2(got, ref)
    assert np.abs(got - ref).max() < ABS_TOL


@pytest.mark.parametrize("T,H,W", [(1, 256, 128), (3, 256, 128), (2, 8192, 64)])
def test_decode_matmul_matches_the_separate_calls(T, H, W):
    """The one-launch decode form (routes + shared tensor, fused SwiGLU) against grouped matmul + swiglu + dense matmul:
    the same values up to the order of the fp32 sums over K.  H = 8192 gives the 2-bit cohort 32 steps: more than
    three items per wave, the variant with a prefetch ring."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_moe import build_moe_route_plan, moe_swiglu
    rng = np.random.default_rng(900 + T + H)
    E, k = 12, 4
    bits = [(2, 3, 4, 5)[i % 4] for i in range(E)]
    _, gu = _moe(rng, E, 2 * W, H, bits)
    _, dn = _moe(rng, E, H, W, bits)
    sg = O.quantize_nint((rng.standard_normal((2 * W, H)) * 0.02).astype(np.float32), 4, 24, 6)
    sd = O.quantize_nint((rng.standard_normal((H, W)) * 0.02).astype(np.float32), 5, 28, 6)
    sgu = R.load_quant_linear("NINT4", O.pack_nint(sg)).weight
    sdn = R.load_quant_linear("NINT5", O.pack_nint(sd)).weight
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    ids[0, 1] = E + 3                                  # invalid id -> zero row
    ids_d = torch.from_numpy(ids).cuda()
    route = build_moe_route_plan(ids_d, E)

    def close(got, want, tol):
        got, want = got.float().cpu().numpy(), want.float().cpu().numpy()
        assert rel_l2(got, want) < tol, rel_l2(got, want)

    for dtype in (torch.bfloat16, torch.float16):
        x = torch.from_numpy(rng.standard_normal((T, H)).astype(np.float32)).to(dtype).cuda()
        assert gu.decode_capable(sgu) and dn.decode_capable(sdn)
        hid = gu.forward_decode(x, ids_d, sgu, swiglu=True)
        want = torch.cat([moe_swiglu(gu(x, route)).reshape(T * k, W), moe_swiglu(R.nint_matmul(sgu, x))])
        close(hid, want, 1e-3)                         # fp16 outputs: half an ulp is 5e-4
        assert torch.all(hid[1] == 0)
        from tyloquant_amd.runtime_moe import moe_geglu
        hid_g = gu.forward_decode(x, ids_d, sgu, swiglu="gelu")   # the same launch with the GELU gate
        want_g = torch.cat([moe_geglu(gu(x, route)).reshape(T * k, W), moe_geglu(R.nint_matmul(sgu, x))])
        close(hid_g, want_g, 1e-3)
        gu_np = gu(x, route).reshape(T * k, 2 * W).cpu().numpy()
        assert rel_l2(moe_geglu(gu(x, route)).reshape(T * k, W).float().cpu().numpy(), O.moe_geglu(gu_np)) < 1e-3
        out = dn.forward_decode(hid, ids_d, sdn, routed=True)
        want = torch.cat([dn(hid[: T * k].reshape(T, k, W), route).reshape(T * k, H), R.nint_matmul(sdn, hid[T * k:])])
        close(out, want, 1e-5)
        plain = gu.forward_decode(x, ids_d)            # no shared tensor, no SwiGLU: the grouped matmul itself
        assert torch.equal(plain.view(torch.int32), gu(x, route).reshape(T * k, 2 * W).view(torch.int32))


def test_decode_matmul_rejects_what_it_cannot_run():
    """Cohorts without a batch-1 unit (6-bit experts) and a shared tensor of another height are refused with a message,
    and the FFN forward then takes the separate calls."""
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_moe import nint_moe_ffn_forward
    rng = np.random.default_rng(77)
    E, H, W, k = 6, 96, 48, 2
    _, gu = _moe(rng, E, 2 * W, H, [4, 6, 3, 4, 6, 2])
    _, dn = _moe(rng, E, H, W, [4, 6, 3, 4, 6, 2])
    ids = torch.from_numpy(np.array([[0, 2]], dtype=np.int32)).cuda()
    x = torch.from_numpy(rng.standard_normal((1, H)).astype(np.float32)).to(torch.bfloat16).cuda()
    assert not gu.decode_capable()
    with pytest.raises(RuntimeError, match="no batch-1 kernel"):
        gu.forward_decode(x, ids)
    tg, gu4 = _moe(rng, E, 2 * W, H, [4, 3, 3, 4, 2, 2])
    td, dn4 = _moe(rng, E, H, W, [4, 3, 3, 4, 2, 2])
    other = R.load_quant_linear("NINT4", O.pack_nint(O.quantize_nint(
        (rng.standard_normal((W, H)) * 0.02).astype(np.float32), 4, 24, 6))).weight
    assert not gu4.decode_capable(other)
    with pytest.raises(RuntimeError, match="shared tensor has"):
        gu4.forward_decode(x, ids, other)
    logits = rng.standard_normal((1, E)).astype(np.float32)
    out, _, _ = nint_moe_ffn_forward(gu, dn, x, torch.from_numpy(logits).cuda(), k, delayed_softmax=True)
    assert out.shape == (1, H) and bool(torch.isfinite(out).all())


def test_moe_errors():
    from tyloquant_amd.runtime_moe import NintMoeWeight, build_moe_route_plan
    rng = np.random.default_rng(2)
    t = synth.moe_random(rng, 4, 16, 48, [4, 4, 3, 3])
    blob = O.pack_nint_moe(t)
    with pytest.raises(ValueError, match="invalid NINTM magic"):
        NintMoeWeight.from_blob(b"NIM9" + blob[4:])
    with pytest.raises(ValueError, match="invalid NINTM tail"):
        NintMoeWeight.from_blob(blob + b"\0")
    with pytest.raises(RuntimeError, match="int32"):
        build_moe_route_plan(torch.zeros((2, 2), dtype=torch.int64).cuda(), 4)


def test_expert_cache_keeps_a_working_set_resident():
    """Experts in pinned host memory, a GPU arena of a few slots per cohort: whatever the route, the cached tensor gives
    bit for bit what the fully resident tensor gives (same kernels, same bytes), through decode-size and mapped calls;
    slots are reused least-recently-used first, experts already resident cost nothing, and a route that needs more
    experts of a cohort than its arena holds is refused."""
    from tyloquant_amd.runtime_moe import MoeExpertCache, NintMoeWeight, build_moe_route_plan
    rng = np.random.default_rng(2025)
    E, out, K, R = 12, 32, 96, 2
    bits = [4, 3, 4, 3, 4, 3, 4, 3, 4, 3, 4, 3]           # two cohorts of six experts
    t = synth.moe_random(rng, E, out, K, bits, quantize=True)
    blob = O.pack_nint_moe(t)
    full = NintMoeWeight.from_blob(blob)
    probe = MoeExpertCache(1 << 30)
    per_slot = sum(c.slot_bytes for c in probe.register_source(blob).cohorts)
    cache = MoeExpertCache(3 * per_slot + 64)              # three slots per cohort
    src = cache.register_source(blob, minimum_slots=2)
    with pytest.raises(RuntimeError, match="finalized before inference"):
        cache.prepare(src, [0])
    cache.finalize()
    assert [len(c.free) for c in src.cohorts] == [3, 3] and cache.allocated_bytes <= 3 * per_slot + 2 * 4096
    with pytest.raises(RuntimeError, match="after cache finalization"):
        cache.register_source(blob)
    for step, T in enumerate([1, 2, 20, 1, 3, 20, 2]):
        # experts 2k are 4-bit, 2k+1 are 3-bit: draw at most three of each cohort per call
        even = rng.choice(np.arange(0, E, 2), size=3, replace=False)
        odd = rng.choice(np.arange(1, E, 2), size=3, replace=False)
        ids = np.stack([np.array([rng.choice(even), rng.choice(odd)]) for _ in range(T)]).astype(np.int32)
        x = torch.from_numpy((rng.standard_normal((T, K)) * 0.1).astype(np.float32)).to(torch.bfloat16).cuda()
        route = build_moe_route_plan(torch.from_numpy(ids).cuda(), E)
        got = cache.forward(src, x, route)
        want = full(x, route)
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), (step, T)
    st = cache.stats
    sizes = [c.slot_bytes for c in src.cohorts]
    assert st["misses"] >= 6 and st["evictions"] > 0 and st["hits"] > 0
    assert st["misses"] * min(sizes) <= st["bytes"] <= st["misses"] * max(sizes)     # only missing experts travel
    resident = {int(src.cohorts[ci].expert_ids[l]) for ci in range(2) for l in src.cohorts[ci].slot_of}
    table = src.weight.expert_local.cpu().numpy()
    assert {e for e in range(E) if table[e] >= 0} == resident          # the device table says what is resident
    before = dict(st)
    cache.prepare(src, sorted(resident))                                # all hits: nothing moves
    assert st["bytes"] == before["bytes"] and st["launches"] == before["launches"]
    with pytest.raises(RuntimeError, match="its arena holds 3"):
        cache.prepare(src, [0, 2, 4, 6])


@pytest.mark.parametrize("routed", [False, True])
@pytest.mark.parametrize("activation,out_dtype", [(0, torch.float16), (1, torch.bfloat16)])
def test_grouped_glu_epilogue_matches_the_two_calls(routed, activation, out_dtype):
    """forward_glu (GLU in the epilogue of the mapped prefill kernels) against forward + moe_glu: the same 16-bit values
    but for a last-place flip where the fp32 product sits on a rounding boundary (at most 1 in 1000 values, one unit);
    experts with 0, 1, 15, 30, 45, 60, 70, 90 and 150 pairs (every tile count of the three kernel groups), an invalid id
    (zero row), W = 80 neurons (a partial neuron tile) and ragged K; and against the oracle's loop."""
    from tyloquant_amd.runtime_moe import build_moe_route_plan, moe_glu
    rng = np.random.default_rng(91)
    counts = [0, 1, 15, 30, 45, 60, 70, 90, 150, 33]
    E, W, K, R = len(counts), 80, 776, 2
    t, w = _moe(rng, E, 2 * W, K, [4, 3, 2, 5, 4, 3, 2, 5, 4, 3])
    flat = np.concatenate([np.full(c, e, dtype=np.int32) for e, c in enumerate(counts)])
    if len(flat) % R:
        flat = np.concatenate([flat, np.array([9], dtype=np.int32)])
    rng.shuffle(flat)
    ids = flat.reshape(-1, R)
    ids[3, 1] = 77                      # out of range: a zero row
    T = ids.shape[0]
    shape = (T, R, K) if routed else (T, K)
    x = torch.from_numpy((rng.standard_normal(shape) * 0.1).astype(np.float32)).to(torch.bfloat16).cuda()
    route = build_moe_route_plan(torch.from_numpy(ids).cuda(), E)
    assert route.ids_dst is not None
    fused = w.forward_glu(x, route, activation, out_dtype)
    two = moe_glu(w(x, route), out_dtype, activation)
    assert fused.shape == (T, R, W) and fused.dtype == out_dtype
    ulp = (fused.view(torch.int16).int() - two.view(torch.int16).int()).abs()
    assert int(ulp.max()) <= 1 and float((ulp != 0).float().mean()) < 1e-3
    assert torch.all(fused[3, 1] == 0)
    dense = O.dequantize_expertwise(t)
    gu = O.moe_grouped_matmul(dense, x.float().cpu().numpy(), ids)
    g, u = gu[..., :W], gu[..., W:]
    if activation == 0:
        ref = g / (1.0 + np.exp(-g)) * u
    else:
        ref = 0.5 * g * (1.0 + np.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3))) * u
    got = fused.float().cpu().numpy()
    assert rel_l2(got, ref) < 5e-3 and np.abs(got - ref).max() < ABS_TOL


def test_mapped_path_with_hundreds_of_experts_and_skewed_routes():
    """200 experts (the chunk lists are built 64 experts at a time), top-4 of 600 tokens with a skewed router: a few
    experts receive several hundred pairs (several 128-pair chunks plus a remainder of every size class), most a
    handful, some none.  Every pair against the oracle's loop."""
    from tyloquant_amd.runtime_moe import build_moe_route_plan
    rng = np.random.default_rng(1234)
    E, out, K, T, R = 200, 48, 96, 600, 4
    bits = [(4, 3, 2, 5)[i % 4] for i in range(E)]
    t, w = _moe(rng, E, out, K, bits)
    p = rng.dirichlet(np.full(E, 0.08))
    ids = np.stack([rng.choice(E, size=R, replace=False, p=p) for _ in range(T)]).astype(np.int32)
    counts = np.bincount(ids.reshape(-1), minlength=E)
    assert counts.max() > 256 and (counts == 0).any() and ((counts > 0) & (counts <= 16)).any()
    x = torch.from_numpy((rng.standard_normal((T, K)) * 0.1).astype(np.float32)).to(torch.bfloat16)
    route = build_moe_route_plan(torch.from_numpy(ids).cuda(), E)
    got = w(x.cuda(), route).cpu().numpy()
    ref = O.moe_grouped_matmul(O.dequantize_expertwise(t), x.float().numpy(), ids)
    assert rel_l2(got, ref) < REL_TOL and np.abs(got - ref).max() < ABS_TOL
    fused = w.forward_glu(x.cuda(), route).float().cpu().numpy()
    g, u = ref[..., : out // 2], ref[..., out // 2:]
    assert rel_l2(fused, g / (1.0 + np.exp(-g)) * u) < 5e-3


def _mixed_family_moe(rng, out, K):
    """Nine experts in six cohorts: NINT4 (3 experts), NVQ3J-512 (2), NVQ2J read from its streams (1), NPQ0-S (1),
    NEPQ1-S (1), NEPQ0-S (1)."""
    def pool(ids, dtype, t):
        return O.MoePool(np.asarray(ids, dtype=np.int32), dtype, t)
    pools = [pool([0, 4, 8], "NINT4", synth.nint_random(rng, 3 * out, K, 4, 32, 6)),
             pool([1, 6], "NVQ3J-512", synth.nvq_jsc_random(rng, 2 * out, K, "d4_512", 2)),
             pool([2], "NVQ2J", synth.nvq_jsc_random(rng, out, K, "e8_256", 2)),
             pool([5], "NPQ0-S", synth.npq0_random(rng, "NPQ0-S", out, K)),
             pool([3], "NEPQ1-S", synth.nepq_random(rng, "NEPQ1-S", 1, out, K, 3)),
             pool([7], "NEPQ0-S", synth.nepq_random(rng, "NEPQ0-S", 1, out, K, 4))]
    return O.NintMoeTensor((9, out, K), pools)


def test_mixed_family_cohorts_in_one_tensor():
    """A NINTM tensor whose cohorts belong to different families: the NINT cohort on the grouped kernels, every other
    expert on its family's kernels through the host's per-expert walk.  Dequantized experts bit for bit, the routed
    product against the oracle's loop for a mapped batch, a decode-sized batch and routed (per-pair) inputs; a tensor
    without any NINT cohort; the residency cache declines such a tensor."""
    from tyloquant_amd.runtime_moe import MoeExpertCache, NintMoeWeight, build_moe_route_plan
    rng = np.random.default_rng(77)
    out, K, E, R = 32, 192, 9, 3
    t = _mixed_family_moe(rng, out, K)
    blob = O.pack_nint_moe(t)
    w = NintMoeWeight.from_blob(blob)
    assert len(w.pools) == 1 and [c.dtype for c in w.foreign] == ["NVQ3J-512", "NVQ2J", "NPQ0-S", "NEPQ1-S", "NEPQ0-S"]
    dense = O.dequantize_expertwise(t)
    assert np.array_equal(w.dequantize().cpu().numpy().view(np.uint32), dense.view(np.uint32))
    assert not w.decode_capable(None, 1, R)
    for T in (40, 2):
        ids = np.stack([rng.choice(E, size=R, replace=False) for _ in range(T)]).astype(np.int32)
        x = torch.from_numpy((rng.standard_normal((T, K)) * 0.1).astype(np.float32)).to(torch.bfloat16)
        route = build_moe_route_plan(torch.from_numpy(ids).cuda(), E)
        got = w(x.cuda(), route).cpu().numpy()
        ref = O.moe_grouped_matmul(dense, x.float().numpy(), ids)
        assert rel_l2(got, ref) < REL_TOL and np.abs(got - ref).max() < ABS_TOL
        xr = torch.from_numpy((rng.standard_normal((T, R, K)) * 0.1).astype(np.float32)).to(torch.bfloat16)
        got = w(xr.cuda(), route).cpu().numpy()
        ref = np.stack([np.stack([dense[ids[t_, r]] @ xr[t_, r].float().numpy() for r in range(R)]) for t_ in range(T)])
        assert rel_l2(got, ref) < REL_TOL
        h = w.forward_glu(x.cuda(), route).float().cpu().numpy()
        y = O.moe_grouped_matmul(dense, x.float().numpy(), ids)
        assert rel_l2(h, O.moe_swiglu(y)) < 5e-3
    # no NINT cohort at all; a NINT8-0 pool; a native MXFP4 pool (one [experts * out, K] tensor, its experts row ranges of it)
    only = O.NintMoeTensor((6, out, K), [O.MoePool(np.array([5], dtype=np.int32), "NINT8-0", O.quantize_nint8_zero(
                                             (rng.standard_normal((out, K)) * 0.02).astype(np.float32))),O.MoePool(np.array([2, 0], dtype=np.int32), "NVQ3J-512",
                                                   synth.nvq_jsc_random(rng, 2 * out, K, "d4_512", 2)),
                                         O.MoePool(np.array([1], dtype=np.int32), "NVQ1-S",
                                                   synth.nvq1_random(rng, "NVQ1-S", out, K)),
                                         O.MoePool(np.array([4, 3], dtype=np.int32), "MXFP4",
                                                   synth.mx_random(rng, "MXFP4", 2 * out, K, 120, 124))])
    w2 = NintMoeWeight.from_blob(O.pack_nint_moe(only))
    assert [c.dtype for c in w2.foreign] == ["NINT8-0", "NVQ3J-512", "NVQ1-S", "MXFP4"]
    d2 = O.dequantize_expertwise(only)
    assert np.array_equal(w2.dequantize().cpu().numpy().view(np.uint32), d2.view(np.uint32))
    for T in (20, 2):
        ids = np.stack([rng.choice(6, size=2, replace=False) for _ in range(T)]).astype(np.int32)
        x = torch.from_numpy((rng.standard_normal((T, K)) * 0.1).astype(np.float32)).to(torch.bfloat16)
        got = w2(x.cuda(), build_moe_route_plan(torch.from_numpy(ids).cuda(), 6)).cpu().numpy()
        ref = O.moe_grouped_matmul(d2, x.float().numpy(), ids)
        assert rel_l2(got, ref) < REL_TOL and np.abs(got - ref).max() < ABS_TOL * max(1.0, float(np.sqrt(np.mean(ref * ref))))
    bad = O.NintMoeTensor((1, 128, 128), [O.MoePool(np.array([0], dtype=np.int32), "MXFP8", synth.mx_random(rng, "MXFP8", 128, 128))])
    with pytest.raises(ValueError, match="NINTM supports native MXFP4 expert pools, got MXFP8"):
        NintMoeWeight.from_blob(O.pack_nint_moe(bad))
    with pytest.raises(NotImplementedError, match="NINT cohorts only"):
        MoeExpertCache(1 << 20).register_source(blob)


def test_mixed_family_decode_step_reads_the_routing_table_on_the_device():
    """A decode-sized batch on a tensor with NVQ, stream-NVQ, 1-bit and NEPQ cohorts takes one launch per cohort over all
    pairs (mfq_hip_*_gemv_pairs): the result agrees with the per-expert walk on the host; the whole call is captured
    into a HIP graph and replayed with other routing tables and activations written into the same device buffers --
    every replay equals the eager call, which only holds if nothing of the routing table is read by the host.  Ids
    outside the table give zero rows."""
    from tyloquant_amd.runtime_moe import ForeignCohort, MoeRoutePlan, NintMoeWeight, build_moe_route_plan
    rng = np.random.default_rng(78)
    out, K, E, R, T = 32, 192, 9, 3, 4
    t = _mixed_family_moe(rng, out, K)
    w = NintMoeWeight.from_blob(O.pack_nint_moe(t))
    dense = O.dequantize_expertwise(t)
    draws = []
    for i in range(3):
        ids = np.stack([rng.choice(E, size=R, replace=False) for _ in range(T)]).astype(np.int32)
        if i == 2:
            ids[0, 0], ids[1, 2] = -1, E + 5
        draws.append((ids, torch.from_numpy((rng.standard_normal((T, K)) * 0.1).astype(np.float32)).to(torch.bfloat16)))
    ids_d = torch.from_numpy(draws[0][0]).cuda()
    x_d = draws[0][1].cuda()
    route = build_moe_route_plan(ids_d, E)
    assert route.ids_dst is None                         # a decode step: no route map
    eager = w(x_d, route).clone()
    saved, ForeignCohort.PAIRS_MAX = ForeignCohort.PAIRS_MAX, 0
    try:
        walked = w(x_d, route).clone()                   # the host's walk over the experts
    finally:
        ForeignCohort.PAIRS_MAX = saved
    assert rel_l2(eager.cpu().numpy(), walked.cpu().numpy()) < REL_TOL    # other kernels, other fp16 roundings
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        y_g = w(x_d, route)
    for ids, x in draws:
        ids_d.copy_(torch.from_numpy(ids))
        x_d.copy_(x)
        want = w(x_d, route).clone()
        torch.cuda.synchronize()
        y_g.zero_()
        (y_g.sum() + 1).item()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_g, want)
        ok = (ids >= 0) & (ids < E)
        ref = np.zeros((T, R, out), np.float32)
        for t_ in range(T):
            for r in range(R):
                if ok[t_, r]:
                    ref[t_, r] = dense[ids[t_, r]] @ x[t_].float().numpy()
        got = want.cpu().numpy()
        assert rel_l2(got, ref) < REL_TOL and np.abs(got - ref).max() < ABS_TOL
        assert not got[~ok].any()
    # a tensor without any NINT cohort, with a NINT8-0 cohort and a native MXFP4 pool: the same, captured and replayed
    only = O.NintMoeTensor((6, out, K), [O.MoePool(np.array([5], dtype=np.int32), "NINT8-0", O.quantize_nint8_zero(
                                             (rng.standard_normal((out, K)) * 0.02).astype(np.float32))),
                                         O.MoePool(np.array([2, 0], dtype=np.int32), "NVQ3J-512",
                                                   synth.nvq_jsc_random(rng, 2 * out, K, "d4_512", 2)),
                                         O.MoePool(np.array([1], dtype=np.int32), "NVQ1-S", synth.nvq1_random(rng, "NVQ1-S", out, K)),
                                         O.MoePool(np.array([4, 3], dtype=np.int32), "MXFP4",
                                                   synth.mx_random(rng, "MXFP4", 2 * out, K, 120, 124))])
    w2 = NintMoeWeight.from_blob(O.pack_nint_moe(only))
    d2 = O.dequantize_expertwise(only)
    ids2 = torch.from_numpy(np.stack([rng.choice(6, size=2, replace=False) for _ in range(T)]).astype(np.int32)).cuda()
    route2 = build_moe_route_plan(ids2, 6)
    w2(x_d, route2)                                      # builds the cohorts' device tables
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g2):
        y2 = w2(x_d, route2)
    for _ in range(2):
        idn = np.stack([rng.choice(6, size=2, replace=False) for _ in range(T)]).astype(np.int32)
        ids2.copy_(torch.from_numpy(idn))
        g2.replay()
        torch.cuda.synchronize()
        ref = O.moe_grouped_matmul(d2, x_d.float().cpu().numpy(), idn)
        got = y2.cpu().numpy()
        assert rel_l2(got, ref) < REL_TOL and np.abs(got - ref).max() < ABS_TOL * max(1.0, float(np.sqrt(np.mean(ref * ref))))


@pytest.mark.parametrize("scale", [1e-6, 3e6])
def test_decode_pairs_take_bf16_rows_of_any_magnitude(scale):
    """The one-row kernels behind a decode step on cohorts of other families (NVQ, NEPQ1 and NINT8-0 rescale every bf16
    row by a power of two before the fp16 conversion; the stream families and MX multiply in fp32): rows 1e-6 and 3e6
    times an ordinary row come out with the relative accuracy of an ordinary one."""
    from tyloquant_amd.runtime_moe import NintMoeWeight, build_moe_route_plan
    rng = np.random.default_rng(79)
    out, K, E, R, T = 32, 192, 6, 2, 3
    def pool(ids, dtype, t):
        return O.MoePool(np.asarray(ids, dtype=np.int32), dtype, t)
    t = O.NintMoeTensor((E, out, K), [
        pool([0], "NINT8-0", O.quantize_nint8_zero((rng.standard_normal((out, K)) * 0.02).astype(np.float32))),
        pool([1, 2], "NVQ3J-512", synth.nvq_jsc_random(rng, 2 * out, K, "d4_512", 2)),
        pool([3], "NEPQ1-S", synth.nepq_random(rng, "NEPQ1-S", 1, out, K, 3)),
        pool([4], "NVQ1-S", synth.nvq1_random(rng, "NVQ1-S", out, K)),
        pool([5], "MXFP4", synth.mx_random(rng, "MXFP4", out, K, 120, 124))])
    w = NintMoeWeight.from_blob(O.pack_nint_moe(t))
    dense = O.dequantize_expertwise(t)
    ids = np.array([[0, 1], [2, 3], [4, 5]], dtype=np.int32)
    x = torch.from_numpy((rng.standard_normal((T, K)) * scale).astype(np.float32)).to(torch.bfloat16)
    got = w(x.cuda(), build_moe_route_plan(torch.from_numpy(ids).cuda(), E)).cpu().numpy()
    ref = O.moe_grouped_matmul(dense, x.float().numpy(), ids)
    for t_ in range(T):
        for r in range(R):
            assert rel_l2(got[t_, r], ref[t_, r]) < REL_TOL, (t_, r, rel_l2(got[t_, r], ref[t_, r]))


def test_expert_overlay_cohorts_take_over_their_experts():
    """An NINTMD expert overlay (magic NID2: cohorts for some experts only) on a mixed-family NINTM tensor: the overlay's
    cohorts are appended and own the experts they list -- here a NINT3 cohort takes a NINT4 expert and an NVQ expert, an
    NEPQ1-S cohort a stream-NVQ expert.  Dequantized experts bit for bit against the oracle's overlaid tensor; a decode
    step (one launch per cohort) and a mapped batch against the oracle's loop; the delta alone is not a tensor."""
    from tyloquant_amd.runtime_moe import NintMoeWeight, build_moe_route_plan
    rng = np.random.default_rng(80)
    out, K, E, R = 32, 192, 9, 3
    base = _mixed_family_moe(rng, out, K)
    def pool(ids, dtype, t):
        return O.MoePool(np.asarray(ids, dtype=np.int32), dtype, t)
    delta = O.NintMoeTensor((E, out, K), [pool([4, 1], "NINT3", synth.nint_random(rng, 2 * out, K, 3, 24, 5)),
                                          pool([2], "NEPQ1-S", synth.nepq_random(rng, "NEPQ1-S", 1, out, K, 3))])
    blob, dblob = O.pack_nint_moe(base), O.pack_nint_moe(delta, delta=True)
    assert dblob[:4] == b"NID2"
    with pytest.raises(ValueError, match="delta cannot be loaded as a full tensor"):
        NintMoeWeight.from_blob(dblob)
    with pytest.raises(ValueError, match="delta cannot be loaded as a full tensor"):
        O.unpack_nint_moe(dblob)
    back = O.unpack_nint_moe(dblob, allow_partial=True)
    assert [p.dtype for p in back.pools] == ["NINT3", "NEPQ1-S"] and back.pools[0].expert_ids.tolist() == [4, 1]
    w = NintMoeWeight.from_blob(blob, expert_overlay=dblob)
    over = O.apply_expert_overlay(base, delta)
    dense = O.dequantize_expertwise(over)
    assert not np.array_equal(dense, O.dequantize_expertwise(base))
    assert np.array_equal(w.dequantize().cpu().numpy().view(np.uint32), dense.view(np.uint32))
    assert w.expert_bits[4] == 3 and w.expert_bits[1] == 3 and w.expert_bits[0] == 4
    with pytest.raises(ValueError, match="expert overlay shape mismatch"):
        NintMoeWeight.from_blob(blob, expert_overlay=O.pack_nint_moe(O.NintMoeTensor((E, out, 2 * K), [pool(
            [0], "NINT4", synth.nint_random(rng, out, 2 * K, 4, 32, 6))]), delta=True))
    for T in (40, 2):
        ids = np.stack([rng.choice(E, size=R, replace=False) for _ in range(T)]).astype(np.int32)
        ids[0] = [4, 1, 2]                                # the three experts that changed hands
        x = torch.from_numpy((rng.standard_normal((T, K)) * 0.1).astype(np.float32)).to(torch.bfloat16)
        got = w(x.cuda(), build_moe_route_plan(torch.from_numpy(ids).cuda(), E)).cpu().numpy()
        ref = O.moe_grouped_matmul(dense, x.float().numpy(), ids)
        assert rel_l2(got, ref) < REL_TOL and np.abs(got - ref).max() < ABS_TOL
