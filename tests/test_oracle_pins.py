"""Pins of the CPU oracle against what the reference fixes without running it: its own constants and
known-answer identities, closed forms, brute force on tiny inputs, library routines, and the golden
vectors written from the reference's numpy quantizer (tests/golden/make_nint_quant_vectors.py)."""
import hashlib
import math
from pathlib import Path

import numpy as np
import pytest

import synth
from oracle import mfq_oracle as O

GOLD = Path(__file__).parent / "golden"
DATA = Path(__file__).resolve().parents[1] / "tyloquant_amd" / "data"


# ---- bit streams ---------------------------------------------------------------------------------
def _bigint_stream(values, bits):
    acc = 0
    for i, v in enumerate(values):
        acc |= int(v) << (i * bits)
    n = (len(values) * bits + 7) // 8
    return acc.to_bytes(n, "little")


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8, 9, 11])
def test_pack_bits_is_a_little_endian_bit_stream(bits):
    rng = np.random.default_rng(bits)
    for n in (1, 7, 8, 24, 257):
        v = rng.integers(0, 1 << bits, n)
        blob = O.pack_bits(v, bits)
        assert blob == _bigint_stream(v, bits)          # value i sits at bit i*bits
        back, off = O.unpack_bits(b"\xff" * 3 + blob, 3, n, bits)
        assert off == 3 + len(blob) and np.array_equal(back, v)


def test_three_bit_stream_matches_the_3_byte_8_value_formula():
    """The explicit unpack of mfq/kernels/cuda/nint_matmul.cu:8219-8231: 8 codes per 3 bytes."""
    v = np.arange(24) % 8
    b = O.pack_bits(v, 3)
    for t in range(3):
        w = b[3 * t] | (b[3 * t + 1] << 8) | (b[3 * t + 2] << 16)
        assert [(w >> (3 * i)) & 7 for i in range(8)] == v[8 * t: 8 * t + 8].tolist()
    assert O.pack_bits([0x3, 0xA], 4) == bytes([0xA3])   # 4-bit: low nibble first (io.py:150-155)


# ---- NINT ------------------------------------------------------------------------------------------
def test_nint_payload_sizes_match_the_reference_identities():
    # tests/test_formats/test_nint.py:18-20, :80 (theoretical bpw) and the BASELINE config sizes
    assert abs((4 + 32 / 5120 + 12 / 24) - (4 + 32.0 / 5120 + 2.0 * 6 / 24)) < 1e-12
    assert O.nint_payload_nbytes(4096, 4096, 3, 24, 5) == 7195648
    assert O.nint_payload_nbytes(12288, 4096, 4, 32, 6) == 27574272
    assert O.nint_payload_nbytes(4096, 12288, 4, 32, 6) == 27541504
    # tests/test_formats/test_io.py:102-107: real payload < 4.55 bpw at 128 x 5120 NINT4(4,24,6)
    t = synth.nint_random(np.random.default_rng(0), 128, 5120, 4, 24, 6)
    assert 8 * len(O.pack_nint(t)) / (128 * 5120) < 4.55
    rng = np.random.default_rng(1)
    for (out, K, bits, gs, sb) in [(8, 96, 4, 24, 6), (17, 257, 3, 24, 5), (5, 100, 5, 28, 7), (3, 73, 2, 16, 5)]:
        t = synth.nint_random(rng, out, K, bits, gs, sb)
        blob = O.pack_nint(t)
        hdr = 14 + 4 + 16 + 8
        assert len(blob) - hdr == O.nint_payload_nbytes(out, K, bits, gs, sb)
        u = O.unpack_nint(blob)
        for f in ("q", "sub_scale", "sub_min", "neuron_scale", "neuron_min"):
            assert np.array_equal(getattr(u, f), getattr(t, f)), f


def test_nint_legacy_tail_and_invalid_tail():
    t = synth.nint_random(np.random.default_rng(2), 8, 96, 4, 24, 6)
    blob = O.pack_nint(t)
    head = blob[: 14 + 4 + 16 + 8 + 32]
    legacy = head + t.sub_scale.tobytes() + t.sub_min.tobytes() + t.q.tobytes()
    u = O.unpack_nint(legacy)
    assert np.array_equal(u.q, t.q) and np.array_equal(u.sub_min, t.sub_min)
    with pytest.raises(ValueError, match="invalid NINT blob tail"):
        O.unpack_nint(blob + b"\0")


def test_nint_dequant_is_four_roundings_brute_force():
    """All (ss, sm, q) for one f16 anchor pair, against exact arithmetic in fp64 rounded to fp32 after
    each of the four operations (fp64 holds every intermediate exactly)."""
    # anchors with full 11-bit significands, so that d_eff * q needs more than 24 bits
    ns, nm = (np.float32(np.array([b], dtype=np.uint16).view(np.float16)[0]) for b in (0x15E3, 0x21DF))
    ssv, smv = np.arange(0, 256, 3), np.arange(0, 256, 37)
    ss, sm = [a.reshape(-1) for a in np.meshgrid(ssv, smv, indexing="ij")]
    n = ss.size
    q = np.tile(np.arange(256, dtype=np.uint8), (n, 1, 1))                    # every 8-bit code in every group
    t = O.NintTensor(8, 256, 8, (n, 256), 0, 256, q, np.full(n, ns), np.full(n, nm),
                     ss.reshape(n, 1).astype(np.uint8), sm.reshape(n, 1).astype(np.uint8))
    got = O.dequantize_nint(t)
    d = np.float32(np.float64(ns) * ss).astype(np.float64)[:, None]
    m = np.float32(np.float64(nm) * sm).astype(np.float64)[:, None]
    qf = np.arange(256, dtype=np.float64)[None, :]
    want = np.float32(np.float32(d * qf).astype(np.float64) - m)
    assert np.array_equal(got, want)
    fused = np.float32(d * qf - m)                         # what an FMA would give: differs somewhere
    assert np.any(fused != want)
    # special cases: q = 0 or ss = 0 give exactly -m_eff
    assert np.array_equal(got[:, 0], -np.float32(m[:, 0]))
    assert np.array_equal(got[ss == 0], np.broadcast_to(-np.float32(m[ss == 0]), (int((ss == 0).sum()), 256)))


def test_nint_quantizer_matches_reference_golden_vectors():
    g = np.load(GOLD / "nint_quant_vectors.npz")
    keys = sorted({n.split("_")[0] for n in g.files})
    assert len(keys) == 8
    for k in keys:
        _, rows, K, bits, gs, sb = (int(v) for v in g[k + "_meta"])
        t = O.quantize_nint(g[k + "_W"], bits, gs, sb)
        assert np.array_equal(t.q, g[k + "_q"]), k
        assert np.array_equal(t.sub_scale, g[k + "_ss"]) and np.array_equal(t.sub_min, g[k + "_sm"]), k
        assert np.array_equal(t.neuron_scale, g[k + "_ns"]) and np.array_equal(t.neuron_min, g[k + "_nm"]), k
        assert np.array_equal(O.dequantize_nint(t), g[k + "_deq"]), k
        back = O.unpack_nint(O.pack_nint(t))
        assert np.array_equal(O.dequantize_nint(back), g[k + "_deq"]), k


def test_nint_quantizer_snr_properties():
    """tests/test_formats/test_nint.py:48-55 (SNR > 18 dB at NINT4) and test_nint_quant.py:31-38 (> 20 dB)."""
    rng = np.random.default_rng(0)
    W = (rng.standard_normal((32, 1024)) * 0.02).astype(np.float32)
    snr = {}
    for bits, gs, sb in [(3, 24, 5), (4, 24, 6), (5, 28, 7)]:
        r = O.dequantize_nint(O.quantize_nint(W, bits, gs, sb))
        snr[bits] = 10 * math.log10(float((W ** 2).sum() / ((W - r) ** 2).sum()))
    assert snr[4] > 20 and snr[3] < snr[4] < snr[5]


# ---- NVQ ---------------------------------------------------------------------------------------------
def test_grid_tables_carry_the_reference_hashes():
    want = {"e8_256": "915952ebc4af8ddba8113583ca1316fc818843f7b825bbf1a25ae1c39bf0e16d",
            "d4_256": "c9678803c61b2210fbd8cbbb3f965a835409cd7d88a04d086d236261bd221d11",
            "d4_512": "353274c58dd7d8dc5ee960dc8fc54ff9164eaf2b49206b841cd49415cf393f81",
            "iq1s_2048": "e9ffebfc997ad6023063a667c0bf4eedd8ebf7f56b3da399cbc7d1b1f7ea52c6",
            "nvq1s_banks": "beb341195ce650979d2640b6a494652047d8a371ea0af66183fc5c9f38a5a37e"}
    for name, h in want.items():
        assert hashlib.sha256((DATA / f"{name}.bin").read_bytes()).hexdigest() == h
    # tests/test_formats/test_nvq.py:26-41: shapes, alphabets, uniqueness
    d4, d5, e8 = O.nvq_grid("d4_256"), O.nvq_grid("d4_512"), O.nvq_grid("e8_256")
    assert d4.shape == (256, 4) and d5.shape == (512, 4) and e8.shape == (256, 8)
    assert set(np.unique(d5)) <= set(range(1, 16, 2)) and set(np.unique(e8)) <= {1, 3, 5, 7}
    assert np.unique(d5, axis=0).shape[0] == 512 and np.unique(d4, axis=0).shape[0] == 256


def test_nvq_payload_identities():
    # tests/test_formats/test_nvq.py:44-50
    assert 8.0 * O.nvq_payload_nbytes("d4_512", 4096, 5120) / (4096 * 5120) == 3.2953125
    assert 8.0 * O.nvq_payload_nbytes("d4_256", 4096, 5120) / (4096 * 5120) == 3.0453125
    assert 8.0 * O.nvq_payload_nbytes("e8_256", 4096, 5120) / (4096 * 5120) == 2.0453125
    assert O.nvq_payload_nbytes("d4_512", 17408, 5120) == 36713472
    assert O.nvq_payload_nbytes("d4_512", 5120, 17408) == 36684800
    # tensor-contiguous 9-bit index stream (tests/test_nvq_kernels_cuda.py:410-449) and JSC accounting
    t = synth.nvq_jsc_random(np.random.default_rng(3), 24, 80, "d4_512", 2)
    blob = O.pack_nvq_jsc(t)
    assert len(O.pack_bits(t.indices, 9)) == (24 * 20 * 9 + 7) // 8
    assert len(blob) == 20 + 16 + 4 + 64 + 2 * 512 * 4 + O.nvq_payload_nbytes("d4_512", 24, 80)
    u = O.unpack_nvq(blob)
    assert np.array_equal(u.indices, t.indices) and np.array_equal(u.signs, t.signs) and np.array_equal(u.state, t.state)
    assert O.tensor_dtype(u) == "NVQ3J-512"
    with pytest.raises(ValueError):
        O.unpack_nvq(blob[:-1])


def test_nvq_sign_rule_is_even_parity():
    masks = np.arange(128, dtype=np.uint8).reshape(1, 128)
    s = O._nvq_signs(masks, 1024).reshape(128, 8)
    assert np.all((s < 0).sum(axis=1) % 2 == 0)          # an even number of negatives in every 8
    assert np.array_equal(s[:, :7] < 0, ((np.arange(128)[:, None] >> np.arange(7)) & 1).astype(bool))


def test_nvq_jsc_dequant_closed_form_on_a_hand_built_tensor():
    cb = np.zeros((2, 512, 4), dtype=np.int8)
    cb[0, 5] = [8, 24, 40, 56]
    cb[1, 5] = [16, 16, 16, 120]
    cb[0, 0] = cb[1, 0] = [1, 1, 1, 1]
    lut = np.linspace(0.5, 2.0, 16).astype(np.float16).astype(np.float32)
    t = O.NvqJscTensor("d4_512", (1, 24), 24, np.array([np.float32(np.float16(0.01))]), lut,
                       (np.arange(16) & 1).astype(np.uint8), np.array([[3]], dtype=np.uint8),
                       np.array([[5, 0, 0, 0, 0, 5]], dtype=np.uint16), np.array([[0b0000101, 0, 0b1000000]], dtype=np.uint8), cb)
    w = O.dequantize_nvq_jsc(O.unpack_nvq(O.pack_nvq_jsc(t)))[0]
    scale = np.float32(np.float32(np.float16(0.01)) * lut[3])      # state 3 -> bank 1
    # mask 0b0000101: elements 0 and 2 negative, parity even -> element 7 positive
    assert w[:8].tolist() == [-(np.float32(16) * scale), np.float32(16) * scale, -(np.float32(16) * scale),
                              np.float32(120) * scale, scale, scale, scale, scale]
    # mask 0b1000000: element 6 negative and, by parity, element 7 too; vector 5 = bank-1 entry 5
    assert w[20:].tolist() == [np.float32(16) * scale, np.float32(16) * scale, -(np.float32(16) * scale),
                               -(np.float32(120) * scale)]


def test_plain_nvq3_equals_jsc_with_analytic_tables():
    """Plain NVQ3 (integer sub-scale, built-in grid) is the one-bank JSC with lut[s] = s."""
    rng = np.random.default_rng(4)
    p = synth.nvq_plain_random(rng, 6, 100)
    j = O.NvqJscTensor("d4_256", p.shape, p.neuron_len, p.neuron_scale, np.arange(16, dtype=np.float32),
                       np.zeros(16, np.uint8), p.sub_scale, p.indices, p.signs, O.nvq_grid("d4_256")[None])
    assert np.array_equal(O.dequantize_nvq(p), O.dequantize_nvq_jsc(j))
    assert O.pack_jsc_tables(j.scale_lut, j.bank_for_state, j.codebooks)[3] == 1   # flagged analytic


# ---- NEPQ --------------------------------------------------------------------------------------------
def test_nepq_payload_size_and_round_trip():
    assert O.nepq_payload_nbytes("NEPQ1-S", 1, 12288, 4096, 0 + 1) - 2048 == 8944128     # 8.94 MB at the FFN shape
    rng = np.random.default_rng(5)
    for label, hdr in (("NEPQ1-S", 36), ("NEPQ1-L", 36)):
        t = synth.nepq_random(rng, label, 2, 16, 200, 3)
        blob = O.pack_nepq(t)
        assert len(blob) - hdr == O.nepq_payload_nbytes(label, 2, 16, 200, 3)
        u = O.unpack_nepq(blob)
        for f in ("state", "indices", "aux", "bank_ids", "table_payloads"):
            assert np.array_equal(getattr(u, f), getattr(t, f)), f
        with pytest.raises(ValueError, match="invalid NEPQ tail"):
            O.unpack_nepq(blob + b"\0")
    t.bank_ids[0, 0, 0] = 3
    with pytest.raises(ValueError, match="bank ID exceeds"):
        O.unpack_nepq(O.pack_nepq(t))


def test_ternary_table_digits_are_code_plus_one():
    codes = np.array([[-1, 0, 1, 1, 0, -1, 0, 1]], dtype=np.int8)
    packed = O.pack_ternary_table(codes)
    assert int.from_bytes(packed, "little") == sum((int(c) + 1) << (2 * i) for i, c in enumerate(codes[0]))
    assert np.array_equal(O.unpack_ternary_table(packed), codes)
    iq = O.unpack_ternary_table((DATA / "iq1s_2048.bin").read_bytes())
    assert iq.shape == (2048, 8) and set(np.unique(iq)) == {-1, 0, 1} and np.unique(iq, axis=0).shape[0] == 2048


def test_nepq_dequant_closed_form():
    """value = fl(anchor * state) * (code -/+ delta); the kernel's integer form (32c + 5d)/32 and (8c + d)/8
    (mfq/kernels/cuda/nvq_matmul.cu:199-219) is the same number."""
    rng = np.random.default_rng(6)
    for label, delta in (("NEPQ1-S", 5 / 32), ("NEPQ1-L", 1 / 8)):
        t = synth.nepq_random(rng, label, 1, 4, 96, 2)
        w = O.dequantize_nepq(O.unpack_nepq(O.pack_nepq(t)))[0]
        for row in range(4):
            for g in range(4):
                bank = t.bank_ids[0, row, 0]
                st, aux = int(t.state[0, row, g]), int(t.aux[0, row, g])
                scale = np.float32(t.neuron_scale[0, row] * np.float32(st))
                for v in range(3):
                    idx = int(t.indices[0, row, 3 * g + v])
                    tbl = t.table_payloads[bank].tobytes()
                    e = int.from_bytes(tbl[2 * idx + (1024 * aux if label == "NEPQ1-S" else 0):][:2], "little")
                    for i in range(8):
                        code = ((e >> (2 * i)) & 3) - 1
                        want = np.float32(scale * np.float32(code + (-delta if aux else delta)))
                        assert w[row, 24 * g + 8 * v + i] == want
                        num = (32 * code + (-5 if aux else 5)) if label == "NEPQ1-S" else (8 * code + (-1 if aux else 1))
                        assert np.float32(code + (-delta if aux else delta)) == np.float32(num / (32 if label == "NEPQ1-S" else 8))


# ---- NINTM / MFQ1 ------------------------------------------------------------------------------------
def test_nintm_round_trip_and_invariants(tmp_path):
    rng = np.random.default_rng(7)
    t = synth.moe_random(rng, 7, 16, 48, [4, 3, 4, 2, 5, 3, 4])
    blob = O.pack_nint_moe(t)
    u = O.unpack_nint_moe(blob)
    assert [p.dtype for p in u.pools] == ["NINT2", "NINT3", "NINT4", "NINT5"]
    assert sorted(np.concatenate([p.expert_ids for p in u.pools]).tolist()) == list(range(7))
    dense = O.dequantize_expertwise(u)
    for p in t.pools:
        assert np.array_equal(dense[p.expert_ids].reshape(-1, 48), O.dequantize_nint(p.tensor))
    with pytest.raises(ValueError, match="invalid NINTM tail"):
        O.unpack_nint_moe(blob + b"\0")
    bad = bytearray(blob)
    bad[20 + 24: 20 + 28] = (6).to_bytes(4, "little")    # repeat an expert id of another pool
    with pytest.raises(ValueError):
        O.unpack_nint_moe(bytes(bad))
    path = tmp_path / "t.mfq"
    O.mfq_file_write(path, {"moe": t, "lin": t.pools[0].tensor})
    back = O.mfq_file_read(path)
    assert back["moe"] == ("NINTM", blob) and back["lin"][0] == "NINT2"


# ---- routing -------------------------------------------------------------------------------------------
def test_topk_matches_torch():
    torch = pytest.importorskip("torch")
    g = torch.Generator().manual_seed(71)
    logits = torch.randn(9, 64, generator=g)
    ids, w = O.moe_topk(logits.numpy(), 6)
    ew, ei = torch.softmax(logits, dim=-1).topk(6, dim=-1)       # tests/test_moe_kernels_cuda.py:155-161
    assert np.array_equal(ids, ei.numpy().astype(np.int32))
    np.testing.assert_allclose(w, ew.numpy(), rtol=2e-6, atol=2e-7)
    logits = torch.randn(1, 256, generator=g)
    ids, w = O.moe_topk(logits.numpy(), 8, delayed_softmax=True)  # :164-171
    ev, ei = logits.topk(8, dim=-1)
    assert np.array_equal(ids, ei.numpy().astype(np.int32))
    np.testing.assert_allclose(w, torch.softmax(ev, dim=-1).numpy(), rtol=2e-6, atol=2e-7)
    # delayed softmax == softmax-then-normalize for softmax routing
    i2, w2 = O.moe_topk(logits.numpy(), 8, normalize=True)
    assert np.array_equal(i2, ids)
    np.testing.assert_allclose(w2, w, rtol=1e-5)
    ids, w = O.moe_topk(logits.numpy(), 4, use_sigmoid=True, normalize=True, scale=2.0)
    sv, si = torch.sigmoid(logits).topk(4, dim=-1)
    assert np.array_equal(ids, si.numpy().astype(np.int32))
    np.testing.assert_allclose(w, (2.0 * sv / sv.sum(-1, keepdim=True)).numpy(), rtol=2e-6)


def test_expert_map_invariants():
    rng = np.random.default_rng(8)
    ids = rng.integers(0, 40, (300, 3)).astype(np.int32)
    ids[5, 1] = -1
    dst, eb, tb, te, counts = O.build_expert_map(ids, 40, 8)
    flat = ids.reshape(-1)
    assert counts.sum() == flat.size - 1 and eb[-1] == counts.sum()
    assert np.array_equal(eb[1:] - eb[:-1], counts) and np.array_equal(tb[1:] - tb[:-1], (counts + 7) // 8)
    assert sorted(dst.tolist()) == sorted(np.flatnonzero(flat >= 0).tolist())      # a permutation of the valid pairs
    for e in range(40):
        seg = dst[eb[e]: eb[e + 1]]
        assert np.all(flat[seg] == e) and np.all(np.diff(seg) > 0)
        assert np.all(te[tb[e]: tb[e + 1]] == e)


def test_moe_reference_loop_and_ffn_pieces():
    rng = np.random.default_rng(9)
    dense = rng.standard_normal((5, 7, 12)).astype(np.float32)
    x = rng.standard_normal((4, 12)).astype(np.float32)
    ids = rng.integers(0, 5, (4, 2)).astype(np.int32)
    out = O.moe_grouped_matmul(dense, x, ids)
    assert np.allclose(out, np.einsum("tk,trok->tro", x, dense[ids]), atol=1e-5)
    gu = rng.standard_normal((3, 8)).astype(np.float32)
    g, u = gu[:, :4].astype(np.float64), gu[:, 4:].astype(np.float64)
    assert np.allclose(O.moe_swiglu(gu), g / (1 + np.exp(-g)) * u, atol=1e-6)
    # input gate: silu(g) = g * sigmoid(g), sigmoid(0) = 1/2, sigmoid(-g) = 1 - sigmoid(g)
    xs, gs_ = rng.standard_normal(9), rng.standard_normal(9)
    assert np.allclose(O.input_mul(xs, gs_, 0), gs_ * O.input_mul(xs, gs_, 1), atol=1e-12)
    assert np.allclose(O.input_mul(xs, np.zeros(9), 1), 0.5 * xs) and np.all(O.input_mul(xs, np.zeros(9), 0) == 0)
    assert np.allclose(O.input_mul(xs, gs_, 1) + O.input_mul(xs, -gs_, 1), xs, atol=1e-12)
    # GEGLU: the tanh form against the erf form it approximates (max difference of the two GELUs is below 5e-4 over
    # the reals), exact zeros, and the large-|g| limits g and 0
    from math import erf
    gg = np.linspace(-6.0, 6.0, 241)
    geglu = O.moe_geglu(np.concatenate([gg, np.ones_like(gg)]).astype(np.float32)[None, :])[0]
    exact = np.array([0.5 * v * (1.0 + erf(v / np.sqrt(2.0))) for v in gg])
    assert np.abs(geglu - exact).max() < 5e-4 and geglu[120] == 0.0
    assert abs(geglu[-1] - 6.0) < 1e-6 and abs(geglu[0]) < 1e-6
    assert np.allclose(O.moe_geglu(np.array([[1.0, 3.0]], np.float32)), 3.0 * 0.8411919906082768, atol=1e-6)
    w = rng.random((4, 2)).astype(np.float32)
    assert np.allclose(O.moe_weighted_reduce(out, w), (out * w[..., None]).sum(1), atol=1e-5)


def test_bf16_rounding_is_nearest_even():
    torch = pytest.importorskip("torch")
    x = np.random.default_rng(10).standard_normal(4096).astype(np.float32) * 3
    assert np.array_equal(O.bf16_round(x), torch.from_numpy(x).to(torch.bfloat16).float().numpy())


def test_c_restatement_matches_the_numpy_oracle_bit_for_bit():
    """oracle/mfq_oracle_c.c (timed as the CPU baseline) against oracle/mfq_oracle.py and the golden vectors."""
    from oracle import c_oracle
    if not c_oracle.LIB.exists():
        pytest.skip("oracle/libmfq_oracle.so is not built (make -C oracle)")
    rng = np.random.default_rng(12)
    for spec in [(3, 24, 5), (4, 32, 6), (5, 28, 7), (8, 24, 8), (2, 16, 5)]:
        t = synth.nint_random(rng, 19, 203, *spec)
        blob = O.pack_nint(t)
        body = blob[14 + 4 + 16 + 8:]
        W = c_oracle.nint_dequant(body, spec[0], spec[2], spec[1], 19, 203)
        assert np.array_equal(W.view(np.uint32), O.dequantize_nint(t).view(np.uint32))
        part = c_oracle.nint_dequant_rows(body, spec[0], spec[2], spec[1], 19, 203, 5, 9)
        assert np.array_equal(part, W[5:14])
    g = np.load(GOLD / "nint_quant_vectors.npz")
    t = O.quantize_nint(g["c7_W"], 3, 24, 5)
    W = c_oracle.nint_dequant(O.pack_nint(t)[42:], 3, 5, 24, 16, 4096)
    assert np.array_equal(W, g["c7_deq"])
    x = rng.standard_normal((3, 4096)).astype(np.float32)
    y = c_oracle.matmul_nt(x, W)
    ref = O.linear_forward_f64(W, x)
    assert np.abs(y - ref).max() < 1e-4 * np.abs(ref).max()


def test_c_twins_of_the_nvq_and_nepq_dequantizers_and_the_moe_loop():
    """The C restatements bench.py times for configs 3, 4 and 5 against the numpy oracle: dequantizers bit for bit
    (ragged K, a second bank, indices that stop short of the last group), the MoE loop against the oracle's moe_ffn up to
    the summation order of its matrix products."""
    from oracle import c_oracle
    if not c_oracle.LIB.exists():
        pytest.skip("oracle/libmfq_oracle.so is not built (make -C oracle)")
    rng = np.random.default_rng(13)
    for out, K, cb, banks in ((7, 203, "d4_512", 2), (16, 384, "d4_512", 2), (5, 100, "d4_256", 1)):
        t = synth.nvq_jsc_random(rng, out, K, cb, banks)
        assert np.array_equal(c_oracle.nvq_jsc_dequant(t).view(np.uint32), O.dequantize_nvq_jsc(t).view(np.uint32))
    for E, out, K, banks in ((1, 9, 192, 3), (2, 5, 360, 2)):
        t = synth.nepq_random(rng, "NEPQ1-S", E, out, K, banks)
        tables = np.stack([np.stack([O.unpack_ternary_table(p.tobytes()[:1024]), O.unpack_ternary_table(p.tobytes()[1024:])])
                           for p in t.table_payloads])
        assert np.array_equal(c_oracle.nepq1s_dequant(t, tables).view(np.uint32), O.dequantize_nepq(t).view(np.uint32))
    E, H, W, T, k = 6, 96, 40, 5, 2
    gu = (rng.standard_normal((E, 2 * W, H)) * 0.1).astype(np.float32)
    dn = (rng.standard_normal((E, H, W)) * 0.1).astype(np.float32)
    x = rng.standard_normal((T, H)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    ref, ids, w = O.moe_ffn(gu, dn, x, logits, k)
    ids[0, 1] = -1                                            # a dropped route contributes nothing
    ref = O.moe_weighted_reduce(O.moe_grouped_matmul(dn, O.moe_swiglu(O.moe_grouped_matmul(gu, x, ids)), ids), w)
    hit = sorted(set(int(e) for e in ids.reshape(-1) if e >= 0))
    got = c_oracle.moe_ffn(x, ids, w, {e: gu[e] for e in hit}, {e: dn[e] for e in hit}, E)
    assert np.abs(got - ref).max() < 1e-5 * np.abs(ref).max()


def test_nint8_zero_is_ggml_q8_0():
    """NINT8-0 restates the textbook GGML Q8_0 block: fp16 scale = max|x| / 127, codes = round-half-away(x / scale),
    34 bytes per 32 weights (8.5 bit/weight).  Known answers on hand-made blocks, the byte layout written out by hand,
    round trips, and the reference's error messages (mfq/formats/nint8_zero.py)."""
    import struct
    blk = np.zeros((2, 64), np.float32)
    blk[0, :32] = np.arange(32) - 10.0            # max |x| = 21 -> scale 21/127, x = -10 -> code round(-60.476) = -60
    blk[0, 32:] = 0.0                             # all-zero block: scale 0, codes 0
    blk[1, 0], blk[1, 1], blk[1, 2] = 127.0, 63.5, -0.5   # scale exactly 1: ties round away from zero
    t = O.quantize_nint8_zero(blk)
    assert t.q.shape == (2, 2, 32) and t.scale.dtype == np.float16
    assert t.scale[0, 0] == np.float16(21.0 / 127.0) and t.scale[0, 1] == 0 and not t.q[0, 1].any()
    assert t.q[0, 0, 0] == -60 and t.q[0, 0, 31] == 127 and t.q[0, 0, 10] == 0
    assert t.scale[1, 0] == 1.0 and list(t.q[1, 0, :3]) == [127, 64, -1]
    # codes use the fp32 scale, the file keeps its fp16 rounding: the reconstruction is scale_f16 * code
    deq = O.dequantize_nint8_zero(t)
    assert deq[0, 31] == np.float32(np.float16(21.0 / 127.0)) * np.float32(127.0) and deq.dtype == np.float32
    blob = O.pack_nint8_zero(t)
    assert blob[:4] == b"NI80" and struct.unpack_from("<iiI", blob, 4) == (0, 64, 2)
    assert struct.unpack_from("<2q", blob, 16) == (2, 64) and struct.unpack_from("<II", blob, 32) == (2, 2)
    assert len(blob) == 40 + 4 * 34                                   # 8.5 bits per weight behind a 40-byte header
    first = blob[40:74]
    assert first[:2] == np.float16(21.0 / 127.0).tobytes() and first[2] == (-60) & 0xff and first[33] == 127
    back = O.unpack_nint8_zero(blob)
    assert np.array_equal(back.q, t.q) and np.array_equal(back.scale, t.scale) and back.shape == (2, 64)
    assert O.tensor_dtype(t) == "NINT8-0" and O.pack_tensor(t) == ("NINT8-0", blob)
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((7, 96)) * 0.02).astype(np.float32)
    tw = O.quantize_nint8_zero(w)
    err = np.abs(O.dequantize_nint8_zero(tw) - w).reshape(7, 3, 32)
    half_step = np.abs(w).reshape(7, 3, 32).max(-1) / 127.0 * 0.5
    # half a step, plus the fp16 rounding of the scale (2^-11) carried by a code of up to 127: 0.062 of a step
    assert np.all(err <= half_step[..., None] * (1.0 + 2 * 127 * 2.0 ** -11) + 1e-9)
    for bad, msg in ((blob[:10], "truncated NINT8-0 header"), (b"XXXX" + blob[4:], "invalid NINT8-0 magic"),
                     (blob[:-1], "invalid NINT8-0 block bytes"), (blob[:8] + struct.pack("<i", 48) + blob[12:], "multiple of 32")):
        with pytest.raises(ValueError, match=msg):
            O.unpack_nint8_zero(bad)
    with pytest.raises(ValueError, match="multiple of 32"):
        O.quantize_nint8_zero(np.zeros((3, 40), np.float32))
    from tyloquant_amd import formats as F
    h = F.parse_nint8_zero(blob)
    assert (h.out, h.ng, h.neuron_len, h.body_off, h.body_bytes) == (2, 2, 64, 40, 136)
    with pytest.raises(ValueError, match="invalid NINT8-0 block bytes"):
        F.parse_nint8_zero(blob + b"\0")


@pytest.mark.parametrize("case", ["mixed", "single"])
def test_expertwise_quantizer_matches_the_reference_fixture(case):
    """quantize_expertwise on the fixture's weights and profiles: the oracle's and the product's NIM2 bytes equal the
    bytes the reference packed (cohort order by first appearance of a precision, experts ascending inside a cohort, every
    pool the flat-cohort NINT quantization), and the oracle dequantizes them to the reference's values bit for bit
    (tests/golden/make_reference_expertwise.py wrote the fixture from mfq/quantize/expert_nint.py:507-578)."""
    from tyloquant_amd.quantize import nint_quantize_expertwise
    fx = np.load(Path(__file__).resolve().parent / "golden" / "reference_expertwise.npz")
    W, profiles = fx[f"{case}_weight"], [tuple(p) for p in fx[f"{case}_profiles"].tolist()]
    want = fx[f"{case}_blob"].tobytes()
    t = O.quantize_expertwise(W, profiles)
    assert O.pack_nint_moe(t) == want
    assert np.concatenate([p.expert_ids for p in t.pools]).tolist() == fx[f"{case}_pool_ids"].tolist()
    assert [len(p.expert_ids) for p in t.pools] == fx[f"{case}_pool_sizes"].tolist()
    deq = O.dequantize_expertwise(t)
    assert np.array_equal(deq.view(np.uint32), fx[f"{case}_deq"].view(np.uint32))
    pools, blob = nint_quantize_expertwise(W, profiles)
    assert blob == want
    # the quantized tensor stays close to the weights it came from: a dropped cohort or a permuted expert would not
    err = np.abs(deq - W).max(axis=(1, 2)) / np.abs(W).max(axis=(1, 2))
    assert (err < 0.35).all(), err
    with pytest.raises(ValueError):
        O.quantize_expertwise(W, profiles[:-1])
    with pytest.raises(ValueError):
        nint_quantize_expertwise(W[0], profiles)
