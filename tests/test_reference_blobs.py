"""Blobs and dequantized arrays written by the reference's own packers and dequantizers (tests/golden/
reference_blobs.npz, made by tests/golden/make_reference_blobs.py) against the oracle and the product: byte-identical
packing, bit-identical values.  This pins what a round trip cannot: the order of the streams inside a blob, the
tensor-wide (not per-row) bit packing, which 96 weights a NEPQ bank id covers, the index-parity sign rule."""
from pathlib import Path

import numpy as np
import pytest

from oracle import mfq_oracle as O

G = np.load(Path(__file__).resolve().parent / "golden" / "reference_blobs.npz")


def _bits_equal(a, b):
    a, b = np.asarray(a, dtype=np.float32), np.asarray(b, dtype=np.float32)
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


def _nint(key):
    rows, K, bits, gs, sb = (int(v) for v in G[f"{key}_meta"])
    return O.NintTensor(bits, gs, sb, (rows, K), 0, K, G[f"{key}_q"], G[f"{key}_ns"], G[f"{key}_nm"], G[f"{key}_ss"],
                        G[f"{key}_sm"])


def _nvq_jsc(key):
    rows, K, banks = (int(v) for v in G[f"{key}_meta"])
    return O.NvqJscTensor(bytes(G[f"{key}_codebook"]).decode(), (rows, K), K, G[f"{key}_anchors"], G[f"{key}_lut"],
                          G[f"{key}_bank_for_state"], G[f"{key}_state"], G[f"{key}_indices"], G[f"{key}_signs"],
                          G[f"{key}_codebooks"])


def _nepq(key, label):
    E, rows, K, banks = (int(v) for v in G[f"{key}_meta"])
    return O.NepqTensor(label, (E, rows, K), G[f"{key}_anchors"], G[f"{key}_state"], G[f"{key}_indices"], G[f"{key}_aux"],
                        G[f"{key}_bank_ids"], G[f"{key}_tables"])


@pytest.mark.parametrize("key", ["nint3", "nint4", "nint5"])
def test_nint_blob_and_values_match_the_reference(key):
    from tyloquant_amd import formats as F
    t = _nint(key)
    blob = bytes(G[f"{key}_blob"])
    assert O.pack_nint(t) == blob
    assert F.nint_blob(t.bits, t.sub_bits, t.groupsize, t.neuron_len, t.neuron_scale, t.neuron_min, t.sub_scale,
                       t.sub_min, t.q) == blob
    back = O.unpack_nint(blob)
    assert np.array_equal(back.q, t.q) and np.array_equal(back.sub_scale, t.sub_scale)
    assert _bits_equal(O.dequantize_nint(back), G[f"{key}_deq"])
    h = F.parse_nint(blob)
    assert (h.bits, h.gs, h.sub_bits, h.out, h.neuron_len, h.legacy) == (t.bits, t.groupsize, t.sub_bits, t.out,
                                                                          t.neuron_len, False)


@pytest.mark.parametrize("key", ["nvq3j512", "nvq3j"])
def test_nvq_jsc_blob_and_values_match_the_reference(key):
    from tyloquant_amd import formats as F
    t = _nvq_jsc(key)
    blob = bytes(G[f"{key}_blob"])
    assert O.pack_nvq_jsc(t) == blob
    assert F.nvq_jsc_blob(t.codebook, t.neuron_len, t.neuron_scale, t.scale_lut, t.bank_for_state, t.codebooks, t.state,
                          t.indices, t.signs) == blob
    assert _bits_equal(O.dequantize_nvq_jsc(O.unpack_nvq(blob)), G[f"{key}_deq"])


def test_plain_nvq3_and_index_parity_signs_match_the_reference():
    rows, K = (int(v) for v in G["nvq3_meta"])
    t = O.NvqTensor("d4_256", (rows, K), K, G["nvq3_anchors"], G["nvq3_sub_scale"], G["nvq3_indices"], G["nvq3_signs"])
    assert O.pack_nvq_plain(t) == bytes(G["nvq3_blob"])
    assert _bits_equal(O.dequantize_nvq(O.unpack_nvq(bytes(G["nvq3_blob"]))), G["nvq3_deq"])
    # e8_256 with the index-parity rule: the eighth sign of a vector = parity of the seven stored bits XOR bit 7 of its index
    rows, K = (int(v) for v in G["nvq2ip_meta"])
    ip = O.unpack_nvq(bytes(G["nvq2ip_blob"]))
    assert ip.sign_mode == "index_parity" and ip.codebook == "e8_256"
    assert np.array_equal(ip.indices, G["nvq2ip_indices"]) and np.array_equal(ip.signs, G["nvq2ip_signs"])
    assert _bits_equal(O.dequantize_nvq(ip), G["nvq2ip_deq"])


@pytest.mark.parametrize("key,label", [("nepq1s", "NEPQ1-S"), ("nepq1l", "NEPQ1-L")])
def test_nepq_blob_and_values_match_the_reference(key, label):
    from tyloquant_amd import formats as F
    t = _nepq(key, label)
    blob = bytes(G[f"{key}_blob"])
    assert O.pack_nepq(t) == blob
    assert F.nepq_blob(label, t.shape, t.table_payloads, t.neuron_scale, t.state, t.indices, t.aux, t.bank_ids) == blob
    assert _bits_equal(O.dequantize_nepq(O.unpack_nepq(blob)), G[f"{key}_deq"])


def test_nintm_container_and_values_match_the_reference():
    from tyloquant_amd import formats as F
    E, rows, K = (int(v) for v in G["nintm_meta"])
    blob = bytes(G["nintm_blob"])
    t = O.unpack_nint_moe(blob)
    assert t.shape == (E, rows, K) and len(t.pools) == 2
    for pi, p in enumerate(t.pools):
        assert np.array_equal(p.expert_ids, G[f"nintm_pool{pi}_ids"]) and np.array_equal(p.tensor.q, G[f"nintm_pool{pi}_q"])
    assert O.pack_nint_moe(t) == blob
    assert _bits_equal(O.dequantize_expertwise(t), G["nintm_deq"])
    h = F.parse_nintm(blob)
    assert (h.n_experts, h.out_per_expert, h.neuron_len) == (E, rows, K)
    assert [p.dtype for p in h.pools] == [p.dtype for p in t.pools]


@pytest.mark.gpu
def test_device_dequantizers_reproduce_the_reference_values():
    """The HIP repack + dequantizer on the reference-written bytes, bit for bit against the reference's own values."""
    pytest.importorskip("torch")
    from tyloquant_amd import runtime as R
    from tyloquant_amd.runtime_moe import NintMoeWeight
    for key, dtype in (("nint3", "NINT3"), ("nint4", "NINT4"), ("nint5", "NINT5"), ("nvq3j512", "NVQ3J-512"),
                       ("nvq3j", "NVQ3J"), ("nvq3", "NVQ3")):
        lin = R.load_quant_linear(dtype, bytes(G[f"{key}_blob"]))
        assert _bits_equal(lin.dequantize().cpu().numpy(), G[f"{key}_deq"]), key
    from tyloquant_amd.runtime_vq import NepqWeight
    for key in ("nepq1s", "nepq1l"):
        w = NepqWeight.from_blob(bytes(G[f"{key}_blob"]))
        assert _bits_equal(w.dequantize().cpu().numpy(), G[f"{key}_deq"]), key
    moe = NintMoeWeight.from_blob(bytes(G["nintm_blob"]))
    assert _bits_equal(moe.dequantize().cpu().numpy(), G["nintm_deq"])
