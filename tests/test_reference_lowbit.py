"""The 1-bit families (NVQ1-L, NVQ1-S, NPQ0-L, NPQ0-S) against blobs and dequantized arrays written by the reference's own
packers and dequantizers (tests/golden/reference_lowbit.npz, made by tests/golden/make_reference_lowbit.py):
byte-identical packing, bit-identical values.  Pins the stream order (anchors, scales / states, indices, delta signs), the
tensor-wide bit packing, which bank and which delta a group's sign bit selects, the index split of the product codebooks
and the vector count of a ragged NVQ1-L row."""
from pathlib import Path

import numpy as np
import pytest

from oracle import mfq_oracle as O

G = np.load(Path(__file__).resolve().parent / "golden" / "reference_lowbit.npz")

NVQ1 = {"nvq1l_grid": "NVQ1-L", "nvq1l_custom": "NVQ1-L", "nvq1s_default": "NVQ1-S", "nvq1s_custom": "NVQ1-S"}
NPQ0 = {"npq0l": "NPQ0-L", "npq0s": "NPQ0-S"}


def _bits_equal(a, b):
    a, b = np.asarray(a, dtype=np.float32), np.asarray(b, dtype=np.float32)
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


def _nvq1(key):
    label = NVQ1[key]
    meta = [int(v) for v in G[f"{key}_meta"]]
    rows, K = meta[0], meta[1]
    sbits = meta[2] if label == "NVQ1-L" else 4
    cb = G[f"{key}_cb"] if G[f"{key}_cb"].size else None
    return O.Nvq1Tensor(label, (rows, K), 0, K, sbits, G[f"{key}_ns"], G[f"{key}_sub"], G[f"{key}_idx"], G[f"{key}_dsg"], cb)


def _npq0(key):
    rows, K = (int(v) for v in G[f"{key}_meta"])
    return O.Npq0Tensor(NPQ0[key], (rows, K), 0, K, G[f"{key}_ns"], G[f"{key}_lut"], G[f"{key}_state"], G[f"{key}_idx"],
                        G[f"{key}_first"], G[f"{key}_second"])


@pytest.mark.parametrize("key", list(NVQ1))
def test_nvq1_blob_and_values_match_the_reference(key):
    t = _nvq1(key)
    blob = bytes(G[f"{key}_blob"])
    assert O.pack_nvq1(t) == blob
    back = O.unpack_nvq1(blob, t.label)
    assert np.array_equal(back.indices, t.indices) and np.array_equal(back.sub_scale, t.sub_scale)
    assert np.array_equal(back.delta_sign, t.delta_sign) and back.state_bits == t.state_bits
    assert _bits_equal(O.dequantize_nvq1(back), G[f"{key}_deq"])
    assert _bits_equal(O.dequantize_tensor(O.unpack_tensor(t.label, blob)), G[f"{key}_deq"])
    with pytest.raises(ValueError, match="blob tail"):
        O.unpack_nvq1(blob + b"\0", t.label)
    with pytest.raises(ValueError, match="magic"):
        O.unpack_nvq1(b"XXXX" + blob[4:], t.label)


@pytest.mark.parametrize("key", list(NPQ0))
def test_npq0_blob_and_values_match_the_reference(key):
    t = _npq0(key)
    blob = bytes(G[f"{key}_blob"])
    assert O.pack_npq0(t) == blob
    back = O.unpack_npq0(blob, t.label)
    assert np.array_equal(back.indices, t.indices) and np.array_equal(back.state, t.state)
    assert np.array_equal(back.first_codebooks, t.first_codebooks) and np.array_equal(back.second_codebooks, t.second_codebooks)
    assert _bits_equal(O.dequantize_npq0(back), G[f"{key}_deq"])
    bad = bytearray(blob)
    bad[O._LOWBIT_HDR.size + 2 * 8 + 4 + 40] = 1      # a reserved byte of the table header
    with pytest.raises(ValueError, match="reserved"):
        O.unpack_npq0(bytes(bad), t.label)


@pytest.mark.parametrize("key,label", [("nepq0s", "NEPQ0-S"), ("nepq0l", "NEPQ0-L")])
def test_nepq0_blob_and_values_match_the_reference(key, label):
    """The expert form: NPQ0 tables in the NEPQ container's pool, one bank id per neuron and 96 weights."""
    E, rows, K, banks = (int(v) for v in G[f"{key}_meta"])
    t = O.NepqTensor(label, (E, rows, K), G[f"{key}_anchors"], G[f"{key}_state"], G[f"{key}_indices"], G[f"{key}_aux"],
                     G[f"{key}_bank_ids"], G[f"{key}_tables"])
    blob = bytes(G[f"{key}_blob"])
    assert O.pack_nepq(t) == blob
    back = O.unpack_nepq(blob)
    assert back.label == label and np.array_equal(back.bank_ids, t.bank_ids) and np.array_equal(back.indices, t.indices)
    assert _bits_equal(O.dequantize_nepq(back), G[f"{key}_deq"])
    bad = bytearray(blob)
    bad[O._NEPQ_HDR.size + 1] ^= 0xFF                       # the state count of the first table's header
    with pytest.raises(ValueError, match="table profile"):
        O.unpack_nepq(bytes(bad))


def test_lowbit_mistakes_the_fixture_would_catch():
    """The checks above are not vacuous: swapping the delta's sign, taking the bank from the wrong bit, or splitting the
    product index the other way round changes the values."""
    t = _nvq1("nvq1s_custom")
    good = O.dequantize_nvq1(t)
    flipped = O.Nvq1Tensor(t.label, t.shape, 0, t.neuron_len, 4, t.neuron_scale, t.sub_scale, t.indices, 1 - t.delta_sign,
                           t.codebook)
    assert not _bits_equal(O.dequantize_nvq1(flipped), good)
    p = _npq0("npq0l")
    swapped = O.Npq0Tensor(p.label, p.shape, 0, p.neuron_len, p.neuron_scale, p.scale_lut, p.state,
                           ((p.indices & 7) << 3 | (p.indices >> 3)) & 127, p.first_codebooks, p.second_codebooks)
    assert not _bits_equal(O.dequantize_npq0(swapped), O.dequantize_npq0(p))
