"""Pins of the oracle's MXFP4 / MXFP8 restatement: a reference-written payload and reference-decoded values
(tests/golden/reference_mx.npz), torch's own float8_e4m3fn conversion, and the closed forms of E2M1 and E8M0."""
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import mfq_oracle as O

G = np.load(Path(__file__).resolve().parent / "golden" / "reference_mx.npz")


def same(a, b):
    """bit-equal, any NaN matching any NaN and -0 matching +0: the E2M1 code 8 decodes to +0 in the reference's Python
    decoder (mfq/quantize/mxfp.py, which wrote the fixture) and to -0 in its runtime (cpp_runtime/mfq_decode.cpp:1943-1945),
    which the oracle follows"""
    a, b = np.asarray(a, np.float32), np.asarray(b, np.float32)
    if a.shape != b.shape or not np.array_equal(np.isnan(a), np.isnan(b)):
        return False
    a, b = np.where(np.isnan(a) | (a == 0), np.float32(0), a), np.where(np.isnan(b) | (b == 0), np.float32(0), b)
    return np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("key,dtype", [("fp4", "MXFP4"), ("fp8", "MXFP8")])
def test_reference_payload_bytes_and_values(key, dtype):
    values, scales, blob = G[f"{key}_values"], G[f"{key}_scales"], G[f"{key}_blob"].tobytes()
    shape = (values.shape[0], values.shape[1] * (2 if dtype == "MXFP4" else 1))
    t = O.MxTensor(dtype, shape, values, scales)
    assert O.pack_mx(t) == blob
    back = O.unpack_mx(dtype, blob)
    assert back.shape == shape and np.array_equal(back.values, values) and np.array_equal(back.scales, scales)
    assert O.unpack_tensor(dtype, blob).dtype == dtype and O.pack_tensor(back) == (dtype, blob)
    want = G[f"{key}_dequant"]
    assert np.isnan(want).any()  # the fixture holds a NaN scale (and, for MXFP8, the NaN codes)
    assert same(O.dequantize_mx(back), want)
    assert same(O.dequantize_tensor(back), want)


def test_e4m3fn_matches_torch_on_every_code():
    raw = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(raw).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert same(O.decode_e4m3fn(raw), want)
    assert np.isnan(want[[0x7F, 0xFF]]).all() and np.isfinite(np.delete(want, [0x7F, 0xFF])).all()
    assert want[0x7E] == 448.0 and want[0x01] == 2.0 ** -9


def test_e2m1_and_e8m0_closed_forms():
    # E2M1: exponent bias 1, one mantissa bit, subnormal step 0.5
    for code in range(8):
        e, m = code >> 1, code & 1
        assert O.FP4_E2M1[code] == (0.5 * m if e == 0 else 2.0 ** (e - 1) * (1 + 0.5 * m))
    raw = np.arange(255, dtype=np.uint8)
    s = O.decode_e8m0(raw)
    mant, exp = np.frexp(s.astype(np.float64))
    assert (mant == 0.5).all() and np.array_equal(exp - 1, raw.astype(np.int64) - 127)
    assert np.isnan(O.decode_e8m0(np.uint8(255)))
    # low nibble = even column, sign bit 8
    t = O.MxTensor("MXFP4", (1, 32), np.array([[0x2F] + [0] * 15], np.uint8), np.array([[128]], np.uint8))
    d = O.dequantize_mx(t)
    assert d[0, 0] == -12.0 and d[0, 1] == 2.0 and not d[0, 2:].any()


def test_mx_geometry_and_header_errors():
    with pytest.raises(ValueError, match="MXFP4 columns must be divisible by 32"):
        O.mx_shapes("MXFP4", (4, 48))
    with pytest.raises(ValueError, match="MXFP8 columns must be divisible by 128"):
        O.mx_shapes("MXFP8", (4, 96))
    assert O.mx_shapes("MXFP8", (129, 256)) == ((129, 256), (2, 2))
    blob = G["fp4_blob"].tobytes()
    with pytest.raises(ValueError, match="truncated MFQ MX tensor header"):
        O.unpack_mx("MXFP4", blob[:20])
    with pytest.raises(ValueError, match="invalid MXFP8 payload header"):
        O.unpack_mx("MXFP8", blob)
    with pytest.raises(ValueError, match="payload size"):
        O.unpack_mx("MXFP4", blob + b"\0")


@pytest.mark.parametrize("key,dtype", [("fp4", "MXFP4"), ("fp8", "MXFP8")])
def test_host_parser_and_writer_on_the_reference_payload(key, dtype):
    """tyloquant_amd.formats: the product's own parser and writer, same bytes, same messages."""
    from tyloquant_amd import formats as F
    blob = G[f"{key}_blob"].tobytes()
    h = F.parse_mx(dtype, blob)
    values, scales = G[f"{key}_values"], G[f"{key}_scales"]
    assert (h.rows, h.cols * (1 if dtype == "MXFP8" else 1)) == (values.shape[0], values.shape[1] * (2 if dtype == "MXFP4" else 1))
    assert blob[h.values_off: h.values_off + h.values_bytes] == values.tobytes()
    assert blob[h.scales_off: h.scales_off + h.scales_bytes] == scales.tobytes()
    assert F.write_mx(dtype, h.rows, h.cols, values, scales) == blob
    other = "MXFP8" if dtype == "MXFP4" else "MXFP4"
    with pytest.raises(ValueError, match=f"invalid {other} payload header"):
        F.parse_mx(other, blob)
    with pytest.raises(ValueError, match="payload size"):
        F.parse_mx(dtype, blob[:-1])
    with pytest.raises(ValueError, match="truncated MFQ MX tensor header"):
        F.parse_mx(dtype, blob[:55])

