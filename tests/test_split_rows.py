"""formats.split_rows: the per-expert blobs cut from a cohort tensor of the NVQ, 1-bit and NINT8-0 families parse on their own and
dequantize (oracle) to the expert's rows of the whole tensor, bit for bit -- for streams whose per-expert share does not
start on a byte boundary."""
import numpy as np
import pytest

import synth
from oracle import mfq_oracle as O
from tyloquant_amd import formats as F

CASES = {
    "NVQ3J-512": lambda rng: synth.nvq_jsc_random(rng, 45, 100, "d4_512", 2),
    "NVQ3J-L": lambda rng: synth.nvq_jsc_random(rng, 45, 100, "d4_1024", 4),
    "NVQ2J-L": lambda rng: synth.nvq_jsc_random(rng, 45, 104, "e8_1024", 2),
    "NVQ3": lambda rng: synth.nvq_plain_random(rng, 45, 100),
    "NVQ2": lambda rng: synth.nvq_plain_e8_random(rng, 45, 100, "index_parity"),
    "NVQ1-L": lambda rng: synth.nvq1_random(rng, "NVQ1-L", 45, 100, 3),
    "NVQ1-S": lambda rng: synth.nvq1_random(rng, "NVQ1-S", 45, 104, custom=True),
    "NPQ0-L": lambda rng: synth.npq0_random(rng, "NPQ0-L", 45, 104),
    "NPQ0-S": lambda rng: synth.npq0_random(rng, "NPQ0-S", 45, 104),
    "NINT8-0": lambda rng: O.quantize_nint8_zero((rng.standard_normal((45, 96)) * 0.02).astype(np.float32)),
}


@pytest.mark.parametrize("dtype", list(CASES))
@pytest.mark.parametrize("parts", [1, 3, 5, 45])
def test_pieces_hold_the_rows_of_the_whole(dtype, parts):
    rng = np.random.default_rng(len(dtype) * 100 + parts)
    got_dtype, blob = O.pack_tensor(CASES[dtype](rng))
    assert got_dtype == dtype
    full = O.dequantize_tensor(O.unpack_tensor(dtype, blob))
    pieces = F.split_rows(dtype, blob, parts)
    assert len(pieces) == parts
    rows = np.concatenate([O.dequantize_tensor(O.unpack_tensor(dtype, p)) for p in pieces])
    assert np.array_equal(rows.view(np.uint32), full.view(np.uint32))
    if parts == 1:
        assert O.dequantize_tensor(O.unpack_tensor(dtype, pieces[0])).shape == full.shape


def test_uneven_split_is_refused():
    _, blob = O.pack_tensor(CASES["NVQ3J-512"](np.random.default_rng(0)))
    with pytest.raises(ValueError, match="do not split"):
        F.split_rows("NVQ3J-512", blob, 4)
