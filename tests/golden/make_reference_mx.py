"""Write reference-made MXFP4 / MXFP8 payloads and their reference-decoded values.

As the other make_reference_*.py scripts: the reference's own modules are imported IN THE BUILD CONTAINER ONLY (from
/root/reference: mfq.formats.mx for the container, mfq.quantize.mxfp for decode_mxfp4 / decode_mxfp8; numpy and CPU
torch, nothing else), fed seeded random bytes, and the inputs, the packed bytes and the decoded fp32 arrays are stored in
tests/golden/reference_mx.npz.  The fixture is data; the reference never travels.

    python tests/golden/make_reference_mx.py
"""
import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
sys.path.insert(0, "/root/reference")
from mfq.formats.mx import MxTensor, pack_mx, unpack_mx  # noqa: E402
from mfq.quantize.mxfp import decode_mxfp4, decode_mxfp8  # noqa: E402

rng = np.random.default_rng(4048)
out = {}

# MXFP4: every nibble value, scales over the whole E8M0 range incl. 0 (2^-127), 254 and 255 (NaN)
rows, cols = 6, 160
v4 = rng.integers(0, 256, (rows, cols // 2), dtype=np.uint8)
s4 = rng.integers(100, 150, (rows, cols // 32), dtype=np.uint8)
s4[0, 0], s4[1, 1], s4[2, 2], s4[3, 3] = 0, 254, 255, 1
blob4 = pack_mx(MxTensor("MXFP4", (rows, cols), v4, s4))
back = unpack_mx("MXFP4", blob4)
assert np.array_equal(back.values, v4) and np.array_equal(back.scales, s4)
out["fp4_values"], out["fp4_scales"] = v4, s4
out["fp4_blob"] = np.frombuffer(blob4, dtype=np.uint8)
out["fp4_dequant"] = decode_mxfp4(v4, s4, device="cpu").numpy()

# MXFP8: all 256 codes in the first rows, two block rows (the second one partial), three block columns
rows, cols = 200, 384
v8 = rng.integers(0, 256, (rows, cols), dtype=np.uint8)
v8[0, :256] = np.arange(256, dtype=np.uint8)
s8 = rng.integers(110, 140, (2, 3), dtype=np.uint8)
s8[1, 2] = 255
blob8 = pack_mx(MxTensor("MXFP8", (rows, cols), v8, s8))
out["fp8_values"], out["fp8_scales"] = v8, s8
out["fp8_blob"] = np.frombuffer(blob8, dtype=np.uint8)
out["fp8_dequant"] = decode_mxfp8(v8, s8, row_start=0, total_rows=rows, device="cpu").numpy()

np.savez_compressed(HERE / "reference_mx.npz", **out)
print({k: v.shape for k, v in out.items()})
