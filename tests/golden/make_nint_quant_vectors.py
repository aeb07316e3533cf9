"""Write golden input/output vectors for the NINT weight-only quantizer.

`nint_quant.quantize` / `make_qkx2` (mfq/quantize/nint_quant.py:745-893,
mfq/formats/nint.py:119-174) depend on numpy's fp32 reduction order and tie
rounding, which no closed form pins.  This script imports the reference's
numpy quantizer IN THE BUILD CONTAINER ONLY (from /root/reference; it needs
numpy and nothing else), runs it on small seeded matrices, and stores inputs
and outputs in tests/golden/nint_quant_vectors.npz.  The fixture is data; the
reference itself never travels.

    python tests/golden/make_nint_quant_vectors.py
"""
import sys
from pathlib import Path

import numpy as np

sys.path.insert(0, "/root/reference")
from mfq.formats.nint import NintSpec  # noqa: E402
from mfq.quantize import nint_quant  # noqa: E402

CASES = [  # (seed, out, K, bits, gs, sub_bits, sigma)
    (0, 8, 96, 4, 24, 6, 0.02), (1, 8, 96, 3, 24, 5, 0.02), (2, 17, 257, 4, 32, 6, 0.02),
    (3, 5, 88, 2, 16, 5, 0.02), (4, 6, 112, 5, 28, 7, 0.02), (5, 4, 100, 6, 24, 6, 1.0),
    (6, 3, 73, 8, 24, 8, 0.5), (7, 16, 4096, 3, 24, 5, 0.02),
]

out = {}
for seed, rows, K, bits, gs, sb, sigma in CASES:
    rng = np.random.default_rng(seed)
    W = (rng.standard_normal((rows, K)) * sigma).astype(np.float32)
    if seed == 5:
        W[1] = 0.0            # degenerate all-zero neuron
        W[2, :24] = 0.25      # constant group
    t = nint_quant.quantize(W, NintSpec(bits=bits, groupsize=gs, sub_bits=sb))
    deq = nint_quant.dequantize(t)
    key = f"c{seed}"
    out[key + "_meta"] = np.array([seed, rows, K, bits, gs, sb], dtype=np.int64)
    out[key + "_W"] = W
    out[key + "_q"] = t.q.astype(np.uint8)
    out[key + "_ns"] = t.neuron_scale.astype(np.float32)
    out[key + "_nm"] = t.neuron_min.astype(np.float32)
    out[key + "_ss"] = t.sub_scale.astype(np.uint8)
    out[key + "_sm"] = t.sub_min.astype(np.uint8)
    out[key + "_deq"] = deq.astype(np.float32)
np.savez_compressed(Path(__file__).with_name("nint_quant_vectors.npz"), **out)
print("wrote", len(CASES), "cases")
