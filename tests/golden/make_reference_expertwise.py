"""Write a reference-made expert-wise (NINTM) quantization of a small seeded [experts, out, K] tensor.

quantize_expertwise groups the experts by precision (cohorts in the order their precision first appears, experts in
ascending order inside a cohort), quantizes each cohort's flattened rows with the NINT quantizer and packs the pools
into one NIM2 blob.  Nothing but the reference itself fixes the cohort order and the blob's pool order, so this script
imports the reference's quantizer IN THE BUILD CONTAINER ONLY (from /root/reference: mfq.quantize.expert_nint,
mfq.formats.{io,nint}; numpy and CPU torch) and stores the weights, the profiles, the packed bytes and the values the
reference dequantizes them to.  The fixture (tests/golden/reference_expertwise.npz) is data; the reference never travels.

    python tests/golden/make_reference_expertwise.py
"""
import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
sys.path.insert(0, "/root/reference")
from mfq.formats import io as rio  # noqa: E402
from mfq.formats.nint import NintSpec  # noqa: E402
from mfq.quantize.expert_nint import dequantize_expertwise, quantize_expertwise  # noqa: E402

rng = np.random.default_rng(77)
out = {}
# two cases: six experts in four cohorts whose precisions first appear out of numeric order, a ragged K;
# and five experts of one precision (a single cohort)
CASES = {
    "mixed": ((6, 16, 100), [(4, 24, 6), (2, 16, 5), (4, 24, 6), (5, 28, 7), (3, 24, 5), (2, 16, 5)]),
    "single": ((5, 8, 72), [(3, 24, 5)] * 5),
}
for key, (shape, profiles) in CASES.items():
    W = (rng.standard_normal(shape) * 0.02).astype(np.float32)
    W[0, 3] = 0.0                      # an all-zero neuron
    W[1, :, 10:20] *= 20.0             # outlier columns in one expert
    specs = [NintSpec(bits=b, groupsize=g, sub_bits=s) for b, g, s in profiles]
    t = quantize_expertwise(W, specs, device="cpu")
    out[f"{key}_weight"] = W
    out[f"{key}_profiles"] = np.asarray(profiles, dtype=np.int32)
    out[f"{key}_blob"] = np.frombuffer(bytes(rio.pack_nint_moe(t)), dtype=np.uint8)
    out[f"{key}_deq"] = dequantize_expertwise(t)
    out[f"{key}_pool_ids"] = np.concatenate([np.asarray(p.expert_ids, dtype=np.int32) for p in t.pools])
    out[f"{key}_pool_sizes"] = np.asarray([len(p.expert_ids) for p in t.pools], dtype=np.int32)

np.savez_compressed(HERE / "reference_expertwise.npz", **out)
print("wrote", len(out), "arrays,", sum(a.nbytes for a in out.values()), "bytes")
